"""Paths of the HIP operator that the shape-matrix tests do not reach:

* float16 with a state beyond the float16 range: the reference keeps its kv state and the inter-block product in
  float32 (lightning_attn2.py:55, 72-74), so it cannot overflow; here the state is float32 too, but the MFMA takes
  it as float16 fragments, which are clamped to +-65504 instead of becoming inf.  Asserted: finite results that
  follow the block recurrence with the clamped state (not the exact one), and bfloat16 on the same inputs exact.
* a chunk plan that wants a workspace, given none / a short one / a misaligned one: the warm-up form must step in,
  bit-identical to the single walk and equal to the oracle to the usual tolerance (through the C ABI).
* `o.sum().backward()`: the upstream gradient autograd hands over is an expanded scalar (all strides zero).
* the first launch of a shape inside a stream capture after la_init() (fresh process)."""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

import oracle
from util import assert_close_scaled, rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops import lightning_attn_func  # noqa: E402
from lightning_attn.ops.hip import _lib  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _recurrence_with_clamped_state(q, k, v, clamp, block=64):
    """Forward by the block recurrence without decay (lightning_attn2_no_decay.py:41-77), float64, with the
    state entering the inter-block product clamped to +-clamp as the float16 fragments of the kernel are."""
    b, h, n, d = q.shape
    e = v.shape[-1]
    q, k, v = q.double(), k.double(), v.double()
    kv = torch.zeros(b, h, d, e, dtype=torch.float64)
    out = torch.zeros(b, h, n, e, dtype=torch.float64)
    for t0 in range(0, n, block):
        sl = slice(t0, min(n, t0 + block))
        Q, K, V = q[:, :, sl], k[:, :, sl], v[:, :, sl]
        out[:, :, sl] = torch.tril(Q @ K.transpose(2, 3)) @ V + Q @ kv.clamp(-clamp, clamp)
        kv = kv + K.transpose(2, 3) @ V
    return out


def test_float16_state_beyond_the_float16_range_saturates():
    b, h, n, d, e = 1, 2, 2048, 64, 64
    g = torch.Generator().manual_seed(9)
    # k = v = 8 in every feature: each token adds 64 to every state entry, 65536 after 1024 tokens
    k = torch.full((b, h, n, d), 8.0)
    v = torch.full((b, h, n, e), 8.0)
    q = torch.zeros(b, h, n, d)
    q[..., 0] = 2.0 ** -11 * (1 + torch.rand(b, h, n, generator=g))  # o stays far inside the float16 range
    exact = oracle.linear_attn_f64(q.half(), k.half(), v.half(), None)
    clamped = _recurrence_with_clamped_state(q.half(), k.half(), v.half(), 65504.0)
    assert exact[:, :, -1].abs().max() < 3e4
    assert ((exact - clamped).abs() / exact.abs().clamp_min(1)).max() > 0.2  # the two models differ late in the sequence
    with torch.no_grad():
        o16 = lightning_attn_func(q.half().to(DEV), k.half().to(DEV), v.half().to(DEV), None)
        obf = lightning_attn_func(q.bfloat16().to(DEV), k.bfloat16().to(DEV), v.bfloat16().to(DEV), None)
    torch.cuda.synchronize()
    assert torch.isfinite(o16.float()).all()
    # float16: the clamped-state recurrence, not the exact sum
    assert rel_norm(o16, clamped) < 5e-3
    assert rel_norm(o16[:, :, 1100:], exact[:, :, 1100:]) > 0.05
    # before the state leaves the range the two agree
    assert rel_norm(o16[:, :, :1000], exact[:, :, :1000]) < 5e-3
    # bfloat16 has the range: the exact sum
    exact_bf = oracle.linear_attn_f64(q.bfloat16(), k.bfloat16(), v.bfloat16(), None)
    assert rel_norm(obf, exact_bf) < 5e-3


def _call_fwd_bwd(L, q, k, v, s, do, ws_ptr, ws_bytes, opts=None):
    b, h, n, d = q.shape
    e = v.shape[-1]
    o = torch.full_like(v, float("nan"))
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
    st = torch.cuda.current_stream().cuda_stream
    rc = L.la_fwd_opts(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), o.data_ptr(), None, b, h, n, d, e, 0,
                       ws_ptr, ws_bytes, opts, st)
    assert rc == 0, L.la_error_string(rc)
    rc = L.la_bwd_opts(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), do.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                       dv.data_ptr(), None, b, h, n, d, e, 0, ws_ptr, ws_bytes, opts, st)
    assert rc == 0, L.la_error_string(rc)
    torch.cuda.synchronize()
    return o, dq, dk, dv


@pytest.mark.parametrize("b, h, n, d", [(1, 8, 4096, 128), (1, 4, 3000, 192)])
def test_scan_plan_without_a_usable_workspace_falls_back_to_warm_up_chunks(b, h, n, d):
    import ctypes

    L = _lib.lib()
    need = max(L.la_workspace_bytes(0, b, h, n, d, d, 0), L.la_workspace_bytes(1, b, h, n, d, d, 0))
    assert need > 0  # the library plans chunks from scanned states for this shape
    g = torch.Generator().manual_seed(17)
    q, k, v, do = (torch.randn(b, h, n, d, generator=g).bfloat16() for _ in range(4))
    s = _build_slope_tensor(h).float().reshape(h)
    want = oracle.linear_attn_fwd_bwd(q[:, :2], k[:, :2], v[:, :2], s[:2], do[:, :2], torch.float32)
    q, k, v, do, s = (t.to(DEV).contiguous() for t in (q, k, v, do, s))
    ws = torch.empty(need + 64, dtype=torch.uint8, device=DEV)
    base = ws.data_ptr()
    assert base % 16 == 0
    single = _lib.LaunchOpts(1, _lib.LA_OPT_OFF, 0, 0, _lib.LA_OPT_OFF)  # one walk per sequence, separate launches
    ref = _call_fwd_bwd(L, q, k, v, s, do, None, 0, ctypes.byref(single))
    for name, ptr, nbytes in (("scanned", base, need), ("no workspace", None, 0), ("short", base, 16),
                              ("misaligned", base + 4, need)):
        print("workspace case", (b, h, n, d), name, flush=True)
        got = _call_fwd_bwd(L, q, k, v, s, do, ptr, nbytes)
        for tname, a, r in zip(("o", "dq", "dk", "dv"), got, want):
            assert_close_scaled(a[:, :2], r, 2e-2, 2e-2, "%s %s" % (name, tname))
            assert rel_norm(a[:, :2], r) < 1e-2
        if name != "scanned":
            # warm-up chunks rebuild the state block by block in the order of the single walk
            for a, r in zip(got, ref):
                assert torch.equal(a, r), name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sum_backward_hands_over_an_expanded_gradient(dtype):
    """configs[0]: b1 h8 n1024 d=e=64, loss = o.sum()."""
    b, h, n, d = 1, 8, 1024, 64
    g = torch.Generator().manual_seed(2024)
    q, k, v = (torch.randn(b, h, n, d, generator=g).to(dtype) for _ in range(3))
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, torch.ones(b, h, n, d), torch.float64 if dtype == torch.float32 else torch.float32)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = lightning_attn_func(qg, kg, vg, s.to(DEV))
    o.sum().backward()
    torch.cuda.synchronize()
    for name, a, r in zip(("o", "dq", "dk", "dv"), (o.detach(), qg.grad, kg.grad, vg.grad), want):
        if dtype == torch.float32:
            assert rel_norm(a, r) < 1e-4, (name, rel_norm(a, r))
        else:
            assert_close_scaled(a, r, 2e-2, 2e-2, name)
            assert rel_norm(a, r) < 1e-2, (name, rel_norm(a, r))


def test_first_launch_inside_a_capture_after_la_init():
    """A fresh process calls la_init() and then records la_fwd + la_bwd of shapes it has never launched straight into
    a graph; three replays on new data must equal what the same entry points give eagerly afterwards."""
    code = textwrap.dedent("""
        import sys
        sys.path[:0] = [%r, %r]
        import torch
        from lightning_attn.ops.hip import _lib
        from lightning_attn.utils import _build_slope_tensor
        L = _lib.lib()
        dev = torch.device("cuda")
        torch.zeros(1, device=dev)
        assert L.la_init() == 0
        for (b, h, n, d) in ((2, 4, 700, 128), (1, 3, 500, 192), (1, 2, 300, 64)):
            gen = torch.Generator(device=dev).manual_seed(1)
            fresh = lambda: tuple(torch.randn(b, h, n, d, generator=gen, device=dev).bfloat16() for _ in range(4))
            q, k, v, do = fresh()
            o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
            s = _build_slope_tensor(h).to(dev).reshape(h).contiguous()
            def enqueue(outs):
                st = _lib.stream_ptr(dev)
                o_, dq_, dk_, dv_ = outs
                assert L.la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), o_.data_ptr(), b, h, n, d, d, 0, None, 0, st) == 0
                assert L.la_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), do.data_ptr(), dq_.data_ptr(), dk_.data_ptr(),
                                dv_.data_ptr(), b, h, n, d, d, 0, None, 0, st) == 0
            print("capture case", (b, h, n, d), flush=True)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                enqueue((o, dq, dk, dv))
            for rep in range(3):
                for dst, src in zip((q, k, v, do), fresh()):
                    dst.copy_(src)
                for t in (o, dq, dk, dv):
                    t.fill_(float("nan"))
                graph.replay()
                torch.cuda.synchronize()
                eager = tuple(torch.empty_like(q) for _ in range(4))
                enqueue(eager)
                torch.cuda.synchronize()
                for a, c in zip((o, dq, dk, dv), eager):
                    assert torch.equal(a, c) and not torch.isnan(a.float()).any(), (b, h, n, d, rep)
        print("capture ok")
    """) % (os.path.join(ROOT, "lightning-attention_amd"), ROOT)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0 and "capture ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
