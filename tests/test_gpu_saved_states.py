"""la_fwd_save / la_bwd_saved: the forward pass leaves its K^T V state at a few token boundaries and the dQ sweep
of the backward pass starts its chunks there (in place of lightning_attn2.py:240-280, which recomputes that
state walking forward).  Checked through the C ABI and through the autograd operators:

* the output of la_fwd_save is la_fwd's, bit for bit (same launch, the state is only written out as well);
* the saved matrices against the closed-form state of the fp64 oracle (oracle.kv_state);
* dk, dv of la_bwd_saved are la_bwd's bit for bit (same launches); dq agrees with la_bwd's to rounding and
  with the oracle to the tolerance of the other parity tests (util.assert_close_scaled, rtol = atol = 2e-2 with
  the absolute term scaled by the sequence RMS, relative Frobenius error < 1e-2);
* shapes the pair is not meant for report 0 bytes and behave exactly as la_fwd / la_bwd."""
import ctypes

import pytest
import torch

import oracle
from util import assert_close_scaled, rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops import lightning_attn_func  # noqa: E402
from lightning_attn.ops.hip import _lib, launch_opts  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"
CODE = {torch.bfloat16: 0, torch.float16: 1}


def _inputs(b, h, n, d, e, dtype, seed, token_major=False):
    g = torch.Generator().manual_seed(seed)

    def mk(c):
        if token_major:  # a (b, n, h*c) projection output viewed as (b, h, n, c)
            return torch.randn(b, n, h, c, generator=g).to(dtype).to(DEV).transpose(1, 2)
        return torch.randn(b, h, n, c, generator=g).to(dtype).to(DEV)

    return mk(d), mk(d), mk(e), mk(e)


def _strides(*ts):
    vals = []
    for t in ts:
        vals += list(t.stride())[:3]
    return (ctypes.c_int64 * len(vals))(*vals)


def _fwd(L, q, k, v, s, saved):
    b, h, n, d = q.shape
    e = v.shape[-1]
    o = torch.full_like(v, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    strides = None if q.is_contiguous() else _strides(q, k, v, o)
    rc = L.la_fwd_save(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None, o.data_ptr(),
                       strides, b, h, n, d, e, CODE[q.dtype], None, 0, None,
                       saved.data_ptr() if saved is not None else None, saved.numel() * 4 if saved is not None else 0, st)
    assert rc == 0, L.la_error_string(rc)
    return o


def _bwd(L, q, k, v, s, do, saved):
    b, h, n, d = q.shape
    e = v.shape[-1]
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
    st = torch.cuda.current_stream().cuda_stream
    strides = None if q.is_contiguous() else _strides(q, k, v, do, dq, dk, dv)
    rc = L.la_bwd_saved(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None, do.data_ptr(),
                        dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), strides, b, h, n, d, e, CODE[q.dtype], None, 0, None,
                        saved.data_ptr() if saved is not None else None, saved.numel() * 4 if saved is not None else 0, st)
    assert rc == 0, L.la_error_string(rc)
    return dq, dk, dv


CASES = [
    # b, h, n, d, e, dtype, decay, token_major
    (4, 32, 1536, 128, 128, torch.bfloat16, True, False),   # the benchmark's b*h: 2 chunks
    (3, 24, 1700, 128, 128, torch.bfloat16, True, False),   # 72 sequences: 3 chunks, the last one short and ragged
    (4, 32, 1555, 128, 104, torch.float16, True, False),    # e < d, fp16, ragged
    (2, 64, 1900, 72, 128, torch.bfloat16, False, False),   # no decay, d off the 64 grid
    (4, 32, 2048, 128, 128, torch.bfloat16, True, True),    # projection layout, used in place
    (4, 25, 1664, 96, 112, torch.bfloat16, True, True),
    # feature dims 129 .. 192: the forward pass in two column slices, dQ with all its columns in one workgroup
    (4, 32, 1536, 192, 192, torch.bfloat16, True, False),
    (4, 30, 1700, 176, 144, torch.float16, True, True),     # ragged, d != e, projection layout
    (3, 40, 1900, 136, 192, torch.bfloat16, False, False),  # no decay
]


@pytest.mark.parametrize("b, h, n, d, e, dtype, decay, token_major", CASES)
def test_saved_states_pair_through_the_c_abi(b, h, n, d, e, dtype, decay, token_major):
    L = _lib.lib()
    code = CODE[dtype]
    nbytes = L.la_saved_state_bytes(b, h, n, d, e, code, None)
    step = L.la_saved_state_interval(b, h, n, d, e, code, None)
    print("saved-state case", (b, h, n, d, e, dtype, decay, token_major), "bytes", nbytes, "interval", step, flush=True)
    assert nbytes > 0 and step > 0 and step % 64 == 0
    m = nbytes // (b * h * d * e * 4)
    assert m >= 1 and nbytes == m * b * h * d * e * 4
    assert m * step < n <= (m + 1) * step + 63  # boundaries inside the sequence, equally spaced
    q, k, v, do = _inputs(b, h, n, d, e, dtype, 31 + n, token_major)
    s = _build_slope_tensor(h).float().to(DEV).contiguous() if decay else None
    saved = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device=DEV)
    o_plain = _fwd(L, q, k, v, s, None)
    o_save = _fwd(L, q, k, v, s, saved)
    torch.cuda.synchronize()
    assert torch.equal(o_plain, o_save)
    # the saved matrices: KV_T at T = step, 2 step, ..., on a few sequences (the oracle is O(n d e) per matrix)
    S = saved.view(b * h, m, d, e)
    assert not torch.isnan(S).any()
    kc, vc, sc = k.cpu(), v.cpu(), (s.cpu() if decay else None)
    for j in range(m):
        want = oracle.kv_state(kc, vc, sc, (j + 1) * step).view(b * h, d, e)
        for u in (0, b * h // 2, b * h - 1):
            # operands rounded to the tensors' dtype (k as is, v scaled by the decay first): a few 1e-3 relative
            assert rel_norm(S[u, j], want[u]) < 5e-3, (u, j, rel_norm(S[u, j], want[u]))
    # backward: with and without the states
    g_plain = _bwd(L, q, k, v, s, do, None)
    g_saved = _bwd(L, q, k, v, s, do, saved)
    torch.cuda.synchronize()
    assert torch.equal(g_plain[1], g_saved[1]) and torch.equal(g_plain[2], g_saved[2])
    assert not torch.isnan(g_saved[0].float()).any()
    assert rel_norm(g_saved[0], g_plain[0].float()) < 3e-3
    # a subset of sequences against the naive oracle
    sel = [0, h - 1] if b == 1 else [0, h // 2, h - 1]
    qs, ks, vs, ds = (t[-1:, sel].cpu().contiguous() for t in (q, k, v, do))
    want = oracle.linear_attn_fwd_bwd(qs, ks, vs, sc[sel] if decay else None, ds, torch.float32)
    got = (o_save[-1:, sel], g_saved[0][-1:, sel], g_saved[1][-1:, sel], g_saved[2][-1:, sel])
    for name, a, r in zip(("o", "dq", "dk", "dv"), got, want):
        assert_close_scaled(a, r, 2e-2, 2e-2, "saved %s" % name)
        assert rel_norm(a, r) < 1e-2, (name, rel_norm(a, r))


def test_saved_states_through_autograd_and_the_opt_out():
    """The operators use the pair by themselves where the library asks for it; launch_opts(save_states=False)
    gives the inputs-only behaviour of the reference.  Same o, dk, dv bit for bit, dq to rounding."""
    b, h, n, d, e = 4, 32, 1536, 128, 128
    assert _lib.lib().la_saved_state_bytes(b, h, n, d, e, 0, None) > 0
    q, k, v, do = _inputs(b, h, n, d, e, torch.bfloat16, 5)
    s = _build_slope_tensor(h).to(DEV)
    per_path = []
    for native in (True, False):  # the C++ autograd nodes (where built), then the Python ones
        prev = _lib.use_native_ops(native)
        try:
            res = []
            for save in (True, False):
                qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
                with launch_opts(save_states=save):
                    o = lightning_attn_func(qg, kg, vg, s)
                    if hasattr(o.grad_fn, "saved_tensors"):  # (Python node)
                        node_saved = [t for t in o.grad_fn.saved_tensors if t is not None and t.dtype == torch.float32
                                      and t.dim() == 1 and t.numel() > h]
                        assert bool(node_saved) == save
                    o.backward(do)
                res.append((o.detach(), qg.grad, kg.grad, vg.grad))
        finally:
            _lib.use_native_ops(prev)
        torch.cuda.synchronize()
        (o1, dq1, dk1, dv1), (o0, dq0, dk0, dv0) = res
        assert torch.equal(o1, o0) and torch.equal(dk1, dk0) and torch.equal(dv1, dv0)
        assert rel_norm(dq1, dq0.float()) < 3e-3
        assert not torch.equal(dq1, dq0)  # the two dQ paths round differently: the states were really used
        per_path.append(res)
    for a, c in zip(per_path[0][0] + per_path[0][1], per_path[1][0] + per_path[1][1]):
        assert torch.equal(a, c)
    o1 = per_path[0][0][0]
    # no gradient wanted: nothing is saved
    with torch.no_grad():
        o = lightning_attn_func(q, k, v, s)
    assert torch.equal(o, o1)


@pytest.mark.parametrize("b, h, n, d, e, dtype", [(1, 8, 4096, 128, 128, torch.bfloat16), (8, 32, 512, 128, 128, torch.bfloat16),
                                                 (4, 32, 1024, 64, 64, torch.bfloat16), (4, 32, 1024, 256, 256, torch.bfloat16),
                                                 (4, 32, 1024, 192, 128, torch.bfloat16),
                                                 (4, 32, 128, 128, 128, torch.bfloat16), (4, 32, 1024, 128, 128, torch.bfloat16),
                                                 (4, 32, 2048, 128, 96, torch.bfloat16)])
def test_shapes_without_saved_states_are_the_plain_entry_points(b, h, n, d, e, dtype):
    L = _lib.lib()
    assert L.la_saved_state_bytes(b, h, n, d, e, CODE[dtype], None) == 0
    assert L.la_saved_state_interval(b, h, n, d, e, CODE[dtype], None) == 0
    q, k, v, do = _inputs(b, h, n, d, e, dtype, 3)
    s = _build_slope_tensor(h).float().to(DEV).contiguous()
    spare = torch.full((1 << 20,), float("nan"), dtype=torch.float32, device=DEV)
    print("no-saved-state case", (b, h, n, d, e), flush=True)
    o0, o1 = _fwd(L, q, k, v, s, None), _fwd(L, q, k, v, s, spare)
    g0, g1 = _bwd(L, q, k, v, s, do, None), _bwd(L, q, k, v, s, do, spare)
    torch.cuda.synchronize()
    assert torch.equal(o0, o1) and all(torch.equal(a, c) for a, c in zip(g0, g1))
    assert torch.isnan(spare).all()  # never touched
