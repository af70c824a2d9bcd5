"""GPU parity of lightning_attn_func / lightning_attn2 (HIP, through the C ABI) against
the naive oracle.  Shape matrix, seed and 1/10 input scale follow the reference's
tests/ops/test_lightning2.py:8-64 and test_lightning2_no_decay.py:7-62 (batch reduced
so that the O(n^2) CPU oracle finishes in seconds).

Tolerances: bf16/fp16  rtol = atol = 2e-2 element-wise (absolute term scaled by
max(1, rms(expected)), see util.assert_close_scaled) plus a relative Frobenius
error below 1e-2; fp32  relative Frobenius error below 1e-4.  The expected value is
the naive formula evaluated in float32 on the same (already rounded) inputs."""
import pytest
import torch

import oracle
from util import assert_close_scaled, rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops import lightning_attn2, lightning_attn2_no_decay, lightning_attn_func  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def make_inputs(b, h, n, d, e, dtype, scale, seed=2024):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = ((torch.randn(b, h, n, x, generator=g) * scale).to(dtype) for x in (d, d, e, e))
    return q, k, v, do


def run_hip(q, k, v, s, do, fn=None):
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    sg = None if s is None else s.to(DEV)
    if fn is None:
        o = lightning_attn_func(qg, kg, vg, sg)
    else:
        o = fn(qg, kg, vg, sg) if sg is not None else fn(qg, kg, vg)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    return o.detach(), qg.grad, kg.grad, vg.grad


def check(got, want, dtype, what):
    for name, a, r in zip(("o", "dq", "dk", "dv"), got, want):
        assert a.dtype == dtype, (what, name, a.dtype)
        if dtype == torch.float32:
            assert rel_norm(a, r) < 1e-4, (what, name, rel_norm(a, r))
        else:
            assert_close_scaled(a, r, 2e-2, 2e-2, "%s %s" % (what, name))
            assert rel_norm(a, r) < 1e-2, (what, name, rel_norm(a, r))


REFERENCE_SHAPES = [
    (2, 8, 256, 128, 64),
    (2, 8, 512, 128, 64),
    (2, 8, 1024, 128, 64),
    (2, 8, 2048, 128, 64),
    (1, 4, 4096, 128, 64),
    (1, 2, 8192, 128, 64),
    (2, 8, 2048, 32, 64),
    (2, 8, 2048, 64, 64),
    (1, 12, 2048, 128, 64),
    (1, 16, 2048, 128, 64),
    (1, 20, 2048, 128, 64),
    (1, 8, 2048, 128, 64),
    (3, 8, 1024, 128, 64),
    (2, 8, 913, 128, 64),
    (2, 8, 513, 128, 64),
    (2, 8, 1213, 128, 64),
    (2, 8, 2048, 16, 64),
]


@pytest.mark.parametrize("b, h, n, d, e", REFERENCE_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_matrix_decay(b, h, n, d, e, dtype):
    q, k, v, do = make_inputs(b, h, n, d, e, dtype, 0.1)
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    got = run_hip(q, k, v, s, do, lightning_attn2)
    check(got, want, dtype, "decay %s" % ((b, h, n, d, e),))
    # at this input scale the plain allclose of the stated tolerance holds as well
    for a, r in zip(got, want):
        torch.testing.assert_close(a.float().cpu(), r, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("b, h, n, d, e", REFERENCE_SHAPES[:4] + REFERENCE_SHAPES[6:8] + REFERENCE_SHAPES[13:])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_matrix_no_decay(b, h, n, d, e, dtype):
    q, k, v, do = make_inputs(b, h, n, d, e, dtype, 0.1)
    want = oracle.linear_attn_fwd_bwd(q, k, v, None, do, torch.float32)
    got = run_hip(q, k, v, None, do, lightning_attn2_no_decay)
    check(got, want, dtype, "no decay %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("b, h, n, d, e", [(1, 8, 1024, 128, 128), (2, 3, 300, 64, 128), (1, 12, 700, 192, 192),
                                           (1, 5, 257, 256, 256), (1, 4, 640, 8, 8), (1, 2, 200, 72, 200)])
@pytest.mark.parametrize("decay", [True, False])
def test_unit_variance_bf16(b, h, n, d, e, decay):
    """N(0,1) inputs (the benchmark's distribution), feature dims off the 64 grid."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0)
    s = _build_slope_tensor(h) if decay else None
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, torch.bfloat16, "N(0,1) %s" % ((b, h, n, d, e, decay),))


@pytest.mark.parametrize("b, h, n, d, e", [(1, 8, 1024, 64, 64), (2, 3, 333, 128, 128), (1, 4, 130, 16, 40), (1, 2, 64, 8, 8),
                                           (1, 2, 200, 96, 128), (1, 3, 257, 128, 72), (2, 2, 100, 32, 64), (1, 1, 70, 72, 104)])
@pytest.mark.parametrize("decay", [True, False])
def test_float32(b, h, n, d, e, decay):
    """Config 1's shape (b1 h8 n1024 d=e=64, fp32, slopes(8)) and neighbours: 1e-4 relative."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.float32, 1.0)
    if (b, h, n, d, e) == (1, 8, 1024, 64, 64):
        do = torch.ones_like(do)  # loss = o.sum()
    s = _build_slope_tensor(h) if decay else None
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float64)
    check(run_hip(q, k, v, s, do), want, torch.float32, "fp32 %s" % ((b, h, n, d, e, decay),))


@pytest.mark.parametrize("b, h, n, d", [(1, 8, 1024, 64), (2, 3, 333, 128), (3, 5, 70, 24), (1, 1, 200, 96)])
@pytest.mark.parametrize("decay", [True, False])
def test_float32_backward_in_one_launch(b, h, n, d, decay, monkeypatch):
    """float32 with d == e: dQ, dK and dV share a launch; LA_SWEEP_UNPAIRED=1 launches them one after
    the other.  Same numbers, bit for bit."""
    q, k, v, do = make_inputs(b, h, n, d, d, torch.float32, 1.0, seed=n)
    s = _build_slope_tensor(h) if decay else None
    together = run_hip(q, k, v, s, do)
    monkeypatch.setenv("LA_SWEEP_UNPAIRED", "1")
    apart = run_hip(q, k, v, s, do)
    monkeypatch.delenv("LA_SWEEP_UNPAIRED", raising=False)
    for a, c in zip(together, apart):
        assert torch.equal(a, c)
    # few sequences: the walk is cut into chunks with warm-up blocks, here as well bit-identical for every count
    for chunks in ("1", "2", "5", "8"):
        monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
        for a, c in zip(run_hip(q, k, v, s, do), together):
            assert torch.equal(a, c), chunks
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    check(together, oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float64), torch.float32, "fp32 one launch")


def test_config4_d192_decay_and_zero_rates():
    """b2 h12 n2048 d=e=192: slopes(12) (non power of two head count), s=None and s=0 agree."""
    b, h, n, d, e = 2, 12, 2048, 192, 192
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0)
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, torch.bfloat16, "config 4 decay")
    want0 = oracle.linear_attn_fwd_bwd(q, k, v, None, do, torch.float32)
    got_none = run_hip(q, k, v, None, do)
    got_zero = run_hip(q, k, v, torch.zeros(h, 1, 1), do)
    check(got_none, want0, torch.bfloat16, "config 4 s=None")
    for a, z in zip(got_none, got_zero):
        assert torch.equal(a, z)


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 127, 129])
def test_short_and_ragged_sequences(n):
    q, k, v, do = make_inputs(2, 3, n, 32, 24, torch.bfloat16, 1.0, seed=n)
    s = _build_slope_tensor(3)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, torch.bfloat16, "n=%d" % n)


def test_empty_batch():
    q = torch.empty(0, 4, 128, 64, dtype=torch.bfloat16, device=DEV)
    o = lightning_attn_func(q, q, q, _build_slope_tensor(4).to(DEV))
    assert o.shape == (0, 4, 128, 64)


def test_strided_inputs_and_slope_layouts():
    """(b,n,h,d) projections transposed to (b,h,n,d) without a copy; s given as (h,), (h,1,1)."""
    b, h, n, d = 2, 4, 192, 64
    g = torch.Generator().manual_seed(5)
    base = [(torch.randn(b, n, h, d, generator=g)).bfloat16() for _ in range(4)]
    q, k, v, do = (t.transpose(1, 2) for t in base)
    assert not q.is_contiguous()
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    got = run_hip(q, k, v, s, do)
    check(got, want, torch.bfloat16, "strided")
    got2 = run_hip(q, k, v, s.reshape(h), do)
    for a, c in zip(got, got2):
        assert torch.equal(a, c)


@pytest.mark.parametrize("b, h, n, d, e", [(2, 4, 300, 128, 128), (1, 3, 1111, 64, 96), (2, 12, 257, 192, 192)])
def test_projection_layout_is_used_in_place(b, h, n, d, e):
    """q, k, v sliced out of one fused (b, n, 3*h*d)-style projection and viewed as (b, h, n, d): the strided entry
    points read them where they are, write o / dq / dk / dv in token-major order (so that
    "b h n d -> b n (h d)" is a view), and give bit-identical values to the plain-layout call."""
    g = torch.Generator().manual_seed(11)
    fused = torch.randn(b, n, h * (2 * d + e), generator=g).bfloat16().to(DEV)
    do_nm = torch.randn(b, n, h * e, generator=g).bfloat16().to(DEV)
    s = _build_slope_tensor(h).to(DEV)
    qs, ks, vs = fused.split([h * d, h * d, h * e], dim=-1)
    views = [t.unflatten(-1, (h, -1)).transpose(1, 2) for t in (qs, ks, vs)]
    assert not any(t.is_contiguous() for t in views)
    qv, kv, vv = (t.detach().requires_grad_() for t in views)
    produced = []  # gradients as the operator's backward hands them over (before autograd accumulates them)
    for t in (qv, kv, vv):
        t.register_hook(produced.append)
    o = lightning_attn_func(qv, kv, vv, s)
    assert o.shape == (b, h, n, e) and o.transpose(1, 2).is_contiguous()
    o.backward(do_nm.unflatten(-1, (h, e)).transpose(1, 2))
    assert len(produced) == 3
    for t in produced:
        assert t.transpose(1, 2).is_contiguous()
    # the same numbers through the plain (b, h, n, d) layout
    qc, kc, vc = (t.detach().contiguous().requires_grad_() for t in views)
    oc = lightning_attn_func(qc, kc, vc, s)
    assert oc.is_contiguous()
    oc.backward(do_nm.unflatten(-1, (h, e)).transpose(1, 2).contiguous())
    torch.cuda.synchronize()
    for a, c in zip((o, qv.grad, kv.grad, vv.grad), (oc, qc.grad, kc.grad, vc.grad)):
        assert torch.equal(a, c)
    want = oracle.linear_attn_fwd_bwd(qc.detach().cpu(), kc.detach().cpu(), vc.detach().cpu(), s.cpu(),
                                      do_nm.unflatten(-1, (h, e)).transpose(1, 2).cpu(), torch.float32)
    check((o.detach(), qv.grad, kv.grad, vv.grad), want, torch.bfloat16, "projection layout")


def test_mixed_layouts_and_unit_dims():
    """One plain tensor whose size-1 batch dim carries an odd stride, one token-major view, one head-sliced
    view of a wider tensor: every tensor keeps its own layout in the same call."""
    h, n, d, e = 4, 200, 64, 64
    g = torch.Generator().manual_seed(17)
    q = (torch.randn(1, h, n, d, generator=g) * 0.5).bfloat16().to(DEV)
    q = q.as_strided(q.shape, (7, n * d, d, 1))                      # the batch stride is never used
    k = (torch.randn(1, n, h, d, generator=g) * 0.5).bfloat16().to(DEV).transpose(1, 2)
    v = (torch.randn(1, h + 2, n, e, generator=g) * 0.5).bfloat16().to(DEV)[:, 1:h + 1]
    do = torch.randn(1, n, h, e, generator=g).bfloat16().to(DEV).transpose(1, 2)
    s = _build_slope_tensor(h).to(DEV)
    qg, kg, vg = (t.detach().requires_grad_() for t in (q, k, v))
    o = lightning_attn_func(qg, kg, vg, s)
    o.backward(do)
    torch.cuda.synchronize()
    want = oracle.linear_attn_fwd_bwd(q.cpu(), k.cpu(), v.cpu(), s.cpu(), do.cpu(), torch.float32)
    check((o.detach(), qg.grad, kg.grad, vg.grad), want, torch.bfloat16, "mixed layouts")


def test_wide_features_are_split_by_the_interface():
    """d, e above the kernels' 256 limit go through the slice-and-add path of lightning_attn_func."""
    q, k, v, do = make_inputs(1, 2, 200, 320, 264, torch.bfloat16, 0.5)
    s = _build_slope_tensor(2)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, torch.bfloat16, "wide")
    qf, kf, vf, dof = make_inputs(1, 2, 150, 192, 136, torch.float32, 1.0)
    want = oracle.linear_attn_fwd_bwd(qf, kf, vf, s, dof, torch.float64)
    check(run_hip(qf, kf, vf, s, dof), want, torch.float32, "wide fp32")


@pytest.mark.parametrize("b, h, n, d, e", [(1, 2, 4096, 128, 64), (2, 3, 1000, 64, 128), (1, 1, 1500, 192, 72)])
def test_sequence_chunking_is_exact(b, h, n, d, e, monkeypatch):
    """Few sequences: the walk is cut into chunks whose workgroups rebuild their incoming state with
    warm-up blocks (the chunk-parallel path without a workspace, LA_SWEEP_SCAN=0).  Every chunk count
    must give bit-identical results, and they must match the oracle."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0, seed=n)
    s = _build_slope_tensor(h)
    monkeypatch.setenv("LA_SWEEP_SCAN", "0")
    outs = {}
    for chunks in ("1", "2", "3", "8", None):  # None = the library's own choice
        if chunks is None:
            monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
        else:
            monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
        outs[chunks] = run_hip(q, k, v, s, do)
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    monkeypatch.delenv("LA_SWEEP_SCAN", raising=False)
    for chunks in ("2", "3", "8", None):
        for a, c in zip(outs["1"], outs[chunks]):
            assert torch.equal(a, c), chunks
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(outs[None], want, torch.bfloat16, "chunked %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("b, h, n, d, e", [(1, 2, 4096, 128, 64), (2, 3, 1000, 64, 128), (1, 2, 2100, 128, 128), (1, 1, 1500, 96, 72),
                                           (3, 1, 831, 16, 128), (1, 2, 900, 64, 64), (1, 2, 1500, 192, 192), (1, 1, 900, 256, 256),
                                           (2, 1, 1100, 160, 136)])
@pytest.mark.parametrize("decay", [True, False])
def test_chunk_states_by_scan(b, h, n, d, e, decay, monkeypatch):
    """With a workspace (the Python operators always pass one) the kernels start every chunk from
    a scanned state instead of rebuilding it: three launches, up to 64 chunks.  The state sums are taken
    in another order, so results agree with the single walk to rounding, not bit for bit."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0, seed=n + d)
    s = _build_slope_tensor(h) if decay else None
    monkeypatch.setenv("LA_SWEEP_CHUNKS", "1")
    one = run_hip(q, k, v, s, do)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    for wide in (None, "0", "1"):  # the library's choice, 64-column, 128-column workgroups
        if wide is None:
            monkeypatch.delenv("LA_SWEEP_WIDE", raising=False)
        else:
            monkeypatch.setenv("LA_SWEEP_WIDE", wide)
        for chunks in ("2", "3", "7", "16", "64", None):
            if chunks is None:
                monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
            else:
                monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
            got = run_hip(q, k, v, s, do)
            for name, a, c in zip(("o", "dq", "dk", "dv"), got, one):
                assert rel_norm(a, c) < 5e-4, (wide, chunks, name, rel_norm(a, c))
            check(got, want, torch.bfloat16, "scan, wide %s, %s chunks %s" % (wide, chunks, (b, h, n, d, e)))
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    monkeypatch.delenv("LA_SWEEP_WIDE", raising=False)


@pytest.mark.parametrize("chunks", ["2", "5"])
def test_chunked_walk_on_projection_layout(chunks, monkeypatch):
    """Chunked walk and token-major tensors together (ragged n, e off the 64 grid): the output tile of
    every chunk's last block and the rows beyond n are the cases the write-back path has to get right."""
    b, h, n, d, e = 1, 3, 1237, 128, 72
    g = torch.Generator().manual_seed(23)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    v, do = (torch.randn(b, n, h, e, generator=g).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    s = _build_slope_tensor(h)
    monkeypatch.setenv("LA_SWEEP_SCAN", "0")  # warm-up chunks: bit-identical to the single walk
    monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
    got = run_hip(q.detach(), k.detach(), v.detach(), s, do)  # fresh leaves for every call
    got_plain = run_hip(q.contiguous(), k.contiguous(), v.contiguous(), s, do.contiguous())
    monkeypatch.setenv("LA_SWEEP_CHUNKS", "1")
    got_one = run_hip(q.detach(), k.detach(), v.detach(), s, do)
    monkeypatch.delenv("LA_SWEEP_SCAN", raising=False)
    monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
    got_scan = run_hip(q.detach(), k.detach(), v.detach(), s, do)  # the same chunks from scanned states
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    for a, c, one, sc in zip(got, got_plain, got_one, got_scan):
        assert torch.equal(a, c) and torch.equal(a, one)
        assert rel_norm(sc, a) < 5e-4
    want = oracle.linear_attn_fwd_bwd(q.cpu(), k.cpu(), v.cpu(), s, do.cpu(), torch.float32)
    check(got, want, torch.bfloat16, "chunked token-major")


@pytest.mark.parametrize("b, h, n, d", [(2, 4, 1000, 128), (1, 3, 777, 64), (1, 2, 500, 192), (1, 2, 300, 256),
                                        (1, 5, 913, 72), (2, 3, 450, 96), (1, 2, 1100, 120)])
def test_paired_backward_launch_matches_separate_launches(b, h, n, d, monkeypatch):
    """With d == e the dK and dV sweeps travel in one launch (their workgroups share the reads of dO
    and q), with 64 or - LA_SWEEP_WIDE=1 - 128 columns per workgroup; LA_SWEEP_UNPAIRED=1 launches
    them one after the other.  Same numbers, bit for bit, also when the walk is cut into chunks."""
    q, k, v, do = make_inputs(b, h, n, d, d, torch.bfloat16, 1.0, seed=d + n)
    s = _build_slope_tensor(h)
    monkeypatch.setenv("LA_SWEEP_SCAN", "0")  # (scanned chunk states agree to rounding only)
    got = {}
    for mode, env in (("narrow", {"LA_SWEEP_WIDE": "0"}), ("wide", {"LA_SWEEP_WIDE": "1"}),
                      ("wide chunked", {"LA_SWEEP_WIDE": "1", "LA_SWEEP_CHUNKS": "3"}), ("separate", {"LA_SWEEP_UNPAIRED": "1"})):
        for name in ("LA_SWEEP_WIDE", "LA_SWEEP_CHUNKS", "LA_SWEEP_UNPAIRED"):
            monkeypatch.delenv(name, raising=False)
        for name, value in env.items():
            monkeypatch.setenv(name, value)
        got[mode] = run_hip(q, k, v, s, do)
    for name in ("LA_SWEEP_WIDE", "LA_SWEEP_CHUNKS", "LA_SWEEP_UNPAIRED", "LA_SWEEP_SCAN"):
        monkeypatch.delenv(name, raising=False)
    for mode in ("narrow", "wide", "wide chunked"):
        for a, c in zip(got[mode], got["separate"]):
            assert torch.equal(a, c), mode
    if d <= 128:
        want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
        check(got["wide"], want, torch.bfloat16, "wide pair d=%d" % d)


@pytest.mark.parametrize("b, h, n, d", [(2, 12, 2048, 192), (1, 8, 1024, 128), (2, 3, 777, 64), (1, 2, 300, 256), (1, 5, 913, 72),
                                        (3, 3, 450, 160), (1, 1, 64, 8), (12, 8, 200, 128)])
@pytest.mark.parametrize("decay", [True, False])
def test_backward_in_one_launch(b, h, n, d, decay, monkeypatch):
    """With d == e and few sequences dQ (walking forward) and dK + dV (walking backward) travel in ONE
    launch and run side by side; LA_SWEEP_ONCE=0 keeps them apart, =1 joins them whatever the size.
    Same numbers, bit for bit, for every chunk count, on plain and token-major tensors."""
    g = torch.Generator().manual_seed(n + d)
    q, k, v, do = ((torch.randn(b, n, h, d, generator=g) * sc).bfloat16().to(DEV) for sc in (0.7, 0.7, 1.0, 1.0))
    s = _build_slope_tensor(h) if decay else None
    monkeypatch.setenv("LA_SWEEP_SCAN", "0")  # (scanned chunk states agree to rounding only)
    got = {}
    for token_major in (False, True):
        tq, tk, tv, tdo = ((t.transpose(1, 2) if token_major else t.transpose(1, 2).contiguous()) for t in (q, k, v, do))
        for once, chunks in (("0", None), ("1", None), ("1", "1"), ("1", "3"), ("1", "8")):
            monkeypatch.setenv("LA_SWEEP_ONCE", once)
            if chunks is None:
                monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
            else:
                monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
            got[token_major, once, chunks] = run_hip(tq.detach(), tk.detach(), tv.detach(), s, tdo)
    monkeypatch.delenv("LA_SWEEP_ONCE", raising=False)
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    got[False, None, None] = run_hip(q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous(), v.transpose(1, 2).contiguous(), s,
                                     do.transpose(1, 2).contiguous())  # the library's own choice
    monkeypatch.delenv("LA_SWEEP_SCAN", raising=False)
    for key, val in got.items():
        for a, c in zip(val, got[False, "0", None]):
            assert torch.equal(a, c), key
    want = oracle.linear_attn_fwd_bwd(*(t.transpose(1, 2).cpu() for t in (q, k, v)), s, do.transpose(1, 2).cpu(), torch.float32)
    check(got[True, "1", "3"], want, torch.bfloat16, "one launch %s" % ((b, h, n, d),))


@pytest.mark.parametrize("b, h, n, d, e", [(2, 8, 1024, 128, 64), (1, 3, 777, 64, 128), (1, 2, 300, 192, 256), (1, 2, 513, 72, 40),
                                           (2, 2, 1100, 256, 128), (12, 8, 200, 128, 64)])
@pytest.mark.parametrize("decay", [True, False])
def test_dq_and_dk_in_one_launch(b, h, n, d, e, decay, monkeypatch):
    """With d != e the dQ sweep (walking forward) and the dK sweep (walking backward) have one shape
    and, with few sequences, share a launch; dV follows.  LA_SWEEP_ONCE=0 / 1 as above; same numbers,
    bit for bit, on plain and token-major tensors."""
    g = torch.Generator().manual_seed(n + d + e)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV) for _ in range(2))
    v, do = (torch.randn(b, n, h, e, generator=g).bfloat16().to(DEV) for _ in range(2))
    s = _build_slope_tensor(h) if decay else None
    monkeypatch.setenv("LA_SWEEP_SCAN", "0")
    got = {}
    for token_major in (False, True):
        tq, tk, tv, tdo = ((t.transpose(1, 2) if token_major else t.transpose(1, 2).contiguous()) for t in (q, k, v, do))
        for once, chunks in (("0", None), ("1", None), ("1", "1"), ("1", "4")):
            monkeypatch.setenv("LA_SWEEP_ONCE", once)
            if chunks is None:
                monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
            else:
                monkeypatch.setenv("LA_SWEEP_CHUNKS", chunks)
            got[token_major, once, chunks] = run_hip(tq.detach(), tk.detach(), tv.detach(), s, tdo)
    monkeypatch.delenv("LA_SWEEP_ONCE", raising=False)
    monkeypatch.delenv("LA_SWEEP_CHUNKS", raising=False)
    got["auto"] = run_hip(*(t.transpose(1, 2).contiguous() for t in (q, k, v)), s, do.transpose(1, 2).contiguous())
    monkeypatch.delenv("LA_SWEEP_SCAN", raising=False)
    for key, val in got.items():
        for a, c in zip(val, got[False, "0", None]):
            assert torch.equal(a, c), key
    want = oracle.linear_attn_fwd_bwd(*(t.transpose(1, 2).cpu() for t in (q, k, v)), s, do.transpose(1, 2).cpu(), torch.float32)
    check(got[True, "1", "4"], want, torch.bfloat16, "dq + dk in one launch %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("dtype, decay", [(torch.bfloat16, True), (torch.float16, True), (torch.bfloat16, False)])
def test_many_sequences_take_the_128_column_workgroups(dtype, decay):
    """b * h >= the number of CUs: the library picks 128-column workgroups for every launch by itself."""
    b, h, n, d = 32, 8, 130, 128
    q, k, v, do = make_inputs(b, h, n, d, d, dtype, 1.0 if dtype == torch.bfloat16 else 0.5, seed=77)
    s = _build_slope_tensor(h) if decay else None
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, dtype, "many sequences")


def test_wide_pair_on_token_major_tensors(monkeypatch):
    """The 128-column workgroups on strided tensors (explicit row masks, ragged n)."""
    b, h, n, d = 1, 3, 1237, 128
    g = torch.Generator().manual_seed(29)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    v, do = (torch.randn(b, n, h, d, generator=g).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    s = _build_slope_tensor(h)
    monkeypatch.setenv("LA_SWEEP_WIDE", "1")
    wide = run_hip(q.detach(), k.detach(), v.detach(), s, do)
    monkeypatch.setenv("LA_SWEEP_WIDE", "0")
    narrow = run_hip(q.detach(), k.detach(), v.detach(), s, do)
    monkeypatch.delenv("LA_SWEEP_WIDE", raising=False)
    for a, c in zip(wide, narrow):
        assert torch.equal(a, c)
    want = oracle.linear_attn_fwd_bwd(q.cpu(), k.cpu(), v.cpu(), s, do.cpu(), torch.float32)
    check(wide, want, torch.bfloat16, "wide token-major")


def test_deterministic():
    q, k, v, do = make_inputs(2, 8, 1000, 128, 128, torch.bfloat16, 1.0)
    s = _build_slope_tensor(8)
    a = run_hip(q, k, v, s, do)
    b = run_hip(q, k, v, s, do)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


# ---- full benchmark sizes: properties that need no O(n^2) oracle ----------------

def _full_inputs(b, h, n, d, seed=2024):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return tuple(torch.randn(b, h, n, d, generator=g, device=DEV, dtype=torch.float32).bfloat16() for _ in range(4))


@pytest.mark.parametrize("n", [4096, 8192, 32768])
def test_full_size_against_block_recurrence_on_head_subset(n):
    """b4 h32 d=e=128 at full length: three (batch, head) pairs (fast, middle and slow decay)
    are checked against the fp64 block-recurrence oracle, itself pinned to the naive formula."""
    b, h, d = 4, 32, 128
    q, k, v, do = _full_inputs(b, h, n, d)
    s = _build_slope_tensor(h)
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    o = lightning_attn_func(qg, kg, vg, s.to(DEV))
    o.backward(do)
    torch.cuda.synchronize()
    for bi, hi in ((0, 0), (1, 13), (3, 31)):
        sub = [t[bi:bi + 1, hi:hi + 1].float().cpu() for t in (q, k, v, do)]
        ss = s[hi:hi + 1]
        want_o = oracle.block_recurrence_fwd(sub[0], sub[1], sub[2], ss, 64)
        want_g = oracle.block_recurrence_bwd(sub[0], sub[1], sub[2], ss, sub[3], 64)
        got = [t[bi:bi + 1, hi:hi + 1] for t in (o.detach(), qg.grad, kg.grad, vg.grad)]
        check(got, (want_o,) + tuple(want_g), torch.bfloat16, "n=%d head (%d,%d)" % (n, bi, hi))


def test_very_long_sequence_few_heads():
    """n = 262144 (4096 blocks), b1 h2: the chunked walk at its longest; the slow-decay head against the
    fp64 block recurrence, and no decay (a state that keeps growing) as well."""
    b, h, n, d = 1, 2, 262144, 128
    g = torch.Generator(device=DEV).manual_seed(31)
    q, k, v, do = ((torch.randn(b, h, n, d, generator=g, device=DEV) * sc).bfloat16() for sc in (0.3, 0.3, 1.0, 1.0))
    for s in (torch.tensor([0.5, 2.0 ** -8]).reshape(h, 1, 1), None):
        qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
        o = lightning_attn_func(qg, kg, vg, None if s is None else s.to(DEV))
        o.backward(do)
        torch.cuda.synchronize()
        sub = [t[:, 1:2].float().cpu() for t in (q, k, v, do)]
        ss = None if s is None else s[1:2]
        want_o = oracle.block_recurrence_fwd(sub[0], sub[1], sub[2], ss, 64)
        want_g = oracle.block_recurrence_bwd(sub[0], sub[1], sub[2], ss, sub[3], 64)
        got = [t[:, 1:2] for t in (o.detach(), qg.grad, kg.grad, vg.grad)]
        check(got, (want_o,) + tuple(want_g), torch.bfloat16, "n=262144 %s" % ("decay" if s is not None else "no decay"))


def test_full_size_prefix_linearity_and_slicing():
    """Config 2 (b4 h32 n4096 d=e=128): causality (a prefix run reproduces the prefix bit for bit),
    linearity in v, and independence of batch/head slices."""
    b, h, n, d = 4, 32, 4096, 128
    q, k, v, v2 = _full_inputs(b, h, n, d, seed=7)
    s = _build_slope_tensor(h).to(DEV)
    o = lightning_attn_func(q, k, v, s)
    o_pre = lightning_attn_func(q[:, :, :1024].contiguous(), k[:, :, :1024].contiguous(), v[:, :, :1024].contiguous(), s)
    assert torch.equal(o[:, :, :1024], o_pre)
    o_pre = lightning_attn_func(q[:, :, :1000].contiguous(), k[:, :, :1000].contiguous(), v[:, :, :1000].contiguous(), s)
    assert torch.equal(o[:, :, :1000], o_pre)
    o_head = lightning_attn_func(q[2:3, 5:7].contiguous(), k[2:3, 5:7].contiguous(), v[2:3, 5:7].contiguous(), s[5:7])
    assert torch.equal(o[2:3, 5:7], o_head)
    o2 = lightning_attn_func(q, k, v2, s)
    osum = lightning_attn_func(q, k, (v.float() + v2.float()).bfloat16(), s)
    assert rel_norm(osum, o.float() + o2.float()) < 1e-2
