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

from lightning_attn.ops import (  # noqa: E402
    lightning_attn2, lightning_attn2_no_decay, lightning_attn2_parallel, lightning_attn_func)
from lightning_attn.ops.hip import launch_opts  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def make_inputs(b, h, n, d, e, dtype, scale, seed=2024):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = ((torch.randn(b, h, n, x, generator=g) * scale).to(dtype) for x in (d, d, e, e))
    return q, k, v, do


def run_hip(q, k, v, s, do, fn=None, **opts):
    """Forward + backward on the device; `opts` are launch options (launch_opts) for both."""
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    sg = None if s is None else s.to(DEV)
    with launch_opts(**opts):
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
def test_float32_backward_in_one_launch(b, h, n, d, decay):
    """float32 with d == e: dQ, dK and dV share a launch; paired=False launches them one after
    the other.  Same numbers, bit for bit."""
    q, k, v, do = make_inputs(b, h, n, d, d, torch.float32, 1.0, seed=n)
    s = _build_slope_tensor(h) if decay else None
    together = run_hip(q, k, v, s, do)
    apart = run_hip(q, k, v, s, do, paired=False)
    for a, c in zip(together, apart):
        assert torch.equal(a, c)
    # few sequences: the walk is cut into chunks with warm-up blocks, here as well bit-identical for every count
    for chunks in (1, 2, 5, 8):
        for a, c in zip(run_hip(q, k, v, s, do, chunks=chunks), together):
            assert torch.equal(a, c), chunks
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
def test_sequence_chunking_is_exact(b, h, n, d, e):
    """Few sequences: the walk is cut into chunks whose workgroups rebuild their incoming state with
    warm-up blocks (the chunk-parallel path without a workspace, scan=False).  Every chunk count
    must give bit-identical results, and they must match the oracle."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0, seed=n)
    s = _build_slope_tensor(h)
    outs = {}
    for chunks in (1, 2, 3, 8, None):  # None = the library's own choice
        outs[chunks] = run_hip(q, k, v, s, do, scan=False, chunks=chunks)
    for chunks in (2, 3, 8, None):
        for a, c in zip(outs[1], outs[chunks]):
            assert torch.equal(a, c), chunks
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(outs[None], want, torch.bfloat16, "chunked %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("b, h, n, d, e", [(1, 2, 4096, 128, 64), (2, 3, 1000, 64, 128), (1, 2, 2100, 128, 128), (1, 1, 1500, 96, 72),
                                           (3, 1, 831, 16, 128), (1, 2, 900, 64, 64), (1, 2, 1500, 192, 192), (1, 1, 900, 256, 256),
                                           (2, 1, 1100, 160, 136)])
@pytest.mark.parametrize("decay", [True, False])
def test_chunk_states_by_scan(b, h, n, d, e, decay):
    """With a workspace (the Python operators always pass one) the kernels start every chunk from
    a scanned state instead of rebuilding it: three launches, up to 64 chunks.  The state sums are taken
    in another order, so results agree with the single walk to rounding, not bit for bit."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 1.0, seed=n + d)
    s = _build_slope_tensor(h) if decay else None
    one = run_hip(q, k, v, s, do, chunks=1)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    for wide in (None, False, True):  # the library's choice, 64-column, 128-column workgroups
        for chunks in (2, 3, 7, 16, 64, None):
            got = run_hip(q, k, v, s, do, wide=wide, chunks=chunks)
            for name, a, c in zip(("o", "dq", "dk", "dv"), got, one):
                assert rel_norm(a, c) < 5e-4, (wide, chunks, name, rel_norm(a, c))
            check(got, want, torch.bfloat16, "scan, wide %s, %s chunks %s" % (wide, chunks, (b, h, n, d, e)))


@pytest.mark.parametrize("chunks", [2, 5])
def test_chunked_walk_on_projection_layout(chunks):
    """Chunked walk and token-major tensors together (ragged n, e off the 64 grid): the output tile of
    every chunk's last block and the rows beyond n are the cases the write-back path has to get right."""
    b, h, n, d, e = 1, 3, 1237, 128, 72
    g = torch.Generator().manual_seed(23)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    v, do = (torch.randn(b, n, h, e, generator=g).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    s = _build_slope_tensor(h)
    # warm-up chunks (scan=False): bit-identical to the single walk; fresh leaves for every call
    got = run_hip(q.detach(), k.detach(), v.detach(), s, do, scan=False, chunks=chunks)
    got_plain = run_hip(q.contiguous(), k.contiguous(), v.contiguous(), s, do.contiguous(), scan=False, chunks=chunks)
    got_one = run_hip(q.detach(), k.detach(), v.detach(), s, do, scan=False, chunks=1)
    got_scan = run_hip(q.detach(), k.detach(), v.detach(), s, do, chunks=chunks)  # the same chunks from scanned states
    for a, c, one, sc in zip(got, got_plain, got_one, got_scan):
        assert torch.equal(a, c) and torch.equal(a, one)
        assert rel_norm(sc, a) < 5e-4
    want = oracle.linear_attn_fwd_bwd(q.cpu(), k.cpu(), v.cpu(), s, do.cpu(), torch.float32)
    check(got, want, torch.bfloat16, "chunked token-major")


@pytest.mark.parametrize("b, h, n, d", [(2, 4, 1000, 128), (1, 3, 777, 64), (1, 2, 500, 192), (1, 2, 300, 256),
                                        (1, 5, 913, 72), (2, 3, 450, 96), (1, 2, 1100, 120)])
def test_paired_backward_launch_matches_separate_launches(b, h, n, d):
    """With d == e the dK and dV sweeps travel in one launch (their workgroups share the reads of dO
    and q), with 64 or - wide=True - 128 columns per workgroup; paired=False launches
    them one after the other.  Same numbers, bit for bit, also when the walk is cut into chunks."""
    q, k, v, do = make_inputs(b, h, n, d, d, torch.bfloat16, 1.0, seed=d + n)
    s = _build_slope_tensor(h)
    got = {}
    # scan=False: scanned chunk states agree to rounding only
    for mode, opts in (("narrow", {"wide": False}), ("wide", {"wide": True}),
                       ("wide chunked", {"wide": True, "chunks": 3}), ("separate", {"paired": False})):
        got[mode] = run_hip(q, k, v, s, do, scan=False, **opts)
    for mode in ("narrow", "wide", "wide chunked"):
        for a, c in zip(got[mode], got["separate"]):
            assert torch.equal(a, c), mode
    if d <= 128:
        want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
        check(got["wide"], want, torch.bfloat16, "wide pair d=%d" % d)


@pytest.mark.parametrize("b, h, n, d", [(2, 12, 2048, 192), (1, 8, 1024, 128), (2, 3, 777, 64), (1, 2, 300, 256), (1, 5, 913, 72),
                                        (3, 3, 450, 160), (1, 1, 64, 8), (12, 8, 200, 128)])
@pytest.mark.parametrize("decay", [True, False])
def test_backward_in_one_launch(b, h, n, d, decay):
    """With d == e and few sequences dQ (walking forward) and dK + dV (walking backward) travel in ONE
    launch and run side by side; once=False keeps them apart, once=True joins them whatever the size.
    Same numbers, bit for bit, for every chunk count, on plain and token-major tensors."""
    g = torch.Generator().manual_seed(n + d)
    q, k, v, do = ((torch.randn(b, n, h, d, generator=g) * sc).bfloat16().to(DEV) for sc in (0.7, 0.7, 1.0, 1.0))
    s = _build_slope_tensor(h) if decay else None
    got = {}
    # scan=False throughout: scanned chunk states agree to rounding only
    for token_major in (False, True):
        tq, tk, tv, tdo = ((t.transpose(1, 2) if token_major else t.transpose(1, 2).contiguous()) for t in (q, k, v, do))
        for once, chunks in ((False, None), (True, None), (True, 1), (True, 3), (True, 8)):
            got[token_major, once, chunks] = run_hip(tq.detach(), tk.detach(), tv.detach(), s, tdo, scan=False, once=once,
                                                     chunks=chunks)
    got[False, None, None] = run_hip(q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous(), v.transpose(1, 2).contiguous(), s,
                                     do.transpose(1, 2).contiguous(), scan=False)  # the library's own choice
    for key, val in got.items():
        for a, c in zip(val, got[False, False, None]):
            assert torch.equal(a, c), key
    want = oracle.linear_attn_fwd_bwd(*(t.transpose(1, 2).cpu() for t in (q, k, v)), s, do.transpose(1, 2).cpu(), torch.float32)
    check(got[True, True, 3], want, torch.bfloat16, "one launch %s" % ((b, h, n, d),))


@pytest.mark.parametrize("b, h, n, d, e", [(2, 8, 1024, 128, 64), (1, 3, 777, 64, 128), (1, 2, 300, 192, 256), (1, 2, 513, 72, 40),
                                           (2, 2, 1100, 256, 128), (12, 8, 200, 128, 64)])
@pytest.mark.parametrize("decay", [True, False])
def test_dq_and_dk_in_one_launch(b, h, n, d, e, decay):
    """With d != e the dQ sweep (walking forward) and the dK sweep (walking backward) have one shape
    and, with few sequences, share a launch; dV follows.  once=False / True as above; same numbers,
    bit for bit, on plain and token-major tensors."""
    g = torch.Generator().manual_seed(n + d + e)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV) for _ in range(2))
    v, do = (torch.randn(b, n, h, e, generator=g).bfloat16().to(DEV) for _ in range(2))
    s = _build_slope_tensor(h) if decay else None
    got = {}
    for token_major in (False, True):
        tq, tk, tv, tdo = ((t.transpose(1, 2) if token_major else t.transpose(1, 2).contiguous()) for t in (q, k, v, do))
        for once, chunks in ((False, None), (True, None), (True, 1), (True, 4)):
            got[token_major, once, chunks] = run_hip(tq.detach(), tk.detach(), tv.detach(), s, tdo, scan=False, once=once,
                                                     chunks=chunks)
    got["auto"] = run_hip(*(t.transpose(1, 2).contiguous() for t in (q, k, v)), s, do.transpose(1, 2).contiguous(), scan=False)
    for key, val in got.items():
        for a, c in zip(val, got[False, False, None]):
            assert torch.equal(a, c), key
    want = oracle.linear_attn_fwd_bwd(*(t.transpose(1, 2).cpu() for t in (q, k, v)), s, do.transpose(1, 2).cpu(), torch.float32)
    check(got[True, True, 4], want, torch.bfloat16, "dq + dk in one launch %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("dtype, decay", [(torch.bfloat16, True), (torch.float16, True), (torch.bfloat16, False)])
def test_many_sequences_take_the_128_column_workgroups(dtype, decay):
    """b * h >= the number of CUs: the library picks 128-column workgroups for every launch by itself."""
    b, h, n, d = 32, 8, 130, 128
    q, k, v, do = make_inputs(b, h, n, d, d, dtype, 1.0 if dtype == torch.bfloat16 else 0.5, seed=77)
    s = _build_slope_tensor(h) if decay else None
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(run_hip(q, k, v, s, do), want, dtype, "many sequences")


def test_wide_pair_on_token_major_tensors():
    """The 128-column workgroups on strided tensors (explicit row masks, ragged n)."""
    b, h, n, d = 1, 3, 1237, 128
    g = torch.Generator().manual_seed(29)
    q, k = ((torch.randn(b, n, h, d, generator=g) * 0.7).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    v, do = (torch.randn(b, n, h, d, generator=g).bfloat16().to(DEV).transpose(1, 2) for _ in range(2))
    s = _build_slope_tensor(h)
    wide = run_hip(q.detach(), k.detach(), v.detach(), s, do, wide=True)
    narrow = run_hip(q.detach(), k.detach(), v.detach(), s, do, wide=False)
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


@pytest.mark.parametrize("n", [512, 1024, 2048, 4096, 8192, 16384, 32768])
def test_full_size_against_block_recurrence_on_head_subset(n):
    """b4 h32 d=e=128 at every length of the long-sequence sweep, all 128 sequences on the device:
    three (batch, head) pairs (fast, middle and slow decay) are checked against the fp64
    block-recurrence oracle, itself pinned to the naive formula."""
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


@pytest.mark.parametrize("b, n, d", [(4, 8192, 192), (8, 4096, 192), (4, 4096, 160)])
def test_full_size_at_feature_dims_129_to_192(b, n, d):
    """h = 32 at d = e = 192 / 160 with 128 and 256 sequences, the shapes the all-column workgroups are planned
    for (dK + dV, dQ from the forward pass's states; from 256 sequences on the forward launch as well): three
    (batch, head) pairs against the fp64 block-recurrence oracle, and the whole result against the run with
    64-column workgroups throughout and no saved states (o, dk, dv bit for bit; dq to rounding where states
    were used)."""
    h = 32
    q, k, v, do = _full_inputs(b, h, n, d)
    s = _build_slope_tensor(h)
    got = run_hip(q, k, v, s, do)
    for bi, hi in ((0, 0), (1, 13), (b - 1, 31)):
        sub = [t[bi:bi + 1, hi:hi + 1].float().cpu() for t in (q, k, v, do)]
        ss = s[hi:hi + 1]
        want_o = oracle.block_recurrence_fwd(sub[0], sub[1], sub[2], ss, 64)
        want_g = oracle.block_recurrence_bwd(sub[0], sub[1], sub[2], ss, sub[3], 64)
        check([t[bi:bi + 1, hi:hi + 1] for t in got], (want_o,) + tuple(want_g), torch.bfloat16,
              "d=%d b=%d n=%d head (%d,%d)" % (d, b, n, bi, hi))
    narrow = run_hip(q, k, v, s, do, wide=False, save_states=False)
    for name, a, c in zip(("o", "dq", "dk", "dv"), got, narrow):
        if name == "dq":
            assert rel_norm(a, c.float()) < 3e-3, name
        else:
            assert torch.equal(a, c), name


@pytest.mark.parametrize("b, h, n, d, e", [(2, 4, 300, 128, 128), (1, 3, 200, 256, 256), (2, 2, 260, 192, 128), (1, 2, 130, 64, 160)])
def test_all_columns_option_is_the_librarys_choice_where_it_has_no_form(b, h, n, d, e):
    """wide="all" (LA_OPT_ALL) names a form that exists for d and e both in 129 .. 192; elsewhere the option is
    accepted and means the library's own choice: same bits as without it."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 0.6, seed=n + d)
    s = _build_slope_tensor(h)
    for a, c in zip(run_hip(q, k, v, s, do, wide="all"), run_hip(q, k, v, s, do)):
        assert torch.equal(a, c)


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


# ---- the tolerance as it is named for this path: |a - ref| <= 2e-2 + 2e-2 |ref|, element-wise -----------

def _literal_fail_fraction(a, ref):
    a, ref = a.double().cpu(), ref.double().cpu()
    return ((a - ref).abs() > 2e-2 + 2e-2 * ref.abs()).double().mean().item()


def _literal_tolerance_case(q, k, v, s, do, got, what):
    """`got` = (o, dq, dk, dv) of the HIP kernels for the CPU tensors q, k, v, do.  Expected values: the
    naive formula in float32 on the same bf16 inputs.  With unit-variance inputs outputs have an RMS of
    10..100, so an absolute term of 2e-2 is a fraction of one bf16 ulp and some elements fall outside
    the literal bound for ANY bf16 pipeline - the reference's own naive path run in bf16
    (lightning_attn/ops/torch/linear_attention.py:30-32) included.  The kernels must not do worse
    than that path does on the same inputs."""
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    ref_bf16 = oracle.linear_attn_fwd_bwd(q, k, v, s, do, None)  # the reference's dataflow, natively in bf16
    for name, a, r, w in zip(("o", "dq", "dk", "dv"), got, ref_bf16, want):
        f_hip, f_ref = _literal_fail_fraction(a, w), _literal_fail_fraction(r, w)
        print("literal rtol=atol=2e-2 failures, %s %s: HIP %.4f %%, reference bf16 dataflow %.4f %%  (rel. error %.2e / %.2e)"
              % (what, name, 100 * f_hip, 100 * f_ref, rel_norm(a, w), rel_norm(r, w)), flush=True)
        assert f_hip <= f_ref + 1e-5, (what, name, f_hip, f_ref)
        assert rel_norm(a, w) <= rel_norm(r, w) * 1.05, (what, name)


def test_literal_tolerance_config2_head_subset():
    """Config 2 (bf16 b4 h32 n4096 d=e=128, N(0,1), slopes(32)) on the device in full; the O(n^2)
    oracles on three (batch, head) pairs: fastest, middle and slowest decay."""
    b, h, n, d = 4, 32, 4096, 128
    q, k, v, do = _full_inputs(b, h, n, d, seed=11)
    s = _build_slope_tensor(h)
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    o = lightning_attn_func(qg, kg, vg, s.to(DEV))
    o.backward(do)
    torch.cuda.synchronize()
    for bi, hi in ((0, 0), (2, 15), (3, 31)):
        sub = [t[bi:bi + 1, hi:hi + 1].cpu() for t in (q, k, v, do)]
        got = [t[bi:bi + 1, hi:hi + 1] for t in (o.detach(), qg.grad, kg.grad, vg.grad)]
        _literal_tolerance_case(sub[0], sub[1], sub[2], s[hi:hi + 1], sub[3], got, "config 2 head (%d,%d)" % (bi, hi))


@pytest.mark.parametrize("decay", [True, False])
def test_literal_tolerance_config4(decay):
    """Config 4 (bf16 b2 h12 n2048 d=e=192, N(0,1)), with slopes(12) and without decay, all 24 sequences.
    Without decay the outputs grow like sqrt(n) * d and only the relative term matters."""
    b, h, n, d = 2, 12, 2048, 192
    q, k, v, do = make_inputs(b, h, n, d, d, torch.bfloat16, 1.0, seed=4)
    s = _build_slope_tensor(h) if decay else None
    got = run_hip(q, k, v, s, do)
    _literal_tolerance_case(q, k, v, s, do, got, "config 4 %s" % ("decay" if decay else "no decay"))


@pytest.mark.parametrize("b, h, n, d, e", [(1, 2, 16384, 128, 128), (1, 3, 5000, 192, 192), (1, 1, 9000, 64, 128)])
def test_parallel_variant_names(b, h, n, d, e):
    """variant="parallel" of lightning_attn_func and lightning_attn2_parallel
    (lightning_attn/ops/lightning_attn_interface.py:20-21, lightning_attn2_parallel.py:1072) on few, long
    sequences - where the walk is cut into chunks that start from scanned states - against the fp64
    block-recurrence oracle, and against the default variant (same kernels: bit-identical)."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 0.5, seed=n)
    s = _build_slope_tensor(h)
    want = (oracle.block_recurrence_fwd(q, k, v, s, 64),) + tuple(oracle.block_recurrence_bwd(q, k, v, s, do, 64))
    by_func = run_hip(q, k, v, s, do, lambda *a: lightning_attn_func(*a, variant="parallel"))
    by_op = run_hip(q, k, v, s, do, lightning_attn2_parallel)
    default = run_hip(q, k, v, s, do)
    check(by_func, want, torch.bfloat16, "variant=parallel %s" % ((b, h, n, d, e),))
    for a, c, dflt in zip(by_func, by_op, default):
        assert torch.equal(a, c) and torch.equal(a, dflt)


def test_tensors_on_different_devices_are_refused():
    """A CPU k or v must raise in Python; its pointer must never reach a launch."""
    q, k, v, do = make_inputs(1, 2, 64, 64, 64, torch.bfloat16, 1.0)
    with pytest.raises(RuntimeError, match="same HIP device"):
        lightning_attn_func(q.to(DEV), k, v.to(DEV), None)
    with pytest.raises(RuntimeError, match="same HIP device"):
        lightning_attn2(q.to(DEV), k.to(DEV), v, _build_slope_tensor(2).to(DEV))


@pytest.mark.parametrize("b, h, n, d, e, dtype", [(1, 3, 300, 64, 100, torch.bfloat16), (2, 2, 130, 36, 36, torch.bfloat16),
                                                  (1, 2, 257, 20, 12, torch.float32), (1, 1, 70, 100, 260, torch.float16)])
def test_feature_dims_off_the_grid_of_8_are_padded(b, h, n, d, e, dtype):
    """d or e not a multiple of 8 (the reference takes any e by padding v to a power of two,
    lightning_attn_interface.py:29-33, 63-64): zero-padded to the next multiple of 8, gradients sliced back."""
    q, k, v, do = make_inputs(b, h, n, d, e, dtype, 0.5, seed=d * e)
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float64 if dtype == torch.float32 else torch.float32)
    got = run_hip(q, k, v, s, do)
    for a, t in zip(got, (v, q, k, v)):
        assert a.shape == t.shape
    check(got, want, dtype, "padded dims %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("b, h, n, d, e", [(2, 3, 700, 192, 192), (1, 2, 450, 256, 256), (1, 3, 513, 160, 160), (2, 2, 300, 136, 200), (2, 2, 333, 176, 144),
                                           (1, 2, 330, 192, 256), (1, 1, 200, 256, 72), (1, 2, 260, 144, 96), (1, 2, 1000, 224, 232)])
@pytest.mark.parametrize("decay", [True, False])
def test_wide_two_barrier_kernel_is_bit_identical_to_the_64_column_form(b, h, n, d, e, decay):
    """Feature dims above 128: 96- / 128-column workgroups (wide=True) against the 64-column ones (wide=False), forward
    and backward, single walk, warm-up chunks and - d == e - the paired dK + dV launch: the same arithmetic per output
    column, so the same bits; from scanned chunk states equal to rounding.  Both against the oracle."""
    q, k, v, do = make_inputs(b, h, n, d, e, torch.bfloat16, 0.7, seed=d + e)
    s = _build_slope_tensor(h) if decay else None
    narrow = run_hip(q, k, v, s, do, wide=False, scan=False, chunks=1, once=False)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check(narrow, want, torch.bfloat16, "64-column %s" % ((b, h, n, d, e),))
    for opts in ({"chunks": 1}, {"chunks": 3}, {"chunks": 2, "paired": False}):
        wide = run_hip(q, k, v, s, do, wide=True, scan=False, once=False, **opts)
        for name, a, c in zip(("o", "dq", "dk", "dv"), wide, narrow):
            assert torch.equal(a, c), (opts, name)
    scanned = run_hip(q, k, v, s, do, wide=True, chunks=4, once=False)
    for name, a, c in zip(("o", "dq", "dk", "dv"), scanned, narrow):
        assert rel_norm(a, c) < 5e-4, name
    check(scanned, want, torch.bfloat16, "wide, scanned chunks %s" % ((b, h, n, d, e),))
    if 128 < d <= 192 and 128 < e <= 192:
        # all (up to 192) columns of a sequence in one workgroup, three accumulator slabs per state wave
        for opts in ({"chunks": 1}, {"chunks": 3}, {"chunks": 2, "paired": False}):
            whole = run_hip(q, k, v, s, do, wide="all", scan=False, once=False, **opts)
            for name, a, c in zip(("o", "dq", "dk", "dv"), whole, narrow):
                assert torch.equal(a, c), ("all columns", opts, name)
        scanned = run_hip(q, k, v, s, do, wide="all", chunks=4, once=False)
        for name, a, c in zip(("o", "dq", "dk", "dv"), scanned, narrow):
            assert rel_norm(a, c) < 5e-4, name
        check(scanned, want, torch.bfloat16, "all columns, scanned chunks %s" % ((b, h, n, d, e),))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_many_sequences_at_192_take_the_wide_workgroups(dtype):
    """b * h = 48 sequences at d = e = 192: three 64-column workgroups per sequence would not fit the CUs in one
    round (a chip of 256 of them is assumed when there are fewer), so the library picks two 96-column ones by itself."""
    b, h, n, d = 6, 16, 200, 192
    q, k, v, do = make_inputs(b, h, n, d, d, dtype, 0.5, seed=5)
    s = _build_slope_tensor(h)
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    got = run_hip(q, k, v, s, do)
    check(got, want, dtype, "many sequences, d = 192")
    for a, c in zip(got, run_hip(q, k, v, s, do, wide=False)):
        assert torch.equal(a, c)


def test_dense_views_off_the_16_byte_grid_are_copied():
    """A contiguous view that starts 8 bytes into a larger buffer: the kernels need 16-byte aligned rows, so the
    operator works on an aligned copy instead of handing the pointer on (which the C entry points refuse)."""
    b, h, n, d = 1, 2, 130, 64
    q, k, v, do = make_inputs(b, h, n, d, d, torch.bfloat16, 0.5, seed=3)
    s = _build_slope_tensor(h)

    def off_grid(t):
        buf = torch.empty(t.numel() + 4, dtype=t.dtype, device=DEV)
        view = buf[4:].view(t.shape)
        view.copy_(t)
        assert view.is_contiguous() and view.data_ptr() % 16 == 8
        return view

    qg, kg, vg = (off_grid(t).requires_grad_() for t in (q, k, v))
    o = lightning_attn_func(qg, kg, vg, s.to(DEV))
    o.backward(off_grid(do))
    torch.cuda.synchronize()
    want = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float32)
    check((o.detach(), qg.grad, kg.grad, vg.grad), want, torch.bfloat16, "views off the 16-byte grid")
