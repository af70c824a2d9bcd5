"""GPU parity of norm_gate (HIP, through the C ABI) against the float32 / float64 oracle:
y = layer_norm(o) * sigmoid(g) and its five gradients.  Tolerance as for SimpleRMSNorm
(atol 5e-2, rtol 1e-2 on bf16 / fp16 outputs), a relative Frobenius error per tensor, and for
the column sums d weight / d bias (sums over all rows, rounded once to the tensor dtype) a relative
error against the float64 oracle."""
import ctypes

import pytest
import torch
from torch.testing import assert_close

import oracle
from util import rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops.hip import _lib, norm_gate, norm_gate_supported  # noqa: E402

DEV = "cuda"


def _inputs(shape, dtype, seed):
    g_ = torch.Generator().manual_seed(seed)
    cols = shape[-1]
    o = (torch.randn(*shape, generator=g_) * 2.5 + 0.3).to(dtype)
    g = (torch.randn(*shape, generator=g_) * 2).to(dtype)
    w = (1 + 0.3 * torch.randn(cols, generator=g_)).to(dtype)
    b = (0.2 * torch.randn(cols, generator=g_)).to(dtype)
    dy = torch.randn(*shape, generator=g_).to(dtype)
    return o, g, w, b, dy


def _run(o, g, w, b, dy, eps=1e-5):
    leaves = [t.to(DEV).requires_grad_() for t in (o, g, w, b)]
    y = norm_gate(*leaves, eps)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    return (y.detach().cpu(),) + tuple(t.grad.cpu() for t in leaves)


@pytest.mark.parametrize("shape", [(2, 384, 512), (1, 1000, 768), (4, 128, 1024), (3, 57, 2048), (2, 33, 4096), (1, 19, 8192),
                                   (5, 8), (1, 1, 64), (700, 264), (3000, 1536)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_norm_gate_matches_oracle(shape, dtype):
    cols = shape[-1]
    if not norm_gate_supported(cols, dtype):
        assert dtype == torch.float32 and cols > 4096
        pytest.skip("float32 rows beyond 4096 columns are not supported")
    o, g, w, b, dy = _inputs(shape, dtype, seed=cols)
    got = _run(o, g, w, b, dy)
    want = oracle.norm_gate_fwd_bwd(o, g, w, b, dy, 1e-5, torch.float32)
    want64 = oracle.norm_gate_fwd_bwd(o, g, w, b, dy, 1e-5, torch.float64)
    names = ("y", "d_o", "d_g", "d_weight", "d_bias")
    for name, a, r, r64 in zip(names, got, want, want64):
        assert a.dtype == dtype and a.shape == r.shape, name
        if dtype == torch.float32:
            assert rel_norm(a, r64) < 2e-5, (name, rel_norm(a, r64))
        else:
            lim = 5e-3 if dtype == torch.bfloat16 else 1e-3
            assert rel_norm(a, r64) < lim, (name, rel_norm(a, r64))
            if name in ("y", "d_o", "d_g"):
                assert_close(a.float(), r, atol=5e-2, rtol=1e-2)


def test_norm_gate_is_deterministic_and_covers_many_rows():
    """More rows than one pass of the grid holds (the kernels walk the rows with a grid stride), twice:
    the column sums are added up in a fixed order, so the results repeat bit for bit."""
    o, g, w, b, dy = _inputs((70000, 256), torch.bfloat16, seed=5)
    a = _run(o, g, w, b, dy)
    c = _run(o, g, w, b, dy)
    for x, y in zip(a, c):
        assert torch.equal(x, y)
    want64 = oracle.norm_gate_fwd_bwd(o, g, w, b, dy, 1e-5, torch.float64)
    for name, x, r in zip(("y", "d_o", "d_g", "d_weight", "d_bias"), a, want64):
        assert rel_norm(x, r) < 5e-3, (name, rel_norm(x, r))


def test_norm_gate_argument_checks():
    L = _lib.lib()
    assert L.norm_gate_supported(1024, 0) == 1 and L.norm_gate_supported(8192, 1) == 1
    assert L.norm_gate_supported(8200, 0) == 0 and L.norm_gate_supported(100, 0) == 0 and L.norm_gate_supported(4100, 2) == 0
    o, g, w, b, dy = (t.to(DEV) for t in _inputs((4, 64), torch.bfloat16, seed=1))
    with pytest.raises(RuntimeError, match="same HIP device"):
        norm_gate(o, g.cpu(), w, b)
    with pytest.raises(ValueError):
        norm_gate(o, g[:, :32], w, b)
    with pytest.raises(RuntimeError, match="not supported"):
        norm_gate(o[:, :60], g[:, :60], w[:60], b[:60])
    # a workspace that is too small is refused before anything is launched
    y = torch.empty_like(o)
    st = torch.empty(8, dtype=torch.float32, device=DEV)
    rc = L.norm_gate_bwd(o.data_ptr(), g.data_ptr(), w.data_ptr(), b.data_ptr(), st.data_ptr(), st.data_ptr(), dy.data_ptr(),
                         y.data_ptr(), y.data_ptr(), w.data_ptr(), b.data_ptr(), None, 0, 4, 64, 0, None)
    assert rc == -4
    empty = norm_gate(o[:0], g[:0], w, b)
    assert empty.shape == (0, 64)


def test_norm_gate_on_views_off_the_16_byte_grid():
    o, g, w, b, dy = _inputs((33, 256), torch.bfloat16, seed=8)

    def off_grid(t):
        buf = torch.empty(t.numel() + 4, dtype=t.dtype, device=DEV)
        view = buf[4:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 8
        return view

    leaves = [off_grid(t).requires_grad_() for t in (o, g, w, b)]
    y = norm_gate(*leaves, 1e-5)
    y.backward(off_grid(dy))
    torch.cuda.synchronize()
    want64 = oracle.norm_gate_fwd_bwd(o, g, w, b, dy, 1e-5, torch.float64)
    for name, a, r in zip(("y", "d_o", "d_g", "d_weight", "d_bias"), [y.detach()] + [t.grad for t in leaves], want64):
        assert rel_norm(a, r) < 5e-3, (name, rel_norm(a, r))
