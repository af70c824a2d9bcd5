"""GPU parity of SimpleRMSNorm (HIP, through the C ABI).  Shape matrix, dtypes, seed and
tolerance (atol 5e-2, rtol 1e-2) are those of the reference's tests/ops/test_srmsnorm.py:8-43."""
import pytest
import torch
from torch.testing import assert_close

import oracle
from util import rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops import SimpleRMSNorm  # noqa: E402

DEV = "cuda"
ATOL, RTOL = 5e-2, 1e-2


def _run(x, dy, eps=1e-6):
    xg = x.to(DEV).requires_grad_()
    y = SimpleRMSNorm(x.shape[-1], eps)(xg)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    return y.detach().cpu(), xg.grad.cpu()


def _params():
    return [(b, n, d) for b in (1, 2, 4, 8) for n in (127, 128, 256, 257, 1024, 1025) for d in (768, 1024)]


@pytest.mark.parametrize("b, n, d", _params())
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_reference_matrix(b, n, d, dtype):
    torch.manual_seed(2024)
    x = torch.randn((b, n, d)).to(dtype)
    dy = torch.randn((b, n, d)).to(dtype)
    eps = 1.6e-5 if dtype == torch.float16 else 1e-6  # the device wrapper's fp16 clamp
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x, dy, eps)
    y, dx = _run(x, dy)
    assert y.dtype == dtype and dx.dtype == dtype and y.shape == x.shape
    assert_close(y, y_ref, atol=ATOL, rtol=RTOL)
    assert_close(dx, dx_ref, atol=ATOL, rtol=RTOL)
    # and much tighter against exact arithmetic: one rounding of the result
    y64, dx64 = oracle.srmsnorm_fwd_bwd(x, dy, eps, torch.float64)
    lim = 1e-6 if dtype == torch.float32 else (1e-3 if dtype == torch.float16 else 5e-3)
    assert rel_norm(y, y64) < lim and rel_norm(dx, dx64) < lim


def test_config5_outliers_full_size():
    """[4*8192, 4096] bf16, 1 % of entries scaled by 50 before the cast, fp32 reduction."""
    g = torch.Generator().manual_seed(2024)
    rows, cols = 32768, 4096
    x = torch.randn(rows, cols, generator=g)
    x = torch.where(torch.rand(rows, cols, generator=g) < 0.01, x * 50, x).bfloat16()
    dy = torch.randn(rows, cols, generator=g).bfloat16()
    y, dx = _run(x, dy)
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x, dy, 1e-6)
    assert_close(y, y_ref, atol=ATOL, rtol=RTOL)
    assert_close(dx, dx_ref, atol=ATOL, rtol=RTOL)
    assert rel_norm(y, y_ref) < 3e-3 and rel_norm(dx, dx_ref) < 3e-3
    # size-independent properties: unit mean square of y, dx orthogonal to x
    ms = y.float().pow(2).mean(-1)
    assert (ms - 1).abs().max() < 2e-2
    cosine = (dx.double() * x.double()).sum(-1) / (dx.double().norm(dim=-1) * x.double().norm(dim=-1))
    assert cosine.abs().max() < 2e-2


@pytest.mark.parametrize("shape", [(5, 1001), (3, 7), (2, 3, 16384), (4, 32768), (1, 1, 8), (9, 2056)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_odd_and_wide_rows(shape, dtype):
    if shape[-1] * torch.empty((), dtype=dtype).element_size() > 65536:
        pytest.skip("beyond the 64 KB row limit")
    g = torch.Generator().manual_seed(3)
    x = torch.randn(*shape, generator=g).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    y, dx = _run(x, dy)
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x, dy, 1e-6)
    assert_close(y, y_ref, atol=ATOL, rtol=RTOL)
    assert_close(dx, dx_ref, atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("cols", [8, 32, 40, 72, 136, 256, 264, 520, 1032, 2056, 4104, 8192, 8200, 16392, 32768])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_every_row_layout(cols, dtype):
    """One width per kernel form: rows that share a wavefront (4, 8, 16, 32 lanes each), one wavefront per
    row with 1 .. 16 chunks per lane, a four-wavefront workgroup per row; 37 rows, so the last wavefront
    of the shared forms is partly empty."""
    if cols * torch.empty((), dtype=dtype).element_size() > 65536:
        pytest.skip("beyond the 64 KB row limit")
    g = torch.Generator().manual_seed(cols)
    x = torch.randn(37, cols, generator=g).to(dtype)
    dy = torch.randn(37, cols, generator=g).to(dtype)
    eps = 1.6e-5 if dtype == torch.float16 else 1e-6
    y, dx = _run(x, dy)
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x, dy, eps)
    assert_close(y, y_ref, atol=ATOL, rtol=RTOL)
    assert_close(dx, dx_ref, atol=ATOL, rtol=RTOL)
    y64, dx64 = oracle.srmsnorm_fwd_bwd(x, dy, eps, torch.float64)
    lim = 1e-6 if dtype == torch.float32 else (1e-3 if dtype == torch.float16 else 5e-3)
    assert rel_norm(y, y64) < lim and rel_norm(dx, dx64) < lim


def test_non_contiguous_input_and_row_limit():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 40, 512, generator=g).bfloat16().transpose(0, 1)
    dy = torch.randn(40, 6, 512, generator=g).bfloat16()
    y, dx = _run(x, dy)
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x, dy, 1e-6)
    assert_close(y, y_ref, atol=ATOL, rtol=RTOL)
    assert_close(dx, dx_ref, atol=ATOL, rtol=RTOL)
    with pytest.raises(RuntimeError, match="64KB"):
        SimpleRMSNorm(40000)(torch.zeros(2, 40000, device=DEV, dtype=torch.bfloat16))
    empty = SimpleRMSNorm(64)(torch.zeros(0, 64, device=DEV, dtype=torch.bfloat16))
    assert empty.shape == (0, 64)


def test_fp16_eps_clamp():
    x = torch.full((4, 256), 1e-4, dtype=torch.float16)
    y, _ = _run(x, torch.ones_like(x), eps=1e-9)
    want = oracle.srmsnorm(x, 1.6e-5)
    assert_close(y, want, atol=1e-3, rtol=1e-2)


@pytest.mark.parametrize("cols, stride", [(1024, 0), (1000, 0), (1024, 7)])
def test_single_row_with_arbitrary_stride(cols, stride):
    """One row: the stride of a dim of size 1 is never used for addressing and may be anything (0 for
    some expanded vectors); it must not reach the kernels as a row stride."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(cols, generator=g).bfloat16()
    dy = torch.randn(1, cols, generator=g).bfloat16()
    xd = x.to(DEV).as_strided((1, cols), (stride, 1)).requires_grad_()
    assert xd.stride(0) == stride
    y = SimpleRMSNorm(cols)(xd)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    y_ref, dx_ref = oracle.srmsnorm_fwd_bwd(x.reshape(1, cols), dy, 1e-6)
    assert_close(y.cpu(), y_ref, atol=ATOL, rtol=RTOL)
    assert_close(xd.grad.cpu(), dx_ref, atol=ATOL, rtol=RTOL)
