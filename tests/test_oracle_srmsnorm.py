"""Pins the SimpleRMSNorm oracle: library routine, plain C, closed-form backward, invariants."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import c_oracle
from oracle.srmsnorm_oracle import srmsnorm_bwd_closed_form
from lightning_attn.ops import SimpleRMSNormTorch


@pytest.mark.parametrize("shape", [(3, 8), (2, 5, 768), (4, 1025)])
def test_forward_vs_library_and_c(shape):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(*shape, generator=g)
    y = oracle.srmsnorm(x, 1e-6)
    assert torch.allclose(y, F.rms_norm(x, (shape[-1],), None, 1e-6), rtol=1e-5, atol=1e-6)
    assert torch.equal(y, SimpleRMSNormTorch(shape[-1])(x))
    yc, _ = c_oracle.srms_fwd(x.reshape(-1, shape[-1]).double().numpy(), 1e-6)
    assert np.allclose(oracle.srmsnorm_f64(x).reshape(-1, shape[-1]).numpy(), yc, rtol=1e-12, atol=1e-12)
    for dt in (torch.float16, torch.bfloat16):
        assert oracle.srmsnorm(x.to(dt)).dtype == dt


def test_backward_closed_form_and_c():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(7, 96, generator=g, dtype=torch.float64)
    dy = torch.randn(7, 96, generator=g, dtype=torch.float64)
    _, dx = oracle.srmsnorm_fwd_bwd(x, dy, 1e-6, torch.float64)
    assert torch.allclose(dx, srmsnorm_bwd_closed_form(x, dy, 1e-6), rtol=1e-10, atol=1e-12)
    assert np.allclose(dx.numpy(), c_oracle.srms_bwd(x.numpy(), dy.numpy(), 1e-6), rtol=1e-10, atol=1e-12)
    xx = x[:2, :8].clone().requires_grad_()
    assert torch.autograd.gradcheck(lambda t: oracle.srmsnorm_f64(t, 1e-6), (xx,), eps=1e-6, atol=1e-6)


def test_invariants():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 512, generator=g, dtype=torch.float64)
    dy = torch.randn(5, 512, generator=g, dtype=torch.float64)
    eps = 1e-6
    y = oracle.srmsnorm_f64(x, eps)
    rstd = torch.rsqrt(x.pow(2).mean(-1) + eps)
    assert torch.allclose(y.pow(2).mean(-1), 1 - eps * rstd**2, rtol=1e-12)
    # scale invariance up to eps, and dx orthogonal to x up to eps
    assert torch.allclose(oracle.srmsnorm_f64(3 * x, eps), y, rtol=1e-5)
    _, dx = oracle.srmsnorm_fwd_bwd(x, dy, eps, torch.float64)
    assert ((dx * x).sum(-1).abs() / (dx.norm(dim=-1) * x.norm(dim=-1))).max() < 1e-5
