"""Oracle for SimpleRMSNorm (no affine) -- test infrastructure.

Restates lightning_attn/ops/torch/srmsnorm.py:9-20:
    y = (x.float() * rsqrt(mean(x.float()^2, -1) + eps)).type_as(x)
and the backward the reference's device kernel implements
(lightning_attn/ops/triton/srmsnorm.py:38-74):
    xhat = x*rstd ; c = mean(xhat*dy) ; dx = (dy - xhat*c) * rstd
The fp16 eps clamp max(eps, 1.6e-5) lives in the device wrapper
(ops/triton/srmsnorm.py:80-81), not in the torch module.

Pinned by: torch.nn.functional.rms_norm (library routine), the plain C fp64
restatement in oracle/la_oracle.c, autograd vs the closed-form dx, and the
invariants mean(y^2) = 1 - eps*rstd^2 and sum(dx*x) ~ eps-order.
"""
import torch


def srmsnorm(x, eps=1e-6):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)


def srmsnorm_f64(x, eps=1e-6):
    xf = x.double()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)


def srmsnorm_fwd_bwd(x, dy, eps=1e-6, compute_dtype=None):
    """y, dx through autograd of the one-line norm.  compute_dtype=float64
    gives the exact-arithmetic target on the given inputs."""
    if compute_dtype == torch.float64:
        xx = x.detach().double().requires_grad_()
        y = srmsnorm_f64(xx, eps)
        y.backward(dy.double())
        return y.detach(), xx.grad
    xx = x.detach().clone().requires_grad_()
    y = srmsnorm(xx, eps)
    y.backward(dy)
    return y.detach(), xx.grad


def srmsnorm_bwd_closed_form(x, dy, eps=1e-6, dtype=torch.float64):
    """dx = rstd * (dy - y * mean(y*dy)), the kernel's formula."""
    xf, g = x.to(dtype), dy.to(dtype)
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    y = xf * rstd
    return rstd * (g - y * (y * g).mean(-1, keepdim=True))
