"""Oracle for the gated output norm of the TNL attention block -- test infrastructure.

Restates examples/module/tnl_attn.py:66-69 of the reference,
    output = self.norm(output)                     # nn.LayerNorm(embed_dim), eps = 1e-5
    output_gate = F.sigmoid(self.output_gate(x))
    output = output * output_gate
as one function of the attention output o and the gate pre-activation g:
    y = layer_norm(o, (C,), weight, bias, eps) * sigmoid(g)
computed in float32 (or float64) on the given inputs, gradients through autograd.

Pinned by: ``torch.nn.functional.layer_norm`` and ``torch.sigmoid`` (library routines) on one side
and, on the other, the closed-form expressions the device kernel evaluates
(``norm_gate_closed_form``: mean / variance by explicit sums, the hand-derived gradients), which
tests/test_oracle_norm_gate.py checks against each other and with ``gradcheck`` in float64.
"""
import torch
import torch.nn.functional as F


def norm_gate(o, g, weight, bias, eps=1e-5, dtype=torch.float32):
    o, g, weight, bias = (t.to(dtype) for t in (o, g, weight, bias))
    return F.layer_norm(o, (o.shape[-1],), weight, bias, eps) * torch.sigmoid(g)


def norm_gate_fwd_bwd(o, g, weight, bias, dy, eps=1e-5, dtype=torch.float32):
    """y, d_o, d_g, d_weight, d_bias at precision `dtype` on the given (already rounded) inputs."""
    leaves = [t.detach().to(dtype).requires_grad_() for t in (o, g, weight, bias)]
    y = norm_gate(*leaves, eps=eps, dtype=dtype)
    y.backward(dy.to(dtype))
    return (y.detach(),) + tuple(t.grad for t in leaves)


def norm_gate_closed_form(o, g, weight, bias, dy, eps=1e-5, dtype=torch.float64):
    """The kernel's own formulas, written out: no autograd, no library norm."""
    o, g, w, b, dy = (t.to(dtype) for t in (o, g, weight, bias, dy))
    c = o.shape[-1]
    mu = o.sum(-1, keepdim=True) / c
    var = ((o - mu) ** 2).sum(-1, keepdim=True) / c
    rstd = 1.0 / torch.sqrt(var + eps)
    xh = (o - mu) * rstd
    ln = xh * w + b
    sg = 1.0 / (1.0 + torch.exp(-g))
    y = ln * sg
    dln = dy * sg
    d_g = dy * ln * sg * (1.0 - sg)
    dxh = dln * w
    d_o = rstd * (dxh - dxh.mean(-1, keepdim=True) - xh * (dxh * xh).mean(-1, keepdim=True))
    flat = lambda t: t.reshape(-1, c)
    return y, d_o, d_g, (flat(dln) * flat(xh)).sum(0), flat(dln).sum(0)
