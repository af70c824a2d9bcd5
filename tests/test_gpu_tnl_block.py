"""TNL attention block (examples/module/tnl_attn.py of the reference, :12-74) built on the HIP operator:
forward and input / weight gradients against the same block evaluated on the CPU in float32 with
the naive oracle in place of the operator.  Tolerance: relative Frobenius error below 2e-2 (bf16
weights and activations through four projections, a LayerNorm and the operator)."""
import importlib.util
import os

import pytest
import torch
import torch.nn.functional as F

import oracle
from util import rel_norm

pytestmark = pytest.mark.gpu

_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lightning-attention_amd", "examples",
                     "module", "tnl_attn.py")
_spec = importlib.util.spec_from_file_location("tnl_attn_example", _PATH)
tnl = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(tnl)


def _reference_block(block, x):
    """The block's arithmetic in float32 on the CPU; the operator is the naive oracle."""
    p = {k: v.detach().float().cpu().requires_grad_() for k, v in block.named_parameters()}
    x = x.detach().float().cpu().requires_grad_()
    h, d = block.num_heads, block.head_dim

    def lin(name, t):
        return F.linear(t, p[name + ".weight"], p.get(name + ".bias"))

    q, k, v = (F.silu(lin(n, x)).unflatten(-1, (h, d)).transpose(1, 2) for n in ("q_proj", "k_proj", "v_proj"))
    o = oracle.linear_attn(q, k, v, block.slope_rate.float().cpu())
    o = o.transpose(1, 2).flatten(-2)
    o = F.layer_norm(o, (h * d,), p["norm.weight"], p["norm.bias"])
    gate = torch.sigmoid(lin("output_gate.1", lin("output_gate.0", x)))
    return lin("o_proj", o * gate), x, p


@pytest.mark.parametrize("b, n, embed, heads, layer", [(2, 384, 512, 4, 0), (1, 1000, 768, 12, 5)])
def test_tnl_block_matches_float32_reference(b, n, embed, heads, layer):
    torch.manual_seed(3)
    block = tnl.TnlAttention(embed, heads, layer_idx=layer, num_layers=12).cuda().bfloat16()
    x = torch.randn(b, n, embed, device="cuda", dtype=torch.bfloat16).requires_grad_()
    g = torch.randn(b, n, embed, device="cuda", dtype=torch.bfloat16)
    y = block(x)
    y.backward(g)
    torch.cuda.synchronize()
    want, xr, pr = _reference_block(block, x)
    want.backward(g.float().cpu())
    assert y.shape == (b, n, embed) and y.dtype == torch.bfloat16
    assert rel_norm(y.detach().float().cpu(), want.detach()) < 2e-2
    assert rel_norm(x.grad.float().cpu(), xr.grad) < 2e-2
    for name, prm in block.named_parameters():
        assert rel_norm(prm.grad.float().cpu(), pr[name].grad) < 3e-2, name


def test_state_dict_names_follow_the_reference():
    block = tnl.TnlAttention(256, 4)
    names = set(block.state_dict().keys())
    assert names == {"q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight", "norm.weight", "norm.bias",
                     "output_gate.0.weight", "output_gate.1.weight"}
    assert block.slope_rate.shape == (4, 1, 1)


def test_float32_norm_parameters_take_the_unfused_path():
    """A LayerNorm kept in float32 beside bf16 activations (master weights, autocast) cannot go through the fused
    kernel, which takes one dtype: the block then runs the three PyTorch operators of tnl_attn.py:66-69 instead
    of raising, and agrees with the fused path on bf16 parameters to bf16 rounding."""
    torch.manual_seed(4)
    block = tnl.TnlAttention(512, 4).cuda().bfloat16()
    x = torch.randn(2, 200, 512, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        fused = block(x)
    block.norm.float()
    gate = block.output_gate(x)
    assert not block._can_fuse(x, gate)
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        y = block(x)
    torch.cuda.synchronize()
    assert y.shape == fused.shape
    assert rel_norm(y.float(), fused.float()) < 2e-2
    # a norm without bias is not the fused kernel's either
    block2 = tnl.TnlAttention(512, 4).cuda().bfloat16()
    block2.norm = torch.nn.LayerNorm(512, bias=False).cuda().bfloat16()
    assert not block2._can_fuse(x, gate)
    with torch.no_grad():
        assert block2(x).shape == x.shape
