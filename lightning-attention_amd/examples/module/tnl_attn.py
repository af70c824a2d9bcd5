"""TransNormerLLM attention block around ``lightning_attn_func`` (https://arxiv.org/abs/2405.17381).

Mirror of the reference's examples/module/tnl_attn.py:12-74 — same constructor arguments,
parameter names (``q_proj, k_proj, v_proj, o_proj, norm, output_gate``) and arithmetic, so a
state dict moves over unchanged.  What differs is data movement: the projections' ``(b, n, h*d)``
outputs are handed to the operator as strided ``(b, h, n, d)`` views and its output comes back
token-major, so neither the head split before the operator nor the head merge after it copies
anything (the reference's two ``rearrange`` calls, :56-64, each end in a copy kernel), and the
output LayerNorm, the sigmoid of the gate and their product (:66-69) are one fused row kernel
(``lightning_attn.ops.hip.norm_gate``) where the embedding width allows it.  In inference (no gradient
wanted) the SiLU on q, k, v (:51-54) runs inside the forward kernel's tile load (``lightning_attn_silu_func``).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from lightning_attn.ops import lightning_attn_func, lightning_attn_silu_func
from lightning_attn.ops.hip import norm_gate, norm_gate_supported
from lightning_attn.utils import _build_slope_tensor


class TnlAttention(nn.Module):
    def __init__(self, embed_dim: int, num_heads: int, bias: bool = False, norm_type: str = "layernorm",
                 layer_idx: int = 0, num_layers: int = 12, causal: bool = True):
        super().__init__()
        if embed_dim % num_heads:
            raise ValueError("embed_dim must be a multiple of num_heads")
        self.num_heads = num_heads
        self.head_dim = embed_dim // num_heads
        self.layer_idx = layer_idx
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            setattr(self, name, nn.Linear(embed_dim, embed_dim, bias=bias))
        self.norm = nn.LayerNorm(embed_dim)
        # low-rank gate: embed_dim -> head_dim -> embed_dim
        self.output_gate = nn.Sequential(nn.Linear(embed_dim, self.head_dim, bias=bias),
                                         nn.Linear(self.head_dim, embed_dim, bias=bias))
        # per-head decay rates, shrinking towards the last layer (tnl_attn.py:36-38)
        depth_scale = 1 - layer_idx / (num_layers - 1) + 1e-5
        self.register_buffer("slope_rate", _build_slope_tensor(num_heads) * depth_scale, persistent=False)
        self.fused_norm_gate = True  # False: LayerNorm, sigmoid and product as separate PyTorch operators
        self.fused_silu = True       # False: SiLU on q, k, v as separate PyTorch operators also without gradients

    def _heads(self, t):
        """(b, n, h*d) -> (b, h, n, d) as a view."""
        return t.unflatten(-1, (self.num_heads, self.head_dim)).transpose(-3, -2)

    def forward(self, x, **kwargs):
        # SiLU on the projections and the operator (tnl_attn.py:51-56); one kernel when no gradient is wanted
        q, k, v = (self._heads(proj(x)) for proj in (self.q_proj, self.k_proj, self.v_proj))
        if self.fused_silu:
            mixed = lightning_attn_silu_func(q, k, v, self.slope_rate)  # (b, h, n, d), token-major memory
        else:
            mixed = lightning_attn_func(F.silu(q), F.silu(k), F.silu(v), self.slope_rate)
        mixed = mixed.transpose(-3, -2).flatten(-2)            # (b, n, h*d): a view of that memory
        gate = self.output_gate(x)
        if self._can_fuse(mixed, gate):
            return self.o_proj(norm_gate(mixed, gate, self.norm.weight, self.norm.bias, self.norm.eps))
        return self.o_proj(self.norm(mixed) * torch.sigmoid(gate))

    def _can_fuse(self, mixed, gate):
        """The fused kernel takes one dtype for the activations and the norm's parameters; anything else
        (float32 LayerNorm parameters under autocast, a norm without bias, a width the kernel does not
        take) goes through the three PyTorch operators, as in the reference."""
        w, b = self.norm.weight, self.norm.bias
        return (self.fused_norm_gate and mixed.is_cuda and w is not None and b is not None
                and mixed.dtype == gate.dtype == w.dtype == b.dtype
                and norm_gate_supported(mixed.shape[-1], mixed.dtype))


if __name__ == "__main__":
    dev, dt = torch.device("cuda"), torch.bfloat16
    block = TnlAttention(embed_dim=1024, num_heads=8).to(dev).to(dt)
    x = torch.randn(2, 1024, 1024, device=dev, dtype=dt).requires_grad_()
    y = block(x)
    y.sum().backward()
    print(tuple(y.shape), tuple(x.grad.shape))
