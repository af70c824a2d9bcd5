"""Public dispatch function, lightning_attn/ops/lightning_attn_interface.py:16-65.

The reference pads e to a power of two and splits d > 128 into <= 64-wide
slices because its Triton tiles need that; the HIP kernels tile any multiple of
8 up to 256 natively (128 for float32), so neither happens here (other sizes are
zero-padded to the next multiple of 8, which is exact).  Larger feature
dims are split into slices of q/k whose partial outputs add up (the scores are
additive over feature slices) and into column groups of v."""
import torch

from .hip.lightning_attn2 import lightning_attn2, lightning_attn2_no_decay, lightning_attn_silu, silu_fused_ok

_VARIANTS = ("chunk_loop", "parallel")


def is_support(dim):
    """True when a feature dim is usable: any positive size.  Multiples of 8 run as they are, other
    sizes are zero-padded to the next multiple of 8 (the reference's gate, ``16 % dim``, rejects the
    divisors of 16 and pads e to a power of two, lightning_attn_interface.py:8-9, 29-33)."""
    return dim > 0


def _pad8(t):
    """Last dim zero-padded to the next multiple of 8: zero features add nothing to q . k, zero
    columns of v give zero columns of o."""
    extra = -t.shape[-1] % 8
    return torch.nn.functional.pad(t, (0, extra)) if extra else t


def lightning_attn_func(q, k, v, s=None, variant="chunk_loop"):
    """o = (q k^T * M) v with M[i,j] = exp(-s_h (i-j)) [i >= j]; s=None means no decay.

    q, k: (b, h, n, d); v: (b, h, n, e); s: h float32 rates (any shape with h
    elements) or None.  Returns (b, h, n, e) in q.dtype; differentiable in
    q, k, v."""
    if variant not in _VARIANTS:
        raise ValueError("variant must be one of %s, got %r" % (_VARIANTS, variant))
    b, h, n, d = q.shape
    e = v.shape[-1]
    assert is_support(d) and is_support(e), "feature dims must be positive (got d=%d, e=%d)" % (d, e)
    if d % 8 or e % 8:
        return lightning_attn_func(_pad8(q), _pad8(k), _pad8(v), s, variant)[..., :e]

    _MAX_DIM = 128 if q.dtype == torch.float32 else 256

    def run(q1, k1, v1):
        if s is None:
            return lightning_attn2_no_decay(q1, k1, v1)
        return lightning_attn2(q1, k1, v1, s)

    if e > _MAX_DIM:
        # output columns are independent: cut v
        outs = [lightning_attn_func(q, k, v[..., c : c + _MAX_DIM], s, variant) for c in range(0, e, _MAX_DIM)]
        return torch.cat(outs, dim=-1)
    if d > _MAX_DIM:
        o = None
        for c in range(0, d, _MAX_DIM):
            part = run(q[..., c : c + _MAX_DIM], k[..., c : c + _MAX_DIM], v)
            o = part if o is None else o + part
        return o
    return run(q, k, v)


def lightning_attn_silu_func(q, k, v, s=None, variant="chunk_loop"):
    """lightning_attn_func(silu(q), silu(k), silu(v), s): what the reference's attention block computes from its
    projections (examples/module/tnl_attn.py:51-56).  Without a gradient to compute (inference), bf16 / fp16 and
    feature dims that are multiples of 8 up to 128, the activation is applied inside the forward kernel and the
    three activation passes disappear; otherwise this is the three PyTorch calls followed by lightning_attn_func."""
    if variant not in _VARIANTS:
        raise ValueError("variant must be one of %s, got %r" % (_VARIANTS, variant))
    d, e = q.shape[-1], v.shape[-1]
    if d % 8 == 0 and e % 8 == 0 and silu_fused_ok(q, k, v):
        return lightning_attn_silu(q, k, v, s)
    f = torch.nn.functional.silu
    return lightning_attn_func(f(q), f(k), f(v), s, variant)
