"""Naive O(n^2) decayed linear attention in plain PyTorch: the public
``linear_attn`` of lightning_attn/ops/torch/linear_attention.py:4-34.  It runs on
whatever device its inputs live on and is never called by the HIP operators."""
import torch


def get_mask(n, slope=1):
    """(n, n) float32 matrix exp(-slope*(i-j)) on and below the diagonal, 0 above."""
    pos = torch.arange(n)
    lag = pos.view(n, 1) - pos.view(1, n)
    decay = torch.exp(-(lag.clamp(min=0).float() * slope))
    return decay.masked_fill(lag < 0, 0.0)


def get_full_mask(n, slopes):
    """(h, n, n) stack of per-head masks, or tril(ones) when slopes is None."""
    if slopes is None:
        return torch.tril(torch.ones((n, n)))
    return torch.stack([get_mask(n, rate.item()) for rate in slopes.reshape(-1)], dim=0)


def linear_attn(q, k, v, s=None):
    """o = ((q k^T) * mask) v with scores kept in q.dtype and the mask applied in float32."""
    n = q.shape[2]
    mask = get_full_mask(n, s).to(q.device).to(torch.float32)
    scores = torch.matmul(q, k.transpose(2, 3))
    scores = (scores.to(torch.float32) * mask).to(q.dtype)
    return torch.matmul(scores, v)
