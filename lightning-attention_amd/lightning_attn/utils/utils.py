"""Host helpers with the semantics of lightning_attn/utils/utils.py:6-38."""
import math

import torch


def _pow2_head_rates(count):
    # geometric sequence base^(i+1) with base = 2^(-8/count), accumulated the way
    # the reference does (float multiply of start and ratio**i) so that the
    # float32 values agree bit for bit
    base = 2.0 ** (-(2.0 ** -(math.log2(count) - 3)))
    return [base * base**i for i in range(count)]


def _head_rates(count):
    if count & (count - 1) == 0:
        return _pow2_head_rates(count)
    below = 1 << (count.bit_length() - 1)
    extra = _head_rates(2 * below)[0::2][: count - below]
    return _pow2_head_rates(below) + extra


def _build_slope_tensor(n_attention_heads: int):
    """Per-head decay rates s_h, float32, shape (h, 1, 1), on the CPU.

    Power-of-two head counts give 2^(-8(i+1)/h); other counts take the rates of
    the next lower power of two and append every other rate of the next higher
    one (lightning_attn/utils/utils.py:6-31)."""
    if n_attention_heads < 1:
        raise ValueError("n_attention_heads must be >= 1")
    return torch.tensor(_head_rates(int(n_attention_heads))).reshape(n_attention_heads, 1, 1)


def get_memory(device):
    """Peak allocated device memory in MiB since the last call, then reset
    (lightning_attn/utils/utils.py:34-38)."""
    mb_used = torch.cuda.max_memory_allocated(device) / 1024 / 1024
    torch.cuda.reset_peak_memory_stats(device)
    return mb_used
