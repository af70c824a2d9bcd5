"""Operator surface of lightning_attn/ops/__init__.py:1-3."""
from .lightning_attn_interface import lightning_attn_func, lightning_attn_silu_func, is_support  # noqa: F401
from .torch import linear_attn, SimpleRMSNormTorch  # noqa: F401
from .hip import (  # noqa: F401
    lightning_attn2,
    lightning_attn2_no_decay,
    lightning_attn2_parallel,
    LightningAttention2,
    LightningAttention2NoDecay,
    SimpleRMSNorm,
)
