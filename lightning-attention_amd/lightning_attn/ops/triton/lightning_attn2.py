"""lightning_attn/ops/triton/lightning_attn2.py:398-507 by name; the operator is the HIP one."""
from ..hip.lightning_attn2 import LightningAttention2, lightning_attn2  # noqa: F401
