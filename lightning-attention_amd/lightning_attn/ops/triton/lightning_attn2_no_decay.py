"""lightning_attn/ops/triton/lightning_attn2_no_decay.py:367-471 by name; the operator is the HIP one."""
from ..hip.lightning_attn2 import LightningAttention2NoDecay, lightning_attn2_no_decay  # noqa: F401
