"""lightning_attn/ops/triton/lightning_attn2_parallel.py:835-1072 by name: the HIP sweep kernels cut the
sequence into chunks by themselves, so the chunk-parallel variant is the same operator."""
from ..hip.lightning_attn2 import LightningAttention2 as LightningAttention2Parallel, lightning_attn2_parallel  # noqa: F401
