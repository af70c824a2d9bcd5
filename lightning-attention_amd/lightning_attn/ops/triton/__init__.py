"""Import path of the reference's backend package (lightning_attn/ops/triton/__init__.py:1-4), kept so that
``from lightning_attn.ops.triton import lightning_attn2`` and friends keep working.  Nothing here is
Triton: every name is a re-export of the HIP operators in ``lightning_attn.ops.hip``."""
from ..hip.lightning_attn2 import (  # noqa: F401
    LightningAttention2,
    LightningAttention2NoDecay,
    lightning_attn2,
    lightning_attn2_no_decay,
    lightning_attn2_parallel,
)
from ..hip.srmsnorm import SimpleRMSNorm, _SrmsNorm  # noqa: F401
from . import lightning_attn2 as _m1, lightning_attn2_no_decay as _m2, lightning_attn2_parallel as _m3, srmsnorm as _m4  # noqa: F401,E402
