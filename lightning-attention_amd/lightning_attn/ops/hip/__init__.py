from .lightning_attn2 import (  # noqa: F401
    LightningAttention2,
    LightningAttention2NoDecay,
    lightning_attn2,
    lightning_attn2_no_decay,
    lightning_attn2_parallel,
    lightning_attn_silu,
    silu_fused_ok,
)
from .srmsnorm import SimpleRMSNorm, _SrmsNorm  # noqa: F401
from ._lib import launch_opts  # noqa: F401
from .norm_gate import norm_gate, norm_gate_supported  # noqa: F401
