"""lightning_attn/ops/triton/srmsnorm.py:76-185 by name; the operator is the HIP one."""
from ..hip.srmsnorm import SimpleRMSNorm, _SrmsNorm  # noqa: F401
