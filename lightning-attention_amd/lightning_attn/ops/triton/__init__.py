"""Import path of the reference's backend package (lightning_attn/ops/triton/__init__.py:1-4), kept so that
``from lightning_attn.ops.triton import lightning_attn2`` and friends keep working.  Nothing here is
Triton: every name is a re-export of the HIP operators in ``lightning_attn.ops.hip``.

The operator names are also the names of this package's submodules.  Importing a submodule sets the
package attribute of that name to the module, so the submodules are imported first and the names are
bound to the operators afterwards, as the reference's package does: the operators then stay in
place whatever a caller imports later."""
from .lightning_attn2 import LightningAttention2, lightning_attn2  # noqa: F401
from .lightning_attn2_no_decay import LightningAttention2NoDecay, lightning_attn2_no_decay  # noqa: F401
from .lightning_attn2_parallel import lightning_attn2_parallel  # noqa: F401
from .srmsnorm import SimpleRMSNorm, _SrmsNorm  # noqa: F401
