"""Lightning Attention for MI355X (gfx950): the reference's Python operator API
(lightning_attn/__init__.py:1-2) over hand-written HIP kernels."""
from .ops import *  # noqa: F401,F403
from .utils import *  # noqa: F401,F403
from .utils import _build_slope_tensor, get_memory  # noqa: F401

__version__ = "0.1.0"
