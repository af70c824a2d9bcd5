from .utils import _build_slope_tensor, get_memory  # noqa: F401
