from .custom_gn import GN_NHWC_Func, GN_NHWC  # noqa: F401  (same exports as src/gnnhwc/__init__.py:1)
from .custom_gn import group_norm_nhwc  # noqa: F401  (traceable functional form; no counterpart in the reference)
from .custom_gn import GN_NCHW_Func  # noqa: F401  (channels-first input; the reference falls back to torch there)
