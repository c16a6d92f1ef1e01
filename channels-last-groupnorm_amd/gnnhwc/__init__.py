from .custom_gn import GN_NHWC_Func, GN_NHWC  # noqa: F401  (same exports as src/gnnhwc/__init__.py:1)
