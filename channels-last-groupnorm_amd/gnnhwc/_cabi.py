"""ctypes binding of libgnnhwc_hip.so (C ABI declared in include/gnnhwc.h).

The library is built ahead of time, in-tree, by ``make -C channels-last-groupnorm_amd/csrc`` (or
``__graft_entry__.build()``).  There is no fallback: if the shared object is missing or does not
export the expected symbols, importing this module raises.
"""
import ctypes
import os

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
# With GNNHWC_TRACE set (1 or 2) at import, the twin library with the in-kernel phase stamps compiled in is loaded instead
# (bench.py --timeline); the library proper carries no trace code at all.
TRACING = os.environ.get("GNNHWC_TRACE", "0") not in ("", "0")
LIB_PATH = os.path.join(_CSRC, "libgnnhwc_hip_trace.so" if TRACING else "libgnnhwc_hip.so")

# dtype / activation codes of include/gnnhwc.h
F32, F64, F16, BF16 = 0, 1, 2, 3
STATIC_SCRATCH_BYTES = 4 << 20  # GNNHWC_STATIC_SCRATCH_BYTES
NUM_KERNEL_KINDS = 15

SYMBOLS = (
    "gnnhwc_version",
    "gnnhwc_last_error",
    "gnnhwc_fwd_workspace_bytes",
    "gnnhwc_bwd_workspace_bytes",
    "gnnhwc_fwd",
    "gnnhwc_fwd_cast",
    "gnnhwc_fwd_add",
    "gnnhwc_fwd_static",
    "gnnhwc_fwd_static_scratch_bytes",
    "gnnhwc_bwd",
    "gnnhwc_bwd_cast",
    "gnnhwc_nchw_workspace_bytes",
    "gnnhwc_fwd_nchw",
    "gnnhwc_bwd_nchw",
    "gnnhwc_profile_enable",
    "gnnhwc_profile_collect",
    "gnnhwc_kernel_kind_name",
    "gnnhwc_set_resident",
    "gnnhwc_resident_status",
    "gnnhwc_debug_read_trace",
    "gnnhwc_debug_plan",
    "gnnhwc_debug_last_launch",
    "gnnhwc_debug_load_tile",
)


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "gnnhwc: %s not found. Build the HIP extension first: make -C %s   "
            "(there is deliberately no non-HIP fallback)" % (LIB_PATH, _CSRC)
        )
    lib = ctypes.CDLL(LIB_PATH)
    i64, vp, ci, sz, dbl = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_double
    for name in SYMBOLS:
        if not hasattr(lib, name):
            raise ImportError("gnnhwc: %s does not export %s" % (LIB_PATH, name))
    lib.gnnhwc_version.restype = ci
    lib.gnnhwc_last_error.restype = ctypes.c_char_p
    lib.gnnhwc_fwd_workspace_bytes.argtypes = [i64, i64, i64, i64, ci]
    lib.gnnhwc_fwd_workspace_bytes.restype = sz
    lib.gnnhwc_bwd_workspace_bytes.argtypes = [i64, i64, i64, i64, ci]
    lib.gnnhwc_bwd_workspace_bytes.restype = sz
    lib.gnnhwc_fwd.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, dbl, ci, ci, ci, ci, vp, sz, vp]
    lib.gnnhwc_fwd.restype = ci
    lib.gnnhwc_fwd_cast.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, dbl, ci, ci, ci, ci, ci, vp, sz, vp]
    lib.gnnhwc_fwd_cast.restype = ci
    lib.gnnhwc_fwd_add.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, dbl, ci, ci, ci, ci, ci, vp, sz, vp]
    lib.gnnhwc_fwd_add.restype = ci
    lib.gnnhwc_fwd_static.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, dbl, ci, ci, ci, ci, vp]
    lib.gnnhwc_fwd_static.restype = ci
    lib.gnnhwc_fwd_static_scratch_bytes.argtypes = [i64, i64, i64, i64, ci]
    lib.gnnhwc_fwd_static_scratch_bytes.restype = sz
    lib.gnnhwc_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, ci, ci, ci, vp, sz, vp]
    lib.gnnhwc_bwd.restype = ci
    lib.gnnhwc_bwd_cast.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, ci, ci, ci, ci, vp, sz, vp]
    lib.gnnhwc_bwd_cast.restype = ci
    lib.gnnhwc_nchw_workspace_bytes.argtypes = [i64, i64, i64, i64, ci, ci]
    lib.gnnhwc_nchw_workspace_bytes.restype = sz
    lib.gnnhwc_fwd_nchw.argtypes = list(lib.gnnhwc_fwd.argtypes)
    lib.gnnhwc_fwd_nchw.restype = ci
    lib.gnnhwc_bwd_nchw.argtypes = list(lib.gnnhwc_bwd.argtypes)
    lib.gnnhwc_bwd_nchw.restype = ci
    lib.gnnhwc_profile_enable.argtypes = [ci]
    lib.gnnhwc_profile_enable.restype = ci
    lib.gnnhwc_profile_collect.argtypes = [ctypes.POINTER(i64), ctypes.POINTER(dbl)]
    lib.gnnhwc_profile_collect.restype = ci
    lib.gnnhwc_set_resident.argtypes = [ci]
    lib.gnnhwc_set_resident.restype = ci
    lib.gnnhwc_resident_status.argtypes = []
    lib.gnnhwc_resident_status.restype = ci
    lib.gnnhwc_debug_read_trace.argtypes = [vp, i64]
    lib.gnnhwc_debug_read_trace.restype = ci
    lib.gnnhwc_debug_set_spin_limit.argtypes = [ci]
    lib.gnnhwc_debug_set_spin_limit.restype = ci
    lib.gnnhwc_debug_load_tile.argtypes = [vp, vp, vp, i64, i64, i64, ci, vp]
    lib.gnnhwc_debug_load_tile.restype = ci
    lib.gnnhwc_debug_copy.argtypes = [vp, vp, sz, vp]
    lib.gnnhwc_debug_copy.restype = ci
    lib.gnnhwc_debug_plan.argtypes = [i64, i64, i64, i64, ci, ci, ci, ctypes.POINTER(i64)]
    lib.gnnhwc_debug_plan.restype = ci
    lib.gnnhwc_debug_last_launch.argtypes = [ctypes.POINTER(i64)]
    lib.gnnhwc_debug_last_launch.restype = ci
    lib.gnnhwc_kernel_kind_name.argtypes = [ci]
    lib.gnnhwc_kernel_kind_name.restype = ctypes.c_char_p
    return lib


lib = _load()


def last_error():
    return lib.gnnhwc_last_error().decode("utf-8", "replace")


def check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, last_error()))


def kernel_kind_names():
    return [lib.gnnhwc_kernel_kind_name(k).decode() for k in range(NUM_KERNEL_KINDS)]


def last_launch():
    """What the calling thread's most recent forward / backward call launched: e.g. 'fused_bwd rows=22 window=0 parked=0
    two_level=0 launches=1' for a single-launch kernel, 'multi-launch' for the streaming kernels."""
    out = (ctypes.c_int64 * 7)()
    check(lib.gnnhwc_debug_last_launch(out), "gnnhwc_debug_last_launch")
    if out[0] < 0:
        return "multi-launch"
    return "%s rows=%d window=%d parked=%d two_level=%d launches=%d" % (kernel_kind_names()[out[0]], out[1], out[2], out[6], out[3], out[4])


def set_resident(on):
    """Allow (True) or forbid (False) the single-launch kernels; returns the previous setting."""
    return bool(lib.gnnhwc_set_resident(1 if on else 0))


def profile_enable(on):
    check(lib.gnnhwc_profile_enable(1 if on else 0), "gnnhwc_profile_enable")


def profile_collect():
    """Returns {kind name: (launches, total milliseconds)} since the previous collect."""
    n = (ctypes.c_int64 * NUM_KERNEL_KINDS)()
    ms = (ctypes.c_double * NUM_KERNEL_KINDS)()
    check(lib.gnnhwc_profile_collect(n, ms), "gnnhwc_profile_collect")
    names = kernel_kind_names()
    return {names[k]: (int(n[k]), float(ms[k])) for k in range(NUM_KERNEL_KINDS)}
