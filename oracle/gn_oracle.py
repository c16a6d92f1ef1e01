"""Python face of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this module; the
product (the gnnhwc package and libgnnhwc_hip.so) never does.

Two checkers live here:

* the C restatement of the reference's algorithm (gn_oracle.c, loaded with ctypes), operating on
  numpy arrays laid out (N, R, C) like the kernels' operands (src/gnnhwc/csrc/custom_gn.cpp:24,64-65);
* ``torch_reference``: ``act(F.group_norm(x))`` plus autograd, the routine the reference's own tests
  compare against (test/check_outputs.py:91-157, test/trailing_dims.py:22-26) and the results contract.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgn_oracle.so")
_lib = None

# same integers as GN_NHWC.act_code (src/gnnhwc/custom_gn.py:52-59)
ACT_CODES = {"identity": 0, "relu": 1, "swish": 2, "silu": 2, "gelu": 3, "gelu_tanh": 4}
ACT_NAMES = ["identity", "relu", "silu", "gelu", "gelu_tanh"]


def build(force=False):
    """Compile libgn_oracle.so with gcc (a few hundred milliseconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libgn_oracle.so"])
    return _LIB_PATH


def load():
    global _lib
    if _lib is not None:
        return _lib
    build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, dbl, vp, ci = ctypes.c_int64, ctypes.c_double, ctypes.c_void_p, ctypes.c_int
    for suf in ("f64", "f32"):
        getattr(lib, "gn_oracle_stats_" + suf).argtypes = [vp, i64, i64, i64, i64, dbl, vp, vp]
        getattr(lib, "gn_oracle_stats_" + suf).restype = None
        getattr(lib, "gn_oracle_fwd_" + suf).argtypes = [vp, vp, vp, i64, i64, i64, i64, dbl, ci, vp, vp, vp]
        getattr(lib, "gn_oracle_fwd_" + suf).restype = None
        getattr(lib, "gn_oracle_bwd_" + suf).argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, vp, vp, vp, vp]
        getattr(lib, "gn_oracle_bwd_" + suf).restype = None
    _lib = lib
    return lib


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64"
    if dtype == np.float32:
        return "f32"
    raise TypeError("the C oracle computes in float64 or float32, not %s" % dtype)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _prep(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def stats(x, G, eps=1e-5, dtype=np.float64):
    """x: (N, R, C).  Returns mean, rstd of shape (N, G)."""
    lib = load()
    x = _prep(x, dtype)
    N, R, C = x.shape
    mean = np.empty((N, G), dtype)
    rstd = np.empty((N, G), dtype)
    getattr(lib, "gn_oracle_stats_" + _suffix(dtype))(_p(x), N, R, C, G, eps, _p(mean), _p(rstd))
    return mean, rstd


def fwd(x, w, b, G, eps=1e-5, act=0, dtype=np.float64):
    """x: (N, R, C); w, b: (C).  Returns y (N, R, C), mean (N, G), rstd (N, G)."""
    lib = load()
    x, w, b = _prep(x, dtype), _prep(w, dtype), _prep(b, dtype)
    N, R, C = x.shape
    assert C % G == 0 and w.shape == (C,) and b.shape == (C,)
    y = np.empty_like(x)
    mean = np.empty((N, G), dtype)
    rstd = np.empty((N, G), dtype)
    getattr(lib, "gn_oracle_fwd_" + _suffix(dtype))(_p(x), _p(w), _p(b), N, R, C, G, eps, int(act), _p(y), _p(mean), _p(rstd))
    return y, mean, rstd


def bwd(dy, x, w, b, mean, rstd, G, act=0, dtype=np.float64):
    """Returns dx (N, R, C), dgamma (C), dbeta (C)."""
    lib = load()
    dy, x, w, b = _prep(dy, dtype), _prep(x, dtype), _prep(w, dtype), _prep(b, dtype)
    mean, rstd = _prep(mean, dtype), _prep(rstd, dtype)
    N, R, C = x.shape
    dx = np.empty_like(x)
    dw = np.empty((C,), dtype)
    db = np.empty((C,), dtype)
    scratch = np.empty((2 * N * C,), dtype)
    getattr(lib, "gn_oracle_bwd_" + _suffix(dtype))(_p(dy), _p(x), _p(w), _p(b), _p(mean), _p(rstd), N, R, C, G, int(act),
                                                    _p(dx), _p(dw), _p(db), _p(scratch))
    return dx, dw, db


def fwd_bwd(x, w, b, dy, G, eps=1e-5, act=0, dtype=np.float64):
    y, mean, rstd = fwd(x, w, b, G, eps, act, dtype)
    dx, dw, db = bwd(dy, x, w, b, mean, rstd, G, act, dtype)
    return dict(y=y, mean=mean, rstd=rstd, dx=dx, dw=dw, db=db)


# ---------------------------------------------------------------------------------------------
# torch: the results contract
# ---------------------------------------------------------------------------------------------
def torch_act(name):
    import torch.nn.functional as F

    return {
        "identity": lambda t: t,
        "relu": F.relu,
        "silu": F.silu,
        "swish": F.silu,
        "gelu": F.gelu,
        "gelu_tanh": lambda t: F.gelu(t, approximate="tanh"),
    }[name]


def torch_reference(x, w, b, G, eps, act, dy=None):
    """act(F.group_norm(x, G, w, b, eps)) on x of shape (N, C, *spatial), any strides, in x's dtype and device.

    Returns dict(y=...) and, when dy is given, dx, dw, db from autograd (test/check_outputs.py:104-157)."""
    import torch
    import torch.nn.functional as F

    name = act if isinstance(act, str) else ACT_NAMES[act]
    xr = x.detach().clone().requires_grad_(dy is not None)
    wr = w.detach().clone().requires_grad_(dy is not None)
    br = b.detach().clone().requires_grad_(dy is not None)
    y = torch_act(name)(F.group_norm(xr, G, wr, br, eps))
    out = {"y": y.detach()}
    if dy is not None:
        dx, dw, db = torch.autograd.grad(y, (xr, wr, br), dy)
        out.update(dx=dx, dw=dw, db=db)
    return out


def to_nrc(t):
    """(N, C, *spatial) torch tensor -> (N, R, C) numpy float64 array (the kernels' operand layout)."""
    import torch

    N, C = t.shape[0], t.shape[1]
    return t.detach().to("cpu", torch.float64).reshape(N, C, -1).permute(0, 2, 1).contiguous().numpy()


def from_nrc(a, shape):
    """(N, R, C) numpy array -> float64 torch tensor of logical shape (N, C, *spatial)."""
    import torch

    N, C = shape[0], shape[1]
    return torch.from_numpy(np.ascontiguousarray(a)).reshape(N, -1, C).permute(0, 2, 1).reshape(shape)
