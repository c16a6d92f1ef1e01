"""Helpers for the GPU parity tests: direct calls through the C ABI on torch-owned device memory, and the
error metrics the tolerances are written in."""
import ctypes

import numpy as np
import torch

from gnnhwc import _cabi

from workloads import DT_CODE, nrc_view  # noqa: F401  (re-exported: the tests import them from here)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def cabi_fwd(x_nrc, w, b, G, eps, act, stats_dtype=None, y=None, ws=None):
    """gnnhwc_fwd on (N, R, C) device tensors.  Returns y, mean, rstd."""
    N, R, C = x_nrc.shape
    dt = DT_CODE[x_nrc.dtype]
    sdtype = stats_dtype or (torch.float32 if x_nrc.dtype in (torch.float16, torch.bfloat16) else x_nrc.dtype)
    pdt = DT_CODE[w.dtype] if w is not None else dt
    y = torch.empty_like(x_nrc) if y is None else y
    mean = torch.empty((N, G), dtype=sdtype, device=x_nrc.device)
    rstd = torch.empty((N, G), dtype=sdtype, device=x_nrc.device)
    lib = _cabi.lib
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, dt)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x_nrc.device) if ws is None else ws
    rc = lib.gnnhwc_fwd(_ptr(x_nrc), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), N, R, C, G, float(eps), int(act),
                        dt, pdt, DT_CODE[sdtype], _ptr(ws), ws.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_fwd")
    return y, mean, rstd


def cabi_fwd_add(x_nrc, residual, channel_bias, w, b, G, eps, act, want_sum=True, sum_out=None, y=None):
    """gnnhwc_fwd_add on (N, R, C) device tensors.  Returns y, sum (or None), mean, rstd."""
    N, R, C = x_nrc.shape
    dt = DT_CODE[x_nrc.dtype]
    sdtype = torch.float32 if x_nrc.dtype in (torch.float16, torch.bfloat16) else x_nrc.dtype
    pdt = DT_CODE[w.dtype] if w is not None else dt
    cbdt = DT_CODE[channel_bias.dtype] if channel_bias is not None else dt
    y = torch.empty_like(x_nrc) if y is None else y
    if sum_out is None and want_sum:
        sum_out = torch.empty_like(x_nrc)
    mean = torch.empty((N, G), dtype=sdtype, device=x_nrc.device)
    rstd = torch.empty((N, G), dtype=sdtype, device=x_nrc.device)
    lib = _cabi.lib
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, dt)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x_nrc.device)
    rc = lib.gnnhwc_fwd_add(_ptr(x_nrc), _ptr(residual), _ptr(channel_bias), _ptr(sum_out), _ptr(w), _ptr(b), _ptr(y),
                            _ptr(mean), _ptr(rstd), N, R, C, G, float(eps), int(act), dt, pdt, DT_CODE[sdtype], cbdt,
                            _ptr(ws), ws.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_fwd_add")
    return y, sum_out, mean, rstd


def cabi_bwd(dy_nrc, x_nrc, w, b, mean, rstd, G, act, dx=None, ws=None, want_dw=True, want_db=True):
    N, R, C = x_nrc.shape
    dt = DT_CODE[x_nrc.dtype]
    pdtype = w.dtype if w is not None else x_nrc.dtype
    dx = torch.empty_like(x_nrc) if dx is None else dx
    dw = torch.empty((C,), dtype=pdtype, device=x_nrc.device) if want_dw else None
    db = torch.empty((C,), dtype=pdtype, device=x_nrc.device) if want_db else None
    lib = _cabi.lib
    nbytes = lib.gnnhwc_bwd_workspace_bytes(N, R, C, G, dt)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x_nrc.device) if ws is None else ws
    rc = lib.gnnhwc_bwd(_ptr(dy_nrc), _ptr(x_nrc), _ptr(w), _ptr(b), _ptr(mean), _ptr(rstd), _ptr(dx), _ptr(dw), _ptr(db),
                        N, R, C, G, int(act), dt, DT_CODE[pdtype], DT_CODE[mean.dtype], _ptr(ws), ws.numel(),
                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_bwd")
    return dx, dw, db


def err(a, truth):
    """max_i |a_i - t_i| / (|t_i| + rms(t)): relative for elements of typical size, and relative to the
    tensor's scale for elements near zero (where a pure ratio is meaningless)."""
    a = torch.as_tensor(a).detach().to("cpu", torch.float64).reshape(-1)
    t = torch.as_tensor(truth).detach().to("cpu", torch.float64).reshape(-1)
    assert a.shape == t.shape, (a.shape, t.shape)
    if t.numel() == 0:
        return 0.0
    rms = float(t.square().mean().sqrt())
    if rms == 0.0:
        rms = 1.0
    return float(((a - t).abs() / (t.abs() + rms)).max())


def rel_err(a, truth):
    """max_i |a_i - t_i| / |t_i| over the elements of typical size, |t_i| >= rms(t): the pure relative error, where
    it is meaningful (near zero a ratio says nothing about accuracy; err() above covers those elements)."""
    a = torch.as_tensor(a).detach().to("cpu", torch.float64).reshape(-1)
    t = torch.as_tensor(truth).detach().to("cpu", torch.float64).reshape(-1)
    assert a.shape == t.shape, (a.shape, t.shape)
    if t.numel() == 0:
        return 0.0
    rms = float(t.square().mean().sqrt())
    big = t.abs() >= rms
    if rms == 0.0 or not bool(big.any()):
        return 0.0
    return float(((a - t).abs()[big] / t.abs()[big]).max())


# Observed errors, one JSON object per line, for the per-configuration result table (profiles/results_all_configs.txt is
# built from it).  Written only when GNNHWC_PARITY_LOG names a file.
def record_errors(**fields):
    import json
    import os

    path = os.environ.get("GNNHWC_PARITY_LOG")
    if path:
        with open(path, "a") as f:
            f.write(json.dumps(fields) + "\n")


def as_np64(t):
    return t.detach().to("cpu", torch.float64).numpy()


def cabi_fwd_nchw(x_ncr, w, b, G, eps, act, y=None):
    """gnnhwc_fwd_nchw on (N, C, R) contiguous device tensors.  Returns y, mean, rstd."""
    N, C, R = x_ncr.shape
    dt = DT_CODE[x_ncr.dtype]
    sdtype = torch.float32 if x_ncr.dtype in (torch.float16, torch.bfloat16) else x_ncr.dtype
    pdt = DT_CODE[w.dtype] if w is not None else dt
    y = torch.empty_like(x_ncr) if y is None else y
    mean = torch.empty((N, G), dtype=sdtype, device=x_ncr.device)
    rstd = torch.empty((N, G), dtype=sdtype, device=x_ncr.device)
    lib = _cabi.lib
    nbytes = lib.gnnhwc_nchw_workspace_bytes(N, C, R, G, dt, 0)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x_ncr.device)
    rc = lib.gnnhwc_fwd_nchw(_ptr(x_ncr), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), N, C, R, G, float(eps), int(act),
                             dt, pdt, DT_CODE[sdtype], _ptr(ws), ws.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_fwd_nchw")
    return y, mean, rstd


def cabi_bwd_nchw(dy_ncr, x_ncr, w, b, mean, rstd, G, act, want_dw=True, want_db=True):
    N, C, R = x_ncr.shape
    dt = DT_CODE[x_ncr.dtype]
    pdtype = w.dtype if w is not None else x_ncr.dtype
    dx = torch.empty_like(x_ncr)
    dw = torch.empty((C,), dtype=pdtype, device=x_ncr.device) if want_dw else None
    db = torch.empty((C,), dtype=pdtype, device=x_ncr.device) if want_db else None
    lib = _cabi.lib
    nbytes = lib.gnnhwc_nchw_workspace_bytes(N, C, R, G, dt, 1)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x_ncr.device)
    rc = lib.gnnhwc_bwd_nchw(_ptr(dy_ncr), _ptr(x_ncr), _ptr(w), _ptr(b), _ptr(mean), _ptr(rstd), _ptr(dx), _ptr(dw), _ptr(db),
                             N, C, R, G, int(act), dt, DT_CODE[pdtype], DT_CODE[mean.dtype], _ptr(ws), ws.numel(),
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_bwd_nchw")
    return dx, dw, db

