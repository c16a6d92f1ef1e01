"""CPU-only checks of the boundary: the shared library loads, exports every symbol include/gnnhwc.h
declares, sizes workspaces, rejects bad arguments without launching anything, and the Python surface
mirrors the reference's (src/gnnhwc/custom_gn.py:29-90)."""
import ctypes
import os
import re

import pytest
import torch

import gnnhwc
from gnnhwc import GN_NHWC, GN_NHWC_Func, _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "gnnhwc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gnnhwc_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert {"gnnhwc_fwd", "gnnhwc_fwd_add", "gnnhwc_bwd", "gnnhwc_fwd_workspace_bytes", "gnnhwc_bwd_workspace_bytes", "gnnhwc_last_error",
            "gnnhwc_version", "gnnhwc_profile_enable", "gnnhwc_profile_collect", "gnnhwc_kernel_kind_name",
            "gnnhwc_debug_read_trace", "gnnhwc_set_resident", "gnnhwc_debug_copy", "gnnhwc_debug_set_spin_limit",
            "gnnhwc_debug_plan", "gnnhwc_fwd_nchw", "gnnhwc_bwd_nchw", "gnnhwc_nchw_workspace_bytes"} <= set(names)
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    # the twin built with the in-kernel phase stamps (loaded instead when GNNHWC_TRACE is set) exports the same interface
    twin = ctypes.CDLL(os.path.join(os.path.dirname(_cabi.LIB_PATH), "libgnnhwc_hip_trace.so"))
    for n in names:
        assert hasattr(twin, n), n
    if not _cabi.TRACING:  # the library proper has no stamps to read
        assert _cabi.lib.gnnhwc_debug_read_trace(None, 8) == -1 and "trace" in _cabi.last_error()


def test_version_and_kind_names():
    assert _cabi.lib.gnnhwc_version() >> 16 == 1
    names = _cabi.kernel_kind_names()
    assert len(names) == _cabi.NUM_KERNEL_KINDS and all(names)


@pytest.mark.parametrize("dtype", [0, 1, 2, 3])
def test_workspace_sizes(dtype):
    lib = _cabi.lib
    for (N, R, C, G) in [(1, 16384, 640, 32), (4, 16384, 320, 32), (1, 262144, 128, 32), (3, 1961, 96, 24), (8, 289, 1920, 32),
                         (1, 1, 1, 1), (2, 5, 7, 7)]:
        f = lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, dtype)
        b = lib.gnnhwc_bwd_workspace_bytes(N, R, C, G, dtype)
        assert f > 0 and f % 256 == 0, (N, R, C, G, f)
        assert b > 0 and b % 256 == 0, (N, R, C, G, b)
        # scratch stays a small fraction of the tensors it serves
        S = N * R * C * (8 if dtype == 1 else 4 if dtype == 0 else 2)
        assert f < 16 * 2 ** 20 and b < 48 * 2 ** 20, (N, R, C, G, f, b, S)
    assert lib.gnnhwc_fwd_workspace_bytes(0, 16, 8, 2, dtype) == 256  # empty batch
    assert lib.gnnhwc_fwd_workspace_bytes(1, 16, 7, 3, dtype) == 0
    assert "divisible" in _cabi.last_error()
    assert lib.gnnhwc_fwd_workspace_bytes(1, 16, 8, 2, 9) == 0
    assert "dtype" in _cabi.last_error()


def test_invalid_arguments_are_rejected_before_any_launch():
    lib = _cabi.lib
    null = None
    # C % G != 0
    rc = lib.gnnhwc_fwd(null, null, null, null, null, null, 1, 16, 7, 3, 1e-5, 0, 0, 0, 0, null, 0, null)
    assert rc == -1 and "divisible" in _cabi.last_error()
    # unknown activation
    rc = lib.gnnhwc_fwd(null, null, null, null, null, null, 1, 16, 8, 2, 1e-5, 7, 0, 0, 0, null, 0, null)
    assert rc == -1 and "activation" in _cabi.last_error()
    # parameter dtype that may not differ from the data dtype
    rc = lib.gnnhwc_fwd(null, null, null, null, null, null, 1, 16, 8, 2, 1e-5, 0, 0, 3, 0, null, 0, null)
    assert rc == -1 and "weight/bias dtype" in _cabi.last_error()
    rc = lib.gnnhwc_bwd(null, null, null, null, null, null, null, null, null, 1, 16, 8, 2, 0, 2, 2, 1, null, 0, null)
    assert rc == -1 and "mean/rstd dtype" in _cabi.last_error()
    # null tensors
    rc = lib.gnnhwc_fwd(null, null, null, null, null, null, 1, 16, 8, 2, 1e-5, 0, 0, 0, 0, null, 0, null)
    assert rc == -1 and "null" in _cabi.last_error()
    # workspace too small (non-null dummy pointers; nothing is dereferenced or launched)
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = lib.gnnhwc_fwd(p, null, null, p, p, p, 1, 16, 8, 2, 1e-5, 0, 0, 0, 0, p, 16, null)
    assert rc == -2 and "workspace" in _cabi.last_error()
    rc = lib.gnnhwc_bwd(p, p, null, null, p, p, p, null, null, 1, 16, 8, 2, 0, 0, 0, 0, null, 0, null)
    assert rc == -2
    with pytest.raises(RuntimeError):
        _cabi.check(rc, "gnnhwc_bwd")


def test_python_surface_matches_the_reference():
    assert gnnhwc.GN_NHWC is GN_NHWC and gnnhwc.GN_NHWC_Func is GN_NHWC_Func
    m = GN_NHWC(4, 8, activation="silu", eps=1e-6)
    assert isinstance(m, torch.nn.GroupNorm)
    assert (m.activation, m.act_code, m.eps) == ("silu", 2, 1e-6)
    assert {k: GN_NHWC(1, 2, activation=k).act_code for k in ("identity", "relu", "swish", "silu", "gelu", "gelu_tanh")} == {
        "identity": 0, "relu": 1, "swish": 2, "silu": 2, "gelu": 3, "gelu_tanh": 4}
    assert repr(m) == "GN_NHWC(4, 8, eps=1e-06, affine=True, activation=silu)"
    assert sorted(m.state_dict()) == ["bias", "weight"]  # loads nn.GroupNorm checkpoints unchanged
    with pytest.raises(KeyError):
        GN_NHWC(4, 8, activation="tanh")
    with pytest.raises(ValueError):
        GN_NHWC(3, 8)
    assert GN_NHWC(2, 4, affine=False).weight is None


def test_ops_are_registered_and_reject_host_tensors():
    x = torch.zeros(1, 8, 4).permute(0, 2, 1).contiguous().permute(0, 2, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        torch.ops.gnop.fwd(x, torch.ones(8), torch.zeros(8), 4, 1e-5, 0)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        torch.ops.gnop.bwd(x, x, torch.ones(8), torch.zeros(8), torch.zeros(1, 4), torch.ones(1, 4), 4, 0)
    # a channels-last CPU tensor reaches the device check through the module as well
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        GN_NHWC(4, 8)(torch.zeros(1, 8, 2, 2).to(memory_format=torch.channels_last))


@pytest.mark.parametrize("act", ["identity", "relu", "silu", "gelu", "gelu_tanh"])
def test_channels_first_host_input_takes_the_torch_expression(act):
    """custom_gn.py:75-79: in the reference channels-first input never reaches a kernel, so that path also serves
    host tensors; here device tensors get the channels-first kernels and host tensors keep the torch expression."""
    from oracle import gn_oracle as orc

    torch.manual_seed(1)
    m = GN_NHWC(4, 8, activation=act)
    x = torch.randn(2, 8, 3, 5, requires_grad=True)
    y = m(x)
    want = orc.torch_act(act)(torch.nn.functional.group_norm(x, 4, m.weight, m.bias, m.eps))
    assert torch.allclose(y, want, rtol=1e-6, atol=1e-7)
    y.sum().backward()
    assert x.grad is not None and m.weight.grad is not None
    m2 = GN_NHWC(4, 8, activation=act, affine=False)
    assert torch.allclose(m2(x), orc.torch_act(act)(torch.nn.functional.group_norm(x, 4, None, None, m2.eps)), rtol=1e-5, atol=1e-6)


def test_operator_metadata_on_meta_tensors():
    """gnop::fwd / gnop::bwd report the shapes, dtypes and channels-last strides of their outputs for meta tensors
    (what fake-tensor tracing sees); no kernel runs."""
    import torch
    import gnnhwc  # noqa: F401  (registers the operators)

    N, C, R, G = 3, 8, 20, 2
    for dtype, sdtype in ((torch.float32, torch.float32), (torch.bfloat16, torch.float32), (torch.float64, torch.float64)):
        X = torch.empty((N, R, C), dtype=dtype, device="meta").permute(0, 2, 1)
        w = torch.empty((C,), dtype=dtype, device="meta")
        Y, mean, rstd = torch.ops.gnop.fwd(X, w, w, G, 1e-5, 2)
        assert Y.shape == (N, C, R) and Y.stride() == (R * C, 1, C) and Y.dtype == dtype
        assert mean.shape == (N, G) and rstd.shape == (N, G) and mean.dtype == sdtype
        dX, dw, db = torch.ops.gnop.bwd(X, X, w, w, mean, rstd, G, 2)
        assert dX.shape == (N, C, R) and dX.stride() == (R * C, 1, C) and dw.shape == (C,) and db.dtype == dtype


def test_operator_autograd_on_meta_tensors():
    """gnop::fwd carries its own autograd formula: differentiating through the traceable functional form on meta
    tensors yields gradients of the right shapes, dtypes and strides without running a kernel."""
    from gnnhwc import group_norm_nhwc

    N, C, H, W, G = 2, 8, 5, 3, 4
    x = torch.empty((N, H, W, C), dtype=torch.bfloat16, device="meta").permute(0, 3, 1, 2).requires_grad_()
    w = torch.empty((C,), dtype=torch.bfloat16, device="meta", requires_grad=True)
    b = torch.empty((C,), dtype=torch.bfloat16, device="meta", requires_grad=True)
    y = group_norm_nhwc(x, w, b, G, 1e-5, "silu")
    assert y.shape == x.shape and y.stride() == x.stride() and y.dtype == x.dtype
    gx, gw, gb = torch.autograd.grad(y, (x, w, b), torch.empty_like(y))
    assert gx.shape == x.shape and gx.stride() == x.stride()
    assert gw.shape == (C,) and gb.shape == (C,) and gw.dtype == torch.bfloat16
    with pytest.raises(RuntimeError):
        group_norm_nhwc(torch.empty((N, C, H, W), device="meta"), w, b, G)
    with pytest.raises(KeyError):
        group_norm_nhwc(x, w, b, G, 1e-5, "tanh")


def test_fused_addition_operator_on_meta_tensors():
    """gnop::fwd_add (additions fused into the forward): output metadata and the shapes of all five gradients,
    on meta tensors (no kernel runs)."""
    from gnnhwc import group_norm_nhwc

    N, C, H, W, G = 2, 8, 5, 3, 4
    mk = lambda *shape: torch.empty(shape, dtype=torch.bfloat16, device="meta")  # noqa: E731
    x = mk(N, H, W, C).permute(0, 3, 1, 2).requires_grad_()
    r = mk(N, H, W, C).permute(0, 3, 1, 2).requires_grad_()
    t = mk(N, C).requires_grad_()
    w = mk(C).requires_grad_()
    b = mk(C).requires_grad_()
    y, s = group_norm_nhwc(x, w, b, G, 1e-5, "silu", residual=r, channel_bias=t, return_sum=True)
    assert y.shape == x.shape and y.stride() == x.stride() and s.shape == x.shape and s.stride() == x.stride()
    grads = torch.autograd.grad((y, s), (x, r, t, w, b), (torch.empty_like(y), torch.empty_like(s)))
    assert [tuple(g.shape) for g in grads] == [tuple(x.shape), tuple(x.shape), (N, C), (C,), (C,)]
    y2 = group_norm_nhwc(x, w, b, G, 1e-5, "silu", channel_bias=t)
    gx, gt = torch.autograd.grad(y2, (x, t), torch.empty_like(y2))
    assert gx.shape == x.shape and gt.shape == (N, C) and gt.dtype == torch.bfloat16
    with pytest.raises(RuntimeError):
        group_norm_nhwc(x, w, b, G, 1e-5, "silu", residual=mk(N, C, H, W + 1))


def _plan(N, R, C, G, dtype, vector, backward):
    out = (ctypes.c_int64 * 12)()
    rc = _cabi.lib.gnnhwc_debug_plan(N, R, C, G, dtype, vector, backward, out)
    assert rc == 0, _cabi.last_error()
    keys = ("vec", "cv", "lpr", "nchunk", "rpi", "tile_rows", "tiles", "gmax", "nblocks", "compaction", "bytes", "D")
    return dict(zip(keys, (int(v) for v in out)))


def test_tiling_invariants_over_many_shapes():
    """Host-side planning (the replacement of calc_block_params / closest_factor, gn_kernel.cu:37-60,121-128) on the
    benchmark shapes and a seeded sample of awkward ones: the tiles cover the tensor exactly once, a workgroup's
    lanes fit its chunk, the grid stays within the launch limits, and the workspace the public size query reports
    holds what the tiling needs."""
    import random

    rng = random.Random(5)
    shapes = [(1, 4096, 320, 32), (2, 1024, 640, 32), (1, 16384, 640, 32), (1, 4096, 1280, 32), (4, 16384, 320, 32),
              (1, 262144, 128, 32), (1, 65536, 256, 32), (3, 1961, 96, 24), (8, 289, 1920, 32), (2, 2048, 256, 16),
              (1, 1, 1, 1), (2, 5, 7, 7), (70000, 3, 8, 2), (1, 3, 4096, 1), (1, 10 ** 7, 8, 8)]
    for _ in range(300):
        G = rng.choice([1, 2, 3, 4, 7, 8, 16, 24, 32, 64])
        D = rng.choice([1, 2, 3, 4, 5, 8, 10, 12, 20, 33, 40, 60, 128])
        shapes.append((rng.randint(1, 9), rng.choice([1, 2, 7, 64, 289, 1000, 1961, 4096, 16384, 100003]), G * D, G))
    elem = {0: 4, 1: 8, 2: 2, 3: 2}
    for (N, R, C, G) in shapes:
        for dtype in (0, 1, 2, 3):
            for vector in (0, 1):
                if vector and C % (16 // elem[dtype]) != 0:
                    continue
                for backward in (0, 1):
                    p = _plan(N, R, C, G, dtype, vector, backward)
                    ctx = (N, R, C, G, dtype, vector, backward, p)
                    assert p["vec"] == (16 // elem[dtype] if vector else 1) and p["cv"] * p["vec"] == C, ctx
                    assert p["D"] * G == C, ctx
                    assert 1 <= p["lpr"] <= 256 and p["rpi"] == 256 // p["lpr"] and p["rpi"] >= 1, ctx
                    assert (p["nchunk"] - 1) * p["lpr"] < p["cv"] <= p["nchunk"] * p["lpr"], ctx  # chunks cover the row once
                    assert p["tile_rows"] >= 1 and p["tile_rows"] % p["rpi"] == 0 or p["tile_rows"] >= R, ctx
                    assert (p["tiles"] - 1) * p["tile_rows"] < R <= p["tiles"] * p["tile_rows"], ctx  # tiles cover the rows once
                    assert p["nblocks"] == N * p["tiles"] * p["nchunk"], ctx
                    assert p["tiles"] < 2 ** 31 and p["nchunk"] <= 65535, ctx  # grid x / y limits
                    assert 1 <= p["gmax"] <= G, ctx
                    query = (_cabi.lib.gnnhwc_bwd_workspace_bytes if backward else _cabi.lib.gnnhwc_fwd_workspace_bytes)(N, R, C, G, dtype)
                    assert p["bytes"] <= query, ctx
    # a large tensor is cut into about a resident wave's worth of workgroups, not more
    big = _plan(1, 262144, 128, 32, 2, 1, 1)
    assert 256 <= big["nblocks"] <= 2048, big
    out = (ctypes.c_int64 * 12)()
    assert _cabi.lib.gnnhwc_debug_plan(1, 16, 12, 4, 3, 1, 0, out) == -1 and "vector width" in _cabi.last_error()



def test_channels_first_operators_on_meta_tensors():
    """gnop::fwd_nchw / gnop::bwd_nchw: contiguous outputs of x's shape, statistics in float32 for 16-bit data."""
    N, C, R, G = 2, 12, 30, 3
    X = torch.empty((N, C, R), dtype=torch.float16, device="meta")
    w = torch.empty((C,), dtype=torch.float32, device="meta")
    Y, mean, rstd = torch.ops.gnop.fwd_nchw(X, w, w, G, 1e-5, 4)
    assert Y.shape == X.shape and Y.is_contiguous() and Y.dtype == torch.float16
    assert mean.shape == (N, G) and mean.dtype == torch.float32 and rstd.shape == (N, G)
    dX, dw, db = torch.ops.gnop.bwd_nchw(X, X, w, w, mean, rstd, G, 4)
    assert dX.shape == X.shape and dw.shape == (C,) and dw.dtype == torch.float32 and db.dtype == torch.float32


def test_channels_first_argument_checks_need_no_gpu():
    lib = _cabi.lib
    assert lib.gnnhwc_nchw_workspace_bytes(2, 8, 100, 2, 3, 0) % 256 == 0
    assert lib.gnnhwc_nchw_workspace_bytes(2, 8, 100, 3, 3, 0) == 0 and "divisible" in _cabi.last_error()
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails validation first
    rc = lib.gnnhwc_fwd_nchw(one, None, None, one, None, None, 1, 8, 16, 2, 1e-5, 9, 0, 0, 0, one, 1 << 20, None)
    assert rc == -1 and "activation" in _cabi.last_error()
    rc = lib.gnnhwc_fwd_nchw(one, None, None, one, None, None, 1, 8, 16, 2, 1e-5, 0, 3, 2, 0, one, 1 << 20, None)
    assert rc == -1 and "dtype" in _cabi.last_error()
    rc = lib.gnnhwc_bwd_nchw(None, one, None, None, one, one, one, None, None, 1, 8, 16, 2, 0, 0, 0, 0, one, 1 << 20, None)
    assert rc == -1 and "must not be null" in _cabi.last_error()
    rc = lib.gnnhwc_fwd_nchw(one, None, None, one, None, None, 1, 2, 2 ** 31, 1, 1e-5, 0, 0, 0, 0, one, 1 << 40, None)
    assert rc == -1 and "beyond the supported range" in _cabi.last_error()

