"""GPU parity of gnnhwc_fwd_cast and gnnhwc_bwd_cast: float32 data, y written / dy read as float16 / bfloat16 by the kernels.

gnnhwc_bwd_cast: dx, dweight, dbias are bit for bit those of gnnhwc_bwd on the same gradient widened to float32 first (the
kernels widen exactly, in registers), for both kernel families and the scalar kernels; errors as gnnhwc_fwd_cast's.

Bars: y is bit for bit gnnhwc_fwd's float32 y rounded once (round to nearest even) to the 16-bit type -- the kernel
rounds the very fp32 value the plain forward stores -- and therefore within one rounding of the float64 oracle's y
(err <= 2^-8 for bfloat16, 2^-11 for float16 -- half a spacing of the type -- plus the fp32 bar of 1e-5); mean / rstd
are the plain forward's (err <= 1e-5 against the oracle).  Through the Python surface the gradients are those of torch's float32 GroupNorm + activation
followed by a cast (err <= 1e-5: the backward runs in float32 on the widened gradient)."""
import ctypes

import pytest
import torch

from oracle import gn_oracle as orc
from gnnhwc import _cabi
from tests.gpu_harness import DT_CODE, _ptr, as_np64, cabi_bwd, cabi_fwd, err

pytestmark = pytest.mark.gpu

EPS = 1e-5
ROUNDING = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}  # half a spacing, relative, at worst
SHAPES = [
    ((1, 4096, 320), 32),   # the float32 SD-UNet forward: single launch
    ((3, 37 * 53, 96), 24),  # odd rows
    ((2, 2048, 256), 16),
    ((2, 5, 6), 3),         # C not a multiple of 4: scalar kernels
    ((4, 289, 1920), 32),
    ((1, 70000, 8), 2),     # long and narrow
]
ACTS = ["identity", "relu", "silu", "gelu", "gelu_tanh"]


def cabi_fwd_cast(x, w, b, G, act, y_dtype, y=None, dtype_code=None):
    N, R, C = x.shape
    dt = DT_CODE[x.dtype] if dtype_code is None else dtype_code
    y = torch.empty((N, R, C), dtype=y_dtype, device=x.device) if y is None else y
    mean = torch.empty((N, G), dtype=torch.float32, device=x.device)
    rstd = torch.empty((N, G), dtype=torch.float32, device=x.device)
    lib = _cabi.lib
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, dt)
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x.device)
    rc = lib.gnnhwc_fwd_cast(_ptr(x), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), N, R, C, G, EPS, int(act), dt,
                             DT_CODE[w.dtype] if w is not None else dt, 0, DT_CODE[y_dtype], _ptr(ws), ws.numel(),
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return rc, y, mean, rstd


def _inputs(shape, device, seed):
    gen = torch.Generator().manual_seed(seed)
    N, R, C = shape
    x = (torch.randn(shape, generator=gen) * 1.7 + torch.randn((C,), generator=gen)).to(device)
    w = (torch.rand((C,), generator=gen) + 0.5).to(device)
    b = (0.1 * torch.randn((C,), generator=gen)).to(device)
    return x, w, b


@pytest.mark.parametrize("y_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,G", SHAPES)
def test_cast_forward_parity(family, shape, G, y_dtype, device):
    act_name = ACTS[(shape[1] + shape[2]) % 5]
    act = orc.ACT_CODES[act_name]
    print("cast", family, shape, G, y_dtype, act_name, flush=True)
    x, w, b = _inputs(shape, device, 500 + shape[2])
    rc, y, mean, rstd = cabi_fwd_cast(x, w, b, G, act, y_dtype)
    assert rc == 0, _cabi.last_error()
    y32, mean32, rstd32 = cabi_fwd(x, w, b, G, EPS, act)
    torch.cuda.synchronize()
    assert y.dtype == y_dtype and torch.equal(y, y32.to(y_dtype))
    assert torch.equal(mean, mean32) and torch.equal(rstd, rstd32)
    ty, tmean, trstd = orc.fwd(as_np64(x), as_np64(w), as_np64(b), G, EPS, act)
    assert err(mean, tmean) <= 1e-5 and err(rstd, trstd) <= 1e-5
    assert err(y, ty) <= ROUNDING[y_dtype] + 1e-5


def test_cast_options_and_errors(device):
    x, w, b = _inputs((2, 300, 64), device, 9)
    # float32 out: the plain forward
    rc, y, mean, rstd = cabi_fwd_cast(x, w, b, 8, 2, torch.float32)
    y32, _, _ = cabi_fwd(x, w, b, 8, EPS, 2)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(y, y32)
    # no parameters; NULL statistics are covered by the plain forward's tests (same code)
    rc, y, _, _ = cabi_fwd_cast(x, None, None, 8, 2, torch.bfloat16)
    y32, _, _ = cabi_fwd(x, None, None, 8, EPS, 2)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(y, y32.bfloat16())
    # 16-bit data keeps its type; unknown codes; in place with another type
    xb = x.bfloat16()
    rc, _, _, _ = cabi_fwd_cast(xb, None, None, 8, 2, torch.float32, y=torch.empty_like(x))
    assert rc == -1 and "y_dtype" in _cabi.last_error()
    rc, _, _, _ = cabi_fwd_cast(xb, None, None, 8, 2, torch.float16, y=torch.empty_like(xb))
    assert rc == -1
    rc, y, _, _ = cabi_fwd_cast(xb, None, None, 8, 2, torch.bfloat16)
    assert rc == 0
    rc, _, _, _ = cabi_fwd_cast(x, None, None, 8, 2, torch.float64, y=torch.empty_like(x, dtype=torch.float64))
    assert rc == -1
    rc, _, _, _ = cabi_fwd_cast(x, None, None, 8, 2, torch.bfloat16, y=x)
    assert rc == -1 and "in place" in _cabi.last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("affine", [True, False])
def test_cast_through_the_python_surface(affine, device):
    """group_norm_nhwc(out_dtype=) and GN_NHWC(out_dtype=): result and gradients against torch's float32 expression
    followed by a cast; the functional form compiles whole."""
    from gnnhwc import GN_NHWC, group_norm_nhwc

    gen = torch.Generator().manual_seed(21)
    x = torch.randn((2, 64, 12, 20), generator=gen).to(device).to(memory_format=torch.channels_last).requires_grad_()
    m = GN_NHWC(8, 64, activation="silu", out_dtype=torch.bfloat16, affine=affine).to(device)
    if affine:
        with torch.no_grad():
            m.weight.copy_(torch.rand((64,), generator=gen) + 0.5)
            m.bias.copy_(torch.randn((64,), generator=gen) * 0.1)
    dy = torch.randn((2, 64, 12, 20), generator=gen).to(device).bfloat16()
    y = m(x)
    assert y.dtype == torch.bfloat16 and y.shape == x.shape and y.stride() == x.stride()
    y.backward(dy)
    xr = x.detach().clone().requires_grad_()
    wr = m.weight.detach().clone().requires_grad_() if affine else None
    br = m.bias.detach().clone().requires_grad_() if affine else None
    yr = torch.nn.functional.silu(torch.nn.functional.group_norm(xr, 8, wr, br, EPS)).bfloat16()
    yr.backward(dy)
    # torch's float32 forward differs from these kernels' in the last bits, so a value may round the other way
    assert err(y, yr) <= 2.0 ** -7
    assert err(x.grad, xr.grad) <= 1e-5
    if affine:
        assert err(m.weight.grad, wr.grad) <= 1e-5 and err(m.bias.grad, br.grad) <= 1e-5
    # functional form, compiled whole
    w = m.weight.detach() if affine else None
    b = m.bias.detach() if affine else None

    def f(t):
        return group_norm_nhwc(t, w, b, 8, EPS, "silu", out_dtype=torch.bfloat16) * 2

    want = f(x.detach())
    got = torch.compile(f, backend="aot_eager", fullgraph=True)(x.detach())
    assert got.dtype == torch.bfloat16 and torch.equal(got, want)
    # other inputs are converted afterwards: 16-bit data to float32 out, channels-first input
    m2 = GN_NHWC(8, 64, activation="silu", out_dtype=torch.float32, affine=affine).to(device)
    assert m2(x.detach().bfloat16()).dtype == torch.float32
    assert m(x.detach().contiguous()).dtype == torch.bfloat16


def cabi_bwd_cast(dy, x, w, b, mean, rstd, G, act, dx=None, dtype_code=None, dy_code=None):
    N, R, C = x.shape
    dt = DT_CODE[x.dtype] if dtype_code is None else dtype_code
    dx = torch.empty_like(x) if dx is None else dx
    dw = torch.empty((C,), dtype=w.dtype, device=x.device) if w is not None else None
    db = torch.empty((C,), dtype=w.dtype, device=x.device) if w is not None else None
    lib = _cabi.lib
    nbytes = lib.gnnhwc_bwd_workspace_bytes(N, R, C, G, DT_CODE[x.dtype])
    assert nbytes > 0, _cabi.last_error()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=x.device)
    rc = lib.gnnhwc_bwd_cast(_ptr(dy), _ptr(x), _ptr(w), _ptr(b), _ptr(mean), _ptr(rstd), _ptr(dx), _ptr(dw), _ptr(db), N, R, C, G,
                             int(act), dt, DT_CODE[w.dtype] if w is not None else dt, DT_CODE[mean.dtype],
                             DT_CODE[dy.dtype] if dy_code is None else dy_code, _ptr(ws), ws.numel(),
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return rc, dx, dw, db


@pytest.mark.parametrize("dy_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,G", SHAPES + [((5, 128 * 128, 320), 32)])  # the last: a backward in two launches
def test_cast_backward_matches_widen_then_backward(family, shape, G, dy_dtype, device):
    act_name = ACTS[(shape[1] + shape[2] + 1) % 5]
    act = orc.ACT_CODES[act_name]
    print("bwd_cast", family, shape, G, act_name, dy_dtype, flush=True)
    x, w, b = _inputs(shape, device, 23)
    gen = torch.Generator().manual_seed(29)
    dy16 = torch.randn(shape, generator=gen).to(dy_dtype).to(device)
    _y, mean, rstd = cabi_fwd(x, w, b, G, EPS, act)
    want = cabi_bwd(dy16.float(), x, w, b, mean, rstd, G, act)  # today's sequence: widen, then the float backward
    rc, dx, dw, db = cabi_bwd_cast(dy16, x, w, b, mean, rstd, G, act)
    _cabi.check(rc, "gnnhwc_bwd_cast")
    torch.cuda.synchronize()
    for name, got, ref in (("dx", dx, want[0]), ("dweight", dw, want[1]), ("dbias", db, want[2])):
        assert torch.equal(got, ref), "%s differs from the backward on the widened gradient" % name
    # without parameters, and float32 dy through the same entry point (= gnnhwc_bwd)
    rc, dx0, _, _ = cabi_bwd_cast(dy16, x, None, None, mean, rstd, G, act)
    _cabi.check(rc, "gnnhwc_bwd_cast")
    want0 = cabi_bwd(dy16.float(), x, None, None, mean, rstd, G, act, want_dw=False, want_db=False)
    rc, dx1, dw1, db1 = cabi_bwd_cast(dy16.float(), x, w, b, mean, rstd, G, act)
    _cabi.check(rc, "gnnhwc_bwd_cast")
    torch.cuda.synchronize()
    assert torch.equal(dx0, want0[0])
    assert torch.equal(dx1, want[0]) and torch.equal(dw1, want[1]) and torch.equal(db1, want[2])


def test_cast_backward_argument_errors(device):
    x, w, b = _inputs((2, 64, 32), device, 3)
    _y, mean, rstd = cabi_fwd(x, w, b, 4, EPS, 2)
    dy = torch.randn_like(x).to(torch.bfloat16)
    assert cabi_bwd_cast(dy, x, w, b, mean, rstd, 4, 2, dy_code=1)[0] == -1        # float64 gradient of float32 data
    assert cabi_bwd_cast(dy, x, w, b, mean, rstd, 4, 2, dy_code=7)[0] == -1        # unknown code
    xb = x.to(torch.bfloat16)
    wb, bb = w.to(torch.bfloat16), b.to(torch.bfloat16)
    assert cabi_bwd_cast(dy.to(torch.float16), xb, wb, bb, mean, rstd, 4, 2)[0] == -1  # 16-bit data take dy in their own type
    assert cabi_bwd_cast(dy, xb, wb, bb, mean, rstd, 4, 2)[0] == 0
    torch.cuda.synchronize()
