"""GPU parity of the channels-first entry points (gnnhwc_fwd_nchw / gnnhwc_bwd_nchw), through the C ABI, against the
CPU oracle (oracle/gn_oracle.c, float64; it works on the (N, R, C) view, so inputs and results are transposed for
it) and, for 16-bit types, against torch's own GroupNorm + activation in that type -- the bars of the channels-last
kernels (tests/test_gpu_parity.py)."""
import numpy as np
import pytest
import torch

from oracle import gn_oracle as orc
from tests.gpu_harness import as_np64, cabi_bwd_nchw, cabi_fwd_nchw, err
from tests.test_gpu_parity import EPS, RELU_BAND, _check

pytestmark = pytest.mark.gpu

ACTS = ["identity", "relu", "silu", "gelu", "gelu_tanh"]
SHAPES = [
    ((2, 64, 256), 8),      # one chunk per row
    ((1, 320, 4096), 32),   # SD-UNet-like, several chunks per row in fp32
    ((3, 96, 37 * 53), 24),  # odd row length: scalar kernels
    ((2, 6, 5), 3),         # tiny
    ((2, 35, 60), 7),       # R a multiple of 4 but not of 8: vector kernels for fp32 only
    ((1, 8, 100000), 2),    # long rows, many chunks per slab
    ((4, 1920, 289), 32),   # many short rows
    ((2, 16, 300), 16),     # one channel per group
    ((2, 24, 520), 1),      # one group
    ((2, 512, 4096), 1),    # one group of many long rows: more partials per slab than a consumer merges itself
    ((1, 16, 70000), 2),    # the same from few, very long rows (fp32: 8 x 69 partials per slab)
]


def _inputs(shape, dtype, device, seed):
    gen = torch.Generator().manual_seed(seed)
    N, C, R = shape
    x = (torch.randn((N, C, R), generator=gen) * 1.6 + torch.randn((C, 1), generator=gen)).to(dtype).to(device)
    dy = torch.randn((N, C, R), generator=gen).to(dtype).to(device)
    w = (torch.rand((C,), generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn((C,), generator=gen)).to(dtype).to(device)
    return x, dy, w, b


def _nrc(t):
    return as_np64(t.permute(0, 2, 1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("shape,G", SHAPES)
def test_channels_first_parity(shape, G, dtype, device):
    act_name = ACTS[(shape[1] + shape[2]) % 5]
    act = orc.ACT_CODES[act_name]
    print("nchw", shape, G, dtype, act_name, flush=True)
    x, dy, w, b = _inputs(shape, dtype, device, 300 + shape[1])
    truth = orc.fwd_bwd(_nrc(x), as_np64(w), as_np64(b), _nrc(dy), G, EPS, act)
    own = None
    if dtype in (torch.float16, torch.bfloat16):
        xs = x.clone().requires_grad_()
        ws, bs = w.clone().requires_grad_(), b.clone().requires_grad_()
        ys = orc.torch_act(act_name)(torch.nn.functional.group_norm(xs, G, ws, bs, EPS))
        gx, gw, gb = torch.autograd.grad(ys, (xs, ws, bs), dy)
        own = {"y": _nrc(ys.detach()), "dx": _nrc(gx), "dw": as_np64(gw), "db": as_np64(gb)}
    y, mean, rstd = cabi_fwd_nchw(x, w, b, G, EPS, act)
    dx, dw, db = cabi_bwd_nchw(dy, x, w, b, mean, rstd, G, act)
    torch.cuda.synchronize()
    sdt = torch.float64 if dtype == torch.float64 else torch.float32
    _check("mean", mean, truth["mean"], None, sdt)
    _check("rstd", rstd, truth["rstd"], None, sdt)
    _check("y", _nrc(y), truth["y"], own and own["y"], dtype)
    mask = None
    if act_name == "relu":
        N, C, R = shape
        D = C // G
        a = np.repeat(truth["rstd"], D, axis=1) * as_np64(w)[None, :]
        z = _nrc(x) * a[:, None, :] + (as_np64(b)[None, :] - np.repeat(truth["mean"], D, axis=1) * a)[:, None, :]
        mask = np.abs(z) > RELU_BAND
    _check("dx", _nrc(dx), truth["dx"], own and own["dx"], dtype, mask)
    _check("dw", dw, truth["dw"], own and own["dw"], dtype)
    _check("db", db, truth["db"], own and own["db"], dtype)


@pytest.mark.parametrize("act_name", ACTS)
def test_channels_first_all_activations_and_options(act_name, device):
    """Every activation in fp32; f32 parameters with bf16 data; NULL parameters; NULL statistics outputs; in place;
    bit-identical repeats."""
    act = orc.ACT_CODES[act_name]
    x, dy, w, b = _inputs((2, 48, 1000), torch.float32, device, 17)
    truth = orc.fwd_bwd(_nrc(x), as_np64(w), as_np64(b), _nrc(dy), 6, EPS, act)
    y, mean, rstd = cabi_fwd_nchw(x, w, b, 6, EPS, act)
    dx, dw, db = cabi_bwd_nchw(dy, x, w, b, mean, rstd, 6, act)
    y2, mean2, rstd2 = cabi_fwd_nchw(x, w, b, 6, EPS, act)
    dx2, dw2, db2 = cabi_bwd_nchw(dy, x, w, b, mean, rstd, 6, act)
    torch.cuda.synchronize()
    assert err(_nrc(y), truth["y"]) <= 1e-5 and err(dw, truth["dw"]) <= 1e-5 and err(db, truth["db"]) <= 1e-5
    if act_name != "relu":
        assert err(_nrc(dx), truth["dx"]) <= 1e-5
    for a, bb in ((y, y2), (mean, mean2), (rstd, rstd2), (dx, dx2), (dw, dw2), (db, db2)):
        assert torch.equal(a, bb)
    # no affine parameters, in place
    buf = x.clone()
    y3, _, _ = cabi_fwd_nchw(buf, None, None, 6, EPS, act, y=buf)
    torch.cuda.synchronize()
    t3 = orc.fwd_bwd(_nrc(x), np.ones(48), np.zeros(48), _nrc(dy), 6, EPS, act)
    assert y3.data_ptr() == buf.data_ptr() and err(_nrc(buf), t3["y"]) <= 1e-5
    # bf16 data with f32 parameters
    xb, dyb = x.bfloat16(), dy.bfloat16()
    tb = orc.fwd_bwd(_nrc(xb), as_np64(w), as_np64(b), _nrc(dyb), 6, EPS, act)
    yb, mb, rb = cabi_fwd_nchw(xb, w, b, 6, EPS, act)
    dxb, dwb, dbb = cabi_bwd_nchw(dyb, xb, w, b, mb, rb, 6, act)
    torch.cuda.synchronize()
    assert dwb.dtype == torch.float32 and err(mb, tb["mean"]) <= 1e-5 and err(_nrc(yb), tb["y"]) <= 2.0 ** -7
    assert err(dwb, tb["dw"]) <= 1e-4 and err(dbb, tb["db"]) <= 1e-4


def test_channels_first_rejects_bad_arguments(device):
    from gnnhwc import _cabi
    import ctypes

    lib = _cabi.lib
    x = torch.empty((1, 8, 16), device=device)
    vp = lambda v: ctypes.c_void_p(v.data_ptr())  # noqa: E731
    assert lib.gnnhwc_fwd_nchw(vp(x), None, None, vp(x), None, None, 1, 7, 16, 3, 1e-5, 0, 0, 0, 0, None, 0, None) == -1
    assert "divisible" in _cabi.last_error()
    assert lib.gnnhwc_fwd_nchw(vp(x), None, None, vp(x), None, None, 1, 8, 16, 2, 1e-5, 0, 0, 0, 0, None, 0, None) == -2
    assert "workspace" in _cabi.last_error()
    assert lib.gnnhwc_nchw_workspace_bytes(0, 8, 16, 2, 0, 0) == 256


def test_channels_first_empty_and_many_samples(device):
    """An empty batch returns empty results (and zero parameter gradients); 70000 one-row samples exceed every grid
    dimension but the first, which is the only one these kernels use."""
    from gnnhwc import GN_NHWC

    m = GN_NHWC(2, 8, activation="silu").to(device)
    x = torch.empty((0, 8, 4, 4), device=device, requires_grad=True)
    y = m(x)
    assert y.shape == x.shape
    y.sum().backward()
    assert float(m.weight.grad.abs().sum()) == 0.0 and float(m.bias.grad.abs().sum()) == 0.0
    gen = torch.Generator().manual_seed(3)
    N, C, R, G = 70000, 4, 6, 2
    xs = torch.randn((N, C, R), generator=gen).to(device)
    w = (torch.rand((C,), generator=gen) + 0.5).to(device)
    b = torch.randn((C,), generator=gen).to(device)
    dy = torch.randn((N, C, R), generator=gen).to(device)
    y2, mean, rstd = cabi_fwd_nchw(xs, w, b, G, EPS, 2)
    dx, dw, db = cabi_bwd_nchw(dy, xs, w, b, mean, rstd, G, 2)
    torch.cuda.synchronize()
    # truth from the CPU oracle: torch's own GroupNorm backward on the device returns wrong dgamma / dbeta for more
    # than 128 samples of so few channels (its CPU result and the oracle agree with each other and with these kernels)
    truth = orc.fwd_bwd(_nrc(xs), as_np64(w), as_np64(b), _nrc(dy), G, EPS, 2)
    assert err(_nrc(y2), truth["y"]) <= 1e-5 and err(_nrc(dx), truth["dx"]) <= 1e-5
    assert err(dw, truth["dw"]) <= 1e-5 and err(db, truth["db"]) <= 1e-5


def test_channels_first_hip_graph_replay(device):
    """Forward + backward recorded into a HIP graph and replayed with eager work in between: every replay equals the
    eager result bit for bit (these kernels keep no state between launches)."""
    x, dy, w, b = _inputs((2, 64, 1024), torch.bfloat16, device, 5)

    def step():
        y, mean, rstd = cabi_fwd_nchw(x, w, b, 8, EPS, 2)
        dx, dw, db = cabi_bwd_nchw(dy, x, w, b, mean, rstd, 8, 2)
        return y, mean, rstd, dx, dw, db

    want = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        got = step()
    for rep in range(3):
        for t in got:
            t.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        for a, ref in zip(got, want):
            assert torch.equal(a, ref), "replay %d differs from the eager result" % rep
        step()
        torch.cuda.synchronize()
