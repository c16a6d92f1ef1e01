"""GPU test of gnnhwc_fwd_static, the forward that allocates nothing (its scratch memory is a device array inside
the library's image): called through the C ABI and checked against gnnhwc_fwd on the same inputs, twice in a row,
the second time with a smaller input, so that whatever the first call left in the shared scratch is in the way.

Bars: bit for bit against gnnhwc_fwd restricted to the same multi-launch kernels (same code on a caller-provided
workspace), and the forward parity bars against the float64 oracle (fp32: err <= 1e-5; bf16: mean / rstd <= 1e-5,
y within half a bf16 ulp of the oracle's value plus the fp32 bar)."""
import ctypes

import pytest
import torch

from gnnhwc import _cabi
from oracle import gn_oracle as orc
from tests.gpu_harness import DT_CODE, as_np64, cabi_fwd, err

pytestmark = pytest.mark.gpu
EPS = 1e-5


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def fwd_static(x, w, b, G, act):
    N, R, C = x.shape
    dt = DT_CODE[x.dtype]
    sd = torch.float32 if x.dtype in (torch.float16, torch.bfloat16) else x.dtype
    y = torch.empty_like(x)
    mean = torch.empty((N, G), dtype=sd, device=x.device)
    rstd = torch.empty((N, G), dtype=sd, device=x.device)
    rc = _cabi.lib.gnnhwc_fwd_static(_ptr(x), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), N, R, C, G, EPS, act, dt,
                                     DT_CODE[w.dtype] if w is not None else dt, DT_CODE[sd],
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return rc, y, mean, rstd


def _inputs(shape, dtype, device, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    N, R, C = shape
    x = (2.0 * torch.randn(shape, generator=g) + torch.randn((1, 1, C), generator=g)).to(dtype).to(device)
    w = (0.5 + torch.rand((C,), generator=g)).to(dtype).to(device)
    b = (0.1 * torch.randn((C,), generator=g)).to(dtype).to(device)
    return x, w, b


# (first problem, second and smaller problem, groups, dtype, activation)
CASES = [
    ((2, 4096, 320), (1, 1000, 320), 32, torch.bfloat16, "silu"),
    ((3, 1961, 96), (2, 289, 96), 24, torch.float32, "gelu"),
    ((1, 16384, 640), (1, 4096, 640), 32, torch.float16, "gelu_tanh"),
    ((4, 777, 30), (1, 55, 30), 3, torch.float32, "relu"),  # C not a multiple of the vector width: scalar kernels
]


@pytest.mark.parametrize("first,second,G,dtype,act_name", CASES)
def test_static_forward_matches_the_workspace_forward_twice_in_a_row(first, second, G, dtype, act_name, device):
    act = orc.ACT_CODES[act_name]
    for i, shape in enumerate((first, second)):
        print("gnnhwc_fwd_static", shape, G, dtype, act_name, "call", i, flush=True)
        x, w, b = _inputs(shape, dtype, device, 100 + i)
        assert 0 < _cabi.lib.gnnhwc_fwd_static_scratch_bytes(*shape, G, DT_CODE[dtype]) <= _cabi.STATIC_SCRATCH_BYTES
        rc, y, mean, rstd = fwd_static(x, w, b, G, act)
        _cabi.check(rc, "gnnhwc_fwd_static")
        # the existing entry point, held to the same kernels: identical bits
        before = _cabi.set_resident(False)
        try:
            y2, mean2, rstd2 = cabi_fwd(x, w, b, G, EPS, act)
        finally:
            _cabi.set_resident(before)
        # and as it runs by default (single-launch kernels where the problem fits)
        y3, mean3, rstd3 = cabi_fwd(x, w, b, G, EPS, act)
        torch.cuda.synchronize()
        assert torch.equal(y, y2) and torch.equal(mean, mean2) and torch.equal(rstd, rstd2)
        ty, tmean, trstd = orc.fwd(as_np64(x), as_np64(w), as_np64(b), G, EPS, act)
        truth = dict(y=ty, mean=tmean, rstd=trstd)
        assert err(mean, truth["mean"]) <= 1e-5 and err(rstd, truth["rstd"]) <= 1e-5
        assert err(mean3, truth["mean"]) <= 1e-5 and err(rstd3, truth["rstd"]) <= 1e-5
        if dtype == torch.float32:
            assert err(y, truth["y"]) <= 1e-5
            assert err(y3, truth["y"]) <= 1e-5
        else:
            # one rounding to the 16-bit type of a value that is within the fp32 bar of the truth
            ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
            t = torch.as_tensor(truth["y"])
            for cand in (y, y3):
                d = (cand.detach().cpu().double() - t).abs()
                assert bool((d <= ulp * t.abs() * 1.001 + 1e-5 * (t.abs() + 1.0) + 2.0 ** -24).all())


def test_static_forward_rejects_what_its_scratch_cannot_hold(device):
    # many samples of many groups: the per-tile statistics alone exceed the library's scratch
    N, R, C, G = 4096, 64, 2048, 512
    need = _cabi.lib.gnnhwc_fwd_static_scratch_bytes(N, R, C, G, 0)
    assert need > _cabi.STATIC_SCRATCH_BYTES
    x = torch.zeros((8,), device=device)  # never dereferenced: the call is refused before anything is launched
    rc, _, _, _ = None, None, None, None
    rc = _cabi.lib.gnnhwc_fwd_static(_ptr(x), None, None, _ptr(x), None, None, N, R, C, G, EPS, 0, 0, 0, 0, None)
    assert rc == -2 and "scratch" in _cabi.last_error()
    with pytest.raises(RuntimeError):
        _cabi.check(rc, "gnnhwc_fwd_static")
    # invalid shapes are refused like everywhere else, and an empty batch is a no-op
    assert _cabi.lib.gnnhwc_fwd_static(None, None, None, None, None, None, 1, 16, 7, 3, EPS, 0, 0, 0, 0, None) == -1
    assert _cabi.lib.gnnhwc_fwd_static(None, None, None, None, None, None, 0, 16, 8, 2, EPS, 0, 0, 0, 0, None) == 0


def test_static_forward_allocates_nothing_under_graph_capture(device):
    """After one warm-up call per device (which looks up the scratch address), the call is recorded into a HIP graph with
    the capture in 'global' error mode -- any allocation, event creation or host-pinned allocation the library made
    while the stream is capturing would invalidate the capture -- and every replay reproduces the eager result bit for bit."""
    shape, G, dtype, act = (2, 4096, 320), 32, torch.bfloat16, orc.ACT_CODES["silu"]
    x, w, b = _inputs(shape, dtype, device, 7)
    rc, y_eager, mean_eager, rstd_eager = fwd_static(x, w, b, G, act)  # warm-up: the only call that may touch set-up paths
    _cabi.check(rc, "gnnhwc_fwd_static")
    torch.cuda.synchronize()
    N, R, C = shape
    y = torch.empty_like(x)
    mean = torch.empty((N, G), dtype=torch.float32, device=device)
    rstd = torch.empty((N, G), dtype=torch.float32, device=device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side, capture_error_mode="global"):
            rc = _cabi.lib.gnnhwc_fwd_static(_ptr(x), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), N, R, C, G, EPS, int(act),
                                             DT_CODE[dtype], DT_CODE[dtype], 0, ctypes.c_void_p(side.cuda_stream))
    _cabi.check(rc, "gnnhwc_fwd_static under capture")
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        y.zero_()
        mean.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_eager) and torch.equal(mean, mean_eager) and torch.equal(rstd, rstd_eager), "replay %d" % replay
        _ = fwd_static(x, w, b, G, act)  # eager work of the same kind between the replays
        torch.cuda.synchronize()
