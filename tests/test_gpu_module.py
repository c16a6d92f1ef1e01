"""GPU tests of the Python surface (GN_NHWC, GN_NHWC_Func, gnop::fwd / gnop::bwd) and of the shapes, layouts and
dtypes the reference's own tests exercise (test/trailing_dims.py, test/nchw_nhwc_equal.py, the shape list of
test/check_outputs.py:161-189), each for both kernel families (single-launch "resident" and streaming).

Truth is torch's GroupNorm + activation evaluated in float64 on the device; tolerances as in test_gpu_parity.py:
fp32 err <= 1e-5, fp64 err <= 1e-12, fp16 / bf16 no worse than torch's own result in that dtype (+2 %).
"""
import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gnnhwc import GN_NHWC, GN_NHWC_Func, _cabi
from oracle import gn_oracle as orc
from tests.gpu_harness import as_np64, cabi_bwd, cabi_fwd, err, nrc_view

pytestmark = pytest.mark.gpu

ACTS = ["identity", "relu", "silu", "gelu", "gelu_tanh"]
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}
HALF_SLACK = 0.02


def channels_last_like(shape, dtype, device, gen, scale=1.0, shift=0.0):
    """Random (N, C, *spatial) tensor whose memory is (N, *spatial, C): stride(1) == 1 for any rank."""
    N, C = shape[0], shape[1]
    t = torch.randn((N, *shape[2:], C), generator=gen) * scale + shift
    nd = len(shape)
    return t.to(dtype).to(device).permute(0, nd - 1, *range(1, nd - 1))


def run_module(x, G, act, w, b, dy, eps=1e-5, affine=True):
    C = x.shape[1]
    m = GN_NHWC(G, C, activation=act, eps=eps, affine=affine).to(x.device).to(x.dtype)
    if affine:
        with torch.no_grad():
            m.weight.copy_(w)
            m.bias.copy_(b)
    xr = x.detach().clone().requires_grad_(True)
    y = m(xr)
    out = {"y": y.detach()}
    if dy is not None:
        y.backward(dy)
        out["dx"] = xr.grad
        if affine:
            out["dw"], out["db"] = m.weight.grad, m.bias.grad
    return out


def check_against_torch(x, G, act, w, b, dy, eps=1e-5, relu_band=1e-4):
    """Compare the module with torch in float64 (truth) and, for 16-bit types, with torch in the same dtype."""
    dtype = x.dtype
    ours = run_module(x, G, act, w, b, dy, eps)
    truth = orc.torch_reference(x.double(), w.double(), b.double(), G, eps, act, None if dy is None else dy.double())
    lib = orc.torch_reference(x, w, b, G, eps, act, dy) if dtype != torch.float64 else None
    mask = None
    if act == "relu" and dy is not None:
        z = F.group_norm(x.double(), G, w.double(), b.double(), eps)
        mask = z.abs() > relu_band
    for k in ours:
        o, t = ours[k].double(), truth[k]
        l = lib[k].double() if lib is not None else None
        if k == "dx" and mask is not None:
            o, t = o * mask, t * mask
            l = l * mask if l is not None else None
        e = err(o, t)
        if dtype == torch.float64:
            assert e <= TOL[dtype], "%s: err %.3g" % (k, e)
        elif dtype == torch.float32:
            # 1e-5; only for ill-conditioned slabs of at most four elements per group (two equal values make the
            # variance vanish) also within twice torch's own fp32 error against the same truth (the reference's
            # second-stage rule, test/check_outputs.py:134)
            per_group = x.numel() // (x.shape[0] * G)
            ok = e <= TOL[dtype] or (per_group <= 4 and e <= 2 * err(l, t))
            assert ok, "%s: err %.3g, torch fp32 %.3g, %d elements per group" % (k, e, err(l, t), per_group)
        else:
            e_lib = err(l, t)
            assert e <= e_lib * (1 + HALF_SLACK) + 1e-12, "%s: err %.3g vs torch's own %.3g" % (k, e, e_lib)
        assert ours[k].shape == truth[k].shape
    if min(x.shape) > 1:  # strides of size-1 dims are arbitrary
        assert ours["y"].stride() == x.stride(), "output keeps the input's (channels-last) strides"
    return ours


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_module_forward_backward(family, act, dtype, device):
    gen = torch.Generator().manual_seed(11)
    shape, G = (2, 64, 23, 19), 8
    x = channels_last_like(shape, dtype, device, gen, 2.0, 0.5)
    dy = channels_last_like(shape, dtype, device, gen)
    w = (torch.rand(64, generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn(64, generator=gen)).to(dtype).to(device)
    check_against_torch(x, G, act, w, b, dy)


# (N, C, spatial..., G): the fp64 shape list of test/check_outputs.py:162-185 that is dead code there, scaled to
# run in seconds: C = 1, prime-ish channel counts, G = C, G = 1, D > 128, D > 1024.
ODD_SHAPES = [
    ((1, 1, 3, 3), 1),
    ((1, 1, 224, 224), 1),
    ((2, 6, 4, 4), 3),
    ((1, 3909, 4, 4), 3),
    ((2, 2062, 3, 5), 1031),
    ((1, 2062, 2, 2), 2),
    ((3, 7, 9, 11), 7),
    ((2, 30, 5, 5), 5),
    ((1, 2680, 6, 6), 8),
    ((1, 536, 7, 3), 67),
    ((5, 256, 1, 1), 32),
    ((2, 128, 2, 1), 128),
    ((13, 2560, 8, 8), 4),
]


@pytest.mark.parametrize("shape,G", ODD_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_shapes(family, shape, G, dtype, device):
    gen = torch.Generator().manual_seed(5)
    C = shape[1]
    x = channels_last_like(shape, dtype, device, gen, 1.5, -0.3)
    dy = channels_last_like(shape, dtype, device, gen)
    w = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(dtype).to(device)
    if shape[2] * shape[3] == 1:
        # H * W == 1 makes the tensor both contiguous and channels-last (test/check_outputs.py:68-69): make sure
        # the kernel path is the one under test, through the autograd function
        xr = x.detach().clone().requires_grad_(True)
        wr, br = w.clone().requires_grad_(True), b.clone().requires_grad_(True)
        y = GN_NHWC_Func.apply(xr, wr, br, G, 1e-5, 2)
        y.backward(dy)
        truth = orc.torch_reference(x.double(), w.double(), b.double(), G, 1e-5, "silu", dy.double())
        lib = orc.torch_reference(x, w, b, G, 1e-5, "silu", dy) if dtype == torch.bfloat16 else None
        for k, o in (("y", y), ("dx", xr.grad), ("dw", wr.grad), ("db", br.grad)):
            e = err(o.double(), truth[k])
            if lib is None:
                assert e <= TOL[dtype], (k, e)
            else:
                assert e <= err(lib[k].double(), truth[k]) * (1 + HALF_SLACK) + 1e-12, (k, e)
        return
    check_against_torch(x, G, "silu", w, b, dy)


def test_trailing_dims(family, device):
    """test/trailing_dims.py:7-33: rank-6 inputs, and the output is unchanged when trailing dims are flattened."""
    for N, C, R_list in [(1, 512, [1, 1, 1, 1]), (1, 256, [4, 2, 8, 1]), (1, 256, [7, 13, 19, 1]), (1, 128, [32, 1, 1, 1]),
                         (1, 32, [32, 128, 32, 1])]:
        R_list = list(R_list)
        x = torch.randn((N, *R_list, C), device=device)
        x = x.permute(0, -1, *range(1, len(R_list) + 1))
        G = 32
        for dtype in (torch.half, torch.float):
            m = GN_NHWC(G, C).to(device).to(dtype)
            m_ref = nn.GroupNorm(G, C).to(device).to(dtype)
            y = m(x.to(dtype))
            y_ref = m_ref(x.to(dtype))
            assert F.mse_loss(y, y_ref) < 1e-6
            xs, dims = x, list(R_list)
            while len(dims) != 1:
                last = dims.pop(-1)
                dims[-1] *= last
                xs = xs.reshape(N, C, *dims)
                assert F.mse_loss(y_ref.reshape(N, C, *dims), m(xs.to(dtype))) < 1e-6


def test_trailing_dims_backward(family, device):
    """The reference's backward only accepts 4-D inputs (custom_gn.py:44); here any rank >= 3 works."""
    gen = torch.Generator().manual_seed(3)
    for shape, G in [((2, 256, 8, 16, 16), 16), ((2, 32, 50), 4), ((1, 16, 3, 2, 2, 5), 2)]:
        x = channels_last_like(shape, torch.float32, device, gen)
        dy = channels_last_like(shape, torch.float32, device, gen)
        C = shape[1]
        w = (torch.rand(C, generator=gen) + 0.5).to(device)
        b = (0.1 * torch.randn(C, generator=gen)).to(device)
        check_against_torch(x, G, "gelu_tanh", w, b, dy)
        # a gradient that arrives in plain contiguous layout is handled as well
        ours = run_module(x, G, "silu", w, b, dy.contiguous())
        truth = orc.torch_reference(x.double(), w.double(), b.double(), G, 1e-5, "silu", dy.double())
        assert err(ours["dx"], truth["dx"]) <= 1e-5


def test_weird_mem_fmt(family, device):
    """test/trailing_dims.py:35-71: pseudo-channels-last (stride(1) == 1, inner dims permuted) and pseudo-contiguous."""
    B, C, G = 2, 32, 8
    for dtype in (torch.half, torch.float):
        m = GN_NHWC(G, C).to(device).to(dtype)
        m_ref = nn.GroupNorm(G, C).to(device).to(dtype)
        for inner in ((3, 5), (3, 5, 7), (3, 5, 7, 11)):
            x = torch.randn((B, *inner, C), device=device)
            x = x.permute(0, -1, *range(len(inner), 0, -1))
            assert x.stride(1) == 1
            assert F.mse_loss(m(x.to(dtype)), m_ref(x.to(dtype))) < 1e-6
            x = torch.randn((B, C, *inner), device=device)
            x = x.permute(0, 1, *range(len(inner), 1, -1), -1)
            assert F.mse_loss(m(x.to(dtype)), m_ref(x.to(dtype))) < 1e-6


def test_nchw_nhwc_equal(family, device):
    """test/nchw_nhwc_equal.py:7-25: the same module fed NCHW (the reference: torch fallback; here: the channels-first
    kernels) and NHWC (the channels-last kernels) agrees."""
    N, R, G, C = 1, 256, 32, 128
    x = torch.randn((N, C, R, R), device=device)
    x_nhwc = x.to(memory_format=torch.channels_last)
    rand_dy = torch.rand_like(x)
    rand_dy_nhwc = rand_dy.to(memory_format=torch.channels_last)
    for act in ("identity", "silu", "gelu", "gelu_tanh"):
        for dtype in (torch.half, torch.float, torch.double, torch.bfloat16):
            m = GN_NHWC(G, C, act).to(device).to(dtype)
            a = x.detach().to(dtype).requires_grad_(True)
            c = x_nhwc.detach().to(dtype).requires_grad_(True)
            out1, out2 = m(a), m(c)
            out1.backward(rand_dy.to(dtype))
            out2.backward(rand_dy_nhwc.to(dtype))
            if dtype != torch.bfloat16:
                # the reference's bound
                assert (out1 - out2).float().square().mean() < 1e-6
                assert (a.grad - c.grad).float().square().mean() < 1e-6
            else:
                # two bf16 results may differ in the last bit of some elements (the two kernel families sum in
                # different orders), which already exceeds 1e-6 in the mean square; each layout is held to the
                # half-precision rule instead: no further from the float64 truth than torch's own bf16 result
                w, b = m.weight.detach(), m.bias.detach()
                truth = orc.torch_reference(x.double(), w.double(), b.double(), G, m.eps, act, rand_dy.double())
                lib = orc.torch_reference(x.to(dtype), w, b, G, m.eps, act, rand_dy.to(dtype))
                for got_y, got_dx in ((out1, a.grad), (out2, c.grad)):
                    assert err(got_y.double(), truth["y"]) <= err(lib["y"].double(), truth["y"]) * (1 + HALF_SLACK)
                    assert err(got_dx.double(), truth["dx"]) <= err(lib["dx"].double(), truth["dx"]) * (1 + HALF_SLACK)


@pytest.mark.parametrize("name", ["c5a_fp32_silu", "c5b_fp32_gelu", "c5c_fp32_relu", "c2", "c3b"])
def test_bit_identical_from_run_to_run(family, name, device):
    """No floating-point atomics and fixed reduction trees: every output is reproduced bit for bit."""
    from tests import configs

    cfg = configs.CONFIGS[name]
    inp = configs.make_inputs(cfg, device)
    x, dy = nrc_view(inp["x"]), nrc_view(inp["dy"])
    act = orc.ACT_CODES[cfg.act]
    first = None
    for rep in range(3):
        y, mean, rstd = cabi_fwd(x, inp["w"], inp["b"], cfg.G, 1e-5, act)
        dx, dw, db = cabi_bwd(dy, x, inp["w"], inp["b"], mean, rstd, cfg.G, act)
        torch.cuda.synchronize()
        cur = [t.clone() for t in (y, mean, rstd, dx, dw, db)]
        if first is None:
            first = cur
        else:
            for a, b_ in zip(first, cur):
                assert torch.equal(a, b_)
        # unrelated work in between, so that scheduling differs
        torch.randn(1 << 20, device=device).sum().item()


def test_unaligned_and_scalar_path(family, device):
    """Base pointers that are not 16-byte aligned and channel counts that are not a multiple of the vector width."""
    gen = torch.Generator().manual_seed(9)
    for dtype in (torch.float32, torch.float16):
        for (N, R, C, G) in [(2, 77, 64, 8), (1, 130, 30, 5)]:
            n = N * R * C
            buf_x = torch.randn(n + 1, generator=gen).to(dtype).to(device)
            buf_dy = torch.randn(n + 1, generator=gen).to(dtype).to(device)
            buf_y = torch.empty(n + 1, dtype=dtype, device=device)
            buf_dx = torch.empty(n + 1, dtype=dtype, device=device)
            x, dy = buf_x[1:].view(N, R, C), buf_dy[1:].view(N, R, C)
            w = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
            b = (0.1 * torch.randn(C, generator=gen)).to(dtype).to(device)
            y, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, 2, y=buf_y[1:].view(N, R, C))
            dx, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, 2, dx=buf_dx[1:].view(N, R, C))
            torch.cuda.synchronize()
            t = orc.fwd_bwd(x.double().cpu().numpy(), w.double().cpu().numpy(), b.double().cpu().numpy(),
                            dy.double().cpu().numpy(), G, 1e-5, 2)
            tol = 1e-5 if dtype == torch.float32 else 2e-3
            for k, o in (("y", y), ("dx", dx), ("dw", dw), ("db", db)):
                assert err(o, t[k]) <= tol, (dtype, (N, R, C, G), k, err(o, t[k]))


def test_mixed_parameter_and_statistics_dtypes(family, device):
    """f32 weight / bias with 16-bit data (the autocast case; the reference rejects it, custom_gn.cpp:35), and
    statistics handed to the backward in the data's own 16-bit type (what the reference stores, custom_gn.cpp:26-27)."""
    gen = torch.Generator().manual_seed(21)
    shape, G = (2, 96, 17, 13), 12
    for dtype in (torch.float16, torch.bfloat16):
        x = channels_last_like(shape, dtype, device, gen, 2.0, 1.0)
        dy = channels_last_like(shape, dtype, device, gen)
        w = (torch.rand(96, generator=gen) + 0.5).to(device)
        b = (0.1 * torch.randn(96, generator=gen)).to(device)
        xn, dyn = nrc_view(x), nrc_view(dy)
        y, mean, rstd = cabi_fwd(xn, w, b, G, 1e-5, 2)
        assert mean.dtype == torch.float32
        dx, dw, db = cabi_bwd(dyn, xn, w, b, mean, rstd, G, 2)
        assert dw.dtype == torch.float32
        torch.cuda.synchronize()
        t = orc.fwd_bwd(xn.double().cpu().numpy(), w.double().cpu().numpy(), b.double().cpu().numpy(), dyn.double().cpu().numpy(),
                        G, 1e-5, 2)
        half_tol = 2e-3 if dtype == torch.float16 else 1.6e-2
        assert err(y, t["y"]) <= half_tol and err(dx, t["dx"]) <= half_tol
        assert err(dw, t["dw"]) <= 1e-4 and err(db, t["db"]) <= 1e-4  # f32 outputs of f32 sums
        # statistics rounded to the data type: still a valid backward, to that type's accuracy
        y2, mean_h, rstd_h = cabi_fwd(xn, w.to(dtype), b.to(dtype), G, 1e-5, 2, stats_dtype=dtype)
        assert mean_h.dtype == dtype and torch.equal(y2, cabi_fwd(xn, w.to(dtype), b.to(dtype), G, 1e-5, 2)[0])
        dx2, _, _ = cabi_bwd(dyn, xn, w.to(dtype), b.to(dtype), mean_h, rstd_h, G, 2)
        torch.cuda.synchronize()
        assert err(dx2, t["dx"]) <= 4 * half_tol


def test_non_affine_and_null_parameters(family, device):
    gen = torch.Generator().manual_seed(2)
    shape, G = (2, 48, 9, 9), 6
    x = channels_last_like(shape, torch.float32, device, gen)
    dy = channels_last_like(shape, torch.float32, device, gen)
    ours = run_module(x, G, "silu", None, None, dy, affine=False)
    ones, zeros = torch.ones(48, device=device), torch.zeros(48, device=device)
    truth = orc.torch_reference(x.double(), ones.double(), zeros.double(), G, 1e-5, "silu", dy.double())
    assert err(ours["y"], truth["y"]) <= 1e-5 and err(ours["dx"], truth["dx"]) <= 1e-5
    # the C ABI takes null weight / bias for gamma = 1, beta = 0, and null dweight / dbias to skip them
    xn, dyn = nrc_view(x), nrc_view(dy)
    y, mean, rstd = cabi_fwd(xn, None, None, G, 1e-5, 2)
    dx, dw, db = cabi_bwd(dyn, xn, None, None, mean, rstd, G, 2, want_dw=False, want_db=False)
    torch.cuda.synchronize()
    assert dw is None and db is None
    assert torch.equal(nrc_view(ours["y"]), y) and torch.equal(nrc_view(ours["dx"]), dx)


def test_empty_and_wrapped_batches(family, device):
    m = GN_NHWC(4, 8, activation="silu").to(device)
    x0 = torch.empty((0, 8, 5, 5), device=device).to(memory_format=torch.channels_last).requires_grad_(True)
    y0 = m(x0)
    assert y0.shape == x0.shape
    y0.sum().backward()
    assert torch.count_nonzero(m.weight.grad) == 0 and torch.count_nonzero(m.bias.grad) == 0
    # more samples than the grid's z extent
    gen = torch.Generator().manual_seed(4)
    shape, G = (65536 + 3, 8, 2, 1), 2
    x = channels_last_like(shape, torch.float32, device, gen)
    dy = channels_last_like(shape, torch.float32, device, gen)
    w = (torch.rand(8, generator=gen) + 0.5).to(device)
    b = (0.1 * torch.randn(8, generator=gen)).to(device)
    xr, wr, br = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    y = GN_NHWC_Func.apply(xr, wr, br, G, 1e-5, 0)
    y.backward(dy)
    # truth from the CPU oracle (torch's own GPU GroupNorm backward is not reliable beyond 65535 samples)
    t = orc.fwd_bwd(orc.to_nrc(x), w.double().cpu().numpy(), b.double().cpu().numpy(), orc.to_nrc(dy), G, 1e-5, 0)
    assert err(orc.to_nrc(y), t["y"]) <= 1e-5 and err(orc.to_nrc(xr.grad), t["dx"]) <= 1e-5
    assert err(wr.grad, t["dw"]) <= 1e-5 and err(br.grad, t["db"]) <= 1e-5


# The reference's own regression list (test/check_outputs.py:161-185: identity activation, float64) and a seeded
# sample of its brute-force grid (test/check_outputs.py:191-211: bfloat16, H == W, batch sizes / channel counts /
# resolutions / group counts from the same lists).
REFERENCE_CUSTOM_INPUTS = [
    (1, 1, 2, 2, 1), (2, 3909, 5, 5, 3), (1, 2062, 5, 5, 1031), (3, 4096, 7, 7, 4), (1, 4096, 7, 7, 4),
    (2, 160, 8, 8, 160), (1, 3, 7, 7, 1), (1, 1, 4, 4, 1), (1, 128, 8, 8, 8), (2, 1280, 8, 8, 32),
    (2, 640, 16, 16, 32), (2, 2560, 8, 8, 32), (2, 1280, 16, 16, 32), (2, 320, 32, 32, 32), (2, 1920, 16, 16, 32),
    (2, 2560, 16, 16, 32), (2, 640, 32, 32, 32), (2, 960, 32, 32, 32), (2, 1280, 32, 32, 32), (2, 320, 64, 64, 32),
    (2, 1920, 32, 32, 32), (2, 640, 64, 64, 32), (8, 128, 64, 64, 32),
]


@pytest.mark.parametrize("B,C,H,W,G", REFERENCE_CUSTOM_INPUTS)
def test_reference_custom_inputs(B, C, H, W, G, device):
    gen = torch.Generator().manual_seed(B * 7919 + C)
    shape = (B, C, H, W)
    x = channels_last_like(shape, torch.float64, device, gen, 1.3, 0.2)
    dy = channels_last_like(shape, torch.float64, device, gen)
    w = (torch.rand(C, generator=gen, dtype=torch.float64) + 0.5).to(device)
    b = (0.1 * torch.randn(C, generator=gen, dtype=torch.float64)).to(device)
    check_against_torch(x, G, "identity", w, b, dy)


def _brute_force_sample(count, seed):
    import itertools
    import random

    Bs = (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 13, 16)
    Cs = (1, 2, 3, 4, 5, 6, 7, 32, 64, 128, 256, 512, 13, 140, 125, 961, 160, 320, 640, 960, 1280, 1600, 1920, 2240, 2560,
          1303, 2602, 3909)
    Rs = (2, 3, 4, 5, 6, 7, 8, 9, 10, 17, 16, 64, 128)
    Gs = (1, 2, 3, 4, 8, 16, 32)
    valid = [(B, C, R, G) for B, C, R, G in itertools.product(Bs, Cs, Rs, Gs) if C % G == 0 and B * C * R * R <= (1 << 24)]
    return random.Random(seed).sample(valid, count)


@pytest.mark.parametrize("B,C,R,G", _brute_force_sample(48, 2024))
def test_reference_brute_force_sample(family, B, C, R, G, device):
    gen = torch.Generator().manual_seed(B * 31 + C * 7 + R)
    shape = (B, C, R, R)
    x = channels_last_like(shape, torch.bfloat16, device, gen, 1.0, 0.0)
    dy = channels_last_like(shape, torch.bfloat16, device, gen)
    w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
    check_against_torch(x, G, "identity", w, b, dy)


@pytest.mark.parametrize("shape,G", [((2, 64, 23, 19), 8), ((4, 320, 128, 128), 32)])
def test_inference_in_place_without_statistics(family, shape, G, device):
    """Forward with y aliasing x and no mean / rstd outputs gives the same y as the ordinary call."""
    import ctypes

    gen = torch.Generator().manual_seed(31)
    C = shape[1]
    x = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen, 1.5, 0.3))
    w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
    y_ref, _, _ = cabi_fwd(x, w, b, G, 1e-5, 2)
    N, R, _ = x.shape
    lib = _cabi.lib
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, 3)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=device)
    buf = x.clone()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    rc = lib.gnnhwc_fwd(vp(buf), vp(w), vp(b), vp(buf), None, None, N, R, C, G, 1e-5, 2, 3, 3, 0, vp(ws), nbytes,
                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _cabi.check(rc, "gnnhwc_fwd")
    torch.cuda.synchronize()
    assert torch.equal(buf, y_ref)


@pytest.mark.parametrize("N,R,C,G,act,dtype", [
    (2, 23 * 19, 64, 8, "silu", torch.bfloat16),
    (4, 128 * 128, 320, 32, "gelu", torch.bfloat16),
    (1, 150037, 192, 24, "silu", torch.bfloat16),      # the backward that keeps g' and streams x through a window
    (6, 128 * 128, 320, 32, "relu", torch.float16),    # a backward in two launches over groups of samples
    (3, 37 * 53, 96, 24, "gelu_tanh", torch.float32),
    (2, 1000, 30, 5, "silu", torch.float32),           # scalar kernels
])
def test_backward_in_place_of_the_incoming_gradient(family, N, R, C, G, act, dtype, device):
    """dx written into dy's own buffer (a caller that has no further use for dy) equals the ordinary call bit for bit,
    in both kernel families."""
    gen = torch.Generator().manual_seed(41 + R)
    x = (torch.randn((N, R, C), generator=gen) * 1.5 + 0.3).to(dtype).to(device)
    dy = torch.randn((N, R, C), generator=gen).to(dtype).to(device)
    w = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(dtype).to(device)
    code = orc.ACT_CODES[act]
    y, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, code)
    dx0, dw0, db0 = cabi_bwd(dy, x, w, b, mean, rstd, G, code)
    buf = dy.clone()
    dx1, dw1, db1 = cabi_bwd(buf, x, w, b, mean, rstd, G, code, dx=buf)
    torch.cuda.synchronize()
    assert dx1.data_ptr() == buf.data_ptr()
    assert torch.equal(dx1, dx0) and torch.equal(dw1, dw0) and torch.equal(db1, db0)


# Shapes for the recovery path of the single-launch kernels: every exchange form (all workgroups poll all tiles; two-level;
# groups straddling chunks; partial last tiles), the backward that keeps g' only, and a backward cut into several launches
# (its dgamma / dbeta stage reads the channel records of earlier launches).
RECOVERY_SHAPES = [
    (2, 2048, 1280, 32, "silu", torch.bfloat16),
    (3, 37 * 53, 96, 24, "gelu", torch.float32),
    (1, 4096, 64, 32, "gelu_tanh", torch.float16),     # 66 records per group and 33 groups per chunk: two-level exchange
    (1, 64 * 64, 1280, 32, "silu", torch.bfloat16),
    (2, 9000, 40, 5, "relu", torch.float32),
    (1, 150037, 192, 24, "silu", torch.bfloat16),      # 58 MB: the windowed backward
    (6, 128 * 128, 320, 32, "silu", torch.bfloat16),   # backward in two launches over groups of samples
]


@pytest.mark.parametrize("N,R,C,G,act,dtype", RECOVERY_SHAPES)
def test_single_launch_kernels_recover_from_expired_waits(N, R, C, G, act, dtype, device):
    """A single-launch kernel whose workgroups cannot wait for each other must still produce the right result.  Forced
    here from the host with the poll limit -2: every wait gives up at its first poll, whether or not the data is there,
    so every workgroup takes the recovery path and RECOMPUTES every record it needs from the inputs (every kernel still
    ends normally).  y, mean, rstd, dx, dweight and dbias meet the same bars as on the fast path, no call reports an
    error, the status query says that it happened, and the process stays on the single-launch kernels."""
    from tests.test_gpu_parity import _check, RELU_BAND

    lib = _cabi.lib
    gen = torch.Generator().manual_seed(11 + R)
    x = (torch.randn((N, R, C), generator=gen) * 2 + torch.randn((C,), generator=gen)).to(dtype).to(device)
    dy = torch.randn((N, R, C), generator=gen).to(dtype).to(device)
    w = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(dtype).to(device)
    code = orc.ACT_CODES[act]

    def torch_ref(t):
        xs = x.to(t).permute(0, 2, 1).contiguous().requires_grad_()
        ws, bs = w.to(t).requires_grad_(), b.to(t).requires_grad_()
        ys = orc.torch_act(act)(torch.nn.functional.group_norm(xs, G, ws, bs, 1e-5))
        gx, gw, gb = torch.autograd.grad(ys, (xs, ws, bs), dy.to(t).permute(0, 2, 1))
        return {"y": ys.detach().permute(0, 2, 1), "dx": gx.permute(0, 2, 1), "dw": gw, "db": gb}

    truth = torch_ref(torch.float64)
    own = torch_ref(dtype) if dtype != torch.float32 else None
    xd = x.double().view(N, R, G, C // G)
    before = _cabi.set_resident(True)
    prev = lib.gnnhwc_debug_set_spin_limit(-2)
    try:
        lib.gnnhwc_resident_status()
        _cabi.profile_collect()
        _cabi.profile_enable(True)
        y, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, code)
        torch.cuda.synchronize()
        assert lib.gnnhwc_resident_status() == 1, "the forward did not take the recovery path"
        assert lib.gnnhwc_resident_status() == 0  # reading clears it
        dx, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, code)
        torch.cuda.synchronize()
        _cabi.profile_enable(False)
        assert lib.gnnhwc_resident_status() == 1, "the backward did not take the recovery path"
        launches = {k: v[0] for k, v in _cabi.profile_collect().items() if v[0]}
        assert set(launches) == {"fused_fwd", "fused_bwd"}, launches  # single-launch kernels only
        assert err(mean, xd.mean(dim=(1, 3))) <= 1e-5
        assert err(rstd, (xd.var(dim=(1, 3), correction=0) + 1e-5).rsqrt()) <= 1e-5
        mask = None
        if act == "relu":
            a = (rstd.double().repeat_interleave(C // G, dim=1) * w.double()[None, :])
            z = x.double() * a[:, None, :] + (b.double()[None, :] - mean.double().repeat_interleave(C // G, dim=1) * a)[:, None, :]
            mask = (z.abs() > RELU_BAND).cpu().numpy()
        for name, ours in (("y", y), ("dx", dx), ("dw", dw), ("db", db)):
            _check(name, ours, as_np64(truth[name]), own and as_np64(own[name]), dtype, mask if name == "dx" else None)
        # and the same calls on the fast path afterwards: nothing was switched off, no error is pending
        lib.gnnhwc_debug_set_spin_limit(prev)
        _cabi.profile_enable(True)
        y2, mean2, rstd2 = cabi_fwd(x, w, b, G, 1e-5, code)
        dx2, dw2, db2 = cabi_bwd(dy, x, w, b, mean2, rstd2, G, code)
        torch.cuda.synchronize()
        _cabi.profile_enable(False)
        launches = {k: v[0] for k, v in _cabi.profile_collect().items() if v[0]}
        assert set(launches) == {"fused_fwd", "fused_bwd"}, launches
        assert lib.gnnhwc_resident_status() == 0
        for name, ours in (("y", y2), ("dx", dx2), ("dw", dw2), ("db", db2)):
            _check(name, ours, as_np64(truth[name]), own and as_np64(own[name]), dtype, mask if name == "dx" else None)
    finally:
        _cabi.profile_enable(False)
        lib.gnnhwc_debug_set_spin_limit(prev)
        lib.gnnhwc_resident_status()
        _cabi.set_resident(before)


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("polls", [0, 2, 16])
@pytest.mark.parametrize("N,R,C,G,act,dtype", RECOVERY_SHAPES)
def test_short_waits_mix_arrived_and_recomputed_records(N, R, C, G, act, dtype, polls, in_place, device):
    """The recovery as it happens in the field: with a poll limit of 0, 2 or 16 (not the forced mode) a wait expires
    only when its record really has not arrived yet, so a launch is a mixture of workgroups on the fast path and
    workgroups that take the records that have arrived and recompute the others.  The results must be those of an
    undisturbed launch up to the rounding of a statistic (a recomputed record sums in another order) -- also when the
    outputs replace the inputs in place (y in x's buffer, dx in dy's), where a recomputed record may only be used if its
    owner has provably not stored anything yet."""
    lib = _cabi.lib
    gen = torch.Generator().manual_seed(77 + R + polls)
    x = (torch.randn((N, R, C), generator=gen) * 2 + torch.randn((C,), generator=gen)).to(dtype).to(device)
    dy = torch.randn((N, R, C), generator=gen).to(dtype).to(device)
    w = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(dtype).to(device)
    code = orc.ACT_CODES[act]
    half = dtype != torch.float32
    before = _cabi.set_resident(True)
    try:
        y0, mean0, rstd0 = cabi_fwd(x, w, b, G, 1e-5, code)
        dx0, dw0, db0 = cabi_bwd(dy, x, w, b, mean0, rstd0, G, code)
        torch.cuda.synchronize()
        prev = lib.gnnhwc_debug_set_spin_limit(polls)
        recovered = 0
        try:
            lib.gnnhwc_resident_status()
            for rep in range(3):
                xin = x.clone() if in_place else x
                dyin = dy.clone() if in_place else dy
                _cabi.profile_collect()
                _cabi.profile_enable(True)
                y, mean, rstd = cabi_fwd(xin, w, b, G, 1e-5, code, y=xin if in_place else None)
                dx, dw, db = cabi_bwd(dyin, x, w, b, mean0, rstd0, G, code, dx=dyin if in_place else None)
                torch.cuda.synchronize()
                _cabi.profile_enable(False)
                launches = {k: v[0] for k, v in _cabi.profile_collect().items() if v[0]}
                assert set(launches) == {"fused_fwd", "fused_bwd"}, launches
                recovered += lib.gnnhwc_resident_status()
                assert err(mean, mean0) <= 1e-5 and err(rstd, rstd0) <= 1e-5, (rep, "statistics")
                # elementwise outputs: a statistic that differs in its last bits moves few elements by one spacing of the type
                for name, a, t in (("y", y, y0), ("dx", dx, dx0)):
                    assert err(a, t) <= (2.0 ** -7 if half else 1e-5), (rep, name, err(a, t))
                    if half:
                        assert float((a.float() != t.float()).float().mean()) < 0.02, (rep, name)
                for name, a, t in (("dw", dw, dw0), ("db", db, db0)):
                    assert err(a, t) <= (2.0 ** -7 if half else 1e-5), (rep, name, err(a, t))
        finally:
            _cabi.profile_enable(False)
            lib.gnnhwc_debug_set_spin_limit(prev)
        if polls == 0:
            assert recovered > 0, "no wait expired although nobody waited at all"
    finally:
        lib.gnnhwc_resident_status()
        _cabi.set_resident(before)


def test_fused_additions_recover_from_expired_waits(device):
    """The same for the forward with fused additions (residual, per-sample channel addend, sum written out): the
    recomputation rebuilds the sum exactly as the fast path forms it."""
    from tests.gpu_harness import cabi_fwd_add

    lib = _cabi.lib
    gen = torch.Generator().manual_seed(5)
    N, R, C, G = 2, 3000, 640, 32
    x = (torch.randn((N, R, C), generator=gen) * 1.5).to(torch.bfloat16).to(device)
    res = torch.randn((N, R, C), generator=gen).to(torch.bfloat16).to(device)
    cb = torch.randn((N, C), generator=gen).to(torch.bfloat16).to(device)
    w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
    before = _cabi.set_resident(True)
    try:
        want = [cabi_fwd_add(x, r_, c_, w, b, G, 1e-5, 2) for r_, c_ in ((res, cb), (res, None), (None, cb))]
        torch.cuda.synchronize()
        prev = lib.gnnhwc_debug_set_spin_limit(-2)
        try:
            lib.gnnhwc_resident_status()
            got = [cabi_fwd_add(x, r_, c_, w, b, G, 1e-5, 2) for r_, c_ in ((res, cb), (res, None), (None, cb))]
            torch.cuda.synchronize()
            assert lib.gnnhwc_resident_status() == 1
        finally:
            lib.gnnhwc_debug_set_spin_limit(prev)
        for (y0, s0, m0, r0), (y1, s1, m1, r1) in zip(want, got):
            assert torch.equal(s0, s1)  # the sum is formed the same way, bit for bit
            assert err(m1, m0) <= 1e-5 and err(r1, r0) <= 1e-5
            # y: the two paths may differ by a rounding of the statistics, i.e. by one bf16 spacing on few elements
            assert err(y1, y0) <= 2.0 ** -7
            assert float((y1.float() != y0.float()).float().mean()) < 0.02
    finally:
        lib.gnnhwc_resident_status()
        _cabi.set_resident(before)


@pytest.mark.parametrize("shape,G", [((2, 64, 23, 19), 8), ((1, 1280, 64, 64), 32), ((5, 320, 128, 128), 32),
                                     ((7, 320, 128, 128), 32)])
def test_hip_graph_replay(family, shape, G, device):
    """Forward + backward recorded into a HIP graph through the C ABI and replayed several times, with eager calls
    on the same workspaces and synchronisations in between; every replay must reproduce the eager result bit for bit
    (the backward of the 5-sample shape is the single-launch form that keeps g' and streams x twice; the 7-sample shape
    runs as two single-launch kernels over groups of samples)."""
    gen = torch.Generator().manual_seed(21)
    N, C = shape[0], shape[1]
    x = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen, 1.5, 0.3))
    dy = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen))
    w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
    lib = _cabi.lib
    R = x.shape[1]
    ws_f = torch.empty((lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, 3),), dtype=torch.uint8, device=device)
    ws_b = torch.empty((lib.gnnhwc_bwd_workspace_bytes(N, R, C, G, 3),), dtype=torch.uint8, device=device)
    y = torch.empty_like(x)
    dx = torch.empty_like(x)

    def step():
        _, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, 2, y=y, ws=ws_f)
        _, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, 2, dx=dx, ws=ws_b)
        return mean, rstd, dw, db

    mean, rstd, dw, db = step()
    torch.cuda.synchronize()
    want = [t.clone() for t in (y, dx, mean, rstd, dw, db)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        mean_g, rstd_g, dw_g, db_g = step()
    for rep in range(4):
        for t in (y, dx, mean_g, rstd_g, dw_g, db_g):
            t.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("y", "dx", "mean", "rstd", "dw", "db"), (y, dx, mean_g, rstd_g, dw_g, db_g), want):
            assert torch.equal(got, ref), "replay %d: %s differs from the eager result" % (rep, name)
        step()  # eager work on the same workspaces between replays
        torch.cuda.synchronize()


@pytest.mark.gpu
def test_hip_graphs_share_a_workspace(device):
    """Captured single-launch kernels take their epoch from a per-replay generation and a per-launch sequence
    number.  Two launches of the same shape on ONE workspace inside one graph (different inputs), and two graphs
    that share that workspace and are replayed alternately with eager calls in between, must each reproduce the
    eager results bit for bit: a launch that mistook another launch's records for its own would normalise with
    the wrong statistics."""
    gen = torch.Generator().manual_seed(33)
    shape, G = (2, 320, 32, 32), 32
    N, C = shape[0], shape[1]
    xs = [nrc_view(channels_last_like(shape, torch.bfloat16, device, gen, 1.0 + i, 0.5 * i)) for i in range(3)]
    dy = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen))
    w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
    b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
    lib = _cabi.lib
    R = xs[0].shape[1]
    nbytes = max(lib.gnnhwc_fwd_workspace_bytes(N, R, C, G, 3), lib.gnnhwc_bwd_workspace_bytes(N, R, C, G, 3))
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=device)
    ys = [torch.empty_like(xs[0]) for _ in xs]
    dx = torch.empty_like(xs[0])

    def step_a():  # two forwards of the same shape on the same workspace, then a backward on it
        _, m0, r0 = cabi_fwd(xs[0], w, b, G, 1e-5, 2, y=ys[0], ws=ws)
        _, m1, r1 = cabi_fwd(xs[1], w, b, G, 1e-5, 2, y=ys[1], ws=ws)
        _, dw, db = cabi_bwd(dy, xs[1], w, b, m1, r1, G, 2, dx=dx, ws=ws)
        return m0, r0, m1, r1, dw, db

    def step_b():
        _, m2, r2 = cabi_fwd(xs[2], w, b, G, 1e-5, 2, y=ys[2], ws=ws)
        return m2, r2

    outs_a = step_a()
    outs_b = step_b()
    torch.cuda.synchronize()
    want_a = [t.clone() for t in (ys[0], ys[1], dx) + tuple(outs_a)]
    want_b = [t.clone() for t in (ys[2],) + tuple(outs_b)]
    assert not torch.equal(want_a[0], want_a[1])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step_a()
        step_b()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ga, gb = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(ga):
        got_a = step_a()
    with torch.cuda.graph(gb):
        got_b = step_b()
    for rep in range(3):
        for t in ys + [dx] + list(got_a) + list(got_b):
            t.fill_(float("nan"))
        ga.replay()
        gb.replay()
        if rep == 1:
            ga.replay()  # the same graph twice in a row
        torch.cuda.synchronize()
        for i, (got, ref) in enumerate(zip((ys[0], ys[1], dx) + tuple(got_a), want_a)):
            assert torch.equal(got, ref), "replay %d: output %d of the first graph differs from the eager result" % (rep, i)
        for i, (got, ref) in enumerate(zip((ys[2],) + tuple(got_b), want_b)):
            assert torch.equal(got, ref), "replay %d: output %d of the second graph differs from the eager result" % (rep, i)
        step_b()  # eager work on the same workspace between replays
        torch.cuda.synchronize()



@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_functional_form_traces_into_one_graph(dtype, device):
    """group_norm_nhwc under torch.compile (fullgraph, so any graph break fails; the 'aot_eager' backend traces
    forward and backward with fake tensors and then runs the traced graphs, i.e. the HIP operators): outputs and
    all three gradients equal the module's bit for bit (same kernels, same inputs)."""
    from gnnhwc import group_norm_nhwc

    gen = torch.Generator().manual_seed(5)
    shape, G = (2, 64, 24, 24), 8
    x0 = channels_last_like(shape, dtype, device, gen, 1.3, 0.2)
    dy = channels_last_like(shape, dtype, device, gen)
    m = GN_NHWC(G, shape[1], activation="silu").to(device=device, dtype=dtype)
    with torch.no_grad():
        m.weight.copy_((torch.rand(shape[1], generator=gen) + 0.5).to(dtype))
        m.bias.copy_((0.1 * torch.randn(shape[1], generator=gen)).to(dtype))
    x = x0.clone().requires_grad_()
    y = m(x)
    gx, gw, gb = torch.autograd.grad(y, (x, m.weight, m.bias), dy)

    def fn(t, w, b):
        return group_norm_nhwc(t * 1.0, w, b, G, m.eps, "silu")

    compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
    x2 = x0.clone().requires_grad_()
    w2 = m.weight.detach().clone().requires_grad_()
    b2 = m.bias.detach().clone().requires_grad_()
    y2 = compiled(x2, w2, b2)
    assert y2.stride() == y.stride()
    gx2, gw2, gb2 = torch.autograd.grad(y2, (x2, w2, b2), dy)
    assert torch.equal(y2, y) and torch.equal(gx2, gx) and torch.equal(gw2, gw) and torch.equal(gb2, gb)


@pytest.mark.gpu
def test_non_affine_module_materialises_no_parameters(device, monkeypatch):
    """affine=False: the reference fills a ones and a zeros tensor on every call (custom_gn.py:83-86); here the absent
    parameters reach the kernels as NULL.  Same bits as the affine module with weight 1 and bias 0, no parameter
    gradients, and no call of torch.ones / torch.zeros during forward or backward."""
    gen = torch.Generator().manual_seed(9)
    for shape, layout in (((2, 48, 9, 9), "last"), ((2, 48, 9, 9), "first")):
        x = channels_last_like(shape, torch.bfloat16, device, gen, 1.5, 0.2)
        dy = channels_last_like(shape, torch.bfloat16, device, gen)
        if layout == "first":
            x, dy = x.contiguous(), dy.contiguous()
        m_ref = GN_NHWC(6, 48, activation="gelu").to(device).to(torch.bfloat16)
        m = GN_NHWC(6, 48, activation="gelu", affine=False).to(device).to(torch.bfloat16)
        xr = x.clone().requires_grad_(True)
        want = m_ref(xr)
        want.backward(dy)

        def forbidden(*a, **k):
            raise AssertionError("a ones / zeros tensor was materialised")

        xa = x.clone().requires_grad_(True)
        with monkeypatch.context() as mp:
            mp.setattr(torch, "ones", forbidden)
            mp.setattr(torch, "zeros", forbidden)
            got = m(xa)
            got.backward(dy)
        assert torch.equal(got, want) and torch.equal(xa.grad, xr.grad)
        assert m.weight is None and m.bias is None


@pytest.mark.gpu
@pytest.mark.parametrize("xdtype", [torch.bfloat16, torch.float16])
def test_module_with_float32_parameters_and_16_bit_input(family, xdtype, device):
    """The autocast / AMP case the reference cannot run (it reads weight as the data type, custom_gn.cpp:35-36): a module
    whose parameters stay float32 while x arrives in a 16-bit type, with and without torch.autocast around the call.
    y and dx come back in x's type, dweight / dbias in float32.  Truth: the float64 oracle on the same values; y / dx
    within half a spacing of the 16-bit type of it (one rounding of a float32-accurate value), dweight / dbias to the
    float32 bar scaled by the 16-bit rounding of dy * act' that autograd's own chain would apply too."""
    gen = torch.Generator().manual_seed(31)
    shape, G = (2, 64, 20, 12), 8
    x = channels_last_like(shape, xdtype, device, gen, 1.7, 0.4)
    dy = channels_last_like(shape, xdtype, device, gen)
    m = GN_NHWC(G, shape[1], activation="silu").to(device)  # float32 parameters
    with torch.no_grad():
        m.weight.copy_(torch.rand(shape[1], generator=gen) + 0.5)
        m.bias.copy_(0.1 * torch.randn(shape[1], generator=gen))
    truth = orc.fwd_bwd(orc.to_nrc(x), m.weight.detach().double().cpu().numpy(), m.bias.detach().double().cpu().numpy(),
                        orc.to_nrc(dy), G, m.eps, orc.ACT_CODES["silu"])
    half = 2.0 ** -8 if xdtype == torch.bfloat16 else 2.0 ** -11

    def close_16(got, want):
        t = torch.as_tensor(want)
        d = (torch.as_tensor(orc.to_nrc(got)) - t).abs()
        return bool((d <= half * 1.001 * t.abs() + 1e-5 * (t.abs() + float(t.square().mean().sqrt())) + 2.0 ** -24).all())

    for use_autocast in (False, True):
        m.zero_grad()
        xr = x.clone().requires_grad_(True)
        if use_autocast:
            with torch.autocast(device_type="cuda", dtype=xdtype):
                y = m(xr)
        else:
            y = m(xr)
        y.backward(dy)
        assert y.dtype == xdtype and xr.grad.dtype == xdtype
        assert m.weight.grad.dtype == torch.float32 and m.bias.grad.dtype == torch.float32
        assert close_16(y, truth["y"]), "y (autocast=%s)" % use_autocast
        # dx carries one more 16-bit rounding: the single-launch backward keeps dy * act'(z) in x's type between its two
        # phases (the rounding an unfused activation backward applies to the same quantity)
        assert err(xr.grad, orc.from_nrc(truth["dx"], shape)) <= 3 * half, "dx (autocast=%s)" % use_autocast
        assert err(m.weight.grad, truth["dw"]) <= 1e-5 and err(m.bias.grad, truth["db"]) <= 1e-5


class _Block(nn.Module):
    """A layer either side of the norm, so that a compiled graph has something of its own to fuse around the operator
    (scalings by powers of two: exact in any type and any evaluation order)."""

    def __init__(self, G, C, act, affine=True):
        super().__init__()
        self.norm = GN_NHWC(G, C, activation=act, affine=affine)

    def forward(self, x):
        return self.norm(x * 2.0) * 0.5


@pytest.mark.gpu
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_model_with_the_module_compiles_whole(backend, device):
    """torch.compile of a model that contains GN_NHWC itself (the reference's forward is a guaranteed graph break,
    custom_gn.py:63): fullgraph=True, so a break is an error; with the default backend (inductor) and with the tracing
    one.  Outputs and all gradients equal the eager module's bit for bit, for channels-last and channels-first input,
    with and without parameters."""
    gen = torch.Generator().manual_seed(17)
    shape, G = (2, 64, 16, 16), 8
    for dtype, layout, affine in ((torch.float32, "last", True), (torch.bfloat16, "last", True),
                                  (torch.bfloat16, "first", True), (torch.float32, "last", False)):
        x0 = channels_last_like(shape, dtype, device, gen, 1.3, 0.2)
        dy = channels_last_like(shape, dtype, device, gen)
        if layout == "first":
            x0, dy = x0.contiguous(), dy.contiguous()
        model = _Block(G, shape[1], "silu", affine).to(device=device, dtype=dtype)
        if affine:
            with torch.no_grad():
                model.norm.weight.copy_((torch.rand(shape[1], generator=gen) + 0.5).to(dtype))
                model.norm.bias.copy_((0.1 * torch.randn(shape[1], generator=gen)).to(dtype))
        params = list(model.parameters())
        x = x0.clone().requires_grad_()
        y = model(x)
        want = torch.autograd.grad(y, [x] + params, dy)
        torch._dynamo.reset()
        compiled = torch.compile(model, backend=backend, fullgraph=True)
        x2 = x0.clone().requires_grad_()
        y2 = compiled(x2)
        got = torch.autograd.grad(y2, [x2] + params, dy)
        assert torch.equal(y2, y), (backend, dtype, layout, affine)
        for g, w in zip(got, want):
            assert torch.equal(g, w), (backend, dtype, layout, affine)


@pytest.mark.gpu
def test_two_streams_take_turns(device):
    """Single-launch kernels issued on two streams with no host synchronisation in between: the library orders each
    behind the previous one on the other stream (each needs the whole device to itself), so every call reproduces
    the result of the same call made alone, and no call has to fall back on its recovery path."""
    lib = _cabi.lib
    gen = torch.Generator().manual_seed(44)
    cases = []
    for shape, G in (((1, 640, 64, 64), 32), ((2, 320, 64, 64), 32)):
        C = shape[1]
        x = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen, 1.5, 0.3))
        dy = nrc_view(channels_last_like(shape, torch.bfloat16, device, gen))
        w = (torch.rand(C, generator=gen) + 0.5).to(torch.bfloat16).to(device)
        b = (0.1 * torch.randn(C, generator=gen)).to(torch.bfloat16).to(device)
        cases.append((x, dy, w, b, G))

    def step(case):
        x, dy, w, b, G = case
        y, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, 2)
        dx, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, 2)
        return y, mean, rstd, dx, dw, db

    before = _cabi.set_resident(True)
    prev = lib.gnnhwc_debug_set_spin_limit(-1)  # the default
    lib.gnnhwc_resident_status()
    try:
        want = [step(c) for c in cases]
        torch.cuda.synchronize()
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        got = []
        for it in range(40):
            for s, c in zip(streams, cases):
                with torch.cuda.stream(s):
                    got.append(step(c))
        torch.cuda.synchronize()
        for i, out in enumerate(got):
            for a, ref in zip(out, want[i % 2]):
                assert torch.equal(a, ref), "call %d differs from the same call made alone" % i
        assert lib.gnnhwc_resident_status() == 0  # no call had to take the recovery path
    finally:
        lib.gnnhwc_debug_set_spin_limit(prev)
        _cabi.set_resident(before)


def _device_err(a, truth):
    """err() of the harness, evaluated on the device (for tensors too large to bring to the host)."""
    a = a.reshape(-1).double()
    t = truth.reshape(-1).double()
    rms = float(t.square().mean().sqrt()) or 1.0
    return float(((a - t).abs() / (t.abs() + rms)).max())


@pytest.mark.gpu
def test_more_than_two_to_the_31_elements(device):
    """(5, 2048 * 2048, 128) bf16 holds 2.7e9 elements: element offsets of the last two samples do not fit 32 bits
    (the reference indexes with int, gn_kernel.cu:21, and overflows here).  Statistics are per sample, so each
    checked sample must agree with the same sample run alone (a tensor whose offsets are small) and with float64
    statistics computed by torch on the device; dgamma / dbeta must be the sum of the single-sample results, and
    dx must sum to zero over every (sample, group) slab."""
    N, R, C, G = 5, 2048 * 2048, 128, 32
    D = C // G
    assert N * R * C > 2 ** 31
    gen = torch.Generator(device=device).manual_seed(7)
    x = torch.empty((N, R, C), dtype=torch.bfloat16, device=device)
    dy = torch.empty((N, R, C), dtype=torch.bfloat16, device=device)
    for n in range(N):
        x[n] = (torch.randn((R, C), generator=gen, device=device) * (1.0 + 0.5 * n) + 0.3 * n).to(torch.bfloat16)
        dy[n] = torch.randn((R, C), generator=gen, device=device).to(torch.bfloat16)
    w = (torch.rand(C, generator=gen, device=device) + 0.5).to(torch.bfloat16)
    b = (0.1 * torch.randn(C, generator=gen, device=device)).to(torch.bfloat16)
    y, mean, rstd = cabi_fwd(x, w, b, G, 1e-5, 2)
    dx, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, 2)
    torch.cuda.synchronize()
    dw_sum = torch.zeros(C, dtype=torch.float64, device=device)
    db_sum = torch.zeros(C, dtype=torch.float64, device=device)
    for n in range(N):
        xs, dys = x[n:n + 1], dy[n:n + 1]
        y1, m1, r1 = cabi_fwd(xs, w, b, G, 1e-5, 2)
        # dgamma / dbeta of one sample in float32, so that their sum can be compared with the bf16 result
        dx1, dw1, db1 = cabi_bwd(dys, xs, w.float(), b.float(), m1, r1, G, 2)
        dw_sum += dw1.double()
        db_sum += db1.double()
        if n in (0, N - 2, N - 1):
            xd = xs.double().view(R, G, D)
            mu = xd.mean(dim=(0, 2))
            var = xd.var(dim=(0, 2), correction=0)
            del xd
            assert _device_err(mean[n], mu) <= 1e-5 and _device_err(rstd[n], (var + 1e-5).rsqrt()) <= 1e-5
            assert _device_err(mean[n], m1[0]) <= 1e-5 and _device_err(rstd[n], r1[0]) <= 1e-5
            assert _device_err(y[n], y1[0]) <= 2.0 ** -7, "sample %d: y differs from the sample run alone" % n
            assert _device_err(dx[n], dx1[0]) <= 2.0 ** -6, "sample %d: dx differs from the sample run alone" % n
            slab = dx[n].double().view(R, G, D)
            total = slab.sum(dim=(0, 2)).abs().max()
            scale = slab.abs().sum(dim=(0, 2)).max()
            del slab
            # every element of dx carries a bf16 rounding error of relative size 2^-9 with random sign
            assert float(total) <= float(scale) * 2.0 ** -9 * 8 / (R * D) ** 0.5
    assert _device_err(dw, dw_sum) <= 2.0 ** -7 and _device_err(db, db_sum) <= 2.0 ** -7


@pytest.mark.gpu
def test_module_on_two_streams(device):
    """The Python surface keeps one scratch buffer per (device, stream): the same module called on two torch streams
    with no synchronisation in between gives, on each, the results of the same calls made alone."""
    gen = torch.Generator().manual_seed(91)
    m = GN_NHWC(32, 640, activation="silu").to(device=device, dtype=torch.bfloat16)
    with torch.no_grad():
        m.weight.copy_((torch.rand(640, generator=gen) + 0.5).to(torch.bfloat16))
        m.bias.copy_((0.1 * torch.randn(640, generator=gen)).to(torch.bfloat16))
    xs = [channels_last_like((1, 640, 48, 48), torch.bfloat16, device, gen, 1.0 + i, 0.3 * i) for i in range(2)]
    with torch.no_grad():
        want = [m(x).clone() for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[], []]
    with torch.no_grad():
        for _ in range(25):
            for i, s in enumerate(streams):
                with torch.cuda.stream(s):
                    got[i].append(m(xs[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for y in got[i]:
            assert torch.equal(y, want[i])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape,G", [((2, 64, 24, 24), 8), ((1, 96, 7, 9, 5), 12), ((3, 30, 50), 5)])
def test_channels_first_module_against_torch(shape, G, dtype, device):
    """Contiguous channels-first input of any rank >= 3 through the module: output contiguous with x's shape, values
    and all gradients those of torch's GroupNorm + activation (float64 truth; bars of the channels-last path)."""
    gen = torch.Generator().manual_seed(13)
    x0 = (torch.randn(shape, generator=gen) * 1.4 + 0.2).to(dtype).to(device)
    dy = torch.randn(shape, generator=gen).to(dtype).to(device)
    for act in ("silu", "gelu", "relu"):
        m = GN_NHWC(G, shape[1], activation=act).to(device=device, dtype=dtype)
        with torch.no_grad():
            m.weight.copy_((torch.rand(shape[1], generator=gen) + 0.5).to(dtype))
            m.bias.copy_((0.1 * torch.randn(shape[1], generator=gen)).to(dtype))
        x = x0.clone().requires_grad_()
        y = m(x)
        assert y.shape == x.shape and y.is_contiguous() and y.dtype == dtype
        gx, gw, gb = torch.autograd.grad(y, (x, m.weight, m.bias), dy)
        xt = x0.double().requires_grad_()
        wt, bt = m.weight.detach().double().requires_grad_(), m.bias.detach().double().requires_grad_()
        yt = orc.torch_act(act)(F.group_norm(xt, G, wt, bt, m.eps))
        tx, tw, tb = torch.autograd.grad(yt, (xt, wt, bt), dy.double())
        tol = 1e-5 if dtype == torch.float32 else 2.0 ** -6
        assert err(y, yt) <= tol and err(gw, tw) <= tol * 4 and err(gb, tb) <= tol * 4
        if act != "relu":
            assert err(gx, tx) <= tol

