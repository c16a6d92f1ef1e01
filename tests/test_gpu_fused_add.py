"""GPU parity of gnnhwc_fwd_add (the forward with its preceding additions fused in), through the C ABI.

Contract: the normalised tensor is s = round_T((x + residual) + channel_bias[n][c]) with fp32 (fp64) arithmetic.
  * sum_out must equal that expression evaluated by torch, bit for bit (an addition and one rounding leave no
    freedom);
  * y, mean, rstd must meet the bars of the plain forward against the CPU oracle (oracle/gn_oracle.c, float64)
    applied to s: fp32 1e-5, fp64 1e-12, fp16/bf16 no worse than the plain kernel on the same s (+2 %).
"""
import numpy as np
import pytest
import torch

from oracle import gn_oracle as orc
from tests.gpu_harness import as_np64, cabi_bwd, cabi_fwd, cabi_fwd_add, err

pytestmark = pytest.mark.gpu

EPS = 1e-5
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}


def _inputs(shape_nrc, dtype, device, seed):
    gen = torch.Generator().manual_seed(seed)
    N, R, C = shape_nrc
    x = (torch.randn((N, R, C), generator=gen) * 1.5 + 0.3).to(dtype).to(device)
    r = (torch.randn((N, R, C), generator=gen) * 0.7 - 0.2).to(dtype).to(device)
    t = torch.randn((N, C), generator=gen).to(dtype).to(device)
    w = (torch.rand((C,), generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn((C,), generator=gen)).to(dtype).to(device)
    return x, r, t, w, b


def _expected_sum(x, r, t):
    wide = torch.float64 if x.dtype == torch.float64 else torch.float32
    s = x.to(wide)
    if r is not None:
        s = s + r.to(wide)
    if t is not None:
        s = s + t.to(wide)[:, None, :]
    return s.to(x.dtype)


def _check_against_oracle(y, mean, rstd, s, w, b, G, act, dtype):
    truth = orc.fwd_bwd(as_np64(s), as_np64(w), as_np64(b), np.zeros(tuple(s.shape)), G, EPS, act)
    stat_tol = 1e-12 if dtype == torch.float64 else 1e-5
    assert err(mean, truth["mean"]) <= stat_tol and err(rstd, truth["rstd"]) <= stat_tol
    e = err(y, truth["y"])
    if dtype in TOL:
        assert e <= TOL[dtype], "y: err %.3g" % e
    else:
        y_plain, _, _ = cabi_fwd(s, w, b, G, EPS, act)
        torch.cuda.synchronize()
        e_plain = err(y_plain, truth["y"])
        assert e <= e_plain * 1.02 + 1e-12, "y: err %.3g vs the plain forward's %.3g on the same sum" % (e, e_plain)


SHAPES = [
    ((2, 64, 64), 8),       # small, single-launch
    ((1, 4096, 320), 32),   # SD-UNet-like
    ((3, 37 * 53, 96), 24),  # odd number of rows
    ((2, 35, 60), 6),       # C not a multiple of the vector width for 16-bit types
    ((5, 16384, 320), 32),  # too large for one launch: the multi-launch form
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("mode", ["residual", "channel_bias", "both"])
@pytest.mark.parametrize("shape,G", SHAPES)
def test_fused_add_parity(family, shape, G, mode, dtype, device):
    if shape[0] * shape[1] * shape[2] > 2 ** 24 and (dtype == torch.float64 or mode != "both"):
        pytest.skip("the large shape is run once per 16/32-bit type")
    print("fwd_add", family, shape, G, mode, dtype, flush=True)
    x, r, t, w, b = _inputs(shape, dtype, device, 100 + shape[1] % 97)
    r = r if mode in ("residual", "both") else None
    t = t if mode in ("channel_bias", "both") else None
    act = 2
    y, s, mean, rstd = cabi_fwd_add(x, r, t, w, b, G, EPS, act)
    torch.cuda.synchronize()
    want = _expected_sum(x, r, t)
    assert torch.equal(s, want), "sum_out differs from x + residual + channel_bias rounded once"
    if shape[0] * shape[1] * shape[2] <= 2 ** 24:
        _check_against_oracle(y, mean, rstd, want, w, b, G, act, dtype)
    else:  # the oracle would take minutes: the plain forward (itself checked against the oracle) on the same sum
        y2, mean2, rstd2 = cabi_fwd(want, w, b, G, EPS, act)
        torch.cuda.synchronize()
        assert err(mean, mean2) <= 1e-5 and err(rstd, rstd2) <= 1e-5
        assert err(y, y2) <= (1e-5 if dtype == torch.float32 else 2.0 ** -7)
    # without sum_out the results are the same bits
    y3, none, mean3, rstd3 = cabi_fwd_add(x, r, t, w, b, G, EPS, act, want_sum=False)
    torch.cuda.synchronize()
    assert none is None and torch.equal(y3, y) and torch.equal(mean3, mean) and torch.equal(rstd3, rstd)


@pytest.mark.parametrize("act", [0, 1, 3, 4])
def test_fused_add_other_activations(family, act, device):
    x, r, t, w, b = _inputs((2, 300, 128), torch.float32, device, 7)
    y, s, mean, rstd = cabi_fwd_add(x, r, t, w, b, 16, EPS, act)
    torch.cuda.synchronize()
    want = _expected_sum(x, r, t)
    assert torch.equal(s, want)
    _check_against_oracle(y, mean, rstd, want, w, b, 16, act, torch.float32)


def test_fused_add_in_place_and_mixed_types(family, device):
    """sum_out may be x itself (h += r), y may be the residual's buffer, channel_bias may be fp32 next to bf16 data
    and fp32 parameters; NULL weight / bias and NULL statistics outputs are accepted as in the plain forward."""
    from gnnhwc import _cabi
    import ctypes

    x, r, t, w, b = _inputs((2, 1024, 256), torch.bfloat16, device, 9)
    t32 = torch.randn((2, 256), generator=torch.Generator().manual_seed(3)).to(device)
    want = _expected_sum(x, r, t32)
    y_ref, s_ref, mean_ref, rstd_ref = cabi_fwd_add(x, r, t32, w.float(), b.float(), 32, EPS, 2)
    torch.cuda.synchronize()
    assert torch.equal(s_ref, want)
    _check_against_oracle(y_ref, mean_ref, rstd_ref, want, w.float(), b.float(), 32, 2, torch.bfloat16)
    xs, rs = x.clone(), r.clone()
    y2, s2, mean2, rstd2 = cabi_fwd_add(xs, rs, t32, w.float(), b.float(), 32, EPS, 2, sum_out=xs, y=rs)
    torch.cuda.synchronize()
    assert s2.data_ptr() == xs.data_ptr() and torch.equal(xs, want) and torch.equal(rs, y_ref)
    assert torch.equal(mean2, mean_ref) and torch.equal(rstd2, rstd_ref)
    # no affine parameters, no statistics outputs
    lib = _cabi.lib
    N, R, C = x.shape
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, 32, 3)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=device)
    y4 = torch.empty_like(x)
    vp = lambda v: ctypes.c_void_p(v.data_ptr())  # noqa: E731
    rc = lib.gnnhwc_fwd_add(vp(x), vp(r), None, None, None, None, vp(y4), None, None, N, R, C, 32, EPS, 0, 3, 3, 0, 3,
                            vp(ws), nbytes, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _cabi.last_error()
    torch.cuda.synchronize()
    s4 = _expected_sum(x, r, None)
    truth = orc.fwd_bwd(as_np64(s4), np.ones(C), np.zeros(C), np.zeros((N, R, C)), 32, EPS, 0)
    y_plain, _, _ = cabi_fwd(s4, None, None, 32, EPS, 0)
    torch.cuda.synchronize()
    assert err(y4, truth["y"]) <= err(y_plain, truth["y"]) * 1.02


def test_fused_add_rejects_bad_arguments(device):
    from gnnhwc import _cabi
    import ctypes

    lib = _cabi.lib
    x, r, t, w, b = _inputs((1, 64, 64), torch.bfloat16, device, 1)
    N, R, C = x.shape
    nbytes = lib.gnnhwc_fwd_workspace_bytes(N, R, C, 8, 3)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=device)
    y = torch.empty_like(x)
    vp = lambda v: ctypes.c_void_p(v.data_ptr())  # noqa: E731
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # sum_out == y
    assert lib.gnnhwc_fwd_add(vp(x), vp(r), None, vp(y), vp(w), vp(b), vp(y), None, None, N, R, C, 8, EPS, 2, 3, 3, 0, 3,
                              vp(ws), nbytes, st) == -1
    assert "sum_out" in _cabi.last_error()
    # fp16 channel bias next to bf16 data
    assert lib.gnnhwc_fwd_add(vp(x), None, vp(t), None, vp(w), vp(b), vp(y), None, None, N, R, C, 8, EPS, 2, 3, 3, 0, 2,
                              vp(ws), nbytes, st) == -1
    assert "channel_bias_dtype" in _cabi.last_error()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_functional_form_with_additions_and_gradients(dtype, device):
    """group_norm_nhwc(residual=, channel_bias=, return_sum=True): forward equals the unfused torch expression's
    sum bit for bit and its normalisation within the forward bar; gradients of x, residual, channel_bias, weight,
    bias equal those of the unfused form built from the same operator (gnop::fwd on the explicit sum)."""
    from gnnhwc import group_norm_nhwc

    gen = torch.Generator().manual_seed(77)
    N, C, H, W, G = 2, 64, 12, 20, 8

    def cl(*shape):
        return torch.randn(shape, generator=gen).to(dtype).to(device)

    x0 = cl(N, H, W, C).permute(0, 3, 1, 2)
    r0 = cl(N, H, W, C).permute(0, 3, 1, 2)
    t0 = cl(N, C)
    w0 = (torch.rand(C, generator=gen) + 0.5).to(dtype).to(device)
    b0 = cl(C)
    dy = cl(N, H, W, C).permute(0, 3, 1, 2)
    ds = cl(N, H, W, C).permute(0, 3, 1, 2)

    leaves = [v.clone().requires_grad_() for v in (x0, r0, t0, w0, b0)]
    y, s = group_norm_nhwc(leaves[0], leaves[3], leaves[4], G, EPS, "silu", residual=leaves[1], channel_bias=leaves[2],
                           return_sum=True)
    grads = torch.autograd.grad((y, s), leaves, (dy, ds))

    leaves2 = [v.clone().requires_grad_() for v in (x0, r0, t0, w0, b0)]
    wide = torch.float32
    s2 = ((leaves2[0].to(wide) + leaves2[1].to(wide)) + leaves2[2].to(wide)[:, :, None, None]).to(dtype)
    y2 = group_norm_nhwc(s2, leaves2[3], leaves2[4], G, EPS, "silu")
    grads2 = torch.autograd.grad((y2, s2), leaves2, (dy, ds))
    assert torch.equal(s, s2)
    assert err(y, y2) <= (1e-5 if dtype == torch.float32 else 2.0 ** -7)
    for name, g, g2 in zip(("x", "residual", "channel_bias", "weight", "bias"), grads, grads2):
        assert g.shape == g2.shape and g.dtype == g2.dtype
        assert err(g, g2) <= (2e-5 if dtype == torch.float32 else 2.0 ** -6), name
    # only a channel bias, sum not returned: the backward rebuilds the sum
    leaves3 = [v.clone().requires_grad_() for v in (x0, t0, w0, b0)]
    y3 = group_norm_nhwc(leaves3[0], leaves3[2], leaves3[3], G, EPS, "silu", channel_bias=leaves3[1])
    g3 = torch.autograd.grad(y3, leaves3, dy)
    leaves4 = [v.clone().requires_grad_() for v in (x0, t0, w0, b0)]
    s4 = (leaves4[0].to(wide) + leaves4[1].to(wide)[:, :, None, None]).to(dtype)
    y4 = group_norm_nhwc(s4, leaves4[2], leaves4[3], G, EPS, "silu")
    g4 = torch.autograd.grad(y4, leaves4, dy)
    assert err(y3, y4) <= (1e-5 if dtype == torch.float32 else 2.0 ** -7)
    for g, g2 in zip(g3, g4):
        assert err(g, g2) <= (2e-5 if dtype == torch.float32 else 2.0 ** -6)
