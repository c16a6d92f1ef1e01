"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle (oracle/gn_oracle.c in float64)
and against torch's own GroupNorm + activation on the same seeded inputs.

Tolerances (the build's stated bar):
  fp32 / fp64 : err <= 1e-5 (fp64: 1e-12), with err = max |ours - truth| / (|truth| + rms(truth)), AND the pure relative
                error max |ours - truth| / |truth| over the elements with |truth| >= rms(truth) within the same bound;
  fp16 / bf16 : err(ours vs float64 truth) <= err(torch's own fp16/bf16 GroupNorm+activation vs the same truth)
                times (1 + HALF_SLACK) -- i.e. no worse than the library routine's own half-precision error.
relu's derivative is discontinuous at 0: dx elements whose pre-activation is within RELU_BAND of 0 are
left out of the element-wise comparison (they may legitimately land on either side).
"""
import re

import numpy as np
import pytest
import torch

from oracle import gn_oracle as orc
from tests import configs
from gnnhwc import _cabi
from tests.gpu_harness import as_np64, cabi_bwd, cabi_fwd, err, nrc_view, record_errors, rel_err

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
FP64_TOL = 1e-12
HALF_SLACK = 0.02
RELU_BAND = 1e-4
EPS = 1e-5


def _truth(inp, G, act_code):
    x = as_np64(nrc_view(inp["x"]))
    dy = as_np64(nrc_view(inp["dy"]))
    return orc.fwd_bwd(x, as_np64(inp["w"]), as_np64(inp["b"]), dy, G, EPS, act_code)


def _torch_same_dtype(inp, G, act):
    """torch's GroupNorm + activation + autograd on the device, in the inputs' own dtype."""
    r = orc.torch_reference(inp["x"], inp["w"], inp["b"], G, EPS, act, inp["dy"])
    return {"y": as_np64(nrc_view(r["y"])), "dx": as_np64(nrc_view(r["dx"])), "dw": as_np64(r["dw"]), "db": as_np64(r["db"])}


def _relu_mask(inp, truth, G):
    x = as_np64(nrc_view(inp["x"]))
    N, R, C = x.shape
    D = C // G
    a = np.repeat(truth["rstd"], D, axis=1) * as_np64(inp["w"])[None, :]
    b = as_np64(inp["b"])[None, :] - np.repeat(truth["mean"], D, axis=1) * a
    z = x * a[:, None, :] + b[:, None, :]
    return np.abs(z) > RELU_BAND


def _check(name, ours, truth, lib_result, dtype, mask=None, log=None):
    """Asserts the bars and returns the observed err.  log: a dict the observed figures are added to, under `name`."""
    o, t = as_np64(ours) if isinstance(ours, torch.Tensor) else ours, truth
    if mask is not None:
        o, t = np.where(mask, o, 0.0), np.where(mask, t, 0.0)
    e = err(o, t)
    r = rel_err(o, t)
    bar = None
    if dtype == torch.float32:
        bar = FP32_TOL
        assert e <= FP32_TOL, "%s: err %.3g > %.1g" % (name, e, FP32_TOL)
        assert r <= FP32_TOL, "%s: relative error %.3g > %.1g" % (name, r, FP32_TOL)
    elif dtype == torch.float64:
        bar = FP64_TOL
        assert e <= FP64_TOL, "%s: err %.3g > %.1g" % (name, e, FP64_TOL)
        assert r <= FP64_TOL, "%s: relative error %.3g > %.1g" % (name, r, FP64_TOL)
    else:
        l = lib_result if mask is None else np.where(mask, lib_result, 0.0)
        e_lib = err(l, t)
        bar = e_lib * (1 + HALF_SLACK)
        assert e <= bar, "%s: err %.3g vs torch's own %s error %.3g" % (name, e, dtype, e_lib)
    if log is not None:
        log[name] = {"err": e, "rel": r, "bar": bar}
    return e


@pytest.mark.parametrize("name", configs.ALL_NAMES)
def test_config_parity(family, name, device):
    cfg = configs.CONFIGS[name]
    print("config", name, cfg, flush=True)
    inp = configs.make_inputs(cfg, device)
    act = orc.ACT_CODES[cfg.act]
    dtype = configs.DT[cfg.dtype]
    x, dy = nrc_view(inp["x"]), nrc_view(inp["dy"])
    truth = _truth(inp, cfg.G, act)
    lib = _torch_same_dtype(inp, cfg.G, cfg.act) if dtype in (torch.float16, torch.bfloat16) else None
    y, mean, rstd = cabi_fwd(x, inp["w"], inp["b"], cfg.G, EPS, act)
    torch.cuda.synchronize()
    log = {}
    _check("mean", mean, truth["mean"], None, torch.float32 if dtype != torch.float64 else dtype, log=log)
    _check("rstd", rstd, truth["rstd"], None, torch.float32 if dtype != torch.float64 else dtype, log=log)
    _check("y", y, truth["y"], lib and lib["y"], dtype, log=log)
    if cfg.passes == "fwd":
        record_errors(config=name, family=family, dtype=cfg.dtype, observed=log)
        return
    dx, dw, db = cabi_bwd(dy, x, inp["w"], inp["b"], mean, rstd, cfg.G, act)
    torch.cuda.synchronize()
    mask = _relu_mask(inp, truth, cfg.G) if cfg.act == "relu" else None
    _check("dx", dx, truth["dx"], lib and lib["dx"], dtype, mask, log=log)
    _check("dw", dw, truth["dw"], lib and lib["dw"], dtype, log=log)
    _check("db", db, truth["db"], lib and lib["db"], dtype, log=log)
    record_errors(config=name, family=family, dtype=cfg.dtype, observed=log)
    # size-independent property: dx sums to zero over every (n, g) slab, relative to the slab's absolute sum
    N, R, C = x.shape
    slab = as_np64(dx).reshape(N, R, cfg.G, C // cfg.G)
    ulp = {torch.float32: 2.0 ** -24, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    assert np.max(np.abs(slab.sum(axis=(1, 3))) / np.abs(slab).sum(axis=(1, 3))) < 4 * ulp


def _medium_shapes(count, seed):
    """Seeded sample of medium-sized problems (1 - 60 MB tensors) with awkward geometry: channels per group that do
    not divide the 64-channel chunks, rows that do not fill the last tile, several samples, one group, G == C / 8."""
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        D = int(rng.choice([1, 2, 3, 5, 8, 10, 12, 20, 40, 45, 64, 96, 160]))
        G = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        C = D * G
        if C % 8 != 0 or C > 2560:
            continue
        N = int(rng.randint(1, 7))
        R = int(rng.choice([rng.randint(200, 20000), 64 * 64, 128 * 128, 96 * 96, 37 * 53]))
        if not (5e5 <= N * R * C <= 3e7):
            continue
        out.append((N, R, C, G, ["identity", "relu", "silu", "gelu", "gelu_tanh"][len(out) % 5],
                    [torch.bfloat16, torch.float32, torch.float16][len(out) % 3]))
    return out


@pytest.mark.parametrize("N,R,C,G,act,dtype", _medium_shapes(36, 31))
def test_random_medium_shapes(family, N, R, C, G, act, dtype, device):
    """The single-launch kernels' tilings (and the streaming ones) on shapes no configuration names.  Truth is
    torch's own GroupNorm + activation + autograd in float64 on the device (the results contract; the C oracle would
    need minutes for these sizes); bars as for the configurations."""
    print("medium", family, N, R, C, G, act, dtype, flush=True)
    _check_against_torch(N, R, C, G, act, dtype, device)


# One sample of 47 - 75 MB: too large for the single-launch backward that keeps x and g' in registers, within reach of
# the one that keeps g' and streams x through a window twice.  Rows that do not fill the last tile, groups that
# straddle the 64-channel chunks, every activation, the three 4-byte-accumulated types.
LARGE_BACKWARD_SHAPES = [
    (1, 150037, 192, 24, "silu", torch.bfloat16),
    (1, 40003, 320, 32, "relu", torch.float32),
    (1, 512 * 512 - 511, 128, 32, "gelu", torch.float16),
    (1, 9001, 3200, 32, "gelu_tanh", torch.bfloat16),
    (1, 100000, 160, 1, "identity", torch.float32),
]


@pytest.mark.parametrize("N,R,C,G,act,dtype", LARGE_BACKWARD_SHAPES)
def test_large_single_sample_backward(family, N, R, C, G, act, dtype, device):
    """The windowed single-launch backward against torch in float64 (bars as for the configurations), and that it is
    the kernel that ran: one launch of the single-launch backward, none of the multi-launch kernels."""
    print("large backward", family, N, R, C, G, act, dtype, flush=True)
    _cabi.profile_collect()
    _cabi.profile_enable(True)
    try:
        _check_against_torch(N, R, C, G, act, dtype, device)
    finally:
        _cabi.profile_enable(False)
    launches = {k: v[0] for k, v in _cabi.profile_collect().items() if v[0]}
    print(launches, flush=True)
    if family == "resident":
        assert launches.get("fused_bwd") == 1 and "bwd_reduce" not in launches and "bwd_dx" not in launches, launches
    else:
        assert launches.get("bwd_dx") == 1 and "fused_bwd" not in launches, launches


@pytest.mark.parametrize("dtype,act", [(torch.bfloat16, "silu"), (torch.float32, "gelu_tanh"), (torch.float16, "relu")])
def test_backward_rows_requested_late_in_short_last_tiles(dtype, act, device):
    """The single-launch backward requests four rows of a lane's tile up front and the others as rows are consumed; rows
    past the end of a sample's last tile are masked where they are requested.  Row counts that leave the last tile's
    lanes with 0 ... all of their rows, around the point where the late requests begin, for the tile heights the sizes
    below select (4 to 32 rows per lane, the form that streams x through a window included), against torch in float64."""
    seen = set()
    before = _cabi.set_resident(True)
    try:
        for base in (3000, 16384, 30000, 45000, 62000):
            for rem in (1, 33, 97, 128, 129, 161):
                R = base - base % 32 + rem
                print("short last tile", dtype, act, R, flush=True)
                _check_against_torch(2, R, 320, 32, act, dtype, device)
                inst = _cabi.last_launch()
                m = re.search(r"fused_bwd rows=(\d+)", inst)
                if m:
                    seen.add(int(m.group(1)))
    finally:
        _cabi.set_resident(before)
    assert len(seen) >= 3 and max(seen) >= 22, seen  # several tile heights, the tall ones among them


def _check_against_torch(N, R, C, G, act, dtype, device):
    gen = torch.Generator().manual_seed(N * 1000003 + R * 101 + C)
    x = (torch.randn((N, R, C), generator=gen) * 1.7 + torch.randn((C,), generator=gen)).to(dtype).to(device)
    dy = torch.randn((N, R, C), generator=gen).to(dtype).to(device)
    w = (torch.rand((C,), generator=gen) + 0.5).to(dtype).to(device)
    b = (0.1 * torch.randn((C,), generator=gen)).to(dtype).to(device)
    code = orc.ACT_CODES[act]

    def torch_ref(t):
        xs = x.to(t).permute(0, 2, 1).contiguous().requires_grad_()
        ws, bs = w.to(t).requires_grad_(), b.to(t).requires_grad_()
        ys = orc.torch_act(act)(torch.nn.functional.group_norm(xs, G, ws, bs, EPS))
        gx, gw, gb = torch.autograd.grad(ys, (xs, ws, bs), dy.to(t).permute(0, 2, 1))
        return {"y": ys.detach().permute(0, 2, 1), "dx": gx.permute(0, 2, 1), "dw": gw, "db": gb}

    truth = torch_ref(torch.float64)
    own = torch_ref(dtype) if dtype != torch.float32 else None
    y, mean, rstd = cabi_fwd(x, w, b, G, EPS, code)
    dx, dw, db = cabi_bwd(dy, x, w, b, mean, rstd, G, code)
    torch.cuda.synchronize()
    xd = x.double().view(N, R, G, C // G)
    assert err(mean, xd.mean(dim=(1, 3))) <= FP32_TOL
    assert err(rstd, (xd.var(dim=(1, 3), correction=0) + EPS).rsqrt()) <= FP32_TOL
    mask = None
    if act == "relu":
        a = (rstd.double().repeat_interleave(C // G, dim=1) * w.double()[None, :])
        z = x.double() * a[:, None, :] + (b.double()[None, :] - mean.double().repeat_interleave(C // G, dim=1) * a)[:, None, :]
        mask = (z.abs() > RELU_BAND).cpu().numpy()
    for name, ours in (("y", y), ("dx", dx), ("dw", dw), ("db", db)):
        _check(name, ours, as_np64(truth[name]), own and as_np64(own[name]), dtype, mask if name == "dx" else None)


def _small_shapes(count, seed):
    """Seeded sample of small problems with many samples and few channels / rows (where the per-channel reductions
    over samples and tiles do most of their work): N up to 400, C up to 96, R up to 300."""
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        G = int(rng.choice([1, 2, 3, 4, 8, 16]))
        D = int(rng.choice([1, 2, 3, 4, 6, 8]))
        C = G * D
        N = int(rng.choice([1, 2, 7, 33, 65, 129, 200, 400]))
        R = int(rng.choice([1, 2, 6, 17, 64, 100, 289, 300]))
        if N * R * C > 2_000_000 or N * R * C < 8:
            continue
        out.append((N, R, C, G, ["identity", "relu", "silu", "gelu", "gelu_tanh"][len(out) % 5],
                    [torch.float32, torch.bfloat16, torch.float64, torch.float16][len(out) % 4]))
    return out


@pytest.mark.parametrize("N,R,C,G,act,dtype", _small_shapes(40, 77))
def test_random_small_shapes_all_layouts(family, N, R, C, G, act, dtype, device):
    """Channels-last (both kernel families) and channels-first entry points against the CPU oracle on the same
    values.  16-bit types are compared with torch's own CPU result in that type, as for the configurations."""
    from tests.gpu_harness import cabi_bwd_nchw, cabi_fwd_nchw

    print("small", family, N, R, C, G, act, dtype, flush=True)
    gen = torch.Generator().manual_seed(N * 7919 + R * 31 + C)
    x = (torch.randn((N, R, C), generator=gen) * 1.3 + torch.randn((C,), generator=gen)).to(dtype)
    dy = torch.randn((N, R, C), generator=gen).to(dtype)
    w = (torch.rand((C,), generator=gen) + 0.5).to(dtype)
    b = (0.1 * torch.randn((C,), generator=gen)).to(dtype)
    code = orc.ACT_CODES[act]
    truth = orc.fwd_bwd(as_np64(x), as_np64(w), as_np64(b), as_np64(dy), G, EPS, code)
    own = None
    if dtype in (torch.float16, torch.bfloat16):
        xs = x.permute(0, 2, 1).contiguous().requires_grad_()  # torch's CPU GroupNorm in the same type
        ws, bs = w.clone().requires_grad_(), b.clone().requires_grad_()
        ys = orc.torch_act(act)(torch.nn.functional.group_norm(xs, G, ws, bs, EPS))
        gx, gw, gb = torch.autograd.grad(ys, (xs, ws, bs), dy.permute(0, 2, 1))
        own = {"y": as_np64(ys.detach().permute(0, 2, 1)), "dx": as_np64(gx.permute(0, 2, 1)), "dw": as_np64(gw), "db": as_np64(gb)}
    mask = None
    if act == "relu":
        D = C // G
        a = np.repeat(truth["rstd"], D, axis=1) * as_np64(w)[None, :]
        z = as_np64(x) * a[:, None, :] + (as_np64(b)[None, :] - np.repeat(truth["mean"], D, axis=1) * a)[:, None, :]
        mask = np.abs(z) > RELU_BAND
    xd, dyd, wd, bd = x.to(device), dy.to(device), w.to(device), b.to(device)
    sdt = torch.float64 if dtype == torch.float64 else torch.float32
    results = {}
    y, mean, rstd = cabi_fwd(xd, wd, bd, G, EPS, code)
    dx, dw, db = cabi_bwd(dyd, xd, wd, bd, mean, rstd, G, code)
    results["channels-last"] = (y, mean, rstd, dx, dw, db)
    if family == "resident":  # the channels-first kernels have one family: run them once
        xc, dyc = xd.permute(0, 2, 1).contiguous(), dyd.permute(0, 2, 1).contiguous()
        yc, meanc, rstdc = cabi_fwd_nchw(xc, wd, bd, G, EPS, code)
        dxc, dwc, dbc = cabi_bwd_nchw(dyc, xc, wd, bd, meanc, rstdc, G, code)
        results["channels-first"] = (yc.permute(0, 2, 1), meanc, rstdc, dxc.permute(0, 2, 1), dwc, dbc)
    torch.cuda.synchronize()
    for layout, (y, mean, rstd, dx, dw, db) in results.items():
        _check(layout + " mean", mean, truth["mean"], None, sdt)
        _check(layout + " rstd", rstd, truth["rstd"], None, sdt)
        _check(layout + " y", as_np64(y), truth["y"], own and own["y"], dtype)
        _check(layout + " dx", as_np64(dx), truth["dx"], own and own["dx"], dtype, mask)
        _check(layout + " dw", dw, truth["dw"], own and own["dw"], dtype)
        _check(layout + " db", db, truth["db"], own and own["db"], dtype)
