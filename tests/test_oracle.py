"""Pins the CPU oracle (oracle/gn_oracle.c): golden vectors, the torch library routine, brute force,
finite differences and invariants.  CPU only."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import gn_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gn_golden.npz")
ACTS = ["identity", "relu", "silu", "gelu", "gelu_tanh"]


def nrc(a):
    """(N, C, *spatial) numpy -> (N, R, C)."""
    N, C = a.shape[:2]
    return np.ascontiguousarray(a.reshape(N, C, -1).transpose(0, 2, 1))


def rel(a, b):
    return float(np.max(np.abs(a - b)) / (np.max(np.abs(b)) + 1e-300))


def test_oracle_matches_golden_vectors():
    z = np.load(GOLDEN, allow_pickle=False)
    eps = float(z["eps"])
    n = int(z["count"])
    assert n == 35
    for i in range(n):
        key = "case%02d" % i
        G = int(z[key + "_meta"][0])
        act = orc.ACT_CODES[str(z[key + "_act"])]
        x, dy = nrc(z[key + "_x"]), nrc(z[key + "_dy"])
        r = orc.fwd_bwd(x, z[key + "_w"], z[key + "_b"], dy, G, eps, act)
        assert rel(r["y"], nrc(z[key + "_y"])) < 1e-12, key
        assert rel(r["mean"], z[key + "_mean"]) < 1e-12, key
        assert rel(r["rstd"], z[key + "_rstd"]) < 1e-12, key
        assert rel(r["dx"], nrc(z[key + "_dx"])) < 1e-10, key
        assert rel(r["dw"], z[key + "_dw"]) < 1e-10, key
        assert rel(r["db"], z[key + "_db"]) < 1e-10, key


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("shape,G", [((3, 96, 37, 53), 24), ((2, 40, 9, 7), 4), ((1, 128, 4, 4, 4), 32), ((2, 7, 11), 7)])
def test_oracle_matches_torch_float64(act, shape, G):
    """The library routine the reference's tests use as their own oracle (test/check_outputs.py:91-157)."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(shape, generator=g, dtype=torch.float64) * 2 + torch.randn(shape[1], generator=g, dtype=torch.float64).view(
        1, -1, *([1] * (len(shape) - 2)))
    w = torch.rand(shape[1], generator=g, dtype=torch.float64) + 0.5
    b = torch.randn(shape[1], generator=g, dtype=torch.float64) * 0.1
    dy = torch.randn(shape, generator=g, dtype=torch.float64)
    ref = orc.torch_reference(x, w, b, G, 1e-5, act, dy)
    r = orc.fwd_bwd(orc.to_nrc(x), w.numpy(), b.numpy(), orc.to_nrc(dy), G, 1e-5, orc.ACT_CODES[act])
    assert rel(r["y"], orc.to_nrc(ref["y"])) < 1e-12
    assert rel(r["dx"], orc.to_nrc(ref["dx"])) < 1e-10
    assert rel(r["dw"], ref["dw"].numpy()) < 1e-10
    assert rel(r["db"], ref["db"].numpy()) < 1e-10
    _, mean, rstd = torch.native_group_norm(x, w, b, shape[0], shape[1], x[0, 0].numel(), G, 1e-5)
    assert rel(r["mean"], mean.numpy()) < 1e-12
    assert rel(r["rstd"], rstd.numpy()) < 1e-12


def _py_act(v, act):
    if act == "identity":
        return v
    if act == "relu":
        return v if v > 0 else 0.0
    if act == "silu":
        return v / (1.0 + math.exp(-v))
    if act == "gelu":
        return 0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0)))
    return 0.5 * v * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (v + 0.044715 * v ** 3)))


def _brute_forward(x, w, b, G, eps, act):
    """Definition of GroupNorm written with Python loops (GN_Naive.forward, test/check_outputs.py:21-32)."""
    N, R, C = x.shape
    D = C // G
    y = np.zeros_like(x)
    for n in range(N):
        for g in range(G):
            vals = [x[n, r, g * D + d] for r in range(R) for d in range(D)]
            mu = sum(vals) / len(vals)
            var = sum((v - mu) ** 2 for v in vals) / len(vals)
            rs = 1.0 / math.sqrt(var + eps)
            for r in range(R):
                for d in range(D):
                    c = g * D + d
                    y[n, r, c] = _py_act((x[n, r, c] - mu) * rs * w[c] + b[c], act)
    return y


TINY = [((2, 5, 6), 3), ((1, 4, 1), 1), ((2, 3, 4), 4), ((2, 4, 6), 1), ((1, 7, 2), 2)]  # (N, R, C), G


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("shape,G", TINY)
def test_oracle_forward_brute_force(act, shape, G):
    rng = np.random.default_rng(3)
    x = rng.normal(size=shape) * 1.5 + 0.7
    w = rng.uniform(0.5, 1.5, size=shape[2])
    b = rng.normal(size=shape[2]) * 0.1
    y, _, _ = orc.fwd(x, w, b, G, 1e-5, orc.ACT_CODES[act])
    assert np.max(np.abs(y - _brute_forward(x, w, b, G, 1e-5, act))) < 1e-12


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("shape,G", TINY[:3])
def test_oracle_backward_finite_differences(act, shape, G):
    """dx, dgamma, dbeta against central differences of L = sum(dy * y), with y from the brute-force forward:
    pins the backward algebra without torch and without the oracle's own forward."""
    rng = np.random.default_rng(11)
    x = rng.normal(size=shape) * 1.5 + 0.7
    w = rng.uniform(0.5, 1.5, size=shape[2])
    b = rng.normal(size=shape[2]) * 0.1
    dy = rng.normal(size=shape)
    eps = 1e-5
    r = orc.fwd_bwd(x, w, b, dy, G, eps, orc.ACT_CODES[act])

    def loss(xx, ww, bb):
        return float(np.sum(dy * _brute_forward(xx, ww, bb, G, eps, act)))

    h = 1e-6
    fd_dx = np.zeros_like(x)
    for idx in np.ndindex(*shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        fd_dx[idx] = (loss(xp, w, b) - loss(xm, w, b)) / (2 * h)
    fd_dw = np.zeros_like(w)
    fd_db = np.zeros_like(b)
    for c in range(shape[2]):
        wp, wm, bp, bm = w.copy(), w.copy(), b.copy(), b.copy()
        wp[c] += h
        wm[c] -= h
        bp[c] += h
        bm[c] -= h
        fd_dw[c] = (loss(x, wp, b) - loss(x, wm, b)) / (2 * h)
        fd_db[c] = (loss(x, w, bp) - loss(x, w, bm)) / (2 * h)
    tol = 2e-6
    assert np.max(np.abs(r["dx"] - fd_dx)) < tol * max(1.0, np.max(np.abs(fd_dx)))
    assert np.max(np.abs(r["dw"] - fd_dw)) < tol * max(1.0, np.max(np.abs(fd_dw)))
    assert np.max(np.abs(r["db"] - fd_db)) < tol * max(1.0, np.max(np.abs(fd_db)))


@pytest.mark.parametrize("act", ACTS)
def test_oracle_invariants(act):
    rng = np.random.default_rng(5)
    N, R, C, G = 2, 33, 24, 6
    D = C // G
    eps = 1e-5
    x = rng.normal(size=(N, R, C)) * 2 + rng.normal(size=C)
    w = rng.uniform(0.5, 1.5, size=C)
    b = rng.normal(size=C) * 0.1
    dy = rng.normal(size=(N, R, C))
    code = orc.ACT_CODES[act]
    r = orc.fwd_bwd(x, w, b, dy, G, eps, code)
    # dx is orthogonal to the constant within every (n, g) slab, whatever the activation
    slab = r["dx"].reshape(N, R, G, D)
    assert np.max(np.abs(slab.sum(axis=(1, 3)))) < 1e-9
    # ... and nearly orthogonal to (x - mean): the residual is O(eps / (var + eps))
    xs = x.reshape(N, R, G, D) - r["mean"][:, None, :, None]
    var = 1.0 / r["rstd"] ** 2 - eps
    assert np.max(np.abs((slab * xs).sum(axis=(1, 3))) * (var + eps) / eps) < 1e3
    # shifting and positively scaling x per group leaves y unchanged up to eps
    shift = rng.normal(size=G).repeat(D)
    y2, _, _ = orc.fwd(3.0 * x + shift, w, b, G, eps * 9.0, code)
    assert np.max(np.abs(y2 - r["y"])) < 1e-10
    if act == "identity":
        y1, mean, rstd = orc.fwd(x, np.ones(C), np.zeros(C), G, eps, code)
        ys = y1.reshape(N, R, G, D)
        assert np.max(np.abs(ys.mean(axis=(1, 3)))) < 1e-12
        assert np.max(np.abs(ys.var(axis=(1, 3)) - var / (var + eps))) < 1e-12


def test_oracle_float32_variant_tracks_float64():
    rng = np.random.default_rng(9)
    N, R, C, G = 2, 64, 32, 8
    x = rng.normal(size=(N, R, C)) * 2 + rng.normal(size=C)
    w = rng.uniform(0.5, 1.5, size=C)
    b = rng.normal(size=C) * 0.1
    dy = rng.normal(size=(N, R, C))
    for act in range(5):
        r64 = orc.fwd_bwd(x, w, b, dy, G, 1e-5, act)
        r32 = orc.fwd_bwd(x, w, b, dy, G, 1e-5, act, dtype=np.float32)
        for k in ("y", "mean", "rstd", "dx", "dw", "db"):
            assert rel(r32[k].astype(np.float64), r64[k]) < 2e-5, (act, k)
