"""The benchmark / parity configurations (seeded synthetic inputs), shared by bench.py and the tests.

Shapes, dtypes, activations and input distributions are the five configuration families the build is
measured on: (c1) the CPU-runnable fp32 forward, (c2) fp16 forward+backward, (c3) the latent-diffusion
UNet sweep in bf16 with per-channel offsets that stress the variance numerics, (c4) large-spatial /
few-channel fp16 with gelu_tanh, (c5) irregular shapes incl. a 5-D input.  The shape grid follows the
reference's own test inputs in spirit (test/check_outputs.py:161-211, test/trailing_dims.py:8-15).
"""
import collections

import torch

Config = collections.namedtuple("Config", "name dtype shape G act passes xdist")

# dtype codes of include/gnnhwc.h
DT_CODE = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.bfloat16: 3}

DT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16, "fp64": torch.float64}

CONFIGS = collections.OrderedDict()


def _add(name, dtype, shape, G, act, passes="fwd+bwd", xdist="normal"):
    CONFIGS[name] = Config(name, dtype, tuple(shape), G, act, passes, xdist)


_add("c1", "fp32", (1, 320, 64, 64), 32, "silu", passes="fwd")
_add("c2", "fp16", (2, 640, 32, 32), 32, "silu")
_add("c3a", "bf16", (1, 640, 128, 128), 32, "silu", xdist="offset")
_add("c3b", "bf16", (1, 1280, 64, 64), 32, "silu", xdist="offset")
_add("c3c", "bf16", (4, 320, 128, 128), 32, "silu", xdist="offset")
_add("c4a", "fp16", (1, 128, 512, 512), 32, "gelu_tanh")
_add("c4b", "fp16", (1, 256, 256, 256), 32, "gelu_tanh")
for _dt in ("fp32", "bf16"):
    for _act in ("identity", "relu", "silu", "gelu", "gelu_tanh"):
        _add("c5a_%s_%s" % (_dt, _act), _dt, (3, 96, 37, 53), 24, _act)
        _add("c5b_%s_%s" % (_dt, _act), _dt, (8, 1920, 17, 17), 32, _act)
        _add("c5c_%s_%s" % (_dt, _act), _dt, (2, 256, 8, 16, 16), 16, _act)

SD_UNET_SWEEP = ("c3a", "c3b", "c3c")
ALL_NAMES = tuple(CONFIGS)

# Measured by bench.py --nchw only (not a parity configuration of its own; tests/test_gpu_nchw.py has its small relatives):
# one group of many long rows, the channels-first case where a slab has thousands of partial sums.
EXTRA = {"one_group": Config("one_group", "bf16", (1, 512, 256, 256), 1, "silu", "fwd+bwd", "normal")}


def _seed(name):
    return 1000 + ALL_NAMES.index(name) if name in ALL_NAMES else 2000 + sorted(EXTRA).index(name)


def make_inputs(cfg, device="cpu", shape=None):
    """Seeded inputs for one configuration.

    Returns dict(x, w, b, dy): x and dy have logical shape (N, C, *spatial) with channels fastest
    (stride(1) == 1, spatial dims contiguous in their logical order); w ~ U(0.5, 1.5), b ~ N(0, 0.1),
    dy ~ N(0, 1); x ~ N(0, 1), or 2 N(0, 1) + a per-channel offset ~ N(0, 1) for the "offset" distribution.
    Values are drawn on the CPU in fp32 and then cast, so every device sees the same numbers.
    `shape` overrides cfg.shape (used to shrink a configuration for CPU-sized checks)."""
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    shape = tuple(shape or cfg.shape)
    N, C = shape[0], shape[1]
    spatial = shape[2:]
    gen = torch.Generator().manual_seed(_seed(cfg.name))
    dtype = DT[cfg.dtype]
    x = torch.randn((N, *spatial, C), generator=gen)
    if cfg.xdist == "offset":
        x = 2.0 * x + torch.randn((C,), generator=gen)
    w = torch.rand((C,), generator=gen) + 0.5
    b = 0.1 * torch.randn((C,), generator=gen)
    dy = torch.randn((N, *spatial, C), generator=gen)
    nd = len(shape)
    perm = (0, nd - 1, *range(1, nd - 1))
    x = x.to(dtype).to(device).permute(*perm)
    dy = dy.to(dtype).to(device).permute(*perm)
    return dict(x=x, w=w.to(dtype).to(device), b=b.to(dtype).to(device), dy=dy)


def tensor_bytes(cfg, shape=None):
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    n = 1
    for s in (shape or cfg.shape):
        n *= s
    return n * torch.finfo(DT[cfg.dtype]).bits // 8


def algorithmic_bytes(cfg, passes=None):
    """Compulsory HBM traffic: forward reads x and writes y (2 S); backward reads x and dy and writes dx (3 S)."""
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    S = tensor_bytes(cfg)
    passes = passes or cfg.passes
    return {"fwd": 2 * S, "bwd": 3 * S, "fwd+bwd": 5 * S}[passes]


def nrc_view(t):
    """(N, C, *spatial) tensor with channels fastest -> (N, R, C) contiguous tensor (no copy when already laid out so)."""
    nd = t.dim()
    u = t.permute(0, *range(2, nd), 1)
    u = u if u.is_contiguous() else u.contiguous()
    return u.reshape(u.shape[0], -1, u.shape[-1])
