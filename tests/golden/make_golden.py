"""Writes tests/golden/gn_golden.npz: small float64 input/output vectors for the CPU oracle.

The vectors come from torch's own CPU routines -- ``F.group_norm`` + the matching torch activation,
``torch.native_group_norm`` for mean / rstd and autograd for the gradients -- which is what the
reference's tests compare their kernels with at run time (test/check_outputs.py:91-157); the reference
itself ships no stored vectors.  The reference package is neither imported nor needed.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

ACTS = {
    "identity": lambda t: t,
    "relu": F.relu,
    "silu": F.silu,
    "gelu": F.gelu,
    "gelu_tanh": lambda t: F.gelu(t, approximate="tanh"),
}
# (N, C, *spatial), G -- includes C = 1, G = C, G = 1, odd sizes and a 5-D input (test/check_outputs.py:162-170 style)
SHAPES = [
    ((2, 6, 5), 3),
    ((2, 12, 7, 5), 4),
    ((1, 8, 3, 3), 8),
    ((2, 6, 2, 2), 1),
    ((1, 1, 3, 3), 1),
    ((2, 8, 2, 3, 2), 2),
    ((3, 24, 5, 3), 6),
]
EPS = 1e-5


def main():
    torch.manual_seed(20240)
    out = {}
    idx = 0
    for shape, G in SHAPES:
        for act in ACTS:
            C = shape[1]
            x = (torch.randn(shape, dtype=torch.float64) * 1.7 + 0.3).requires_grad_(True)
            w = (torch.rand(C, dtype=torch.float64) + 0.5).requires_grad_(True)
            b = (0.1 * torch.randn(C, dtype=torch.float64)).requires_grad_(True)
            dy = torch.randn(shape, dtype=torch.float64)
            y = ACTS[act](F.group_norm(x, G, w, b, EPS))
            dx, dw, db = torch.autograd.grad(y, (x, w, b), dy)
            N = shape[0]
            _, mean, rstd = torch.native_group_norm(x.detach(), w.detach(), b.detach(), N, C, x[0, 0].numel(), G, EPS)
            key = "case%02d" % idx
            out[key + "_meta"] = np.array([G] + list(shape), dtype=np.int64)
            out[key + "_act"] = np.array(act)
            for name, t in (("x", x), ("w", w), ("b", b), ("dy", dy), ("y", y), ("mean", mean), ("rstd", rstd),
                            ("dx", dx), ("dw", dw), ("db", db)):
                out[key + "_" + name] = t.detach().numpy().copy()
            idx += 1
    out["eps"] = np.array(EPS)
    out["count"] = np.array(idx)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gn_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", idx, "cases")


if __name__ == "__main__":
    main()
