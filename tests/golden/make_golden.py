"""Writes tests/golden/dwconv_golden.npz: small fp64 input/output vectors.

The reference ships no fixtures; every expected value in its tests is made at
test time by ``F.conv2d(groups=C)`` (test/test_forward.py:14).  This script
does the same once, in fp64 on the CPU, so that other machines can cross-check
their own torch build, the C oracle and the HIP kernels against fixed numbers.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
from torch.nn import functional as F

# (N, C, H, W, KH, KW, (sh, sw), (ph, pw))
CASES = [
    (2, 3, 6, 7, 3, 3, (1, 1), (1, 1)),
    (2, 3, 9, 8, 5, 5, (2, 2), (2, 2)),
    (1, 4, 7, 7, 7, 7, (1, 1), (3, 3)),
    (2, 2, 11, 13, 3, 3, (2, 2), (0, 0)),
    (1, 2, 10, 9, 5, 3, (2, 1), (2, 0)),
    (2, 3, 14, 14, 5, 5, (1, 1), (2, 2)),
    (1, 5, 8, 12, 1, 1, (1, 1), (0, 0)),
    (1, 2, 12, 10, 4, 4, (3, 3), (1, 1)),
]


def main():
    out = {}
    g = torch.Generator("cpu").manual_seed(20240229)
    for i, (n, c, h, w, kh, kw, s, p) in enumerate(CASES):
        x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64, requires_grad=True)
        k = torch.randn(c, 1, kh, kw, generator=g, dtype=torch.float64, requires_grad=True)
        y = F.conv2d(x, k, stride=s, padding=p, groups=c)
        gy = torch.randn(y.shape, generator=g, dtype=torch.float64)
        gx, gk = torch.autograd.grad(y, (x, k), gy)
        out[f"c{i}_geom"] = np.array([n, c, h, w, kh, kw, s[0], s[1], p[0], p[1]], dtype=np.int64)
        for name, t in (("x", x), ("w", k), ("gy", gy), ("y", y), ("gx", gx), ("gw", gk)):
            out[f"c{i}_{name}"] = t.detach().numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dwconv_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
