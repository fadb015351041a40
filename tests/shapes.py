"""Shape library shared by the tests: the benchmark configurations and the
reference's own test matrix (test/test_forward.py, test/test_grad.py)."""
import torch

# (N, C, H, W, k, stride, padding)
CFG1 = (8, 32, 56, 56, 3, 1, 1)
CFG2 = (16, 64, 256, 256, 5, 1, 2)
# EfficientNet-B0 depthwise stack as (C, H_in, k, stride); batch 128, padding k//2
EFFNET_B0 = [
    (32, 112, 3, 1), (96, 112, 3, 2), (144, 56, 3, 1), (144, 56, 5, 2),
    (240, 28, 5, 1), (240, 28, 3, 2), (480, 14, 3, 1), (480, 14, 5, 1),
    (672, 14, 5, 1), (672, 14, 5, 2), (1152, 7, 5, 1), (1152, 7, 3, 1),
]
EFFNET_B0_BATCH = 128
CFG4 = [(256, 1024, 7, 7, 7, 1, 3), (128, 512, 14, 14, 7, 1, 3)]
CONVNEXT_T = [(64, 96, 56, 56, 7, 1, 3), (64, 192, 28, 28, 7, 1, 3),
              (64, 384, 14, 14, 7, 1, 3), (64, 768, 7, 7, 7, 1, 3)]
STRESS = (64, 256, 128, 96, 5, 2, 2)


def effnet_layers(batch=EFFNET_B0_BATCH):
    return [(batch, c, h, h, k, s, k // 2) for (c, h, k, s) in EFFNET_B0]


# The reference's forward matrix (test/test_forward.py:20-73): N=32
REF_FORWARD = (
    [(32, 32, 64, 64, k, s, p) for k in (3, 5) for s in (1, 2) for p in (k // 2, 0)]
    + [(32, 32, 63, 65, k, s, k // 2) for k in (3, 5) for s in (1, 2)]
    + [(32, 128, 32, 32, k, 1, k // 2) for k in (3, 5)]
)
# The reference's gradient matrix (test/test_grad.py:44-153): N=8, C=8, fp64
REF_GRAD = (
    [(8, 8, 34, 34, k, s, p) for k in (3, 5) for s in (1, 2) for p in (k // 2, 0)]
    + [(8, 8, 33, 35, k, s, k // 2) for k in (3, 5) for s in (1, 2)]
    + [(8, 8, 16, 16, k, 1, k // 2) for k in (3, 5)]
)


def out_hw(h, w, k, s, p):
    return (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1


def make_inputs(shape, seed=0, dtype=torch.float32):
    """Seeded inputs drawn in a fixed order on the CPU: x ~ N(0,1), w ~ N(0,1/k^2), gy ~ N(0,1)."""
    n, c, h, w, k, s, p = shape
    g = torch.Generator("cpu").manual_seed(seed)
    x = torch.randn(n, c, h, w, generator=g, dtype=dtype)
    wt = torch.randn(c, 1, k, k, generator=g, dtype=dtype) / k
    oh, ow = out_hw(h, w, k, s, p)
    gy = torch.randn(n, c, oh, ow, generator=g, dtype=dtype)
    return x, wt, gy


def shape_id(shape):
    n, c, h, w, k, s, p = shape
    return f"N{n}C{c}_{h}x{w}_k{k}s{s}p{p}"
