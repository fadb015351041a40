"""GPU parity: the HIP library (through its C ABI, via torch_dwconv._C) against the CPU oracle.

Tolerances (fp32): forward and grad-input rtol = atol = 1e-5 against the fp64
oracle; grad-weight rtol 1e-4 with atol = 1e-4 * max|gw_ref| (its entries are
sums of up to N*Ho*Wo products, so a bare relative bound fails on entries that
happen to land near zero whatever the summation order), and bit-identical from
run to run.  fp64 kernels: 1e-11.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from shapes import (CFG1, CFG2, CFG4, CONVNEXT_T, REF_FORWARD, REF_GRAD, STRESS, effnet_layers,
                    make_inputs, out_hw, shape_id)

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "dwconv_golden.npz")


@pytest.fixture(scope="module")
def dw(gpu):
    import torch_dwconv.dwconv as m

    return m


def _np(t):
    return t.detach().cpu().numpy()


def _announce(*what):
    print("[case]", *what, flush=True)


def run_three_passes(dw, x, w, gy, stride, padding):
    """forward, grad-input, grad-weight through the autograd Function."""
    from torch_dwconv import _C

    xg = x.detach().clone().requires_grad_(True)
    wg = w.detach().clone().requires_grad_(True)
    y = dw.depthwise_conv2d(xg, wg, stride=stride, padding=padding)
    v_fwd = _C.last_variant()
    gx, gw = torch.autograd.grad(y, (xg, wg), gy)
    return y.detach(), gx, gw, v_fwd


def run_separate_backward(x, w, gy, stride, padding):
    """grad-input and grad-weight through the two entry points the reference's backward calls
    (torch_dwconv/dwconv.py:56-68), not through the combined one."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import make_tuple

    s, p = make_tuple(stride, 2), make_tuple(padding, 2)
    kh, kw = w.shape[2:]
    g_pad = (kh - p[0] - 1, x.shape[2] - gy.shape[2] * s[0] + p[0], kw - p[1] - 1, x.shape[3] - gy.shape[3] * s[1] + p[1])
    gx = _C.dwconv2d(gy, w, s[0], s[1], 1, 1, *g_pad, False)
    gw = _C.dwconv2d_backward_kernel(x, gy, w, 1, 1, s[0], s[1], p[0], p[1])
    return gx, gw


def assert_parity(y, gx, gw, y_ref, gx_ref, gw_ref, dtype):
    if dtype == torch.float32:
        tol = dict(rtol=1e-5, atol=1e-5)
        gw_rtol = 1e-4
    else:
        tol = dict(rtol=1e-11, atol=1e-11)
        gw_rtol = 1e-11
    np.testing.assert_allclose(_np(y).astype(np.float64), y_ref, **tol)
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref, **tol)
    gw_atol = gw_rtol * max(float(np.abs(gw_ref).max()), 1e-30)
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref, rtol=gw_rtol, atol=gw_atol)


def check_against_c_oracle(dw, gpu, shape, dtype=torch.float32, seed=0):
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=seed, dtype=dtype)
    y, gx, gw, variant = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    _announce(shape_id(shape), str(dtype), variant)
    assert y.shape == gy.shape and gx.shape == x.shape and gw.shape == wt.shape
    y_ref = oracle.forward(_np(x), _np(wt), s, p)
    gx_ref = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
    assert_parity(y, gx, gw, y_ref, gx_ref, gw_ref, dtype)
    gx2, gw2 = run_separate_backward(x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    assert_parity(y, gx2, gw2, y_ref, gx_ref, gw_ref, dtype)
    return variant


# Small and awkward shapes: every kernel family, ragged edges, odd extents.
SMALL = [
    (2, 3, 6, 7, 3, 1, 1), (2, 3, 6, 7, 3, 2, 1), (2, 3, 9, 8, 5, 1, 2), (2, 3, 9, 8, 5, 2, 2),
    (1, 2, 7, 7, 7, 1, 3), (3, 5, 7, 7, 5, 1, 2), (3, 5, 7, 7, 3, 1, 1), (1, 2, 12, 11, 7, 2, 3),
    (2, 2, 11, 13, 3, 2, 0), (2, 2, 11, 13, 5, 1, 0), (1, 3, 10, 10, 4, 2, 1), (1, 3, 13, 10, 2, 3, 0),
    (1, 2, 5, 5, 1, 1, 0), (1, 2, 9, 9, 3, 3, 1), (2, 7, 14, 14, 3, 1, 1), (2, 7, 14, 14, 5, 1, 2),
    (2, 7, 14, 14, 5, 2, 2), (2, 7, 14, 14, 7, 1, 3), (2, 5, 28, 28, 5, 1, 2), (2, 5, 28, 28, 3, 2, 1),
    (2, 5, 28, 28, 7, 1, 3), (3, 4, 56, 56, 3, 1, 1), (3, 4, 56, 56, 5, 2, 2), (3, 4, 56, 56, 7, 1, 3),
    (2, 3, 112, 112, 3, 1, 1), (2, 3, 112, 112, 3, 2, 1), (1, 2, 128, 96, 5, 2, 2), (1, 2, 256, 256, 5, 1, 2),
    (1, 1, 1, 1, 3, 1, 1), (1, 1, 3, 300, 3, 1, 1), (1, 1, 300, 3, 5, 2, 2), (1, 2, 40, 1000, 7, 2, 3),
    (2, 3, 57, 59, 7, 2, 3), (2, 3, 58, 60, 5, 2, 1), (2, 3, 61, 64, 3, 2, 0), (1, 3, 64, 64, 7, 1, 0),
    # whole-plane kernels with ragged channel groups, several images per chunk, odd plane sizes
    (3, 12, 7, 7, 5, 1, 2), (5, 20, 7, 7, 3, 1, 1), (3, 8, 7, 7, 7, 1, 3), (2, 13, 14, 14, 3, 1, 1),
    (3, 10, 14, 14, 5, 2, 2), (5, 11, 28, 28, 3, 2, 1), (3, 6, 28, 28, 5, 1, 2), (2, 4, 28, 28, 7, 2, 3),
    (2, 70, 14, 14, 7, 1, 3), (2, 68, 7, 7, 5, 1, 2), (2, 3, 20, 14, 3, 1, 1), (2, 4, 10, 7, 5, 1, 2),
    # whole-plane kernels at the other widths up to 32: exact instances and ragged classes (any width without one), both strides, odd extents (stride 2 of an odd plane: gx is 2*gy - 1 wide), planes that are not a
    # multiple of four elements
    (3, 8, 8, 8, 3, 1, 1), (2, 12, 8, 8, 5, 1, 2), (2, 8, 8, 8, 7, 1, 3), (3, 8, 8, 8, 5, 2, 2),
    (2, 6, 16, 16, 3, 1, 1), (2, 5, 16, 16, 5, 1, 2), (2, 4, 16, 16, 7, 1, 3), (3, 6, 16, 16, 5, 2, 2), (2, 4, 16, 16, 3, 2, 1),
    (2, 3, 32, 32, 3, 1, 1), (2, 4, 32, 32, 5, 1, 2), (1, 3, 32, 32, 7, 1, 3), (2, 3, 32, 32, 3, 2, 1), (2, 2, 32, 32, 7, 2, 3),
    (2, 8, 15, 15, 3, 1, 1), (2, 8, 15, 15, 5, 1, 2), (1, 4, 15, 15, 7, 1, 3), (3, 8, 15, 15, 5, 2, 2), (2, 12, 15, 15, 3, 2, 1),
    (2, 3, 30, 30, 5, 1, 2), (2, 2, 30, 30, 3, 2, 1), (1, 3, 30, 30, 7, 1, 3), (2, 3, 30, 30, 7, 2, 3),
    (2, 4, 12, 12, 5, 1, 2), (2, 3, 24, 24, 3, 1, 1), (2, 5, 20, 20, 5, 2, 2), (2, 4, 9, 9, 3, 1, 1), (3, 8, 9, 9, 5, 2, 2),
    (2, 4, 5, 5, 3, 1, 1), (2, 4, 6, 4, 5, 1, 2), (2, 3, 40, 10, 3, 1, 1), (2, 4, 7, 22, 5, 1, 2), (2, 4, 13, 26, 7, 1, 3),
    (2, 8, 7, 7, 3, 2, 1), (2, 4, 11, 7, 5, 2, 2), (2, 4, 31, 31, 3, 1, 1), (4, 4, 17, 17, 5, 1, 2), (2, 16, 3, 3, 3, 1, 1),
    # runs of planes that start off a 4-element boundary (odd planes, channel groups that are not multiples of four)
    (3, 5, 15, 15, 3, 1, 1), (3, 7, 9, 9, 5, 2, 2), (2, 3, 31, 29, 7, 1, 3), (3, 5, 30, 30, 3, 2, 1), (5, 3, 7, 7, 5, 1, 2),
    (3, 6, 13, 13, 3, 2, 1), (2, 9, 5, 7, 3, 1, 1),
    # ragged even widths (LDS rows at pitch width + 1, element-wise copies), with and without heads
    (2, 6, 24, 24, 5, 1, 2), (3, 5, 24, 24, 3, 2, 1), (2, 8, 12, 12, 5, 1, 2), (3, 7, 12, 12, 5, 2, 2), (2, 8, 6, 6, 3, 1, 1),
    (3, 5, 6, 6, 5, 1, 2), (2, 3, 20, 20, 7, 1, 3), (3, 3, 10, 10, 3, 1, 1), (3, 5, 9, 10, 3, 1, 1), (2, 4, 17, 18, 5, 1, 2),
    (3, 3, 11, 26, 3, 2, 1), (2, 5, 7, 30, 5, 1, 2), (1, 7, 9, 22, 7, 1, 3),
    # widths that keep a ragged class now that 6, 9, 10, 12, 15, 18, 20, 24 and 30 have exact instances
    (3, 5, 11, 22, 3, 1, 1), (2, 3, 27, 26, 5, 2, 2), (3, 4, 19, 21, 5, 1, 2), (2, 6, 13, 11, 3, 1, 1), (3, 3, 23, 27, 7, 1, 3),
    (2, 5, 18, 18, 5, 1, 2), (3, 4, 10, 10, 5, 2, 2), (2, 3, 20, 20, 3, 1, 1), (3, 7, 9, 9, 7, 1, 3),
    # one channel per workgroup over a stack of its images (5x5 / 7x7, stride 1): heights that leave a hanging
    # 4-row unit (one, two or three rows over), tiles that span two and three images, a last tile that is short
    (3, 5, 57, 64, 7, 1, 3), (2, 3, 33, 96, 5, 1, 2), (5, 2, 70, 40, 7, 1, 3), (1, 1, 300, 16, 5, 1, 2), (7, 3, 34, 36, 7, 1, 3),
    (9, 2, 18, 60, 5, 1, 2), (4, 3, 59, 52, 7, 1, 3), (2, 2, 130, 128, 7, 1, 3), (6, 1, 23, 48, 5, 1, 2),
]


@pytest.mark.parametrize("shape", SMALL, ids=shape_id)
def test_small_and_awkward_shapes_fp32(dw, gpu, shape):
    check_against_c_oracle(dw, gpu, shape)


@pytest.mark.parametrize("shape", SMALL[::3], ids=shape_id)
def test_small_and_awkward_shapes_fp64(dw, gpu, shape):
    check_against_c_oracle(dw, gpu, shape, dtype=torch.float64)


@pytest.mark.parametrize("shape", SMALL[::2], ids=shape_id)
def test_generic_kernels_fp32(dw, gpu, shape, monkeypatch):
    monkeypatch.setenv("DWCONV_FORCE_GENERIC", "1")
    variant = check_against_c_oracle(dw, gpu, shape)
    assert variant.startswith("direct")


@pytest.mark.parametrize("shape", REF_FORWARD, ids=shape_id)
def test_reference_forward_matrix(dw, gpu, shape):
    # test/test_forward.py:20-73, same shapes (N=32), all three passes instead of forward only
    check_against_c_oracle(dw, gpu, shape)


@pytest.mark.parametrize("shape", REF_GRAD, ids=shape_id)
def test_reference_grad_matrix_fp64_values(dw, gpu, shape):
    # test/test_grad.py:44-153 shapes in fp64; values against the oracle with a random upstream gradient
    check_against_c_oracle(dw, gpu, shape, dtype=torch.float64)


@pytest.mark.parametrize("shape", [(2, 2) + s[2:] for s in REF_GRAD[::3]], ids=shape_id)
def test_reference_gradcheck_fp64(dw, gpu, shape):
    # the reference's own probe: numerical Jacobian of depthwise_conv2d(...).sum()
    n, c, h, w, k, s, p = shape
    h, w = min(h, 12), min(w, 13)
    g = torch.Generator("cpu").manual_seed(1)
    x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64).to(gpu).requires_grad_(True)
    wt = torch.randn(c, 1, k, k, generator=g, dtype=torch.float64).to(gpu).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a: dw.depthwise_conv2d(a, wt.detach(), stride=s, padding=p).sum(), x)
    assert torch.autograd.gradcheck(lambda b: dw.depthwise_conv2d(x.detach(), b, stride=s, padding=p).sum(), wt)


def test_golden_vectors(dw, gpu):
    z = np.load(GOLDEN)
    ncases = len([k for k in z.files if k.endswith("_geom")])
    for dtype in (torch.float32, torch.float64):
        for i in range(ncases):
            n, c, h, w, kh, kw, sh, sw, ph, pw = (int(v) for v in z[f"c{i}_geom"])
            _announce("golden", i, dtype)
            x, wt, gy = (torch.from_numpy(z[f"c{i}_{k}"]).to(dtype).to(gpu) for k in ("x", "w", "gy"))
            y, gx, gw, _ = run_three_passes(dw, x, wt, gy, (sh, sw), (ph, pw))
            if dtype == torch.float64:
                assert_parity(y, gx, gw, z[f"c{i}_y"], z[f"c{i}_gx"], z[f"c{i}_gw"], dtype)
            else:
                # inputs were rounded to fp32: compare against the oracle on the rounded inputs
                xr, wr, gr = _np(x), _np(wt), _np(gy)
                assert_parity(y, gx, gw, oracle.forward(xr, wr, (sh, sw), (ph, pw)),
                              oracle.grad_input(gr, wr, (h, w), (sh, sw), (ph, pw)),
                              oracle.grad_weight(xr, gr, wt.shape, (sh, sw), (ph, pw)), dtype)


# ---- benchmark configurations at full size ---------------------------------------------
class poisoned_allocations:
    """While active, every tensor the binding allocates with torch.empty / torch.empty_like starts out as NaN
    (0xFF bytes for the workspace), so that an element a kernel fails to store cannot pass by holding a stale
    right answer from an earlier run in the same allocator block."""

    def __enter__(self):
        self._empty, self._empty_like = torch.empty, torch.empty_like

        def poison(t):
            if t.is_cuda and t.numel():
                t.fill_(float("nan") if t.is_floating_point() else 255)
            return t

        torch.empty = lambda *a, **k: poison(self._empty(*a, **k))
        torch.empty_like = lambda *a, **k: poison(self._empty_like(*a, **k))
        return self

    def __exit__(self, *exc):
        torch.empty, torch.empty_like = self._empty, self._empty_like


def assert_close_on_device(got, ref, rtol, atol, what):
    """Every element of `got` (any layout) against the fp64 reference `ref` (numpy or tensor), compared on the device;
    NaN never passes.  On failure names the first offending (n, c, y, x) and how many planes are affected."""
    ref = (torch.from_numpy(np.ascontiguousarray(ref)) if isinstance(ref, np.ndarray) else ref).to(got.device)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    ok = (got.double() - ref).abs() <= atol + rtol * ref.abs()
    if bool(ok.all()):
        return
    bad = (~ok).nonzero()
    first = tuple(bad[0].tolist())
    planes = torch.unique(bad[:, 0] * got.shape[1] + bad[:, 1]).numel() if got.dim() == 4 else "-"
    raise AssertionError(f"{what}: {bad.shape[0]} of {ok.numel()} elements out of tolerance in {planes} planes; "
                         f"first at {first}: got {got[first].item()!r}, expected {ref[first].item()!r}")


# planes up to this many elements per tensor get the C oracle over the whole tensor (seconds with OpenMP)
C_ORACLE_WHOLE_LIMIT = 160 << 20


def boundary_planes(n, c, rng, extra=4):
    """(image, channel) pairs that a remainder bug would hit: the first and last planes, the planes around the last
    few powers of two and multiples of the wavefront / workgroup sizes counted from the end, plus random ones."""
    total = n * c
    flat = {0, 1, total - 1, total - 2, c - 1, c, total - c, total - c - 1}
    for step in (2, 3, 4, 6, 7, 8, 9, 12, 16, 18, 32, 36, 64, 128, 256):
        last = (total - 1) // step * step     # first plane of the last (partial) group of `step`
        flat |= {last - 1, last, last + 1}
    flat |= {int(v) for v in rng.integers(total, size=extra)}
    return sorted((f // c, f % c) for f in flat if 0 <= f < total)


def full_size_references(shape, x, wt, gy, gpu):
    """fp64 references for whole tensors: the C oracle where it finishes in seconds, otherwise the shift-and-add
    closed form on the device (pinned against the C oracle in tests/test_oracle.py) with the C oracle on boundary
    and random planes on top.  16-bit inputs are widened exactly: the references see the rounded values."""
    n, c, h, w, k, s, p = shape
    if x.numel() <= C_ORACLE_WHOLE_LIMIT:
        xn, wn, gn = _np(x.double()), _np(wt.double()), _np(gy.double())
        return (oracle.forward(xn, wn, s, p), oracle.grad_input(gn, wn, (h, w), s, p),
                oracle.grad_weight(xn, gn, wt.shape, s, p), "c-oracle")
    y, gx, gw = oracle.shift_add_reference(x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    return y, gx, gw, "shift-add"


def full_size_tolerances(dtype):
    """(rtol, atol) of y / gx and the relative bound of gw: the fp32 bounds of this file, plus one rounding step of
    the element type for 16-bit tensors (2^-11 for fp16, 2^-8 for bf16; the sums are fp32 and rounded once)."""
    if dtype == torch.float32:
        return 1e-5, 1e-5, 1e-4
    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    return step, 1e-5 + step * 1e-2, step + 1e-4


def check_full_size(dw, gpu, shape, seed=0, layouts=("nchw",), n_planes=4, dtype=torch.float32, expect=None):
    """Full-size run with the planner decisions of the real configuration.  Every element of y, gx and gw is
    compared with an fp64 reference (outputs start as NaN); boundary and random planes are checked against the C
    oracle as well; adjoint identities; grad-weight bit-identical from run to run; both backward routes.
    `expect` = (forward, backward) prefixes the kernel variant strings must start with."""
    from torch_dwconv import _C

    n, c, h, w, k, s, p = shape
    x, wt, gy = (t.to(dtype) for t in make_inputs(shape, seed=seed))
    rtol, atol, gw_rtol = full_size_tolerances(dtype)
    y_ref, gx_ref, gw_ref, how = full_size_references(shape, x, wt, gy, gpu)
    gw_ref_np = gw_ref if isinstance(gw_ref, np.ndarray) else _np(gw_ref)
    gw_atol = gw_rtol * float(np.abs(gw_ref_np).max())
    rng = np.random.default_rng(seed + 1)
    planes = boundary_planes(n, c, rng, extra=n_planes) if how != "c-oracle" else []
    plane_refs = {}
    for b, ch in planes:
        xs, ws, gs = (_np(t.double()) for t in (x[b:b + 1, ch:ch + 1], wt[ch:ch + 1], gy[b:b + 1, ch:ch + 1]))
        plane_refs[(b, ch)] = (oracle.forward(xs, ws, s, p)[0, 0], oracle.grad_input(gs, ws, (h, w), s, p)[0, 0])
    chans = sorted({0, 1, c // 2, c - 2, c - 1} & set(range(c))) if how != "c-oracle" else []
    if chans:
        gw_c = oracle.grad_weight(_np(x[:, chans].double()), _np(gy[:, chans].double()), (len(chans), 1, k, k), s, p)

    def check(tag, y, gx, gw):
        if y is not None:
            assert_close_on_device(y, y_ref, rtol, atol, f"{tag} y")
        assert_close_on_device(gx, gx_ref, rtol, atol, f"{tag} gx")
        assert_close_on_device(gw, gw_ref, gw_rtol, gw_atol, f"{tag} gw")
        for (b, ch), (yp, gxp) in plane_refs.items():
            if y is not None:
                np.testing.assert_allclose(_np(y[b, ch].double()), yp, rtol=rtol, atol=atol)
            np.testing.assert_allclose(_np(gx[b, ch].double()), gxp, rtol=rtol, atol=atol)
        if chans:
            np.testing.assert_allclose(_np(gw[chans].double()), gw_c, rtol=gw_rtol, atol=gw_atol)

    # the inner products below see every rounding of a 16-bit result once
    adj_tol = 1e-6 if dtype == torch.float32 else 1e-2 * rtol
    for layout in layouts:
        fmt = torch.channels_last if layout == "nhwc" else torch.contiguous_format
        xg, wg, gg = x.to(gpu).contiguous(memory_format=fmt), wt.to(gpu), gy.to(gpu).contiguous(memory_format=fmt)
        with poisoned_allocations():
            y, gx, gw, variant = run_three_passes(dw, xg, wg, gg, s, p)
        v_bwd = ""
        if layout == "nchw":
            # (autograd runs the backward on its own thread; the variant note is per thread)
            _C.dwconv2d_backward(xg, gg, wg, s, s, p, p)
            v_bwd = _C.last_variant()
        _announce(shape_id(shape), str(dtype), layout, how, variant, "|", v_bwd)
        if expect is not None:
            assert variant.startswith(expect[0]) and v_bwd.startswith(expect[1]), (variant, v_bwd, expect)
        assert y.dtype == dtype and gx.dtype == dtype and gw.dtype == dtype
        if layout == "nhwc":
            assert y.is_contiguous(memory_format=torch.channels_last) and gx.is_contiguous(memory_format=torch.channels_last)
        check(f"{shape_id(shape)} {layout} [{variant} | {v_bwd}]", y, gx, gw)
        # size-independent property: <y, gy> == <x, gx> == <w, gw>, accumulated in fp64 on the device
        lhs = (y.double() * gg.double()).sum().item()
        mid = (xg.double() * gx.double()).sum().item()
        rhs = (wg.double() * gw.double()).sum().item()
        scale = (y.double().abs() * gg.double().abs()).sum().item()
        # (a 16-bit grad-weight has few elements, each rounded once: with two or three channels those roundings do
        # not average out, and each may be off by half a step of its own size)
        rhs_round = 0.0 if dtype == torch.float32 else rtol * (wg.double().abs() * gw.double().abs()).sum().item()
        assert abs(lhs - mid) <= adj_tol * scale and abs(lhs - rhs) <= adj_tol * scale + rhs_round
        # bit-identical grad-weight on a second run
        with poisoned_allocations():
            _, _, gw2, _ = run_three_passes(dw, xg, wg, gg, s, p)
        assert torch.equal(gw, gw2)
        if layout == "nhwc":
            continue
        # the two separate backward entry points agree with the references as well, and are deterministic too
        with poisoned_allocations():
            gx3, gw3 = run_separate_backward(xg, wg, gg, s, p)
        check(f"{shape_id(shape)} separate backward", None, gx3, gw3)
        _, gw4 = run_separate_backward(xg, wg, gg, s, p)
        assert torch.equal(gw3, gw4)


def test_cfg1_whole_tensor(dw, gpu):
    check_against_c_oracle(dw, gpu, CFG1)


def test_cfg2_large_map(dw, gpu):
    check_full_size(dw, gpu, CFG2)


@pytest.mark.parametrize("shape", effnet_layers(), ids=shape_id)
def test_efficientnet_b0_layers_full_batch(dw, gpu, shape):
    check_full_size(dw, gpu, shape)


@pytest.mark.parametrize("shape", CFG4 + CONVNEXT_T, ids=shape_id)
def test_large_kernel_small_map_layers(dw, gpu, shape):
    check_full_size(dw, gpu, shape)


def effnet_layers_at(res, batch=128):
    """The 12 layers for a res x res network input (224: 112/56/28/14/7; 256: 128/64/32/16/8; 240: 120/60/30/15/8)."""
    from shapes import EFFNET_B0

    shapes, h = [], res // 2
    for (c, _, k, s) in EFFNET_B0:
        shapes.append((batch, c, h, h, k, s, k // 2))
        h = (h + 2 * (k // 2) - k) // s + 1
    return shapes


@pytest.mark.parametrize("shape", effnet_layers_at(256)[4:] + effnet_layers_at(240)[4:10], ids=shape_id)
def test_small_maps_of_other_resolutions_full_batch(dw, gpu, shape):
    """Maps 32, 16, 8, 30 and 15 wide at batch 128 (the whole-plane kernels' exact and ragged width instances):
    whole tensors against the fp64 reference, outputs start as NaN."""
    check_full_size(dw, gpu, shape, seed=51, expect=("small_down", "small_bwd"))


# Rows that are not whole groups of four elements (EfficientNet at a 300-pixel input: maps 150, 75, 38 wide): the tiled
# kernels move them with four-element accesses at element alignment through buffer views (modes "vin3", "vout3", "vgy3",
# "vgx3" of the variant strings).
ANY_WIDTH = [(2, 3, 40, 150, 3, 1, 1), (2, 3, 41, 75, 3, 1, 1), (2, 3, 38, 38, 5, 1, 2), (2, 3, 75, 75, 5, 2, 2),
             (2, 2, 44, 150, 3, 2, 1), (3, 2, 38, 38, 3, 2, 1), (1, 3, 47, 57, 7, 1, 3), (2, 2, 66, 61, 7, 2, 3),
             (2, 3, 35, 33, 3, 1, 0), (1, 2, 90, 201, 5, 1, 2), (2, 5, 34, 37, 5, 2, 1), (1, 2, 130, 65, 3, 1, 1)]


@pytest.mark.parametrize("shape", ANY_WIDTH, ids=shape_id)
def test_rows_of_any_width_fp32(dw, gpu, shape):
    """Forward, both separate backward passes and the fused backward on rows of 33 ... 201 elements, against the C
    oracle; every pass must have taken the view path, not the element-by-element one."""
    from torch_dwconv import _C

    n, c, h, w, k, s, p = shape
    variant = check_against_c_oracle(dw, gpu, shape, seed=61)
    assert " vin3 " in variant and variant.endswith("vout3"), variant
    x, wt, gy = make_inputs(shape, seed=61)
    xg, wg, gg = x.to(gpu), wt.to(gpu), gy.to(gpu)
    ow = gy.shape[3]
    _C.dwconv2d_backward(xg, gg, wg, s, s, p, p)
    fused = _C.last_variant()
    if fused.startswith("bwd_stack"):  # (5x5 / 7x7 stride-1 "same" layers: the stacked kernel's own any-width instance)
        assert fused.endswith(" anywidth"), fused
    else:
        assert "vin3" in fused and ("vgy3" in fused or ow % 4 == 0), fused
    if s == 2:
        assert "vgx3" in fused, fused
    _C.dwconv2d_backward_kernel(xg, gg, wg, 1, 1, s, s, p, p)
    sep = _C.last_variant()
    assert sep.startswith("wgrad_tile") and "vin3" in sep, sep


def test_rows_of_any_width_unaligned_base(dw, gpu):
    """Rows of whole groups of four whose tensor starts one element past a 16-byte boundary: the same view path."""
    from torch_dwconv import _C

    shape = (2, 3, 40, 48, 3, 1, 1)
    x, wt, gy = make_inputs(shape, seed=62)
    y_ref = oracle.forward(_np(x), _np(wt), 1, 1)
    flat = torch.empty(x.numel() + 1, device=gpu)
    flat[1:] = x.to(gpu).flatten()
    xv = flat[1:].view_as(x)
    y = dw.depthwise_conv2d(xv, wt.to(gpu), padding=1)
    assert " vin3 " in _C.last_variant(), _C.last_variant()
    np.testing.assert_allclose(_np(y), y_ref, rtol=1e-5, atol=1e-5)
    gflat = torch.empty(gy.numel() + 1, device=gpu)
    gflat[1:] = gy.to(gpu).flatten()
    gx, gw = _C.dwconv2d_backward(xv, gflat[1:].view_as(gy), wt.to(gpu), 1, 1, 1, 1)
    assert "vin3" in _C.last_variant() and "vgy3" in _C.last_variant(), _C.last_variant()
    np.testing.assert_allclose(_np(gx), oracle.grad_input(_np(gy), _np(wt), (40, 48), 1, 1), rtol=1e-5, atol=1e-5)
    gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, 1, 1)
    np.testing.assert_allclose(_np(gw), gw_ref, rtol=1e-4, atol=1e-4 * float(np.abs(gw_ref).max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_rows_of_any_width_half_precision(dw, gpu, dtype):
    """16-bit tensors, even and odd widths (odd: every other row starts 2 bytes past a 32-bit boundary; such rows are
    loaded from the boundary before and stored element by element), against the fp64 reference on the rounded inputs."""
    from torch_dwconv import _C

    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for shape, mode in (((2, 3, 40, 150, 3, 1, 1), "vin3"), ((2, 3, 38, 38, 5, 2, 2), "vin3"), ((2, 2, 41, 75, 3, 1, 1), "vin3 vout0"),
                        ((3, 3, 37, 39, 5, 2, 2), "vin3"), ((2, 3, 45, 67, 7, 1, 3), "vin3 vout0"), ((1, 5, 33, 35, 3, 2, 0), "vin3"),
                        ((2, 2, 44, 54, 5, 1, 2), "vin3"), ((1, 3, 50, 70, 7, 2, 3), "vin3")):
        n, c, h, w, k, s, p = shape
        x, wt, gy = (t.to(dtype) for t in make_inputs(shape, seed=63))
        y, gx, gw, variant = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
        _announce(shape_id(shape), str(dtype), variant)
        assert mode in variant or variant.endswith(" anywidth"), variant  # (5x5 / 7x7 "same" layers: the stacked kernel)
        y_ref = oracle.forward(_np(x.double()), _np(wt.double()), s, p)
        gx_ref = oracle.grad_input(_np(gy.double()), _np(wt.double()), (h, w), s, p)
        gw_ref = oracle.grad_weight(_np(x.double()), _np(gy.double()), wt.shape, s, p)
        np.testing.assert_allclose(_np(y.double()), y_ref, rtol=step, atol=1e-5 + step * 1e-2)
        np.testing.assert_allclose(_np(gx.double()), gx_ref, rtol=step, atol=1e-5 + step * 1e-2)
        np.testing.assert_allclose(_np(gw.double()), gw_ref, rtol=step + 1e-4, atol=(step + 1e-4) * float(np.abs(gw_ref).max()))


@pytest.mark.parametrize("shape", [effnet_layers_at(300)[i] for i in (0, 1, 3, 4)], ids=shape_id)
def test_rows_of_any_width_full_batch(dw, gpu, shape):
    """Layers of the 300-pixel stack (150x150 3x3 stride 1 and 2, 75x75 5x5 stride 2, 38x38 5x5) at batch 128: whole
    tensors against the fp64 reference, outputs start as NaN."""
    check_full_size(dw, gpu, shape, seed=64, expect=("tile_down<", "bwd_tile"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", [effnet_layers_at(256)[i] for i in (4, 5, 7, 10)] + [effnet_layers_at(240)[i] for i in (4, 5, 8, 9)], ids=shape_id)
def test_small_maps_of_other_resolutions_half_precision(dw, gpu, shape, dtype):
    check_full_size(dw, gpu, shape, seed=52, dtype=dtype, expect=("small_down16", "small_bwd16"))


def test_stress_grad_weight_determinism(dw, gpu):
    n, c, h, w, k, s, p = STRESS
    check_full_size(dw, gpu, STRESS)
    from torch_dwconv import _C

    x, wt, gy = make_inputs(STRESS, seed=4)
    xg, gg, wg = x.to(gpu), gy.to(gpu), wt.to(gpu)
    runs = [_C.dwconv2d_backward_kernel(xg, gg, wg, 1, 1, s, s, p, p) for _ in range(5)]
    torch.cuda.synchronize()
    for r in runs[1:]:
        assert torch.equal(runs[0], r)


# 16-bit tensors at the batch the benchmark runs: chunk counts, planes per tile, the XCD mapping and the remainder
# paths are functions of the tensor sizes, so the small shapes of test_half_precision_io never reach them.
HALF_FULL_SIZE = {
    0: ("tile_down16_dot2", "bwd_tile16_dot2"),    # 112x112 C32 3x3: 16-bit LDS images, fused backward
    1: ("tile_down16_dot2", "bwd_tile_s216"),      # 112x112 C96 3x3 stride 2
    2: ("tile_down16<", "bwd_stack16<k3"),         # 56x56 C144 3x3: backward one channel per workgroup over its stacked images
    3: ("tile_down16_dot2", "bwd_tile_s216"),      # 56x56 C144 5x5 stride 2 (16-bit LDS image from 48 columns on at stride 2)
    4: ("small_down16", "small_bwd16"),            # 28x28 C240 5x5
    5: ("small_down16", "small_bwd16"),            # 28x28 C240 3x3 stride 2
    8: ("small_down16", "small_bwd16"),            # 14x14 C672 5x5
    9: ("small_down16", "small_bwd16"),            # 14x14 C672 5x5 stride 2
    10: ("small_down16", "small_bwd16"),           # 7x7 C1152 5x5
}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("layer", sorted(HALF_FULL_SIZE), ids=lambda i: shape_id(effnet_layers()[i]))
def test_half_precision_full_batch(dw, gpu, layer, dtype):
    """EfficientNet-B0 layers at batch 128 with 16-bit tensors: whole tensors against the fp64 reference on the
    rounded inputs (outputs start as NaN), one rounding step of tolerance, bit-identical grad-weight."""
    check_full_size(dw, gpu, effnet_layers()[layer], seed=41, dtype=dtype, expect=HALF_FULL_SIZE[layer])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_half_precision_full_batch_stacked_forward(dw, gpu, dtype):
    """The 3x3 instance of the stacked-image kernel in the forward pass (taken at the widths where it measured faster
    than the general tiled kernel: 48, 60, 64, 72), at the batch of the benchmark."""
    check_full_size(dw, gpu, (128, 144, 48, 48, 3, 1, 1), seed=45, dtype=dtype, expect=("tile_stack16<k3", "bwd_stack16<k3"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_half_precision_full_batch_general_tiled_kernels(dw, gpu, dtype, monkeypatch):
    """The 16-bit instances of the general tiled kernels on the 56x56 3x3 layer (they serve what the stacked-image
    kernel does not take: rows of odd width, tensors off a 32-bit boundary, small planes)."""
    monkeypatch.setenv("DWCONV_TUNING", "1")
    monkeypatch.setenv("DWCONV_STACK_K3_16", "0")
    check_full_size(dw, gpu, effnet_layers()[2], seed=41, dtype=dtype, expect=("tile_down16<", "bwd_tile16<"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_half_precision_large_maps_full_size(dw, gpu, dtype):
    check_full_size(dw, gpu, CFG2, seed=43, dtype=dtype)
    check_full_size(dw, gpu, CONVNEXT_T[0], seed=44, dtype=dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_half_precision_several_tiles_per_workgroup(dw, gpu, dtype, monkeypatch):
    """A workgroup of the fused 16-bit backward that walks three or more tiles (sums carried over tiles, strided
    chunk walk, grad-input streamed out of LDS between tiles), forced on a small tensor by capping the grid."""
    monkeypatch.setenv("DWCONV_WGRAD_WGS", "8")
    monkeypatch.setenv("DWCONV_TUNING", "1")
    shape = (9, 4, 40, 104, 3, 1, 1)
    check_full_size(dw, gpu, shape, seed=45, dtype=dtype, expect=("tile_down16_dot2", "bwd_tile16_dot2"))
    check_full_size(dw, gpu, (13, 3, 37, 96, 5, 1, 2), seed=46, dtype=dtype, expect=("tile_down16_dot2", "bwd_tile16_dot2"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
def test_stride2_backward_two_step_staging(dw, gpu, dtype, monkeypatch):
    """The fused stride-2 backward whose tile images travel in two steps (loads issued during one arithmetic phase,
    written into LDS after it): the default with 16-bit elements, reachable with fp32 ones through the tuning switch.
    The grid is capped so that every workgroup walks several tiles; heights that leave a partial last band, filters
    3x3 / 5x5 / 7x7."""
    from torch_dwconv import _C

    monkeypatch.setenv("DWCONV_TUNING", "1")
    monkeypatch.setenv("DWCONV_WGRAD_WGS", "8")
    monkeypatch.setenv("DWCONV_S2_PREFETCH", "2")
    for i, shape in enumerate([(9, 4, 40, 104, 3, 2, 1), (7, 3, 37, 96, 5, 2, 2), (5, 2, 70, 64, 7, 2, 3),
                               (4, 3, 130, 128, 3, 2, 1), (3, 2, 300, 72, 5, 2, 2)]):
        x, wt, gy = (t.to(dtype).to(gpu) for t in make_inputs(shape, seed=60 + i))
        _C.dwconv2d_backward(x, gy, wt, shape[5], shape[5], shape[6], shape[6])
        assert _C.last_variant().startswith("bwd_tile_s2") and _C.last_variant().endswith(" pf"), _C.last_variant()
        check_full_size(dw, gpu, shape, seed=60 + i, dtype=dtype)


# ---- closed forms on the device ----------------------------------------------------------
def test_delta_filter_is_identity_bitwise(dw, gpu):
    x = torch.randn(3, 5, 56, 56, device=gpu)
    for k in (3, 5, 7):
        w = torch.zeros(5, 1, k, k, device=gpu)
        w[:, 0, k // 2, k // 2] = 1.0
        assert torch.equal(dw.depthwise_conv2d(x, w, padding=k // 2), x)


def test_linearity_on_device(dw, gpu):
    x1, x2 = torch.randn(2, 4, 30, 33, device=gpu), torch.randn(2, 4, 30, 33, device=gpu)
    w = torch.randn(4, 1, 5, 5, device=gpu) / 5
    a = dw.depthwise_conv2d(x1 + x2, w, stride=2, padding=2)
    b = dw.depthwise_conv2d(x1, w, stride=2, padding=2) + dw.depthwise_conv2d(x2, w, stride=2, padding=2)
    torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)


# ---- boundary behaviour ---------------------------------------------------------------------
def test_empty_and_degenerate_inputs(dw, gpu):
    w = torch.randn(4, 1, 3, 3, device=gpu)
    y = dw.depthwise_conv2d(torch.empty(0, 4, 8, 8, device=gpu), w, padding=1)
    assert y.shape == (0, 4, 8, 8)
    # plane smaller than the filter and no padding: empty output
    x = torch.randn(1, 4, 2, 2, device=gpu, requires_grad=True)
    wp = w.clone().requires_grad_(True)
    y = dw.depthwise_conv2d(x, wp)
    assert y.shape == (1, 4, 0, 0)
    gx, gw = torch.autograd.grad(y, (x, wp), torch.empty_like(y))
    assert torch.count_nonzero(gx) == 0 and torch.count_nonzero(gw) == 0


def test_unaligned_and_noncontiguous_inputs(dw, gpu):
    shape = (2, 3, 20, 24, 3, 1, 1)
    x, wt, gy = make_inputs(shape, seed=8)
    y_ref = oracle.forward(_np(x), _np(wt), 1, 1)
    # contiguous but only 4-byte aligned: a view one element into a flat buffer
    flat = torch.empty(x.numel() + 1, device=gpu)
    flat[1:] = x.to(gpu).flatten()
    xv = flat[1:].view_as(x)
    assert xv.data_ptr() % 16 != 0 and xv.is_contiguous()
    np.testing.assert_allclose(_np(dw.depthwise_conv2d(xv, wt.to(gpu), padding=1)), y_ref, rtol=1e-5, atol=1e-5)
    # non-contiguous (channels-last memory): made contiguous by the binding, like the reference (:855-856)
    xc = x.to(gpu).contiguous(memory_format=torch.channels_last)
    np.testing.assert_allclose(_np(dw.depthwise_conv2d(xc, wt.to(gpu), padding=1)), y_ref, rtol=1e-5, atol=1e-5)


def test_rectangular_filter_stride_and_padding(dw, gpu):
    g = torch.Generator("cpu").manual_seed(11)
    x = torch.randn(2, 3, 12, 10, generator=g)
    wt = torch.randn(3, 1, 5, 2, generator=g)
    s, p = (2, 1), (1, 0)
    oh, ow = (12 + 2 - 5) // 2 + 1, (10 - 2) // 1 + 1
    gy = torch.randn(2, 3, oh, ow, generator=g)
    y, gx, gw, _ = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    assert_parity(y, gx, gw, oracle.forward(_np(x), _np(wt), s, p), oracle.grad_input(_np(gy), _np(wt), (12, 10), s, p),
                  oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p), torch.float32)


def test_c_entry_points_directly(dw, gpu):
    """The generic operator with asymmetric pads / up and down together, and the small entry point."""
    from torch_dwconv import _C

    g = torch.Generator("cpu").manual_seed(5)
    x = torch.randn(2, 3, 9, 11, generator=g)
    for (kh, kw, up, down, pads, fwd) in [(3, 3, 2, 1, (1, 2, 0, 3), False), (5, 5, 2, 2, (2, 1, 3, 0), True),
                                           (4, 3, 3, 2, (0, 0, 1, 1), False), (3, 3, 1, 1, (2, 0, 0, 2), True)]:
        wt = torch.randn(3, 1, kh, kw, generator=g)
        got = _C.dwconv2d(x.to(gpu), wt.to(gpu), up, up, down, down, *pads, fwd)
        ref = oracle.dwconv2d(_np(x), _np(wt), up, up, down, down, *pads, fwd)
        np.testing.assert_allclose(_np(got), ref, rtol=1e-5, atol=1e-5)
    for (kh, kw, ph, pw, fwd) in [(3, 3, 1, 1, True), (5, 5, 2, 2, False), (5, 3, 0, 2, True), (7, 7, 3, 3, False)]:
        wt = torch.randn(3, 1, kh, kw, generator=g)
        got = _C.dwconv2d_small(x.to(gpu), wt.to(gpu), 1, 1, 1, 1, ph, pw, fwd)
        ref = oracle.dwconv2d_small(_np(x), _np(wt), ph, pw, fwd)
        np.testing.assert_allclose(_np(got), ref, rtol=1e-5, atol=1e-5)
    with pytest.raises(RuntimeError, match="stride-1"):
        _C.dwconv2d_small(x.to(gpu), torch.randn(3, 1, 3, 3, device=gpu), 1, 1, 2, 2, 1, 1, True)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.dwconv2d(x, torch.randn(3, 1, 3, 3, device=gpu), 1, 1, 1, 1, 1, 1, 1, 1, True)


# (n, c, h, w, kh, kw, up_h, up_w, down_h, down_w, (pad_h0, pad_h1, pad_w0, pad_w1), forward)
F64_OPERATOR = [
    (2, 3, 9, 11, 3, 3, 1, 1, 1, 1, (1, 1, 1, 1), True), (2, 3, 9, 11, 3, 3, 2, 2, 1, 1, (1, 2, 0, 3), False),
    (2, 3, 23, 17, 5, 5, 2, 2, 2, 2, (2, 1, 3, 0), True), (1, 4, 19, 30, 4, 3, 3, 2, 2, 1, (0, 0, 1, 1), False),
    (2, 2, 40, 37, 3, 3, 1, 1, 1, 1, (2, 0, -1, 2), True), (1, 2, 31, 45, 7, 7, 1, 1, 2, 2, (3, 3, 3, 3), True),
    (3, 5, 7, 7, 5, 5, 1, 1, 1, 1, (2, 2, 2, 2), False), (2, 40, 6, 5, 3, 3, 1, 1, 1, 1, (1, 1, 1, 1), True),
    (1, 2, 70, 130, 9, 5, 1, 1, 3, 2, (4, 1, -2, 4), True), (1, 1, 150, 260, 13, 13, 1, 1, 1, 1, (6, 6, 6, 6), False),
    (2, 3, 28, 28, 5, 5, 2, 2, 1, 1, (2, 3, 2, 3), False), (1, 2, 1, 1, 3, 3, 1, 1, 1, 1, (1, 1, 1, 1), True),
]


@pytest.mark.parametrize("case", F64_OPERATOR, ids=lambda c: "N%d_C%d_%dx%d_k%dx%d_u%dx%d_d%dx%d_%s" % (c[:10] + ("fwd" if c[11] else "rot",)))
def test_fp64_tiled_operator(gpu, case):
    """The raw operator on double tensors through the LDS-tiled fp64 kernel (up- and down-sampling together, pads that
    differ per side and crop, rotated taps, several planes per workgroup, several bands per plane) against the C
    oracle to 1e-12."""
    from torch_dwconv import _C

    n, c, h, w, kh, kw, uh, uw, dh, dw_, pads, fwd = case
    g = torch.Generator("cpu").manual_seed(17)
    x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64)
    wt = torch.randn(c, 1, kh, kw, generator=g, dtype=torch.float64)
    got = _C.dwconv2d(x.to(gpu), wt.to(gpu), uh, uw, dh, dw_, *pads, fwd)
    variant = _C.last_variant()
    _announce(case, variant)
    assert variant.startswith("tile_f64<k%dx%d,u%dx%d,s%dx%d,%s>" % (kh, kw, uh, uw, dh, dw_, "fwd" if fwd else "rot")), variant
    ref = oracle.dwconv2d(_np(x), _np(wt), uh, uw, dh, dw_, *pads, fwd)
    assert _np(got).shape == ref.shape
    np.testing.assert_allclose(_np(got), ref, rtol=1e-12, atol=1e-12)


F64_GRAD_WEIGHT = [(2, 3, 9, 11, 3, 3, 1, 1, 1, 1), (3, 4, 28, 28, 5, 5, 2, 2, 2, 2), (5, 6, 7, 7, 5, 5, 1, 1, 2, 2),
                   (2, 2, 57, 83, 7, 7, 1, 1, 3, 3), (1, 2, 40, 44, 9, 4, 3, 2, 4, 0), (9, 3, 14, 14, 3, 3, 1, 1, 1, 1),
                   (2, 1, 130, 150, 3, 3, 1, 1, 1, 1), (33, 2, 6, 6, 7, 7, 1, 1, 3, 3)]


@pytest.mark.parametrize("case", F64_GRAD_WEIGHT, ids=lambda c: "N%d_C%d_%dx%d_k%dx%d_s%dx%d_p%dx%d" % c)
def test_fp64_tiled_grad_weight(gpu, case):
    """Grad-weight on double tensors through the LDS-tiled fp64 kernel (one to two passes of 32 taps, several images
    per tile on small planes, several bands on large ones) against the C oracle to 1e-11 of the largest sum; the same
    bits on a second run."""
    from torch_dwconv import _C

    n, c, h, w, kh, kw, sh, sw, ph, pw = case
    g = torch.Generator("cpu").manual_seed(23)
    x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64)
    oh, ow = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
    gy = torch.randn(n, c, oh, ow, generator=g, dtype=torch.float64)
    wt = torch.empty(c, 1, kh, kw, dtype=torch.float64)
    got = _C.dwconv2d_backward_kernel(x.to(gpu), gy.to(gpu), wt.to(gpu), 1, 1, sh, sw, ph, pw)
    variant = _C.last_variant()
    _announce(case, variant)
    assert variant.startswith("wgrad_f64<k%dx%d,s%dx%d>" % (kh, kw, sh, sw)), variant
    assert ("passes%d" % ((kh * kw + 31) // 32)) in variant, variant
    ref = oracle.backward_kernel(_np(x), _np(gy), (kh, kw), sh, sw, ph, pw)
    np.testing.assert_allclose(_np(got).reshape(ref.shape), ref, rtol=1e-11, atol=1e-11 * float(np.abs(ref).max()))
    again = _C.dwconv2d_backward_kernel(x.to(gpu), gy.to(gpu), wt.to(gpu), 1, 1, sh, sw, ph, pw)
    assert torch.equal(got, again)


HALF_SHAPES = [(2, 6, 14, 14, 3, 1, 1), (2, 5, 28, 28, 5, 2, 2), (2, 4, 56, 56, 3, 1, 1), (2, 3, 57, 59, 5, 2, 2),
               (1, 8, 7, 7, 5, 1, 2), (2, 4, 112, 112, 3, 2, 1), (1, 2, 33, 35, 7, 1, 3), (2, 8, 14, 14, 5, 2, 2),
               (3, 4, 28, 28, 7, 1, 3), (2, 8, 7, 7, 7, 1, 3), (2, 3, 64, 64, 5, 2, 2), (2, 3, 40, 44, 7, 2, 3),
               (3, 5, 14, 14, 7, 1, 3), (1, 3, 9, 11, 4, 2, 1),
               # whole-plane kernels, other widths (exact 8/16/32, ragged classes)
               (2, 8, 8, 8, 5, 1, 2), (2, 6, 16, 16, 3, 1, 1), (2, 4, 32, 32, 5, 2, 2), (2, 8, 15, 15, 5, 1, 2),
               (2, 8, 15, 15, 3, 2, 1), (2, 4, 30, 30, 7, 1, 3), (2, 4, 20, 12, 3, 1, 1), (3, 5, 15, 15, 5, 1, 2),
               (3, 5, 57, 64, 7, 1, 3), (2, 3, 33, 72, 5, 1, 2),
               (3, 3, 31, 31, 3, 2, 1), (2, 6, 24, 24, 5, 1, 2), (3, 5, 12, 12, 3, 2, 1), (3, 5, 9, 10, 3, 1, 1),
               # rows of at least 96 elements in whole groups of eight: the kernels with 16-bit LDS images and
               # two-element dot products (7-row and 4-row blocks, several planes per workgroup, odd heights)
               (1, 3, 96, 104, 3, 1, 1), (1, 2, 100, 96, 5, 1, 2), (1, 2, 98, 112, 7, 1, 3), (1, 2, 97, 120, 5, 2, 2),
               (1, 12, 8, 96, 3, 1, 1), (2, 5, 6, 128, 5, 1, 2), (1, 2, 61, 104, 7, 2, 3), (1, 3, 30, 96, 3, 2, 1),
               # the same kernels on narrower rows: from 48 columns at stride 2, from 72 at stride 1
               (2, 5, 30, 48, 3, 2, 1), (3, 4, 56, 56, 5, 2, 2), (2, 3, 33, 72, 7, 1, 3), (2, 6, 20, 88, 3, 1, 1),
               (1, 7, 41, 64, 7, 2, 3), (5, 3, 9, 80, 5, 1, 2)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", HALF_SHAPES, ids=shape_id)
def test_half_precision_io(dw, gpu, shape, dtype):
    """16-bit tensors in and out, fp32 arithmetic inside: the only error is the final rounding of each result.
    The oracle runs in fp64 on the already rounded inputs; tolerance = one rounding step of the 16-bit format
    (2^-11 for fp16, 2^-8 for bf16) plus the fp32 bounds used elsewhere."""
    n, c, h, w, k, s, p = shape
    x, wt, gy = (t.to(dtype) for t in make_inputs(shape, seed=17))
    y, gx, gw, variant = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    _announce(shape_id(shape), str(dtype), variant)
    assert y.dtype == dtype and gx.dtype == dtype and gw.dtype == dtype
    xr, wr, gr = (_np(t.double()) for t in (x, wt, gy))
    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    y_ref = oracle.forward(xr, wr, s, p)
    gx_ref = oracle.grad_input(gr, wr, (h, w), s, p)
    gw_ref = oracle.grad_weight(xr, gr, wt.shape, s, p)
    np.testing.assert_allclose(_np(y.double()), y_ref, rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gx.double()), gx_ref, rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gw.double()), gw_ref, rtol=step + 1e-4, atol=(step + 1e-4) * float(np.abs(gw_ref).max()))
    # bit-identical grad-weight from run to run here too
    _, _, gw2, _ = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    assert torch.equal(gw, gw2)
    # the two entry points the reference's backward calls, and tensors whose base is not aligned to four elements
    gx_s, gw_s = run_separate_backward(x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
    np.testing.assert_allclose(_np(gx_s.double()), gx_ref, rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gw_s.double()), gw_ref, rtol=step + 1e-4, atol=(step + 1e-4) * float(np.abs(gw_ref).max()))

    def shifted(t):
        flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=gpu)
        flat[1:] = t.to(gpu).reshape(-1)
        return flat[1:].view(t.shape)

    # (such tensors take another kernel, which adds the fp32 products in another order: the same bound against the
    # oracle, not bit equality with the aligned run)
    y_u, gx_u, gw_u, _ = run_three_passes(dw, shifted(x), wt.to(gpu), shifted(gy), s, p)
    np.testing.assert_allclose(_np(y_u.double()), y_ref, rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gx_u.double()), gx_ref, rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gw_u.double()), gw_ref, rtol=step + 1e-4, atol=(step + 1e-4) * float(np.abs(gw_ref).max()))


def test_half_precision_uses_the_fast_kernels(dw, gpu):
    """fp16 tensors of the benchmark's layer shapes go through the tiled / whole-plane kernels, not the generic one."""
    from torch_dwconv import _C

    for shape, fwd, bwd in [((2, 8, 112, 112, 3, 1, 1), "tile_down16_dot2", "bwd_tile16_dot2"),
                            ((2, 8, 112, 112, 3, 2, 1), "tile_down16_dot2", "bwd_tile_s216"),
                            ((2, 8, 56, 56, 3, 1, 1), "tile_down16<", "bwd_stack16<k3"),
                            ((2, 8, 48, 48, 3, 1, 1), "tile_stack16<k3", "bwd_stack16<k3"),
                            ((2, 8, 56, 54, 3, 1, 1), "tile_down16<", "bwd_stack16<k3"),
                            ((2, 8, 56, 55, 3, 1, 1), "tile_down16<", "bwd_tile16<"),
                            ((2, 8, 14, 14, 5, 1, 2), "small_down16", "small_bwd16"),
                            ((2, 8, 28, 28, 3, 1, 1), "small_down16", "small_bwd16")]:
        n, c, h, w, k, s, p = shape
        x, wt, gy = (t.to(torch.float16).to(gpu) for t in make_inputs(shape, seed=3))
        dw.depthwise_conv2d(x, wt, stride=s, padding=p)
        assert _C.last_variant().startswith(fwd), _C.last_variant()
        _C.dwconv2d_backward(x, gy, wt, s, s, p, p)
        assert _C.last_variant().startswith(bwd), _C.last_variant()


def test_stacked_kernel_routes(dw, gpu):
    """Which stride-1 "same" layers the stacked-image kernel takes: fp32 forward only 7x7 filters on aligned rows up to
    116 elements (the general tiled kernel measured faster elsewhere); the fused backward 5x5 and 7x7 at any width,
    with its own instance for rows that are not whole groups of four."""
    from torch_dwconv import _C

    for shape, fwd, bwd in [((2, 4, 64, 64, 5, 1, 2), "tile_down<k5", "bwd_stack<k5"),
                            ((2, 4, 56, 56, 7, 1, 3), "tile_stack<k7", "bwd_stack<k7"),
                            ((1, 3, 40, 128, 7, 1, 3), "tile_down<k7", "bwd_stack<k7"),
                            ((2, 3, 57, 57, 5, 1, 2), "tile_down<k5", "bwd_stack<k5"),
                            ((2, 3, 46, 66, 7, 1, 3), "tile_down<k7", "bwd_stack<k7")]:
        n, c, h, w, k, s, p = shape
        variant = check_against_c_oracle(dw, gpu, shape, seed=71)
        assert variant.startswith(fwd), variant
        x, wt, gy = (t.to(gpu) for t in make_inputs(shape, seed=71))
        _C.dwconv2d_backward(x, gy, wt, s, s, p, p)
        assert _C.last_variant().startswith(bwd), _C.last_variant()
        assert _C.last_variant().endswith(" anywidth") == (w % 4 != 0), _C.last_variant()


LARGE_FILTERS = [(2, 3, 20, 24, 9, 1, 4), (3, 2, 33, 57, 9, 1, 4), (1, 4, 9, 12, 9, 1, 4), (2, 2, 41, 40, 11, 1, 5),
                 (2, 3, 14, 14, 11, 1, 5), (1, 2, 70, 31, 11, 1, 5), (2, 2, 28, 28, 13, 1, 6), (3, 1, 37, 66, 13, 1, 6),
                 (1, 3, 5, 8, 13, 1, 6), (5, 2, 6, 97, 13, 1, 6)]


@pytest.mark.parametrize("shape", LARGE_FILTERS, ids=shape_id)
def test_large_filters_take_the_stacked_kernels(dw, gpu, shape):
    """9x9, 11x11 and 13x13 stride-1 "same" layers (planes from 5 rows and 8 columns on, any width): forward, both
    separate passes and the fused backward through the stacked-image kernels, against the C oracle."""
    from torch_dwconv import _C

    n, c, h, w, k, s, p = shape
    variant = check_against_c_oracle(dw, gpu, shape, seed=81)
    assert variant.startswith("tile_stack<k%d,d1,s1,fwd>" % k), variant
    x, wt, gy = (t.to(gpu) for t in make_inputs(shape, seed=81))
    gx, gw = _C.dwconv2d_backward(x, gy, wt, s, s, p, p)
    assert _C.last_variant().startswith("bwd_stack<k%d,d1,s1>" % k), _C.last_variant()
    gx2, gw2 = _C.dwconv2d_backward(x, gy, wt, s, s, p, p)
    assert torch.equal(gw, gw2) and torch.equal(gx, gx2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_large_filters_half_precision(dw, gpu, dtype):
    from torch_dwconv import _C

    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for shape in [(2, 3, 20, 24, 9, 1, 4), (2, 2, 33, 58, 11, 1, 5), (2, 2, 28, 28, 13, 1, 6)]:
        n, c, h, w, k, s, p = shape
        x, wt, gy = (t.to(dtype) for t in make_inputs(shape, seed=82))
        y, gx, gw, variant = run_three_passes(dw, x.to(gpu), wt.to(gpu), gy.to(gpu), s, p)
        _announce(shape_id(shape), str(dtype), variant)
        assert variant.startswith("tile_stack16<k%d" % k), variant
        y_ref = oracle.forward(_np(x.double()), _np(wt.double()), s, p)
        gx_ref = oracle.grad_input(_np(gy.double()), _np(wt.double()), (h, w), s, p)
        gw_ref = oracle.grad_weight(_np(x.double()), _np(gy.double()), wt.shape, s, p)
        np.testing.assert_allclose(_np(y.double()), y_ref, rtol=step, atol=1e-5 + step * 2e-2)
        np.testing.assert_allclose(_np(gx.double()), gx_ref, rtol=step, atol=1e-5 + step * 2e-2)
        np.testing.assert_allclose(_np(gw.double()), gw_ref, rtol=step + 1e-4, atol=(step + 1e-4) * float(np.abs(gw_ref).max()))


@pytest.mark.parametrize("shape", [(64, 96, 56, 56, 9, 1, 4), (64, 192, 28, 28, 11, 1, 5), (64, 384, 14, 14, 13, 1, 6)], ids=shape_id)
def test_large_filters_full_size(dw, gpu, shape):
    """ConvNeXt-T's first three stages with 9x9, 11x11 and 13x13 filters at batch 64: whole tensors against the fp64
    reference, outputs start as NaN."""
    k = shape[4]
    check_full_size(dw, gpu, shape, seed=83, expect=("tile_stack<k%d" % k, "bwd_stack<k%d" % k))


# (N, C, H, W, KH, KW, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w): what only the any-geometry tiled kernels serve
ANY_GEOMETRY = [
    (2, 3, 40, 48, 1, 7, 1, 1, 0, 3, 1, 1), (2, 3, 40, 48, 7, 1, 1, 1, 3, 0, 1, 1), (1, 2, 33, 57, 1, 21, 1, 1, 0, 10, 1, 1),
    (1, 2, 57, 33, 21, 1, 1, 1, 10, 0, 1, 1), (2, 2, 30, 30, 4, 4, 1, 1, 1, 2, 1, 1), (2, 3, 21, 26, 2, 2, 2, 2, 0, 0, 1, 1),
    (2, 2, 50, 61, 3, 5, 1, 2, 1, 2, 1, 1), (1, 3, 64, 64, 3, 3, 3, 3, 1, 1, 1, 1), (1, 2, 45, 47, 5, 5, 4, 4, 2, 2, 1, 1),
    (1, 2, 40, 44, 10, 10, 1, 1, 4, 5, 1, 1), (1, 1, 36, 40, 15, 15, 1, 1, 7, 7, 1, 1),
    (2, 2, 33, 33, 3, 3, 1, 1, 6, 6, 6, 6), (1, 2, 65, 65, 3, 3, 1, 1, 18, 18, 18, 18), (2, 2, 40, 52, 3, 3, 1, 1, 3, 3, 3, 3),
    (1, 3, 50, 38, 5, 3, 2, 1, 4, 2, 2, 3), (2, 2, 12, 70, 1, 1, 1, 1, 0, 0, 1, 1),
    # rows of taps walked four at a time (column stride and dilation 1, wider than the register windows)
    (1, 2, 40, 44, 31, 31, 1, 1, 15, 15, 1, 1), (2, 2, 37, 51, 9, 17, 1, 1, 4, 8, 1, 1), (1, 3, 61, 43, 17, 3, 2, 1, 16, 1, 2, 1),
    (2, 2, 29, 66, 3, 9, 1, 1, 1, 4, 1, 1), (1, 2, 48, 39, 5, 6, 3, 1, 2, 3, 1, 1),
    # tap offsets at every position within a 16-byte LDS read, column strides 1 and 2
    (2, 2, 41, 53, 3, 3, 1, 1, 5, 5, 5, 5), (1, 3, 47, 45, 3, 3, 1, 1, 7, 7, 7, 7), (2, 3, 41, 53, 4, 4, 2, 2, 1, 1, 1, 1),
    (1, 2, 50, 38, 3, 3, 2, 2, 3, 3, 3, 3), (2, 2, 33, 70, 2, 5, 1, 2, 0, 5, 1, 3),
    # small planes: grad-weight with several channels to a workgroup (the last group short of channels)
    (3, 7, 14, 14, 15, 15, 1, 1, 7, 7, 1, 1), (2, 40, 7, 7, 9, 9, 1, 1, 4, 4, 1, 1), (2, 5, 20, 24, 4, 4, 1, 1, 1, 2, 1, 1),
    (2, 7, 33, 33, 3, 3, 1, 1, 6, 6, 6, 6), (4, 9, 12, 10, 1, 7, 1, 1, 0, 3, 1, 1), (3, 11, 9, 13, 3, 3, 2, 2, 2, 2, 2, 2),
]


def any_geometry_walks(kh, kw, sh, sw, dh, dw_):
    """Whether the any-geometry kernels walk the filter rows four taps at a time: column stride and dilation 1, three
    taps a row or more, and no register-window instance that holds the filter."""
    plain = (sh, sw, dh, dw_) == (1, 1, 1, 1)
    windowed = plain and ((kh == 1 and kw <= 24) or (kw == 1 and kh <= 24) or (kh <= 8 and kw <= 8))
    return not windowed and sw == 1 and dw_ == 1 and kw >= 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", ANY_GEOMETRY, ids=lambda c: "N%d_C%d_%dx%d_k%dx%d_s%dx%d_p%dx%d_d%dx%d" % c)
def test_any_geometry_tiled_kernels(dw, gpu, case, dtype):
    """Rectangular, even-sized and strip filters, strides above 2 and dilations above 2: forward, grad-input (the
    correlation with the rotated taps where the stride is 1) and grad-weight through the tiled kernels that loop over
    their taps at run time, against fp64 autograd on the rounded inputs; bit-identical grad-weight."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_general

    n, c, h, w, kh, kw, sh, sw, ph, pw, dh, dw_ = case
    step = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    g = torch.Generator("cpu").manual_seed(91)
    x = torch.randn(n, c, h, w, generator=g).to(dtype)
    wt = (torch.randn(c, 1, kh, kw, generator=g) / (kh * kw) ** 0.5).to(dtype)
    xr, wr = x.double().requires_grad_(True), wt.double().requires_grad_(True)
    y_ref = torch.nn.functional.conv2d(xr, wr, stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw_), groups=c)
    gy = torch.randn(y_ref.shape, generator=g).to(dtype)
    gx_ref, gw_ref = torch.autograd.grad(y_ref, (xr, wr), gy.double())
    xg, wg = x.to(gpu).requires_grad_(True), wt.to(gpu).requires_grad_(True)
    if (dh, dw_) == (1, 1):
        y = dw.depthwise_conv2d(xg, wg, stride=(sh, sw), padding=(ph, pw))
    else:
        y = depthwise_conv2d_general(xg, wg, stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw_))
    v_fwd = _C.last_variant()
    _announce(case, str(dtype), v_fwd)
    sfx = "" if dtype == torch.float32 else "16"
    assert v_fwd.startswith("tile_any%s<k%dx%d,s%dx%d,d%dx%d,fwd>" % (sfx, kh, kw, sh, sw, dh, dw_)), v_fwd
    walks = any_geometry_walks(kh, kw, sh, sw, dh, dw_)
    assert v_fwd.endswith(" walk4") == walks, v_fwd
    gx, gw = torch.autograd.grad(y, (xg, wg), gy.to(gpu))
    # (the variant note is per thread and autograd runs the backward on its own: the same calls again from here)
    if (dh, dw_) == (1, 1):
        _, gw2 = _C.dwconv2d_backward(xg.detach(), gy.to(gpu), wg.detach(), sh, sw, ph, pw)
    else:
        _, gw2 = _C.dwconv2d_general_backward(xg.detach(), gy.to(gpu), wg.detach(), sh, sw, ph, pw, dh, dw_)
    v_bwd = _C.last_variant()
    assert "wgrad_any%s<k%dx%d" % (sfx, kh, kw) in v_bwd, v_bwd
    # grad-input: the same kernel with rotated taps at stride 1, above it the up-sampling tiled kernel
    # (dilated layers above stride 1: the per-element kernel)
    assert ("tile_any%s<" % sfx in v_bwd and ",rot>" in v_bwd) == ((sh, sw) == (1, 1)), v_bwd
    assert ("tile_gen%s<k%dx%d,u%dx%d,s1x1,rot>" % (sfx, kh, kw, sh, sw) in v_bwd) == ((sh, sw) != (1, 1) and (dh, dw_) == (1, 1)), v_bwd
    # sixty-four sums a pass: sixteen groups of four taps of a row where the rows are walked, else sixty-four taps
    passes = (kh * ((kw + 3) // 4) + 15) // 16 if walks else (kh * kw + 63) // 64
    assert ("passes%d " % passes) in v_bwd, v_bwd
    assert v_bwd.endswith(" walk4") == walks, v_bwd
    assert torch.equal(gw, gw2)
    tol = 1e-5 + step
    np.testing.assert_allclose(_np(y.detach().double()), y_ref.detach().numpy(), rtol=tol, atol=tol)
    np.testing.assert_allclose(_np(gx.double()), gx_ref.numpy(), rtol=tol, atol=tol)
    gtol = 1e-4 + step
    np.testing.assert_allclose(_np(gw.double()), gw_ref.numpy(), rtol=gtol, atol=gtol * float(gw_ref.abs().max()))


def test_tuning_overrides_need_the_master_switch(dw, gpu, monkeypatch):
    """DWCONV_* overrides of the planners are ignored unless DWCONV_TUNING=1 is set too, and ill-formed values always."""
    from torch_dwconv import _C

    x, wt, _ = make_inputs((2, 8, 14, 14, 3, 1, 1), seed=2)
    xg, wg = x.to(gpu), wt.to(gpu)
    monkeypatch.setenv("DWCONV_NO_SMALL", "1")
    dw.depthwise_conv2d(xg, wg, padding=1)
    assert _C.last_variant().startswith("small_down"), _C.last_variant()
    monkeypatch.setenv("DWCONV_TUNING", "1")
    dw.depthwise_conv2d(xg, wg, padding=1)
    assert _C.last_variant().startswith("tile_down"), _C.last_variant()
    monkeypatch.setenv("DWCONV_NO_SMALL", "yes")   # not a number: ignored
    dw.depthwise_conv2d(xg, wg, padding=1)
    assert _C.last_variant().startswith("small_down"), _C.last_variant()
    monkeypatch.setenv("DWCONV_NO_SMALL", "-1")    # out of range: ignored
    dw.depthwise_conv2d(xg, wg, padding=1)
    assert _C.last_variant().startswith("small_down"), _C.last_variant()


def test_combined_backward_entry_point(dw, gpu):
    """dwconv2d_backward: fused kernels where they exist, the two separate passes otherwise; errors as status codes."""
    from torch_dwconv import _C

    cases = [(2, 6, 14, 14, 3, 1, 1), (2, 6, 30, 33, 5, 2, 2), (2, 3, 40, 44, 3, 1, 0), (1, 4, 64, 64, 5, 1, 2),
             (2, 4, 64, 48, 3, 2, 1), (1, 2, 20, 20, 4, 2, 1), (2, 3, 31, 29, 7, 2, 3), (2, 3, 48, 52, 5, 2, 0),
             (2, 3, 64, 64, 3, 1, 1)]
    seen = set()
    for shape in cases:
        n, c, h, w, k, s, p = shape
        x, wt, gy = make_inputs(shape, seed=13)
        gx, gw = _C.dwconv2d_backward(x.to(gpu), gy.to(gpu), wt.to(gpu), s, s, p, p)
        seen.add(_C.last_variant().split("<")[0])
        _announce(shape_id(shape), _C.last_variant())
        gx_ref = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
        gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
        np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())
    assert {"small_bwd", "bwd_tile", "bwd_stack", "bwd_tile_s2"} <= seen, seen
    # an out_grad whose extent does not belong to the geometry is refused
    x, wt, gy = make_inputs((1, 2, 16, 16, 3, 1, 1), seed=1)
    with pytest.raises(RuntimeError, match="does not match the convolution geometry"):
        _C.dwconv2d_backward(x.to(gpu), gy[:, :, :15].contiguous().to(gpu), wt.to(gpu), 1, 1, 1, 1)
    # a workspace that is too small comes back as DWCONV_ERR_WORKSPACE, not as a fault
    xg, gg, wg = x.to(gpu), gy.to(gpu), wt.to(gpu)
    gxo, gwo = torch.empty_like(xg), torch.empty_like(wg)
    tiny = torch.empty(4, dtype=torch.uint8, device=gpu)
    rc = _C._lib.dwconv2d_backward_f32(xg.data_ptr(), gg.data_ptr(), wg.data_ptr(), gxo.data_ptr(), gwo.data_ptr(),
                                       tiny.data_ptr(), 4, 1, 2, 16, 16, 16, 16, 3, 3, 1, 1, 1, 1, None)
    assert rc == 3 and b"workspace" in _C._lib.dwconv_last_error()


def test_module_matches_plain_conv(dw, gpu):
    m = dw.DepthwiseConv2d(16, 16, 3, stride=1, padding=1).to(gpu)
    x = torch.randn(4, 16, 40, 40, device=gpu, requires_grad=True)
    y = m(x)
    y.square().mean().backward()
    gx, gw = x.grad.clone(), m.weight.grad.clone()
    x.grad = None
    m.weight.grad = None
    m.custom = False
    y2 = m(x)
    y2.square().mean().backward()
    torch.testing.assert_close(y, y2, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(gx, x.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(gw, m.weight.grad, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_autocast_casts_both_operands(dw, gpu, dtype):
    """Under torch.autocast an fp32 activation and an fp32 parameter run in the autocast dtype, like F.conv2d; the
    gradients come back in the dtypes of the leaves."""
    shape = (2, 8, 28, 28, 3, 1, 1)
    x, wt, gy = make_inputs(shape, seed=31)
    xg = x.to(gpu).requires_grad_(True)
    wg = wt.to(gpu).requires_grad_(True)
    with torch.autocast("cuda", dtype=dtype):
        y = dw.depthwise_conv2d(xg, wg, padding=1)
        y_torch = torch.nn.functional.conv2d(xg, wg, padding=1, groups=8)
    assert y.dtype == dtype == y_torch.dtype
    gx, gw = torch.autograd.grad(y, (xg, wg), gy.to(gpu).to(dtype))
    assert gx.dtype == torch.float32 and gw.dtype == torch.float32
    y_ref, gx_ref, gw_ref = oracle.torch_reference(x.to(dtype), wt.to(dtype), gy.to(dtype), 1, 1)
    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    np.testing.assert_allclose(_np(y.double()), _np(y_ref), rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gx.double()), _np(gx_ref), rtol=step, atol=1e-5 + step * 1e-2)
    np.testing.assert_allclose(_np(gw.double()), _np(gw_ref), rtol=step + 1e-4, atol=(step + 1e-4) * float(gw_ref.abs().max()))
    # outside autocast nothing is cast
    assert dw.depthwise_conv2d(xg, wg, padding=1).dtype == torch.float32


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
def test_only_the_requested_gradients_are_computed(dw, gpu, layout):
    """A leaf that does not require a gradient gets none (and costs no kernel); the other gradient is unchanged."""
    shape = (3, 8, 28, 28, 5, 2, 2)
    x, wt, gy = (t.to(gpu) for t in make_inputs(shape, seed=37))
    if layout == "nhwc":
        x, gy = (t.contiguous(memory_format=torch.channels_last) for t in (x, gy))
    _, gx_both, gw_both, _ = run_three_passes(dw, x, wt, gy, 2, 2)
    for need_x, need_w in [(True, False), (False, True)]:
        xg = x.detach().clone().requires_grad_(need_x)
        wg = wt.detach().clone().requires_grad_(need_w)
        dw.depthwise_conv2d(xg, wg, stride=2, padding=2).backward(gy)
        if need_x:
            assert wg.grad is None
            torch.testing.assert_close(xg.grad, gx_both, rtol=1e-6, atol=1e-6)
        else:
            assert xg.grad is None
            torch.testing.assert_close(wg.grad, gw_both, rtol=1e-5, atol=1e-5)


def test_runs_on_the_current_stream(dw, gpu):
    x = torch.randn(4, 8, 64, 64, device=gpu)
    w = torch.randn(8, 1, 3, 3, device=gpu)
    ref = dw.depthwise_conv2d(x, w, padding=1)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        out = dw.depthwise_conv2d(x, w, padding=1)
    side.synchronize()
    assert torch.equal(out, ref)


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
def test_hip_graph_capture_and_replay(dw, gpu, layout):
    """The entry points launch kernels only (no allocation, no synchronisation, no memset node), so a step made of
    them can be captured into a HIP graph.  Every replay, with eager work and synchronisations in between and fresh
    values in the static input buffers, must reproduce the eager results bit for bit (all three passes are
    deterministic)."""
    from torch_dwconv import _C

    # a whole-plane kernel, the tiled ones at stride 1 and 2, and the per-element fallback (4x4 filter)
    for shape in [(4, 16, 28, 28, 5, 1, 2), (2, 8, 56, 56, 3, 1, 1), (2, 8, 56, 60, 3, 2, 1), (2, 8, 9, 11, 4, 2, 1)]:
        n, c, h, w, k, s, p = shape
        x, wt, gy = (t.to(gpu) for t in make_inputs(shape, seed=23))
        if layout == "nhwc":
            x, gy = (t.contiguous(memory_format=torch.channels_last) for t in (x, gy))

        def step():
            if layout == "nhwc":
                return (_C.dwconv2d_nhwc(x, wt, s, s, p, p), *_C.dwconv2d_backward_nhwc(x, gy, wt, s, s, p, p))
            return (_C.dwconv2d(x, wt, 1, 1, s, s, p, p, p, p, True), *_C.dwconv2d_backward(x, gy, wt, s, s, p, p))

        side = torch.cuda.Stream(device=gpu)
        side.wait_stream(torch.cuda.current_stream(gpu))
        with torch.cuda.stream(side):
            step()  # warm-up outside the capture
        torch.cuda.current_stream(gpu).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = step()
        gen = torch.Generator("cpu").manual_seed(29)
        for replay in range(4):
            _announce(shape_id(shape), layout, "replay", replay)
            x.copy_(torch.randn(x.shape, generator=gen))
            gy.copy_(torch.randn(gy.shape, generator=gen))
            graph.replay()
            torch.cuda.synchronize(gpu)
            eager = step()
            torch.cuda.synchronize(gpu)
            for name, a, b in zip(("out", "in_grad", "kernel_grad"), captured, eager):
                assert torch.equal(a, b), (shape, layout, replay, name)
        y_ref, gx_ref, gw_ref = oracle.torch_reference(x, wt, gy, s, p)
        assert_parity(*captured, _np(y_ref), _np(gx_ref), _np(gw_ref), torch.float32)


# ---- channels-last tensors ---------------------------------------------------------------------------------
NHWC_SHAPES = [
    # (N, C, H, W, k, stride, pad): C % 4 == 0 and k in {3,5,7} take the vector kernels, the rest the per-element ones
    (2, 8, 14, 14, 3, 1, 1), (2, 32, 20, 24, 3, 1, 1), (1, 96, 17, 19, 3, 2, 1), (2, 144, 9, 11, 5, 2, 2),
    (2, 240, 7, 7, 5, 1, 2), (1, 12, 28, 28, 7, 1, 3), (2, 16, 15, 13, 7, 2, 3), (2, 8, 12, 12, 3, 1, 0),
    (2, 8, 12, 12, 5, 2, 0), (1, 4, 10, 9, 3, 2, 2), (2, 20, 6, 5, 5, 1, 4), (1, 260, 5, 5, 3, 1, 1),
    (3, 1152, 7, 7, 3, 1, 1), (2, 8, 1, 9, 3, 1, 1), (2, 8, 9, 1, 3, 2, 1), (2, 4, 33, 35, 5, 2, 1),
    (2, 3, 9, 11, 3, 1, 1), (1, 6, 8, 8, 4, 2, 1), (2, 5, 7, 7, 1, 1, 0), (1, 2, 12, 10, 9, 1, 4),
    # channel groups of whole 128-byte lines whose last group is partly idle (C / 4 = 60 lanes in groups of 16, 18 in groups of 8)
    (2, 240, 28, 28, 5, 1, 2), (2, 240, 28, 28, 3, 2, 1), (1, 72, 14, 14, 3, 1, 1),
    # 5x5 forward lane shapes: one channel per lane with 7 x 8 pixel blocks (C % 32 == 0, 14 or 28 rows; a width that is
    # not a multiple of 8), 4 x 2 blocks for stride 2 onto small maps
    (2, 96, 14, 14, 5, 1, 2), (1, 64, 28, 20, 5, 1, 2), (2, 672, 14, 14, 5, 2, 2),
]


def _channels_last(t, gpu):
    return t.to(gpu).contiguous(memory_format=torch.channels_last)


@pytest.mark.parametrize("shape", NHWC_SHAPES, ids=shape_id)
def test_channels_last_matches_oracle(dw, gpu, shape):
    """Channels-last input: same values as the NCHW oracle, channels-last results, bit-identical grad-weight."""
    from torch_dwconv import _C

    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=23)
    xg = _channels_last(x, gpu).requires_grad_(True)
    wg = wt.to(gpu).requires_grad_(True)
    y = dw.depthwise_conv2d(xg, wg, stride=s, padding=p)
    v_fwd = _C.last_variant()
    gx, gw = torch.autograd.grad(y, (xg, wg), _channels_last(gy, gpu))
    _announce(shape_id(shape), v_fwd, "|", _C.last_variant())
    assert v_fwd.startswith("nhwc_"), v_fwd
    fast = c % 4 == 0 and k in (3, 5, 7)
    assert v_fwd.startswith("nhwc_down") == fast, v_fwd
    if c > 1 and y.shape[2] * y.shape[3] > 1:
        assert y.is_contiguous(memory_format=torch.channels_last)
    if c > 1 and h * w > 1:
        assert gx.is_contiguous(memory_format=torch.channels_last)
    y_ref = oracle.forward(_np(x), _np(wt), s, p)
    gx_ref = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
    np.testing.assert_allclose(_np(y.detach()).astype(np.float64), y_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())
    _, gw2 = torch.autograd.grad(dw.depthwise_conv2d(xg, wg, stride=s, padding=p), (xg, wg), _channels_last(gy, gpu))
    assert torch.equal(gw, gw2)


FUSED_NHWC_SHAPES = [(2, 8, 14, 14, 3, 1, 1), (3, 32, 9, 11, 3, 1, 1), (1, 72, 15, 6, 3, 1, 1), (2, 144, 56, 56, 3, 1, 1),
                     (5, 260, 7, 7, 3, 1, 1), (2, 4, 1, 5, 3, 1, 1), (1, 12, 29, 30, 3, 1, 1)]


@pytest.mark.parametrize("shape", FUSED_NHWC_SHAPES, ids=shape_id)
def test_channels_last_fused_backward(dw, gpu, shape, monkeypatch):
    """3x3 stride-1 'same' layers, channels-last: one kernel makes both gradients.  Against the oracle, against the two
    separate kernels, bit-identical from run to run; one gradient alone still takes the separate kernels; the autograd
    route returns the same bits as the direct entry point."""
    from torch_dwconv import _C

    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=41)
    xg, wg, gyg = _channels_last(x, gpu), wt.to(gpu), _channels_last(gy, gpu)
    gx, gw = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    _announce(shape_id(shape), _C.last_variant())
    assert _C.last_variant().startswith("nhwc_bwd<k3,s1"), _C.last_variant()
    assert gx.is_contiguous(memory_format=torch.channels_last) or c == 1 or h * w == 1
    gx_ref = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())
    gx2, gw2 = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    assert torch.equal(gw, gw2) and torch.equal(gx, gx2)
    xa, wa = xg.clone().requires_grad_(True), wg.clone().requires_grad_(True)
    gxa, gwa = torch.autograd.grad(dw.depthwise_conv2d(xa, wa, stride=s, padding=p), (xa, wa), gyg)
    assert torch.equal(gxa, gx) and torch.equal(gwa, gw)
    gx_only, none = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p, need_kernel_grad=False)
    assert none is None and not _C.last_variant().startswith("nhwc_bwd"), _C.last_variant()
    np.testing.assert_allclose(_np(gx_only), _np(gx), rtol=1e-6, atol=1e-6)
    monkeypatch.setenv("DWCONV_NHWC_FUSED_BWD", "0")
    monkeypatch.setenv("DWCONV_TUNING", "1")
    gx3, gw3 = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    assert "nhwc_wgrad" in _C.last_variant(), _C.last_variant()
    np.testing.assert_allclose(_np(gx3), _np(gx), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(_np(gw3), _np(gw), rtol=1e-5, atol=1e-5 * float(gw.abs().max()))
    monkeypatch.delenv("DWCONV_NHWC_FUSED_BWD")
    for dtype, tol in ((torch.float16, 4e-3), (torch.bfloat16, 3e-2)):
        xh, wh, gh = xg.to(dtype), wg.to(dtype), gyg.to(dtype)
        gxh, gwh = _C.dwconv2d_backward_nhwc(xh, gh, wh, s, s, p, p)
        assert _C.last_variant().startswith("nhwc_bwd16<k3,s1"), _C.last_variant()
        _, gx_r, gw_r = oracle.torch_reference(xh.cpu(), wh.cpu(), gh.cpu(), s, p)
        np.testing.assert_allclose(_np(gxh.float()).astype(np.float64), _np(gx_r), rtol=tol, atol=tol)
        np.testing.assert_allclose(_np(gwh.float()).astype(np.float64), _np(gw_r), rtol=tol,
                                   atol=tol * max(1.0, float(np.abs(_np(gw_r)).max())))


FUSED_NHWC_OTHER = [
    # (shape, variant prefix): 5x5 stride 1, and stride 2 on even extents (3x3 in 7 x 4 blocks, 5x5 in 4 x 2 blocks)
    ((2, 8, 14, 14, 5, 1, 2), "nhwc_bwd<k5,s1"), ((1, 36, 9, 11, 5, 1, 2), "nhwc_bwd<k5,s1"),
    ((2, 8, 14, 14, 3, 2, 1), "nhwc_bwd<k3,s2"), ((1, 24, 30, 18, 3, 2, 1), "nhwc_bwd<k3,s2"),
    ((3, 4, 2, 2, 3, 2, 1), "nhwc_bwd<k3,s2"), ((1, 96, 112, 112, 3, 2, 1), "nhwc_bwd<k3,s2"),
    ((2, 8, 14, 14, 5, 2, 2), "nhwc_bwd<k5,s2"), ((1, 40, 22, 10, 5, 2, 2), "nhwc_bwd<k5,s2"),
    ((2, 144, 56, 56, 5, 2, 2), "nhwc_bwd<k5,s2"), ((5, 260, 2, 6, 5, 2, 2), "nhwc_bwd<k5,s2"),
    # odd extents are not covered by the fused stride-2 kernel
    ((2, 8, 15, 14, 3, 2, 1), "nhwc_up2"),
]


@pytest.mark.parametrize("case", FUSED_NHWC_OTHER, ids=lambda c: shape_id(c[0]))
def test_channels_last_fused_backward_other_layers(dw, gpu, case, monkeypatch):
    """The one-kernel backward for 5x5 stride-1 and for stride-2 layers, channels-last fp32: against the oracle,
    against the two separate kernels, bit-identical from run to run (outputs start as NaN)."""
    from torch_dwconv import _C

    shape, prefix = case
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=53)
    xg, wg, gyg = _channels_last(x, gpu), wt.to(gpu), _channels_last(gy, gpu)
    with poisoned_allocations():
        gx, gw = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    _announce(shape_id(shape), _C.last_variant())
    assert _C.last_variant().startswith(prefix), _C.last_variant()
    gx_ref = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    gw_ref = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())
    gx2, gw2 = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    assert torch.equal(gw, gw2) and torch.equal(gx, gx2)
    monkeypatch.setenv("DWCONV_NHWC_FUSED_BWD", "0")
    monkeypatch.setenv("DWCONV_TUNING", "1")
    gx3, gw3 = _C.dwconv2d_backward_nhwc(xg, gyg, wg, s, s, p, p)
    assert "nhwc_wgrad" in _C.last_variant() and not _C.last_variant().startswith("nhwc_bwd"), _C.last_variant()
    np.testing.assert_allclose(_np(gx3), _np(gx), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(_np(gw3), _np(gw), rtol=1e-5, atol=1e-5 * float(gw.abs().max()))


def test_channels_last_forward_lane_shapes(dw, gpu):
    """5x5 forward: one channel per lane and 7 x 8 blocks on 14-row maps with C % 32 == 0, 4 x 2 blocks for stride 2
    onto a 7x7 map, four channels per lane and 4 x 4 blocks otherwise."""
    from torch_dwconv import _C

    for (c, hw, s, want) in [(96, 14, 1, "nhwc_down<k5,s1,fwd,7x8,cv1>"), (672, 14, 2, "nhwc_down<k5,s2,fwd,4x2>"),
                             (240, 28, 1, "nhwc_down<k5,s1,fwd,4x4>"), (96, 12, 1, "nhwc_down<k5,s1,fwd,4x4>")]:
        x = _channels_last(torch.randn(2, c, hw, hw), gpu)
        dw.depthwise_conv2d(x, torch.randn(c, 1, 5, 5, device=gpu), stride=s, padding=2)
        assert _C.last_variant().startswith(want), (_C.last_variant(), want)


def test_channels_last_channel_groups_are_whole_lines(dw, gpu):
    """C = 240 on a 28x28 map: the workgroups take 16 channel lanes (256 bytes per pixel), not the 15 that divide C / 4."""
    from torch_dwconv import _C

    x = _channels_last(torch.randn(2, 240, 28, 28), gpu)
    dw.depthwise_conv2d(x, torch.randn(240, 1, 5, 5, device=gpu), padding=2)
    assert _C.last_variant().endswith("lanes_c16"), _C.last_variant()


@pytest.mark.parametrize("dtype", [torch.float64, torch.float16, torch.bfloat16], ids=["f64", "f16", "bf16"])
def test_channels_last_other_dtypes(dw, gpu, dtype):
    step = {torch.float64: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    for shape in [(2, 16, 14, 14, 3, 1, 1), (2, 8, 13, 15, 5, 2, 2), (1, 12, 9, 9, 7, 1, 3), (2, 6, 9, 8, 3, 2, 1)]:
        n, c, h, w, k, s, p = shape
        x, wt, gy = (t.to(dtype) for t in make_inputs(shape, seed=29))
        xg = _channels_last(x, gpu).requires_grad_(True)
        wg = wt.to(gpu).requires_grad_(True)
        y = dw.depthwise_conv2d(xg, wg, stride=s, padding=p)
        gx, gw = torch.autograd.grad(y, (xg, wg), _channels_last(gy, gpu))
        assert y.dtype == dtype and gx.dtype == dtype and gw.dtype == dtype
        xr, wr, gr = (_np(t.double()) for t in (x, wt, gy))
        y_ref = oracle.forward(xr, wr, s, p)
        gx_ref = oracle.grad_input(gr, wr, (h, w), s, p)
        gw_ref = oracle.grad_weight(xr, gr, wt.shape, s, p)
        tol = dict(rtol=max(step, 1e-12), atol=(1e-5 + step * 1e-2) if step else 1e-12)
        np.testing.assert_allclose(_np(y.detach().double()), y_ref, **tol)
        np.testing.assert_allclose(_np(gx.double()), gx_ref, **tol)
        gtol = (step + 1e-4) if step else 1e-12
        np.testing.assert_allclose(_np(gw.double()), gw_ref, rtol=gtol, atol=gtol * float(np.abs(gw_ref).max()))


def test_channels_last_entry_points(dw, gpu):
    """The C entry points directly: rectangular filters and strides, one gradient at a time, status codes."""
    from torch_dwconv import _C

    g = torch.Generator("cpu").manual_seed(31)
    x = torch.randn(2, 8, 11, 13, generator=g)
    wt = torch.randn(8, 1, 3, 5, generator=g)
    xg, wg = _channels_last(x, gpu), wt.to(gpu)
    ref = torch.nn.functional.conv2d(x.double(), wt.double(), stride=(2, 1), padding=(1, 2), groups=8)
    out = torch.empty(ref.shape, device=gpu).contiguous(memory_format=torch.channels_last)
    lib = _C._lib
    rc = lib.dwconv2d_nhwc_f32(xg.data_ptr(), wg.data_ptr(), out.data_ptr(), 2, 8, 11, 13, 3, 5, 2, 1, 1, 2, None)
    assert rc == 0, lib.dwconv_last_error()
    torch.cuda.synchronize()
    np.testing.assert_allclose(_np(out).astype(np.float64), ref.numpy(), rtol=1e-5, atol=1e-5)
    # grad-weight alone (in_grad = NULL), then grad-input alone
    gy = torch.randn(ref.shape, generator=g)
    gyg = _channels_last(gy, gpu)
    xr = x.double().requires_grad_(True)
    wr = wt.double().requires_grad_(True)
    gx_ref, gw_ref = torch.autograd.grad(torch.nn.functional.conv2d(xr, wr, stride=(2, 1), padding=(1, 2), groups=8),
                                         (xr, wr), gy.double())
    ws_bytes = lib.dwconv2d_backward_nhwc_workspace_bytes(2, 8, 11, 13, 3, 5, 2, 1, 1, 2, 4)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=gpu)
    gw = torch.empty_like(wg)
    gx = torch.empty_like(xg)
    geom = (2, 8, 11, 13, ref.shape[2], ref.shape[3], 3, 5, 2, 1, 1, 2)
    assert lib.dwconv2d_backward_nhwc_f32(xg.data_ptr(), gyg.data_ptr(), None, None, gw.data_ptr(), ws.data_ptr(),
                                          ws_bytes, *geom, None) == 0
    assert lib.dwconv2d_backward_nhwc_f32(None, gyg.data_ptr(), wg.data_ptr(), gx.data_ptr(), None, None, 0,
                                          *geom, None) == 0
    torch.cuda.synchronize()
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref.numpy(), rtol=1e-4, atol=1e-4 * float(gw_ref.abs().max()))
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref.numpy(), rtol=1e-5, atol=1e-5)
    # errors come back as status codes
    assert lib.dwconv2d_backward_nhwc_f32(xg.data_ptr(), gyg.data_ptr(), wg.data_ptr(), None, None, None, 0, *geom, None) == 1
    assert lib.dwconv2d_backward_nhwc_f32(xg.data_ptr(), gyg.data_ptr(), wg.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                          ws.data_ptr(), 4, *geom, None) == 3
    bad = list(geom)
    bad[4] += 1
    assert lib.dwconv2d_backward_nhwc_f32(xg.data_ptr(), gyg.data_ptr(), wg.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                          ws.data_ptr(), ws_bytes, *bad, None) == 1
    # empty batch
    e = dw.depthwise_conv2d(torch.empty(0, 8, 5, 5, device=gpu).contiguous(memory_format=torch.channels_last), wg[:, :, :, :3].contiguous(), padding=1)
    assert e.shape == (0, 8, 5, 5)


@pytest.mark.parametrize("shape", effnet_layers(), ids=shape_id)
def test_channels_last_full_size_layers(dw, gpu, shape):
    """Every EfficientNet-B0 layer at batch 128, channels-last: whole tensors against the fp64 reference (outputs
    start as NaN), adjoint identities, bit-identical grad-weight."""
    check_full_size(dw, gpu, shape, seed=37, layouts=("nhwc",))


@pytest.mark.parametrize("shape", CFG4 + CONVNEXT_T + [STRESS], ids=shape_id)
def test_channels_last_full_size_large_filters(dw, gpu, shape):
    """The 7x7 workloads and the grad-weight stress case in channels-last at full size."""
    check_full_size(dw, gpu, shape, seed=38, layouts=("nhwc",))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("layer", [0, 1, 3, 4, 7, 9, 10], ids=lambda i: shape_id(effnet_layers()[i]))
def test_channels_last_half_precision_full_batch(dw, gpu, layer, dtype):
    check_full_size(dw, gpu, effnet_layers()[layer], seed=39, layouts=("nhwc",), dtype=dtype)


# ---- forward with a fused per-channel scale / shift and activation -------------------------------------------
FUSED_CASES = [
    # (shape, channels_last, expected kernel family)
    ((2, 8, 56, 56, 3, 1, 1), False, "tile_down"), ((2, 6, 57, 44, 5, 2, 2), False, "tile_down"),
    ((3, 8, 14, 14, 5, 1, 2), False, "small_down"), ((2, 12, 28, 28, 3, 2, 1), False, "small_down"),
    ((2, 3, 9, 11, 4, 1, 1), False, "tile_any"), ((2, 16, 20, 24, 3, 1, 1), True, "nhwc_down"),
    ((2, 8, 15, 13, 5, 2, 2), True, "nhwc_down"), ((2, 5, 9, 9, 3, 1, 1), True, "nhwc_fwd_direct"),
]


@pytest.mark.parametrize("activation", [None, "relu", "relu6", "silu"])
@pytest.mark.parametrize("case", FUSED_CASES, ids=lambda c: shape_id(c[0]) + ("_nhwc" if c[1] else ""))
def test_fused_epilogue(dw, gpu, case, activation):
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    shape, nhwc, family = case
    n, c, h, w, k, s, p = shape
    x, wt, _ = make_inputs(shape, seed=43)
    x = x * 2  # enough spread to reach both sides of relu6
    g = torch.Generator("cpu").manual_seed(44)
    scale = torch.randn(c, generator=g) + 1.5
    shift = torch.randn(c, generator=g)
    xg = _channels_last(x, gpu) if nhwc else x.to(gpu)
    for sc, sh in [(scale, shift), (None, shift), (scale, None), (None, None)]:
        y = depthwise_conv2d_fused(xg, wt.to(gpu), bias=None if sh is None else sh.to(gpu),
                                   scale=None if sc is None else sc.to(gpu), activation=activation, stride=s, padding=p)
        assert _C.last_variant().startswith(family), _C.last_variant()
        assert y.is_contiguous(memory_format=torch.channels_last) == nhwc or y.is_contiguous()
        ref = oracle.torch_reference_fused(x, wt, sc, sh, activation, s, p)
        np.testing.assert_allclose(_np(y).astype(np.float64), ref.numpy(), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("route", ["direct", "tile_gen"])
@pytest.mark.parametrize("activation", [None, "relu6", "silu"])
def test_fused_epilogue_per_element_kernel(dw, gpu, activation, route, monkeypatch):
    """The epilogue inside the per-element kernel and inside the last tiled stop before it (here: forced, and with the
    any-geometry tiled kernel switched off)."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    if route == "direct":
        monkeypatch.setenv("DWCONV_FORCE_GENERIC", "1")
    else:
        monkeypatch.setenv("DWCONV_TUNING", "1")
        monkeypatch.setenv("DWCONV_FIR_ANY", "0")
    shape = (2, 3, 9, 11, 4, 1, 1)
    n, c, h, w, k, s, p = shape
    x, wt, _ = make_inputs(shape, seed=43)
    x = x * 2
    g = torch.Generator("cpu").manual_seed(44)
    scale, shift = torch.randn(c, generator=g) + 1.5, torch.randn(c, generator=g)
    y = depthwise_conv2d_fused(x.to(gpu), wt.to(gpu), bias=shift.to(gpu), scale=scale.to(gpu), activation=activation, stride=s, padding=p)
    assert _C.last_variant().startswith(route), _C.last_variant()
    ref = oracle.torch_reference_fused(x, wt, scale, shift, activation, s, p)
    np.testing.assert_allclose(_np(y).astype(np.float64), ref.numpy(), rtol=1e-5, atol=1e-5)


def test_fused_epilogue_other_dtypes_and_autograd(dw, gpu):
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    shape = (2, 8, 14, 14, 3, 1, 1)
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=45)
    scale, shift = torch.linspace(0.5, 2.0, c), torch.linspace(-1.0, 1.0, c)
    # fp64 (generic kernel, double parameters) to 1e-12; fp16 / bf16 to one rounding step
    y64 = depthwise_conv2d_fused(x.double().to(gpu), wt.double().to(gpu), shift.to(gpu), scale.to(gpu), "silu", s, p)
    ref64 = oracle.torch_reference_fused(x.double(), wt.double(), scale.double(), shift.double(), "silu", s, p)
    np.testing.assert_allclose(_np(y64), ref64.numpy(), rtol=1e-12, atol=1e-12)
    for dtype, step in [(torch.float16, 2.0 ** -11), (torch.bfloat16, 2.0 ** -8)]:
        xs, ws = x.to(dtype), wt.to(dtype)
        y = depthwise_conv2d_fused(xs.to(gpu), ws.to(gpu), shift.to(gpu), scale.to(gpu), "relu6", s, p)
        assert y.dtype == dtype
        ref = oracle.torch_reference_fused(xs, ws, scale, shift, "relu6", s, p)
        np.testing.assert_allclose(_np(y.double()), ref.numpy(), rtol=step, atol=1e-5 + step * 1e-2)
    # with gradients: the same fused forward kernel, gradients as torch's
    xg = x.to(gpu).requires_grad_(True)
    wg = wt.to(gpu).requires_grad_(True)
    bg = shift.to(gpu).requires_grad_(True)
    y = depthwise_conv2d_fused(xg, wg, bg, scale.to(gpu), "silu", s, p)
    with torch.no_grad():
        y_fused = depthwise_conv2d_fused(xg, wg, bg, scale.to(gpu), "silu", s, p)
    assert _C.last_variant().startswith("small_down")
    np.testing.assert_allclose(_np(y.detach()), _np(y_fused), rtol=1e-5, atol=1e-6)
    gx, gw, gb = torch.autograd.grad(y, (xg, wg, bg), gy.to(gpu))
    xr, wr, br = (t.double().requires_grad_(True) for t in (x, wt, shift))
    yr = torch.nn.functional.silu(torch.nn.functional.conv2d(xr, wr, stride=s, padding=p, groups=c)
                                  * scale.double().view(1, -1, 1, 1) + br.view(1, -1, 1, 1))
    rx, rw, rb = torch.autograd.grad(yr, (xr, wr, br), gy.double())
    np.testing.assert_allclose(_np(gx).astype(np.float64), rx.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(_np(gw).astype(np.float64), rw.numpy(), rtol=1e-4, atol=1e-4 * float(rw.abs().max()))
    np.testing.assert_allclose(_np(gb).astype(np.float64), rb.numpy(), rtol=1e-4, atol=1e-4 * float(rb.abs().max()))
    # argument errors
    with pytest.raises(ValueError, match="unknown activation"):
        depthwise_conv2d_fused(xg, wg, activation="gelu")
    with pytest.raises(RuntimeError, match="one entry per channel"):
        with torch.no_grad():
            depthwise_conv2d_fused(xg, wg, bias=torch.zeros(c + 1, device=gpu))
    rc = _C._lib.dwconv2d_fused_f32(xg.data_ptr(), wg.data_ptr(), None, None, y_fused.data_ptr(), n, c, h, w, k, k,
                                    s, s, p, p, 9, None)
    assert rc == 1 and b"activation" in _C._lib.dwconv_last_error()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 3, 36, 112, 3, 1, 1), (1, 4, 50, 96, 5, 2, 2)], ids=shape_id)
def test_fused_epilogue_16bit_wide_rows(dw, gpu, shape, dtype):
    """The fused epilogue inside the kernel with 16-bit LDS images (rows of at least 96 elements): every
    activation, with and without scale and shift, to one rounding step of the element type."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    n, c, h, w, k, s, p = shape
    x, wt, _ = make_inputs(shape, seed=47)
    xs, ws = (x * 2).to(dtype), wt.to(dtype)
    scale, shift = torch.linspace(0.5, 2.0, c), torch.linspace(-1.0, 1.0, c)
    step = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for activation in (None, "relu", "relu6", "silu"):
        for sc, sh in [(scale, shift), (None, shift), (scale, None)]:
            y = depthwise_conv2d_fused(xs.to(gpu), ws.to(gpu), None if sh is None else sh.to(gpu),
                                       None if sc is None else sc.to(gpu), activation, s, p)
            assert _C.last_variant().startswith("tile_down16_dot2"), _C.last_variant()
            ref = oracle.torch_reference_fused(xs, ws, sc, sh, activation, s, p)
            np.testing.assert_allclose(_np(y.double()), ref.numpy(), rtol=step, atol=1e-5 + step * 1e-2)


def _fused_reference_grads(x, wt, scale, shift, gy, activation, s, p):
    """fp64 CPU autograd of PyTorch's own composition conv -> * scale -> + shift -> activation."""
    import torch.nn.functional as F

    act = {None: lambda v: v, "relu": F.relu, "relu6": F.relu6, "silu": F.silu}[activation]
    leaves = [t.double().requires_grad_(True) if t is not None else None for t in (x, wt, scale, shift)]
    xr, wr, sr, br = leaves
    y = F.conv2d(xr, wr, stride=s, padding=p, groups=x.shape[1])
    if sr is not None:
        y = y * sr.view(1, -1, 1, 1)
    if br is not None:
        y = y + br.view(1, -1, 1, 1)
    y = act(y)
    wanted = [t for t in leaves if t is not None]
    grads = iter(torch.autograd.grad(y, wanted, gy.double()))
    return y.detach(), [next(grads) if t is not None else None for t in leaves]


FUSED_TRAIN_CASES = [
    # shape, channels_last: every backward kernel family behind the fused training path
    ((3, 8, 56, 56, 3, 1, 1), False), ((2, 6, 30, 33, 5, 2, 2), False), ((4, 12, 14, 14, 5, 1, 2), False),
    ((3, 8, 7, 7, 3, 1, 1), False), ((2, 5, 9, 11, 4, 2, 1), False), ((2, 16, 20, 24, 3, 1, 1), True),
    ((2, 8, 15, 13, 5, 2, 2), True), ((2, 5, 9, 9, 3, 1, 1), True),
]


@pytest.mark.parametrize("activation", [None, "relu", "relu6", "silu"])
@pytest.mark.parametrize("case", FUSED_TRAIN_CASES, ids=lambda c: shape_id(c[0]) + ("_nhwc" if c[1] else ""))
def test_fused_epilogue_training_path(dw, gpu, case, activation):
    """Training through the fused forward: one forward kernel (no saved pre-activation), and a backward that
    recomputes the convolution and runs the epilogue-backward sweep; all four gradients against fp64 autograd of
    PyTorch's own composition, layouts preserved, parameter gradients bit-identical from run to run."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    shape, nhwc = case
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=47)
    x = x * 2
    g = torch.Generator("cpu").manual_seed(48)
    scale = torch.randn(c, generator=g) + 1.5
    shift = torch.randn(c, generator=g)
    fmt = torch.channels_last if nhwc else torch.contiguous_format
    for sc, sh in [(scale, shift), (None, shift), (scale, None)]:
        leaves = [x.to(gpu).contiguous(memory_format=fmt).requires_grad_(True), wt.to(gpu).requires_grad_(True),
                  sc.to(gpu).requires_grad_(True) if sc is not None else None,
                  sh.to(gpu).requires_grad_(True) if sh is not None else None]
        xg, wg, sg, bg = leaves
        y = depthwise_conv2d_fused(xg, wg, bg, sg, activation, s, p)
        assert y.grad_fn is not None and "Fused" in type(y.grad_fn).__name__
        assert y.is_contiguous(memory_format=fmt)
        wanted = [t for t in leaves if t is not None]
        got = iter(torch.autograd.grad(y, wanted, gy.to(gpu).contiguous(memory_format=fmt), retain_graph=True))
        got = [next(got) if t is not None else None for t in leaves]
        _announce(shape_id(shape), "nhwc" if nhwc else "nchw", activation, _C.last_variant())
        y_ref, ref = _fused_reference_grads(x, wt, sc, sh, gy, activation, s, p)
        np.testing.assert_allclose(_np(y).astype(np.float64), y_ref.numpy(), rtol=1e-5, atol=1e-5)
        assert got[0].is_contiguous(memory_format=fmt)
        np.testing.assert_allclose(_np(got[0]).astype(np.float64), ref[0].numpy(), rtol=1e-4, atol=2e-5)
        for a, b in zip(got[1:], ref[1:]):
            if b is None:
                assert a is None
                continue
            assert a.shape == b.shape and a.dtype == torch.float32
            np.testing.assert_allclose(_np(a).astype(np.float64), b.numpy(), rtol=1e-4, atol=1e-4 * float(b.abs().max()))
        again = iter(torch.autograd.grad(y, wanted, gy.to(gpu).contiguous(memory_format=fmt)))
        again = [next(again) if t is not None else None for t in leaves]
        for a, b in zip(got, again):
            assert (a is None and b is None) or torch.equal(a, b)


def test_fused_epilogue_training_partial_gradients_and_dtypes(dw, gpu):
    """Only the gradients that are asked for come back; 16-bit tensors train through the same path."""
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    shape = (3, 8, 28, 28, 5, 2, 2)
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=49)
    scale, shift = torch.linspace(0.5, 2.0, c), torch.linspace(-1.0, 1.0, c)
    _, ref = _fused_reference_grads(x, wt, scale, shift, gy, "silu", s, p)
    # frozen filter and scale: gradients of the input and the bias only
    xg = x.to(gpu).requires_grad_(True)
    bg = shift.to(gpu).requires_grad_(True)
    y = depthwise_conv2d_fused(xg, wt.to(gpu), bg, scale.to(gpu), "silu", s, p)
    y.backward(gy.to(gpu))
    np.testing.assert_allclose(_np(xg.grad).astype(np.float64), ref[0].numpy(), rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(_np(bg.grad).astype(np.float64), ref[3].numpy(), rtol=1e-4, atol=1e-4 * float(ref[3].abs().max()))
    # frozen input: gradients of the filter and the scale
    wg = wt.to(gpu).requires_grad_(True)
    sg = scale.to(gpu).requires_grad_(True)
    depthwise_conv2d_fused(x.to(gpu), wg, shift.to(gpu), sg, "silu", s, p).backward(gy.to(gpu))
    np.testing.assert_allclose(_np(wg.grad).astype(np.float64), ref[1].numpy(), rtol=1e-4, atol=1e-4 * float(ref[1].abs().max()))
    np.testing.assert_allclose(_np(sg.grad).astype(np.float64), ref[2].numpy(), rtol=1e-4, atol=1e-4 * float(ref[2].abs().max()))
    for dtype, step in [(torch.float16, 2.0 ** -11), (torch.bfloat16, 2.0 ** -8)]:
        xs, ws, gs = x.to(dtype), wt.to(dtype), gy.to(dtype)
        # a smooth activation: with ReLU6 an element whose pre-activation sits within a rounding step of a corner
        # can land on the other side when the recomputed convolution result is rounded to 16 bits
        _, refh = _fused_reference_grads(xs, ws, scale, shift, gs, "silu", s, p)
        leaves = [xs.to(gpu).requires_grad_(True), ws.to(gpu).requires_grad_(True), scale.to(gpu).requires_grad_(True),
                  shift.to(gpu).requires_grad_(True)]
        y = depthwise_conv2d_fused(leaves[0], leaves[1], leaves[3], leaves[2], "silu", s, p)
        got = torch.autograd.grad(y, leaves, gs.to(gpu))
        assert got[0].dtype == dtype and got[1].dtype == dtype and got[2].dtype == torch.float32
        # the recomputed convolution result and its gradient are rounded to the 16-bit format on the way (as the
        # intermediate tensors of PyTorch's own composition would be): a few rounding steps of tolerance
        np.testing.assert_allclose(_np(got[0].double()), refh[0].numpy(), rtol=4 * step, atol=4 * step * float(refh[0].abs().max()))
        for a, b in zip(got[1:], refh[1:]):
            np.testing.assert_allclose(_np(a.double()), b.numpy(), rtol=4 * step + 1e-3, atol=(4 * step + 1e-3) * float(b.abs().max()))


@pytest.mark.parametrize("activation", ["relu", "relu6"])
@pytest.mark.parametrize("dtype,step", [(torch.float16, 2.0 ** -11), (torch.bfloat16, 2.0 ** -8)], ids=["f16", "bf16"])
def test_fused_epilogue_training_16bit_piecewise_activations(dw, gpu, dtype, step, activation):
    """ReLU / ReLU6 training on 16-bit tensors.  The backward pass takes the activation's mask from the recomputed
    convolution result, which is rounded to 16 bits, whereas the fused forward applied the activation to the fp32 sum:
    an output whose pre-activation lies within one rounding step of a corner (0, or 6 for ReLU6) may get the slope of
    the other side.  Those outputs, and only those, are given the full size of their contribution as extra tolerance;
    everywhere else the gradients meet the bounds of the smooth-activation test."""
    import torch.nn.functional as F
    from torch_dwconv.dwconv import depthwise_conv2d_fused

    shape = (3, 8, 28, 28, 5, 1, 2)
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=53)
    scale, shift = torch.linspace(0.5, 2.0, c), torch.linspace(-1.0, 3.0, c)
    xs, ws, gs = x.to(dtype), wt.to(dtype), gy.to(dtype)
    _, ref = _fused_reference_grads(xs, ws, scale, shift, gs, activation, s, p)
    xd, wd, gd, sd = xs.double(), ws.double(), gs.double(), scale.double().view(1, -1, 1, 1)
    conv = F.conv2d(xd, wd, stride=s, padding=p, groups=c)
    z = conv * sd + shift.double().view(1, -1, 1, 1)
    reach = conv.abs() * sd * step * 1.01  # how far rounding the convolution result can move z
    near = z.abs() <= reach
    if activation == "relu6":
        near |= (z - 6).abs() <= reach
    frac = float(near.double().mean())
    assert 0 < frac < 0.02, frac  # some such outputs exist, and they are few
    flipped = near.double() * gd.abs()  # the most a flipped slope changes the gradient of the activation's input
    extra = [F.conv_transpose2d(flipped * sd, wd.abs(), stride=s, padding=p, groups=c),
             (flipped * sd).sum((0, 2, 3)).view(c, 1, 1, 1) * float(xd.abs().max()),
             (flipped * conv.abs()).sum((0, 2, 3)), flipped.sum((0, 2, 3))]
    leaves = [xs.to(gpu).requires_grad_(True), ws.to(gpu).requires_grad_(True), scale.to(gpu).requires_grad_(True),
              shift.to(gpu).requires_grad_(True)]
    y = depthwise_conv2d_fused(leaves[0], leaves[1], leaves[3], leaves[2], activation, s, p)
    got = torch.autograd.grad(y, leaves, gs.to(gpu))
    for i, (a, b, e) in enumerate(zip(got, ref, extra)):
        rel = 4 * step + (1e-3 if i else 0.0)
        bound = rel * b.abs() + rel * float(b.abs().max()) + e.expand_as(b)
        worst = ((a.double().cpu() - b).abs() - bound).max()
        assert float(worst) <= 0.0, (i, float(worst))
    # where no such output is in reach the input gradient is as exact as under a smooth activation
    clean = extra[0] == 0
    assert float(clean.double().mean()) > 0.3
    err = (got[0].double().cpu() - ref[0]).abs()[clean]
    assert float(err.max()) <= 4 * step * float(ref[0].abs().max()) * 2


def test_plane_beyond_two_gib(dw, gpu):
    """One fp32 plane of more than 2 GiB: byte offsets inside it pass 2^31, where the kernels' 32-bit buffer-view
    offsets end, so the library must take its 64-bit addressing path.  Corners (with their zero padding) and an
    interior window are compared with the oracle on crops."""
    from torch_dwconv import _C

    hh, ww = 540000, 1024  # 540000 * 1024 * 4 B = 2.2 GB, narrow enough for the tiled kernels
    free, _ = torch.cuda.mem_get_info()
    if free < 12 * 1024 ** 3:
        pytest.skip("needs 12 GiB of free device memory")
    g = torch.Generator(device=gpu).manual_seed(5)
    x = torch.randn(1, 1, hh, ww, device=gpu, generator=g)
    wt = torch.randn(1, 1, 3, 3, generator=torch.Generator("cpu").manual_seed(6))
    y = dw.depthwise_conv2d(x, wt.to(gpu), stride=1, padding=1)
    variant = _C.last_variant()
    _announce("2.2 GB plane", variant)
    assert "vin1" in variant and "vout1" in variant, variant  # vector accesses, but not through a 2 GiB view
    for (r0, c0) in [(0, 0), (hh - 64, ww - 64), (hh // 2 + 3, ww // 2 - 5), (hh - 64, 0)]:
        # crop with a one-pixel halo where the plane has one
        ra, rb_ = max(r0 - 1, 0), min(r0 + 64 + 1, hh)
        ca, cb_ = max(c0 - 1, 0), min(c0 + 64 + 1, ww)
        crop = x[:, :, ra:rb_, ca:cb_].cpu().contiguous()
        ref = oracle.forward(_np(crop), _np(wt), 1, 1)
        got = _np(y[:, :, r0:r0 + 64, c0:c0 + 64].cpu())
        np.testing.assert_allclose(got.astype(np.float64), ref[:, :, r0 - ra:r0 - ra + 64, c0 - ca:c0 - ca + 64],
                                   rtol=1e-5, atol=1e-5)
    del y
    # grad-input of the same plane (the transposed problem) on the same crops, grad-weight against an fp64 sum
    gy = torch.randn(1, 1, hh, ww, device=gpu, generator=g)
    gx, gw = _C.dwconv2d_backward(x, gy, wt.to(gpu), 1, 1, 1, 1)
    _announce("2.2 GB plane backward", _C.last_variant())
    for (r0, c0) in [(0, 0), (hh - 64, ww - 64)]:
        ra, rb_ = max(r0 - 1, 0), min(r0 + 64 + 1, hh)
        ca, cb_ = max(c0 - 1, 0), min(c0 + 64 + 1, ww)
        crop = gy[:, :, ra:rb_, ca:cb_].cpu().contiguous()
        ref = oracle.grad_input(_np(crop), _np(wt), crop.shape[2:], 1, 1)
        got = _np(gx[:, :, r0:r0 + 64, c0:c0 + 64].cpu())
        np.testing.assert_allclose(got.astype(np.float64), ref[:, :, r0 - ra:r0 - ra + 64, c0 - ca:c0 - ca + 64],
                                   rtol=1e-5, atol=1e-5)
    # gw[i,j] = <gy, x shifted by (i-1, j-1)>: torch's fp64 reductions on the device as the independent sum
    ref_gw = torch.zeros(3, 3, dtype=torch.float64)
    for i in range(3):
        for j in range(3):
            di, dj = i - 1, j - 1
            ys = slice(max(0, -di), hh - max(0, di))
            xs = slice(max(0, -dj), ww - max(0, dj))
            yi = slice(max(0, di), hh - max(0, -di))
            xi = slice(max(0, dj), ww - max(0, -dj))
            ref_gw[i, j] = torch.sum(gy[0, 0, ys, xs].double() * x[0, 0, yi, xi].double()).item()
    np.testing.assert_allclose(_np(gw.cpu())[0, 0].astype(np.float64), ref_gw.numpy(), rtol=1e-4,
                               atol=1e-4 * float(ref_gw.abs().max()))


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
def test_tensor_beyond_two_gib(dw, gpu, layout):
    """A batch whose input tensor exceeds 2 GiB (planes themselves are small): the buffer views start at the
    workgroup's own planes / images, so their 32-bit offsets stay small while the bases pass 2^31 bytes.  The last
    images (largest addresses) and the first are compared with the oracle; grad-weight over the whole batch is
    checked through the adjoint identity."""
    free, _ = torch.cuda.mem_get_info()
    if free < 16 * 1024 ** 3:
        pytest.skip("needs 16 GiB of free device memory")
    n, c, h, w, k, s, p = 520, 96, 112, 112, 3, 2, 1  # 520 * 96 * 112 * 112 * 4 B = 2.5 GB
    g = torch.Generator(device=gpu).manual_seed(9)
    x = torch.randn(n, c, h, w, device=gpu, generator=g)
    wt = (torch.randn(c, 1, k, k, generator=torch.Generator("cpu").manual_seed(10)) / k).to(gpu)
    if layout == "nhwc":
        x = x.contiguous(memory_format=torch.channels_last)
    xg = x.requires_grad_(True)
    wg = wt.clone().requires_grad_(True)
    y = dw.depthwise_conv2d(xg, wg, stride=s, padding=p)
    gy = torch.randn(y.shape, device=gpu, generator=g)
    if layout == "nhwc":
        gy = gy.contiguous(memory_format=torch.channels_last)
    gx, gw = torch.autograd.grad(y, (xg, wg), gy)
    for img in (0, n - 1):
        for ch in (0, c - 1):
            xs = x.detach()[img:img + 1, ch:ch + 1].cpu().contiguous()
            ws = wt[ch:ch + 1].cpu().contiguous()
            gs = gy[img:img + 1, ch:ch + 1].cpu().contiguous()
            np.testing.assert_allclose(_np(y.detach()[img:img + 1, ch:ch + 1].cpu()).astype(np.float64),
                                       oracle.forward(_np(xs), _np(ws), s, p), rtol=1e-5, atol=1e-5)
            np.testing.assert_allclose(_np(gx[img:img + 1, ch:ch + 1].cpu()).astype(np.float64),
                                       oracle.grad_input(_np(gs), _np(ws), (h, w), s, p), rtol=1e-5, atol=1e-5)
    lhs = (y.detach().double() * gy.double()).sum().item()
    assert abs(lhs - (wg.detach().double() * gw.double()).sum().item()) <= 1e-6 * abs(lhs) + 1e-2
    assert abs(lhs - (x.detach().double() * gx.double()).sum().item()) <= 1e-6 * abs(lhs) + 1e-2


# ---- dilation and depth multiplier ---------------------------------------------------------------------------
# depth multiplier on maps large enough for one plane per tile: the tiled kernels (forward with the input plane c / M,
# grad-input summed over the M planes of out_grad, grad-weight against the shared input plane); both strides, 3x3 / 5x5 /
# 7x7, odd extents and widths that are not whole groups of four (scalar loads and stores), no padding
MULTIPLIED_TILED = [
    (2, 3, 2, 56, 56, 3, 3, 1, 1, 1), (2, 2, 3, 113, 120, 3, 3, 2, 1, 1), (3, 2, 2, 64, 48, 5, 5, 1, 2, 1),
    (2, 2, 4, 140, 144, 5, 5, 2, 2, 1), (1, 3, 2, 130, 128, 3, 3, 2, 1, 1), (2, 2, 2, 50, 49, 3, 3, 1, 1, 1),
    (2, 2, 2, 60, 64, 3, 3, 1, 0, 1), (2, 2, 2, 56, 56, 7, 7, 1, 3, 1), (2, 1, 5, 127, 130, 3, 3, 2, 1, 1),
]
GENERAL_CASES = [
    # (N, C, M, H, W, KH, KW, stride, pad, dilation)
    (2, 4, 1, 14, 14, 3, 3, 1, 2, 2), (2, 3, 2, 9, 11, 3, 3, 1, 1, 1), (1, 5, 3, 13, 12, 5, 3, 2, 2, 2),
    (2, 8, 1, 16, 16, 3, 3, 2, 3, 3), (2, 2, 4, 7, 7, 3, 3, 1, 0, 1), (1, 3, 2, 6, 6, 3, 3, 1, 1, 3),
    (2, 6, 1, 20, 24, 3, 3, 1, 1, 1),
    # dilation 2, stride 1, "same" padding on maps wide enough for the stacked-image kernels (3x3 and 5x5 taps): heights
    # that leave a hanging unit, tiles across two and three images
    (2, 3, 1, 40, 48, 3, 3, 1, 2, 2), (3, 2, 1, 33, 64, 5, 5, 1, 4, 2), (5, 2, 1, 57, 52, 3, 3, 1, 2, 2),
    (7, 1, 1, 18, 96, 5, 5, 1, 4, 2), (2, 2, 1, 130, 128, 3, 3, 1, 2, 2),
    # the same on rows that are not whole groups of four elements
    (2, 3, 1, 40, 50, 3, 3, 1, 2, 2), (2, 2, 1, 45, 75, 5, 5, 1, 4, 2), (3, 2, 1, 37, 33, 3, 3, 1, 2, 2),
    # dilation 2 on maps up to 32 wide: the whole-plane kernels (exact and ragged widths, odd planes)
    (3, 8, 1, 14, 14, 3, 3, 1, 2, 2), (2, 6, 1, 28, 28, 5, 5, 1, 4, 2), (3, 8, 1, 7, 7, 3, 3, 1, 2, 2), (2, 4, 1, 16, 16, 5, 5, 1, 4, 2),
    (2, 8, 1, 15, 15, 3, 3, 1, 2, 2), (3, 5, 1, 9, 30, 5, 5, 1, 4, 2), (2, 3, 1, 32, 32, 3, 3, 1, 2, 2), (2, 4, 1, 20, 24, 3, 3, 1, 2, 2),
] + MULTIPLIED_TILED


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", GENERAL_CASES, ids=lambda c: "N%d_C%d_M%d_%dx%d_k%dx%d_s%d_p%d_d%d" % c)
def test_dilation_and_depth_multiplier(dw, gpu, case, dtype):
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_general

    n, c, m, h, w, kh, kw, s, p, d = case
    g = torch.Generator("cpu").manual_seed(53)
    x = torch.randn(n, c, h, w, generator=g).to(dtype)
    wt = (torch.randn(c * m, 1, kh, kw, generator=g) / kh).to(dtype)
    xg = x.to(gpu).requires_grad_(True)
    wg = wt.to(gpu).requires_grad_(True)
    y = depthwise_conv2d_general(xg, wg, stride=s, padding=p, dilation=d)
    v_fwd = _C.last_variant()
    gy = torch.randn(y.shape, generator=g).to(dtype)
    gx, gw = torch.autograd.grad(y, (xg, wg), gy.to(gpu))
    _announce(case, str(dtype), v_fwd, "|", _C.last_variant())
    plain = m == 1 and d == 1
    stacked = (m == 1 and d == 2 and s == 1 and kh == kw and kh in (3, 5) and p == d * (kh // 2) and w >= 16
               and h >= 8 and 2 * ((h + 3) // 4) * ((w + 3) // 4) > 256 and dtype != torch.float64)
    small = (m == 1 and d == 2 and s == 1 and kh == kw and kh in (3, 5) and p == d * (kh // 2) and w <= 32 and h <= 64
             and dtype != torch.float64)
    if case in MULTIPLIED_TILED and dtype != torch.float64:
        # (autograd runs the backward on its own thread; the variant note is per thread)
        _C.dwconv2d_general_backward(xg.detach(), gy.to(gpu), wg.detach(), s, s, p, p, d, d)
        v_bwd = _C.last_variant()
        assert v_fwd.startswith("tile_down") and v_fwd.endswith(" m%d" % m), v_fwd
        assert v_bwd.startswith("tile_down" if s == 1 else "tile_up2") and "wgrad_tile" in v_bwd and v_bwd.count(" m%d" % m) == 2, v_bwd
    elif stacked:
        assert v_fwd.startswith("tile_stack") and _C.last_variant() is not None, v_fwd
        assert v_fwd.endswith(" anywidth") == (w % 4 != 0), v_fwd
    elif small:
        assert v_fwd.startswith("small_down") and ",d2" in v_fwd, v_fwd
    elif plain:
        assert not v_fwd.startswith("general_fwd"), v_fwd  # the plain case runs the tuned kernels
    elif m == 1 and dtype != torch.float64:
        assert v_fwd.startswith("tile_any<k%dx%d,s%dx%d,d%dx%d" % (kh, kw, s, s, d, d)), v_fwd  # any other dilation / stride
    elif m == 1:
        # double tensors: the fp64 tiled kernels, with dilated taps; backward as two passes (grad-input of a stride-1
        # layer through the same kernel with rotated taps)
        assert v_fwd.startswith("tile_f64<k%dx%d,u1x1,s%dx%d,fwd>" % (kh, kw, s, s)) and v_fwd.endswith(" d%dx%d" % (d, d)), v_fwd
        _C.dwconv2d_general_backward(xg.detach(), gy.to(gpu), wg.detach(), s, s, p, p, d, d)
        v_bwd = _C.last_variant()
        assert ("tile_f64<" in v_bwd and ",rot>" in v_bwd) == (s == 1), v_bwd
        assert "wgrad_f64<k%dx%d,s%dx%d>" % (kh, kw, s, s) in v_bwd and v_bwd.endswith(" d%dx%d" % (d, d)), v_bwd
    else:
        assert v_fwd.startswith("general_fwd"), v_fwd
    y_ref, gx_ref, gw_ref = oracle.torch_reference_general(x, wt, gy, s, p, d)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(_np(y.detach()).astype(np.float64), y_ref.numpy(), **tol)
    np.testing.assert_allclose(_np(gx).astype(np.float64), gx_ref.numpy(), **tol)
    gtol = 1e-4 if dtype == torch.float32 else 1e-12
    np.testing.assert_allclose(_np(gw).astype(np.float64), gw_ref.numpy(), rtol=gtol, atol=gtol * float(gw_ref.abs().max()))
    _, gw2 = torch.autograd.grad(depthwise_conv2d_general(xg, wg, stride=s, padding=p, dilation=d), (xg, wg), gy.to(gpu))
    assert torch.equal(gw, gw2)


@pytest.mark.parametrize("dtype,step", [(torch.float16, 2.0 ** -11), (torch.bfloat16, 2.0 ** -8)], ids=["f16", "bf16"])
def test_depth_multiplier_tiled_half_precision(dw, gpu, dtype, step):
    """The tiled kernels' depth-multiplier route with 16-bit tensors (fp32 sums, one rounding per result): forward,
    grad-input summed over the M planes of out_grad, grad-weight, against fp64 on the rounded inputs."""
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_general

    for case in [(2, 3, 2, 56, 56, 3, 3, 1, 1, 1), (2, 2, 3, 113, 120, 3, 3, 2, 1, 1), (2, 2, 4, 140, 144, 5, 5, 2, 2, 1),
                 (2, 2, 2, 50, 49, 3, 3, 1, 1, 1), (2, 2, 2, 56, 56, 7, 7, 1, 3, 1)]:
        n, c, m, h, w, kh, kw, s, p, d = case
        g = torch.Generator("cpu").manual_seed(59)
        x = torch.randn(n, c, h, w, generator=g).to(dtype)
        wt = (torch.randn(c * m, 1, kh, kw, generator=g) / kh).to(dtype)
        xg = x.to(gpu).requires_grad_(True)
        wg = wt.to(gpu).requires_grad_(True)
        y = depthwise_conv2d_general(xg, wg, stride=s, padding=p, dilation=d)
        v_fwd = _C.last_variant()
        assert v_fwd.startswith("tile_down16") and v_fwd.endswith(" m%d" % m), v_fwd
        gy = torch.randn(y.shape, generator=g).to(dtype)
        gx, gw = torch.autograd.grad(y, (xg, wg), gy.to(gpu))
        assert y.dtype == dtype and gx.dtype == dtype and gw.dtype == dtype
        y_ref, gx_ref, gw_ref = oracle.torch_reference_general(x.double(), wt.double(), gy.double(), s, p, d)
        for got, ref in ((y.detach(), y_ref), (gx, gx_ref)):
            np.testing.assert_allclose(_np(got.double()), ref.numpy(), rtol=1e-5 + step, atol=1e-5 + step * float(ref.abs().max()))
        np.testing.assert_allclose(_np(gw.double()), gw_ref.numpy(), rtol=1e-4 + step, atol=(1e-4 + step) * float(gw_ref.abs().max()))


def test_general_entry_point_errors(dw, gpu):
    from torch_dwconv import _C
    from torch_dwconv.dwconv import depthwise_conv2d_general

    x = torch.randn(1, 4, 8, 8, device=gpu)
    with pytest.raises(RuntimeError, match="multiplier"):
        depthwise_conv2d_general(x, torch.randn(6, 1, 3, 3, device=gpu))
    y = depthwise_conv2d_general(x.half(), torch.randn(8, 1, 3, 3, device=gpu).half(), padding=2, dilation=2)
    assert y.shape == (1, 8, 8, 8) and y.dtype == torch.float16
    ref = oracle.torch_reference_general(x.half(), torch.zeros(8, 1, 3, 3), None, 1, 2, 2)[0]
    assert ref.shape == y.shape
    lib = _C._lib
    o = torch.empty(1, 8, 8, 8, device=gpu)
    k = torch.randn(8, 1, 3, 3, device=gpu)
    assert lib.dwconv2d_general_f32(x.data_ptr(), k.data_ptr(), o.data_ptr(), 1, 4, 8, 8, 0, 3, 3, 1, 1, 1, 1, 1, 1, None) == 1
    assert b"multiplier" in lib.dwconv_last_error()
    assert lib.dwconv2d_general_f32(x.data_ptr(), k.data_ptr(), o.data_ptr(), 1, 4, 8, 8, 2, 3, 3, 1, 1, 1, 1, 0, 1, None) == 1
    # a dilated filter larger than the padded input gives an empty output, not an error
    e = depthwise_conv2d_general(x, k, dilation=5)
    assert e.shape == (1, 8, 0, 0)

