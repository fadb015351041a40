"""GPU parity on seeded random problems: the HIP library (through its C ABI, via torch_dwconv) against the CPU oracles.

Bounds as in test_gpu_parity.py: fp32 forward / grad-input rtol = atol = 1e-5 against fp64, grad-weight rtol 1e-4 with
atol = 1e-4 * max|gw_ref|; fp64 1e-11; 16-bit element types add one rounding step of the format (2^-11 / 2^-8) to
rtol and a hundredth of it to atol (their arithmetic is fp32, the oracle runs in fp64 on the rounded inputs).
"""
import random

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

STEP = {torch.float32: 0.0, torch.float64: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}
DTYPES = [torch.float32, torch.float32, torch.float16, torch.bfloat16, torch.float64]


@pytest.fixture(scope="module")
def dw(gpu):
    import torch_dwconv.dwconv as m

    return m


def _np(t):
    return t.detach().cpu().numpy()


def _announce(*what):
    print("[case]", *what, flush=True)


def _bounds(dtype):
    base = 1e-11 if dtype == torch.float64 else 1e-5
    return dict(rtol=base + STEP[dtype], atol=base + STEP[dtype] * 1e-2)


def _assert_grad_weight(gw, gw_ref, dtype, case):
    gw_ref = np.asarray(gw_ref, dtype=np.float64)
    tol = (1e-11 if dtype == torch.float64 else 1e-4) + STEP[dtype]
    np.testing.assert_allclose(_np(gw.double()), gw_ref, rtol=tol, atol=tol * max(float(np.abs(gw_ref).max()), 1e-30),
                               err_msg=case)


# ---- randomised geometry sweep --------------------------------------------------------------------
def _draw_case(rng):
    """One random problem: about two thirds in the geometry the tuned kernels take (square 3/5/7 filter, stride 1 or
    2, mostly 'same' padding), the rest anything the operator accepts (rectangular filters up to 11, strides up to 3,
    per-axis padding up to one more than the filter)."""
    def extent():
        r = rng.random()
        if r < 0.35:
            return rng.choice([7, 14, 28])
        if r < 0.6:
            return rng.randint(1, 33)
        if r < 0.9:
            return rng.randint(34, 130)
        return rng.randint(131, 400)

    if rng.random() < 0.65:
        kh = kw = rng.choice([3, 3, 5, 5, 7])
        sh = sw = rng.choice([1, 1, 2])
        ph = pw = kh // 2 if rng.random() < 0.75 else rng.randint(0, kh - 1)
        if rng.random() < 0.15:
            ph = rng.randint(0, kh - 1)
    else:
        kh = rng.choice([1, 2, 3, 3, 3, 4, 5, 5, 7, 7, 9, 11])
        kw = kh if rng.random() < 0.7 else rng.choice([1, 2, 3, 5, 7])
        sh = rng.choice([1, 1, 1, 2, 2, 3])
        sw = sh if rng.random() < 0.8 else rng.choice([1, 2, 3])
        ph = rng.choice([0, kh // 2, kh // 2, kh - 1, rng.randint(0, kh + 1)])
        pw = rng.choice([0, kw // 2, kw // 2, kw - 1, rng.randint(0, kw + 1)])
    h = extent()
    w = h if rng.random() < 0.5 else extent()
    n = rng.choice([1, 2, 3, 5, 8])
    c = rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 24, 40, 64, 96])
    while n * c * h * w > 3_000_000:  # keeps the fp64 CPU check of one case in the milliseconds
        if c > 1:
            c //= 2
        else:
            n, h = 1, max(1, h // 2)
    dtype = rng.choice([torch.float32] * 4 + [torch.float16, torch.bfloat16, torch.float64])
    layout = rng.choice(["nchw", "nchw", "nhwc"])
    return n, c, h, w, kh, kw, sh, sw, ph, pw, dtype, layout


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_randomised_geometry_sweep(dw, gpu, seed):
    """300 seeded random problems per seed over filter extent, stride and padding per axis, plane size, element type
    and layout, each checked in all three passes against PyTorch's fp64 CPU convolution (the oracle of the
    reference's own tests, test/test_forward.py:14) to the bounds used elsewhere in this file.  Odd cases go through
    autograd, even ones through the combined backward entry points directly."""
    from torch_dwconv import _C

    rng = random.Random(seed)
    families = set()
    for it in range(300):
        n, c, h, w, kh, kw, sh, sw, ph, pw, dtype, layout = _draw_case(rng)
        oh, ow = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
        if oh <= 0 or ow <= 0:
            continue  # empty outputs: test_empty_and_degenerate_inputs
        g = torch.Generator("cpu").manual_seed(seed * 100003 + it)
        x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64).to(dtype)
        wt = (torch.randn(c, 1, kh, kw, generator=g, dtype=torch.float64) / (kh * kw) ** 0.5).to(dtype)
        gy = torch.randn(n, c, oh, ow, generator=g, dtype=torch.float64).to(dtype)
        case = f"seed{seed} it{it} N{n}C{c} {h}x{w} k{kh}x{kw} s{sh}x{sw} p{ph}x{pw} {dtype} {layout}"
        _announce(case)
        xg, gyg, wg = x.to(gpu), gy.to(gpu), wt.to(gpu)
        if layout == "nhwc":
            xg = xg.contiguous(memory_format=torch.channels_last)
            gyg = gyg.contiguous(memory_format=torch.channels_last)
        nhwc = _C.is_channels_last(xg)  # false for planes of one pixel or one channel, where the layouts coincide
        xg.requires_grad_(True)
        wg.requires_grad_(True)
        y = dw.depthwise_conv2d(xg, wg, stride=(sh, sw), padding=(ph, pw))
        families.add(_C.last_variant().split("<")[0].split(" ")[0])
        if dtype == torch.float64 or it % 2:
            gx, gw = torch.autograd.grad(y, (xg, wg), gyg)
        elif nhwc:
            gx, gw = _C.dwconv2d_backward_nhwc(xg.detach(), gyg, wg.detach(), sh, sw, ph, pw)
        else:
            gx, gw = _C.dwconv2d_backward(xg.detach(), gyg.contiguous(), wg.detach(), sh, sw, ph, pw)
        assert y.dtype == dtype and gx.dtype == dtype and gw.dtype == dtype, case
        if nhwc:
            assert y.is_contiguous(memory_format=torch.channels_last), case
            assert gx.is_contiguous(memory_format=torch.channels_last), case
        y_ref, gx_ref, gw_ref = oracle.torch_reference(x, wt, gy, (sh, sw), (ph, pw))
        np.testing.assert_allclose(_np(y.double()), _np(y_ref), err_msg=case, **_bounds(dtype))
        np.testing.assert_allclose(_np(gx.double()), _np(gx_ref), err_msg=case, **_bounds(dtype))
        _assert_grad_weight(gw, _np(gw_ref), dtype, case)
    # the sweep is only worth its name if it reaches every forward kernel family
    assert {"tile_down", "small_down", "nhwc_down", "tile_any", "tile_f64", "nhwc_fwd_direct"} <= families, families


# ---- the other entry points ---------------------------------------------------------------------------
def _extent(rng, hi=120):
    r = rng.random()
    if r < 0.3:
        return rng.choice([7, 14, 28])
    if r < 0.6:
        return rng.randint(1, 33)
    return rng.randint(34, hi)


def _raw_operator(rng, gen, gpu, dw, _C):
    """dwconv2d_*: up- and down-sampling together, four independent pads (negative ones crop), either tap order;
    against the C oracle's closed form of torch_dwconv/dwconv_kernel.cu:69-181."""
    kh = rng.choice([1, 2, 3, 3, 4, 5, 5, 7])
    kw = kh if rng.random() < 0.7 else rng.choice([1, 2, 3, 5, 7])
    mode = rng.random()
    if mode < 0.4:  # the grad-input of a stride-2 layer
        up, down = (2, 2), (1, 1)
    elif mode < 0.6:
        d = rng.choice([1, 2, 3])
        up, down = (1, 1), (d, d)
    else:
        up, down = (rng.choice([1, 2, 3]), rng.choice([1, 2, 3])), (rng.choice([1, 2, 3]), rng.choice([1, 2]))
    pads = [rng.randint(-2, kh + 1), rng.randint(-2, kh + 1), rng.randint(-2, kw + 1), rng.randint(-2, kw + 1)]
    if rng.random() < 0.5:
        pads = [max(p, 0) for p in pads]
    h, w, n, c = _extent(rng), _extent(rng), rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 5, 8, 16])
    dtype, fwd = rng.choice(DTYPES), rng.random() < 0.5
    if oracle.out_size(h, up[0], down[0], pads[0], pads[1], kh) <= 0 or oracle.out_size(w, up[1], down[1], pads[2], pads[3], kw) <= 0:
        return None
    x = torch.randn(n, c, h, w, generator=gen, dtype=torch.float64).to(dtype)
    wt = (torch.randn(c, 1, kh, kw, generator=gen, dtype=torch.float64) / (kh * kw) ** 0.5).to(dtype)
    case = f"operator N{n}C{c} {h}x{w} k{kh}x{kw} up{up} down{down} pads{pads} forward={fwd} {dtype}"
    _announce(case)
    got = _C.dwconv2d(x.to(gpu), wt.to(gpu), *up, *down, *pads, fwd)
    ref = oracle.dwconv2d(_np(x.double()), _np(wt.double()), *up, *down, *pads, fwd)
    np.testing.assert_allclose(_np(got.double()), ref, err_msg=case, **_bounds(dtype))
    return _C.last_variant()


def _grad_weight(rng, gen, gpu, dw, _C):
    """dwconv2d_backward_kernel_*: rectangular filters, per-axis decimation, pads 0..K; against the C oracle's closed
    form of torch_dwconv/dwconv_kernel.cu:444-588, and bit-identical on a second call."""
    kh = rng.choice([1, 2, 3, 3, 4, 5, 5, 7, 9])
    kw = kh if rng.random() < 0.7 else rng.choice([1, 2, 3, 5, 7])
    dn_h = rng.choice([1, 1, 2, 3])
    dn_w = dn_h if rng.random() < 0.8 else rng.choice([1, 2])
    ph, pw = (kh // 2, kw // 2) if rng.random() < 0.5 else (rng.randint(0, kh), rng.randint(0, kw))
    h, w, n, c = _extent(rng, 200), _extent(rng, 200), rng.choice([1, 2, 3, 7]), rng.choice([1, 2, 3, 5, 8, 16, 33])
    dtype = rng.choice(DTYPES)
    oh, ow = (h + 2 * ph - kh) // dn_h + 1, (w + 2 * pw - kw) // dn_w + 1
    if oh <= 0 or ow <= 0:
        return None
    x = torch.randn(n, c, h, w, generator=gen, dtype=torch.float64).to(dtype)
    gy = torch.randn(n, c, oh, ow, generator=gen, dtype=torch.float64).to(dtype)
    wt = torch.zeros(c, 1, kh, kw, dtype=dtype, device=gpu)
    case = f"grad-weight N{n}C{c} {h}x{w} k{kh}x{kw} down{dn_h}x{dn_w} pad{ph}x{pw} {dtype}"
    _announce(case)
    got = _C.dwconv2d_backward_kernel(x.to(gpu), gy.to(gpu), wt, 1, 1, dn_h, dn_w, ph, pw)
    variant = _C.last_variant()
    again = _C.dwconv2d_backward_kernel(x.to(gpu), gy.to(gpu), wt, 1, 1, dn_h, dn_w, ph, pw)
    assert torch.equal(got, again), case
    ref = oracle.backward_kernel(_np(x.double()), _np(gy.double()), tuple(wt.shape), dn_h, dn_w, ph, pw)
    _assert_grad_weight(got, ref, dtype, case)
    return variant


def _fused(rng, gen, gpu, dw, _C):
    """dwconv2d_fused_* in both layouts: optional per-channel scale and shift, each activation; against PyTorch's conv
    followed by PyTorch's own elementwise functions in fp64."""
    k = rng.choice([3, 3, 5, 5, 7, 2, 4])
    s = rng.choice([1, 1, 2])
    p = k // 2 if rng.random() < 0.7 else rng.randint(0, k - 1)
    h, w, n, c = _extent(rng), _extent(rng), rng.choice([1, 2, 5]), rng.choice([1, 3, 4, 8, 16, 40])
    dtype, layout, act = rng.choice(DTYPES), rng.choice(["nchw", "nhwc"]), rng.choice([None, "relu", "relu6", "silu"])
    if (h + 2 * p - k) // s + 1 <= 0 or (w + 2 * p - k) // s + 1 <= 0:
        return None
    x = torch.randn(n, c, h, w, generator=gen, dtype=torch.float64).to(dtype)
    wt = (torch.randn(c, 1, k, k, generator=gen, dtype=torch.float64) / k).to(dtype)
    pdt = torch.float64 if dtype == torch.float64 else torch.float32
    scale = (torch.rand(c, generator=gen, dtype=torch.float64) + 0.5).to(pdt) if rng.random() < 0.7 else None
    shift = torch.randn(c, generator=gen, dtype=torch.float64).to(pdt) if rng.random() < 0.7 else None
    case = (f"fused N{n}C{c} {h}x{w} k{k} s{s} p{p} {dtype} {layout} act={act} scale={scale is not None} "
            f"shift={shift is not None}")
    _announce(case)
    xg = x.to(gpu).contiguous(memory_format=torch.channels_last) if layout == "nhwc" else x.to(gpu)
    with torch.no_grad():
        got = dw.depthwise_conv2d_fused(xg, wt.to(gpu), bias=None if shift is None else shift.to(gpu),
                                        scale=None if scale is None else scale.to(gpu), activation=act, stride=s,
                                        padding=p)
    ref = oracle.torch_reference_fused(x, wt, scale, shift, act, s, p)
    tol = _bounds(dtype)
    if dtype == torch.float32 and act == "silu":
        tol = dict(rtol=3e-5, atol=3e-5)  # hardware exp and reciprocal in the fp32 sigmoid
    np.testing.assert_allclose(_np(got.double()), _np(ref), err_msg=case, **tol)
    return _C.last_variant()


def _general(rng, gen, gpu, dw, _C):
    """dwconv2d_general_* through autograd: dilation and depth multiplier; against PyTorch's fp64 grouped conv."""
    kh = rng.choice([1, 2, 3, 3, 5, 7])
    kw = kh if rng.random() < 0.7 else rng.choice([1, 2, 3, 5])
    m, dil = rng.choice([1, 1, 2, 3, 4]), (rng.choice([1, 2, 3]), rng.choice([1, 2, 3]))
    st = (rng.choice([1, 1, 2, 3]), rng.choice([1, 1, 2]))
    pad = (rng.randint(0, dil[0] * (kh - 1) // 2 + 1), rng.randint(0, dil[1] * (kw - 1) // 2 + 1))
    h, w, n, c = _extent(rng, 80), _extent(rng, 80), rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 5, 8])
    dtype = rng.choice(DTYPES)
    oh = (h + 2 * pad[0] - dil[0] * (kh - 1) - 1) // st[0] + 1
    ow = (w + 2 * pad[1] - dil[1] * (kw - 1) - 1) // st[1] + 1
    if oh <= 0 or ow <= 0:
        return None
    x = torch.randn(n, c, h, w, generator=gen, dtype=torch.float64).to(dtype)
    wt = (torch.randn(c * m, 1, kh, kw, generator=gen, dtype=torch.float64) / (kh * kw) ** 0.5).to(dtype)
    gy = torch.randn(n, c * m, oh, ow, generator=gen, dtype=torch.float64).to(dtype)
    case = f"general N{n}C{c}M{m} {h}x{w} k{kh}x{kw} stride{st} pad{pad} dilation{dil} {dtype}"
    _announce(case)
    xg, wg = x.to(gpu).requires_grad_(True), wt.to(gpu).requires_grad_(True)
    y = dw.depthwise_conv2d_general(xg, wg, stride=st, padding=pad, dilation=dil)
    variant = _C.last_variant()
    gx, gw = torch.autograd.grad(y, (xg, wg), gy.to(gpu))
    y_ref, gx_ref, gw_ref = oracle.torch_reference_general(x, wt, gy, st, pad, dil)
    np.testing.assert_allclose(_np(y.double()), _np(y_ref), err_msg=case, **_bounds(dtype))
    np.testing.assert_allclose(_np(gx.double()), _np(gx_ref), err_msg=case, **_bounds(dtype))
    _assert_grad_weight(gw, _np(gw_ref), dtype, case)
    return variant


@pytest.mark.parametrize("kind", [_raw_operator, _grad_weight, _fused, _general], ids=lambda f: f.__name__.strip("_"))
def test_randomised_entry_point_sweep(dw, gpu, kind):
    """400 seeded random problems per entry-point family (see the drawing functions above for the ranges)."""
    from torch_dwconv import _C

    rng = random.Random(kind.__name__)
    families = {}
    for it in range(400):
        gen = torch.Generator("cpu").manual_seed(7919 * it + 13)
        variant = kind(rng, gen, gpu, dw, _C)
        if variant is not None:
            name = variant.split("<")[0].split(" ")[0]
            families[name] = families.get(name, 0) + 1
    _announce(kind.__name__, families)
    assert sum(families.values()) > 300 and len(families) >= 2, families
