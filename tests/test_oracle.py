"""Pins the CPU oracle (oracle/) before anything is checked against it.

Independent anchors, chosen so that a dropped term, a wrong sign/index, a
transposed operand or an un-flipped filter fails at least one of them:
  * torch's fp64 grouped conv and its autograd (the reference's own test oracle,
    test/test_forward.py:14, test/test_grad.py:23-39),
  * torch's fp64 conv_transpose2d for the backward-direction operator,
  * a pure-Python 7-loop brute force on tiny shapes,
  * closed forms: delta filter, box filter == avg_pool2d, 1x1 filter,
  * adjoint identities <y,gy> == <x,gx> == <w,gw>,
  * the committed golden vectors,
  * integer identities for the geometry helpers and a hand truth table for the
    small-path predicate.
"""
import itertools
import os

import numpy as np
import pytest
import torch
from torch.nn import functional as F

import oracle
from shapes import REF_FORWARD, REF_GRAD, make_inputs, shape_id

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "dwconv_golden.npz")


# --------------------------------------------------------------------------
# geometry
# --------------------------------------------------------------------------
def test_out_size_equals_pytorch_formula():
    for h, k, s, p in itertools.product(range(1, 40), (1, 2, 3, 4, 5, 7), (1, 2, 3), (0, 1, 2, 3)):
        if h + 2 * p < k:
            continue
        assert oracle.out_size(h, 1, s, p, p, k) == (h + 2 * p - k) // s + 1


def test_g_pad_identity_recovers_input_size():
    # dwconv.py:39-44: the backward-direction op with up=stride and g_pad must
    # produce exactly the input extent.
    for h, k, s, p in itertools.product(range(1, 40), (1, 3, 4, 5, 7), (1, 2, 3), (0, 1, 2, 3)):
        if h + 2 * p < k or p >= k:
            continue
        oh = (h + 2 * p - k) // s + 1
        gp = oracle.host_logic.g_pad((h, h), (oh, oh), (k, k), (s, s), (p, p))
        assert oracle.out_size(oh, s, 1, gp[0], gp[1], k) == h
        assert gp[0] == k - p - 1 and gp[1] == h - oh * s + p


# (H, W, KH, KW, down, pad) -> expected; evaluated by hand from dwconv_kernel.cu:658-661
SMALL_TRUTH = [
    ((7, 7, 5, 5, 1, 2), True),      # 25 <= ceil(7/2)*7 = 28
    ((7, 7, 7, 7, 1, 3), False),     # 49 > 28
    ((7, 7, 3, 3, 1, 1), True),
    ((14, 14, 7, 7, 1, 3), True),    # 49 <= 7*14
    ((14, 14, 5, 5, 2, 2), False),   # stride 2
    ((28, 28, 3, 3, 2, 1), False),
    ((28, 28, 5, 5, 1, 2), True),
    ((32, 32, 3, 3, 1, 1), True),
    ((33, 32, 3, 3, 1, 1), False),   # H > 32
    ((32, 33, 3, 3, 1, 1), False),   # W > 32
    ((16, 16, 3, 3, 1, 0), False),   # output smaller than input
    ((16, 16, 5, 5, 1, 2), True),
    ((56, 56, 3, 3, 1, 1), False),
    ((4, 4, 3, 3, 1, 1), False),     # 9 > ceil(4/2)*4 = 8
    ((5, 4, 3, 3, 1, 1), True),      # 9 <= 3*4 = 12
]


@pytest.mark.parametrize("geom,expected", SMALL_TRUTH)
def test_small_predicate_truth_table(geom, expected):
    h, w, kh, kw, down, pad = geom
    assert oracle.use_dwconv2d_small(h, w, kh, kw, 1, 1, down, down, pad, pad) is expected


# --------------------------------------------------------------------------
# host logic restatement
# --------------------------------------------------------------------------
def test_expand_semantics():
    e = oracle.host_logic.expand
    assert e(3, 2) == (3, 3)
    assert e((1, 2), 2) == (1, 2)
    assert e([4], 2) == [4, 4]
    with pytest.raises(ValueError):
        e((1, 2, 3), 2)


def test_rejection_order():
    fr = oracle.host_logic.first_rejection
    assert fr(8, 8, 1, None, None) is None
    assert fr(8, 8, 1, 8, False) is None
    assert fr(8, 8, 2, 4, True) == "dilation"
    assert fr(8, 8, (1, 2), None, None) == "dilation"
    assert fr(8, 16, 1, 4, True) == "groups"
    assert fr(8, 16, 1, 8, True) == "channels"
    assert fr(8, 8, 1, None, True) == "bias"
    assert fr(8, 8, 1, None, None, "reflect") == "padding_mode"


# --------------------------------------------------------------------------
# values: torch fp64
# --------------------------------------------------------------------------
def _np(t):
    return t.detach().numpy()


SMALL_MATRIX = [
    (2, 3, 6, 7, 3, 1, 1), (2, 3, 6, 7, 3, 2, 1), (2, 3, 9, 8, 5, 1, 2), (2, 3, 9, 8, 5, 2, 2),
    (1, 2, 7, 7, 7, 1, 3), (1, 2, 12, 11, 7, 2, 3), (2, 2, 11, 13, 3, 2, 0), (2, 2, 11, 13, 5, 1, 0),
    (1, 3, 10, 10, 4, 2, 1), (1, 3, 13, 10, 2, 3, 0), (1, 2, 5, 5, 1, 1, 0), (1, 2, 9, 9, 3, 3, 1),
]


@pytest.mark.parametrize("shape", SMALL_MATRIX + [(2, 4) + s[2:] for s in REF_GRAD], ids=shape_id)
def test_three_passes_equal_torch_fp64(shape):
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=3, dtype=torch.float64)
    y_ref, gx_ref, gw_ref = oracle.torch_reference(x, wt, gy, stride=s, padding=p)
    y = oracle.forward(_np(x), _np(wt), s, p)
    gx = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    gw = oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p)
    np.testing.assert_allclose(y, _np(y_ref), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gx, _np(gx_ref), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gw, _np(gw_ref), rtol=1e-12, atol=1e-11)


@pytest.mark.parametrize("shape", [(2, 4) + s[2:] for s in REF_FORWARD], ids=shape_id)
def test_reference_forward_matrix_shapes(shape):
    n, c, h, w, k, s, p = shape
    x, wt, _ = make_inputs(shape, seed=5, dtype=torch.float64)
    y_ref, _, _ = oracle.torch_reference(x, wt, None, stride=s, padding=p)
    np.testing.assert_allclose(oracle.forward(_np(x), _np(wt), s, p), _np(y_ref), rtol=1e-12, atol=1e-12)


def test_non_square_kernel_stride_and_padding():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 3, 12, 10, generator=g, dtype=torch.float64, requires_grad=True)
    wt = torch.randn(3, 1, 5, 2, generator=g, dtype=torch.float64, requires_grad=True)
    s, p = (2, 1), (1, 0)
    y_ref = F.conv2d(x, wt, stride=s, padding=p, groups=3)
    gy = torch.randn(y_ref.shape, generator=g, dtype=torch.float64)
    gx_ref, gw_ref = torch.autograd.grad(y_ref, (x, wt), gy)
    np.testing.assert_allclose(oracle.forward(_np(x), _np(wt), s, p), _np(y_ref), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.grad_input(_np(gy), _np(wt), (12, 10), s, p), _np(gx_ref), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.grad_weight(_np(x), _np(gy), wt.shape, s, p), _np(gw_ref), rtol=1e-12, atol=1e-11)


@pytest.mark.parametrize("k,s,p", [(3, 1, 1), (3, 2, 1), (5, 2, 2), (4, 2, 1), (5, 3, 0)])
def test_backward_direction_is_conv_transpose(k, s, p):
    # The backward-direction operator with up=stride is a transposed conv.
    g = torch.Generator().manual_seed(k * 10 + s)
    c, oh, ow = 3, 6, 5
    gy = torch.randn(2, c, oh, ow, generator=g, dtype=torch.float64)
    wt = torch.randn(c, 1, k, k, generator=g, dtype=torch.float64)
    full = F.conv_transpose2d(gy, wt, stride=s, padding=p, groups=c)
    h, w = full.shape[-2:]
    got = oracle.grad_input(_np(gy), _np(wt), (h, w), s, p)
    np.testing.assert_allclose(got, _np(full), rtol=1e-12, atol=1e-12)
    # one extra trailing row/column of input (the remainder a stride leaves) gets zero gradient
    got2 = oracle.grad_input(_np(gy), _np(wt), (h + s - 1, w + s - 1), s, p)
    ref2 = F.conv_transpose2d(gy, wt, stride=s, padding=p, groups=c, output_padding=s - 1)
    np.testing.assert_allclose(got2, _np(ref2), rtol=1e-12, atol=1e-12)


RAW_MODES = [
    # (kh, kw, up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward)
    (3, 3, 2, 2, 2, 2, 1, 1, 1, 1, True),       # up and down together
    (5, 5, 2, 2, 2, 2, 2, 1, 3, 0, True),
    (4, 3, 3, 2, 2, 3, 0, 0, 1, 1, False),      # rectangular everything, rotated taps
    (3, 3, 2, 2, 1, 1, 1, 2, 0, 3, True),       # forward direction with up > 1 (taps not rotated)
    (5, 4, 1, 3, 2, 1, 4, 0, 0, 5, True),
    (3, 3, 1, 1, 1, 1, -1, 2, 1, -2, True),     # negative pads crop the input
    (5, 5, 2, 2, 1, 1, -2, 3, -1, -1, False),
    (4, 4, 2, 2, 3, 3, -1, -1, 2, 2, False),
    (1, 1, 3, 3, 2, 2, 0, 0, 0, 0, True),
    (7, 7, 2, 1, 1, 2, 3, 3, 3, 3, False),
]


@pytest.mark.parametrize("mode", RAW_MODES, ids=lambda m: "k%dx%d_u%d%d_d%d%d_p%d.%d.%d.%d_%s" % (m[:10] + ("fwd" if m[10] else "rot",)))
def test_raw_operator_modes_equal_zero_stuffing_plus_strided_conv(mode):
    """The raw operator of dwconv_kernel.cu:69-181 in the modes the autograd path never uses (up and down
    together, forward with up > 1, negative pads), against PyTorch: zero-stuff the input by hand (up - 1 zeros after
    every sample: mid = out*down + up - 1 - pad0, in = floor(mid / up), tap = (in + 1)*up - mid - 1 at :122-178
    places sample i at position i*up), pad (crop for negative pads), then a strided grouped correlation with the
    taps as given (forward) or rotated by 180 degrees (backward, :108-113)."""
    kh, kw, uh, uw, dh, dw_, ph0, ph1, pw0, pw1, fwd = mode
    g = torch.Generator("cpu").manual_seed(kh * 100 + kw * 10 + uh + dh)
    n, c, h, w = 2, 3, 9, 11
    x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64)
    k = torch.randn(c, 1, kh, kw, generator=g, dtype=torch.float64)
    stuffed = torch.zeros(n, c, h * uh, w * uw, dtype=torch.float64)
    stuffed[:, :, ::uh, ::uw] = x
    padded = F.pad(stuffed, (pw0, pw1, ph0, ph1))
    taps = k if fwd else torch.flip(k, dims=(2, 3))
    want = F.conv2d(padded, taps, stride=(dh, dw_), groups=c)
    got = oracle.dwconv2d(x.numpy(), k.numpy(), uh, uw, dh, dw_, ph0, ph1, pw0, pw1, fwd)
    assert got.shape == tuple(want.shape)
    assert got.size > 0
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-12)


def test_small_operator_equals_large_operator():
    g = torch.Generator().manual_seed(2)
    x = _np(torch.randn(2, 3, 9, 11, generator=g, dtype=torch.float64))
    for kh, kw, ph, pw in [(3, 3, 1, 1), (5, 5, 2, 2), (5, 3, 0, 2), (4, 4, 3, 0)]:
        wt = _np(torch.randn(3, 1, kh, kw, generator=g, dtype=torch.float64))
        for fwd in (True, False):
            small = oracle.dwconv2d_small(x, wt, ph, pw, fwd)
            large = oracle.dwconv2d(x, wt, 1, 1, 1, 1, ph, kh - 1 - ph, pw, kw - 1 - pw, fwd)
            np.testing.assert_array_equal(small, large)


# --------------------------------------------------------------------------
# values: brute force and closed forms
# --------------------------------------------------------------------------
def _brute(x, w, gy, s, p):
    n, c, h, wd = x.shape
    kh, kw = w.shape[-2:]
    oh, ow = (h + 2 * p - kh) // s + 1, (wd + 2 * p - kw) // s + 1
    y = np.zeros((n, c, oh, ow))
    gx = np.zeros_like(x)
    gw = np.zeros_like(w)
    for b in range(n):
        for ch in range(c):
            for oy in range(oh):
                for ox in range(ow):
                    for i in range(kh):
                        for j in range(kw):
                            iy, ix = oy * s - p + i, ox * s - p + j
                            if 0 <= iy < h and 0 <= ix < wd:
                                y[b, ch, oy, ox] += x[b, ch, iy, ix] * w[ch, 0, i, j]
                                gx[b, ch, iy, ix] += gy[b, ch, oy, ox] * w[ch, 0, i, j]
                                gw[ch, 0, i, j] += gy[b, ch, oy, ox] * x[b, ch, iy, ix]
    return y, gx, gw


@pytest.mark.parametrize("k,s,p", [(1, 1, 0), (3, 1, 1), (3, 2, 1), (5, 1, 2), (5, 2, 0), (3, 2, 0)])
def test_brute_force_tiny(k, s, p):
    shape = (2, 3, 6, 7, k, s, p)
    x, wt, gy = (_np(t) for t in make_inputs(shape, seed=9, dtype=torch.float64))
    y, gx, gw = _brute(x, wt, gy, s, p)
    np.testing.assert_allclose(oracle.forward(x, wt, s, p), y, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.grad_input(gy, wt, (6, 7), s, p), gx, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.grad_weight(x, gy, wt.shape, s, p), gw, rtol=1e-12, atol=1e-12)


def test_delta_filter_is_identity():
    x = np.random.default_rng(0).standard_normal((2, 3, 8, 9))
    for k in (3, 5, 7):
        w = np.zeros((3, 1, k, k))
        w[:, 0, k // 2, k // 2] = 1.0
        np.testing.assert_array_equal(oracle.forward(x, w, 1, k // 2), x)
        np.testing.assert_array_equal(oracle.grad_input(x, w, (8, 9), 1, k // 2), x)


def test_off_centre_delta_shifts_the_right_way():
    # catches a flipped filter: tap (0,2) of a 3x3 picks x[y-1, x+1] in the forward direction
    x = np.random.default_rng(1).standard_normal((1, 1, 6, 6))
    w = np.zeros((1, 1, 3, 3))
    w[0, 0, 0, 2] = 1.0
    y = oracle.forward(x, w, 1, 1)
    assert y[0, 0, 3, 2] == x[0, 0, 2, 3]
    gx = oracle.grad_input(x, w, (6, 6), 1, 1)
    assert gx[0, 0, 2, 3] == x[0, 0, 3, 2]


def test_box_filter_is_avg_pool():
    x = torch.randn(2, 3, 12, 10, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    for k, s, p in [(3, 1, 1), (3, 2, 1), (5, 2, 2), (2, 2, 0)]:
        w = np.full((3, 1, k, k), 1.0 / (k * k))
        ref = F.avg_pool2d(x, k, stride=s, padding=p, count_include_pad=True)
        np.testing.assert_allclose(oracle.forward(_np(x), w, s, p), _np(ref), rtol=1e-12, atol=1e-13)


def test_one_by_one_filter_scales_channels():
    x = np.random.default_rng(2).standard_normal((2, 4, 5, 6))
    w = np.arange(1, 5, dtype=np.float64).reshape(4, 1, 1, 1)
    np.testing.assert_allclose(oracle.forward(x, w, 1, 0), x * w.reshape(1, 4, 1, 1), rtol=0, atol=0)


@pytest.mark.parametrize("shape", [(2, 3, 33, 35, 5, 2, 2), (2, 3, 33, 35, 3, 2, 1), (2, 3, 14, 14, 7, 1, 3), (1, 2, 20, 17, 4, 3, 2)], ids=shape_id)
def test_adjoint_identities(shape):
    n, c, h, w, k, s, p = shape
    x, wt, gy = (_np(t) for t in make_inputs(shape, seed=21, dtype=torch.float64))
    y = oracle.forward(x, wt, s, p)
    gx = oracle.grad_input(gy, wt, (h, w), s, p)
    gw = oracle.grad_weight(x, gy, wt.shape, s, p)
    lhs = float((y * gy).sum())
    assert abs(lhs - float((x * gx).sum())) <= 1e-10 * max(1.0, abs(lhs))
    assert abs(lhs - float((wt * gw).sum())) <= 1e-10 * max(1.0, abs(lhs))


def test_linearity():
    shape = (2, 3, 10, 9, 3, 2, 1)
    x, wt, gy = (_np(t) for t in make_inputs(shape, seed=1, dtype=torch.float64))
    x2 = np.random.default_rng(5).standard_normal(x.shape)
    a = oracle.forward(x + 2 * x2, wt, 2, 1)
    b = oracle.forward(x, wt, 2, 1) + 2 * oracle.forward(x2, wt, 2, 1)
    np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------
# golden vectors
# --------------------------------------------------------------------------
def _golden_cases():
    z = np.load(GOLDEN)
    n = len([k for k in z.files if k.endswith("_geom")])
    return z, n


def test_golden_vectors_c_oracle_and_torch():
    z, ncases = _golden_cases()
    assert ncases >= 6
    for i in range(ncases):
        n, c, h, w, kh, kw, sh, sw, ph, pw = (int(v) for v in z[f"c{i}_geom"])
        x, wt, gy = z[f"c{i}_x"], z[f"c{i}_w"], z[f"c{i}_gy"]
        np.testing.assert_allclose(oracle.forward(x, wt, (sh, sw), (ph, pw)), z[f"c{i}_y"], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(oracle.grad_input(gy, wt, (h, w), (sh, sw), (ph, pw)), z[f"c{i}_gx"], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(oracle.grad_weight(x, gy, wt.shape, (sh, sw), (ph, pw)), z[f"c{i}_gw"], rtol=1e-12, atol=1e-11)
        # the local torch build reproduces the committed vectors too
        y_t, gx_t, gw_t = oracle.torch_reference(torch.from_numpy(x), torch.from_numpy(wt), torch.from_numpy(gy), (sh, sw), (ph, pw))
        np.testing.assert_allclose(_np(y_t), z[f"c{i}_y"], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(_np(gx_t), z[f"c{i}_gx"], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(_np(gw_t), z[f"c{i}_gw"], rtol=1e-12, atol=1e-11)


def test_fused_reference_closed_forms():
    """torch_reference_fused = torch's conv followed by torch's elementwise functions; pinned by numpy closed forms."""
    g = torch.Generator("cpu").manual_seed(41)
    x = torch.randn(2, 3, 9, 8, generator=g, dtype=torch.float64) * 3
    w = torch.randn(3, 1, 3, 3, generator=g, dtype=torch.float64)
    scale = torch.tensor([0.5, -2.0, 3.0], dtype=torch.float64)
    shift = torch.tensor([1.0, 0.25, -4.0], dtype=torch.float64)
    plain = oracle.torch_reference(x, w, None, 2, 1)[0].numpy()
    assert np.array_equal(oracle.torch_reference_fused(x, w, None, None, None, 2, 1).numpy(), plain)
    z = plain * scale.numpy().reshape(1, 3, 1, 1) + shift.numpy().reshape(1, 3, 1, 1)
    np.testing.assert_allclose(oracle.torch_reference_fused(x, w, scale, shift, None, 2, 1).numpy(), z, rtol=1e-14)
    np.testing.assert_allclose(oracle.torch_reference_fused(x, w, scale, shift, "relu", 2, 1).numpy(), np.maximum(z, 0), rtol=1e-14)
    np.testing.assert_allclose(oracle.torch_reference_fused(x, w, scale, shift, "relu6", 2, 1).numpy(), np.clip(z, 0, 6), rtol=1e-14)
    np.testing.assert_allclose(oracle.torch_reference_fused(x, w, scale, shift, "silu", 2, 1).numpy(), z / (1 + np.exp(-z)),
                               rtol=1e-12, atol=1e-14)
    assert (z < 0).any() and (z > 6).any()  # every branch of the activations is exercised


def test_general_reference_against_brute_force():
    """torch_reference_general (torch's dilated, multiplied grouped conv) pinned by plain loops on a tiny case,
    and its gradients by the adjoint identities."""
    g = torch.Generator("cpu").manual_seed(47)
    n, c, m, h, w, kh, kw, s, p, d = 2, 3, 2, 9, 8, 3, 2, 2, 2, 2
    x = torch.randn(n, c, h, w, generator=g, dtype=torch.float64)
    wt = torch.randn(c * m, 1, kh, kw, generator=g, dtype=torch.float64)
    y, _, _ = oracle.torch_reference_general(x, wt, None, s, p, d)
    oh = (h + 2 * p - d * (kh - 1) - 1) // s + 1
    ow = (w + 2 * p - d * (kw - 1) - 1) // s + 1
    assert tuple(y.shape) == (n, c * m, oh, ow)
    ref = np.zeros((n, c * m, oh, ow))
    xn, wn = x.numpy(), wt.numpy()
    for b in range(n):
        for oc in range(c * m):
            for oy in range(oh):
                for ox in range(ow):
                    acc = 0.0
                    for ty in range(kh):
                        for tx in range(kw):
                            iy, ix = oy * s - p + ty * d, ox * s - p + tx * d
                            if 0 <= iy < h and 0 <= ix < w:
                                acc += xn[b, oc // m, iy, ix] * wn[oc, 0, ty, tx]
                    ref[b, oc, oy, ox] = acc
    np.testing.assert_allclose(y.numpy(), ref, rtol=1e-12, atol=1e-12)
    gy = torch.randn(y.shape, generator=g, dtype=torch.float64)
    _, gx, gw = oracle.torch_reference_general(x, wt, gy, s, p, d)
    lhs = float((y * gy).sum())
    assert abs(lhs - float((x * gx).sum())) < 1e-9 * max(1.0, abs(lhs))
    assert abs(lhs - float((wt * gw).sum())) < 1e-9 * max(1.0, abs(lhs))
    # multiplier 1, dilation 1 is the plain depthwise convolution
    w1 = torch.randn(c, 1, 3, 3, generator=g, dtype=torch.float64)
    np.testing.assert_array_equal(oracle.torch_reference_general(x, w1, None, 1, 1, 1)[0].numpy(),
                                  oracle.torch_reference(x, w1, None, 1, 1)[0].numpy())



# --------------------------------------------------------------------------
# the whole-tensor reference of the full-size GPU tests, and the routing restatement
# --------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(2, 3, 9, 8, 3, 1, 1), (2, 3, 9, 8, 3, 2, 1), (1, 4, 13, 11, 5, 2, 2),
                                   (2, 2, 7, 7, 7, 1, 3), (1, 2, 12, 15, 5, 1, 0), (2, 2, 11, 10, 4, 3, 1),
                                   (1, 3, 10, 9, 3, 2, 0)], ids=shape_id)
def test_shift_add_reference_equals_c_oracle(shape):
    n, c, h, w, k, s, p = shape
    x, wt, gy = make_inputs(shape, seed=41, dtype=torch.float64)
    y, gx, gw = oracle.shift_add_reference(x, wt, gy, s, p)
    np.testing.assert_allclose(y.numpy(), oracle.forward(x.numpy(), wt.numpy(), s, p), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gx.numpy(), oracle.grad_input(gy.numpy(), wt.numpy(), (h, w), s, p), rtol=1e-12,
                               atol=1e-12)
    np.testing.assert_allclose(gw.numpy(), oracle.grad_weight(x.numpy(), gy.numpy(), wt.shape, s, p), rtol=1e-12,
                               atol=1e-12)
    # rectangular filter, stride and padding as well
    g = torch.Generator("cpu").manual_seed(43)
    x = torch.randn(2, 3, 12, 10, generator=g, dtype=torch.float64)
    wt = torch.randn(3, 1, 5, 2, generator=g, dtype=torch.float64)
    gy = torch.randn(2, 3, 5, 9, generator=g, dtype=torch.float64)
    y, gx, gw = oracle.shift_add_reference(x, wt, gy, (2, 1), (1, 0))
    np.testing.assert_allclose(y.numpy(), oracle.forward(x.numpy(), wt.numpy(), (2, 1), (1, 0)), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gx.numpy(), oracle.grad_input(gy.numpy(), wt.numpy(), (12, 10), (2, 1), (1, 0)),
                               rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gw.numpy(), oracle.grad_weight(x.numpy(), gy.numpy(), wt.shape, (2, 1), (1, 0)),
                               rtol=1e-12, atol=1e-12)


# Which of its three paths the reference takes for every benchmark layer, read off torch_dwconv/dwconv.py:123-130
# and dwconv_kernel.cu:652-662 by hand: (H, k, stride) -> path ("native_conv2d" = the F.conv2d hand-off).
ROUTING_TABLE = [
    ((56, 3, 1), "large"), ((256, 5, 1), "large"), ((112, 3, 1), "large"), ((112, 3, 2), "large"),
    ((56, 5, 2), "large"), ((28, 5, 1), "small"), ((28, 3, 2), "native_conv2d"), ((14, 3, 1), "small"),
    ((14, 5, 1), "small"), ((14, 5, 2), "native_conv2d"), ((7, 5, 1), "small"), ((7, 3, 1), "small"),
    ((7, 7, 1), "native_conv2d"),    # 49 taps > ceil(7/2)*7 = 28 lanes
    ((14, 7, 1), "small"), ((56, 7, 1), "large"), ((28, 7, 1), "small"),
    ((33, 3, 1), "large"), ((32, 3, 1), "small"), ((4, 3, 1), "native_conv2d"),
]


@pytest.mark.parametrize("geom,expected", ROUTING_TABLE)
def test_route_matches_the_reference_routing_table(geom, expected):
    h, k, s = geom
    p = k // 2
    small = oracle.use_dwconv2d_small(h, h, k, k, 1, 1, s, s, p, p)
    assert oracle.host_logic.route((h, h), (k, k), (s, s), (p, p), small) == expected


def test_route_rectangular_planes():
    # one axis above 32 is enough for the large path (dwconv.py:125: `and`)
    assert oracle.host_logic.route((40, 8), (3, 3), (2, 2), (1, 1), False) == "large"
    assert oracle.host_logic.route((8, 40), (3, 3), (2, 2), (1, 1), False) == "large"
    assert oracle.host_logic.route((32, 32), (3, 3), (2, 2), (1, 1), False) == "native_conv2d"
