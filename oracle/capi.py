"""ctypes front-end of dwconv_oracle.c (fp64 numpy arrays in and out)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdwconv_oracle.so")
_lib = None

_dp = ctypes.POINTER(ctypes.c_double)


def build(force=False):
    """Compile dwconv_oracle.c with gcc (a second or two)."""
    if force or not os.path.exists(_SO) or (
        os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "dwconv_oracle.c"))
    ):
        subprocess.run(["make", "-s", "-B", "-C", _HERE, "libdwconv_oracle.so"], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_SO)
        lib.oracle_out_size.restype = ctypes.c_int
        lib.oracle_out_size.argtypes = [ctypes.c_int] * 6
        lib.oracle_use_dwconv2d_small.restype = ctypes.c_int
        lib.oracle_use_dwconv2d_small.argtypes = [ctypes.c_int] * 10
        lib.oracle_dwconv2d_f64.restype = None
        lib.oracle_dwconv2d_f64.argtypes = [_dp, _dp, _dp] + [ctypes.c_int] * 15
        lib.oracle_dwconv2d_small_f64.restype = None
        lib.oracle_dwconv2d_small_f64.argtypes = [_dp, _dp, _dp] + [ctypes.c_int] * 9
        lib.oracle_backward_kernel_f64.restype = None
        lib.oracle_backward_kernel_f64.argtypes = [_dp, _dp, _dp] + [ctypes.c_int] * 12
        _lib = lib
    return _lib


def _f64(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.float64)


def _ptr(a):
    return a.ctypes.data_as(_dp)


def _pair(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]), int(v[1])
    return int(v), int(v)


def out_size(in_size, up, down, pad0, pad1, k):
    return _load().oracle_out_size(in_size, up, down, pad0, pad1, k)


def use_dwconv2d_small(in_h, in_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w, pad_h, pad_w):
    return bool(
        _load().oracle_use_dwconv2d_small(
            in_h, in_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w, pad_h, pad_w
        )
    )


def dwconv2d(x, kernel, up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward):
    """Generic up/FIR/down operator of the large-map kernel (either direction)."""
    x, kernel = _f64(x), _f64(kernel)
    n, c, h, w = x.shape
    kh, kw = kernel.shape[-2:]
    assert kernel.shape[0] == c
    oh = out_size(h, up_h, down_h, pad_h0, pad_h1, kh)
    ow = out_size(w, up_w, down_w, pad_w0, pad_w1, kw)
    out = np.zeros((n, c, max(oh, 0), max(ow, 0)), dtype=np.float64)
    if out.size:
        _load().oracle_dwconv2d_f64(
            _ptr(x), _ptr(kernel), _ptr(out), n, c, h, w, kh, kw,
            up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, int(bool(forward)),
        )
    return out


def dwconv2d_small(x, kernel, pad_h, pad_w, forward):
    """Same-size stride-1 operator of the small-map kernel (either direction)."""
    x, kernel = _f64(x), _f64(kernel)
    n, c, h, w = x.shape
    kh, kw = kernel.shape[-2:]
    out = np.zeros_like(x)
    if out.size:
        _load().oracle_dwconv2d_small_f64(
            _ptr(x), _ptr(kernel), _ptr(out), n, c, h, w, kh, kw, pad_h, pad_w, int(bool(forward))
        )
    return out


def backward_kernel(x, out_grad, kernel_shape, down_h, down_w, pad_h, pad_w):
    x, out_grad = _f64(x), _f64(out_grad)
    n, c, h, w = x.shape
    oh, ow = out_grad.shape[-2:]
    kh, kw = kernel_shape[-2:]
    gw = np.zeros((c, 1, kh, kw), dtype=np.float64)
    if gw.size and x.size and out_grad.size:
        _load().oracle_backward_kernel_f64(
            _ptr(x), _ptr(out_grad), _ptr(gw), n, c, h, w, oh, ow, kh, kw, down_h, down_w, pad_h, pad_w
        )
    return gw


# -- the three passes as the autograd Function strings them together -----------
# (torch_dwconv/dwconv.py:17-70)

def forward(x, w, stride=1, padding=0):
    """dwconv.py:33-35: large op, up=1, down=stride, symmetric padding."""
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    return dwconv2d(x, w, 1, 1, sh, sw, ph, ph, pw, pw, True)


def grad_input(gy, w, in_hw, stride=1, padding=0):
    """dwconv.py:39-44 (g_pad) and :61-64: backward-direction op with up=stride."""
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    in_h, in_w = in_hw
    kh, kw = np.asarray(w).shape[-2:]
    oh, ow = np.asarray(gy).shape[-2:]
    g_pad = (kh - ph - 1, in_h - oh * sh + ph, kw - pw - 1, in_w - ow * sw + pw)
    return dwconv2d(gy, w, sh, sw, 1, 1, g_pad[0], g_pad[1], g_pad[2], g_pad[3], False)


def grad_weight(x, gy, kernel_shape, stride=1, padding=0):
    """dwconv.py:66-68."""
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    return backward_kernel(x, gy, kernel_shape, sh, sw, ph, pw)
