"""Binding of libdwconv_hip.so that stands where the reference's pybind11
module ``torch_dwconv._C`` stands (torch_dwconv/dwconv.cpp:60-67).

The four functions keep the reference's names, argument order and error
behaviour (a non-GPU tensor raises ``RuntimeError('... must be a CUDA
tensor')``, torch_dwconv/dwconv.cpp:24-25).  They allocate the result with
torch, pass raw device pointers plus the current HIP stream through the C ABI
declared in include/dwconv_hip.h, and return immediately (no synchronisation).

There is no CPU implementation behind this module: if the shared library is
missing, importing it raises ImportError.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libdwconv_hip.so")

if not os.path.exists(LIBRARY_PATH):
    raise ImportError(
        f"{LIBRARY_PATH} is missing: build it with `make -C depthwise-conv-pytorch_amd/csrc` "
        "(hipcc, --offload-arch=gfx950). torch_dwconv has no fallback implementation."
    )

_lib = ctypes.CDLL(LIBRARY_PATH)

_i, _p, _z = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
_lib.dwconv_last_error.restype = ctypes.c_char_p
_lib.dwconv_last_variant.restype = ctypes.c_char_p
_lib.dwconv_version.restype = ctypes.c_char_p
_lib.dwconv_out_size.restype = _i
_lib.dwconv_out_size.argtypes = [_i] * 6
_lib.dwconv_use_dwconv2d_small.restype = _i
_lib.dwconv_use_dwconv2d_small.argtypes = [_i] * 10
for _name in ("dwconv2d_f32", "dwconv2d_f64", "dwconv2d_f16", "dwconv2d_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p] + [_i] * 15 + [_p]
for _name in ("dwconv2d_small_f32", "dwconv2d_small_f64", "dwconv2d_small_f16", "dwconv2d_small_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p] + [_i] * 13 + [_p]
_lib.dwconv2d_backward_kernel_workspace_bytes.restype = _z
_lib.dwconv2d_backward_kernel_workspace_bytes.argtypes = [_i] * 13
for _name in ("dwconv2d_backward_kernel_f32", "dwconv2d_backward_kernel_f64", "dwconv2d_backward_kernel_f16",
              "dwconv2d_backward_kernel_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p, _p, _z] + [_i] * 14 + [_p]

for _name in ("dwconv2d_backward_f32", "dwconv2d_backward_f16", "dwconv2d_backward_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p, _p, _p, _p, _z] + [_i] * 12 + [_p]

# the entry point that allocates nothing: no workspace argument (include/dwconv_hip.h)
NOALLOC_SCRATCH_BYTES = 32 << 20
_lib.dwconv2d_backward_noalloc_f32.restype = _i
_lib.dwconv2d_backward_noalloc_f32.argtypes = [_p] * 5 + [_i] * 12 + [_p]

for _name in ("dwconv2d_nhwc_f32", "dwconv2d_nhwc_f64", "dwconv2d_nhwc_f16", "dwconv2d_nhwc_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p] + [_i] * 10 + [_p]
_lib.dwconv2d_backward_nhwc_workspace_bytes.restype = _z
_lib.dwconv2d_backward_nhwc_workspace_bytes.argtypes = [_i] * 11
for _name in ("dwconv2d_backward_nhwc_f32", "dwconv2d_backward_nhwc_f64", "dwconv2d_backward_nhwc_f16",
              "dwconv2d_backward_nhwc_bf16"):
    getattr(_lib, _name).restype = _i
    getattr(_lib, _name).argtypes = [_p, _p, _p, _p, _p, _p, _z] + [_i] * 12 + [_p]

for _sfx in ("f32", "f64", "f16", "bf16"):
    for _name in ("dwconv2d_fused_" + _sfx, "dwconv2d_fused_nhwc_" + _sfx):
        getattr(_lib, _name).restype = _i
        getattr(_lib, _name).argtypes = [_p, _p, _p, _p, _p] + [_i] * 11 + [_p]

_lib.dwconv2d_epilogue_backward_workspace_bytes.restype = _z
_lib.dwconv2d_epilogue_backward_workspace_bytes.argtypes = [_i] * 5
for _sfx in ("f32", "f16", "bf16"):
    getattr(_lib, "dwconv2d_epilogue_backward_" + _sfx).restype = _i
    getattr(_lib, "dwconv2d_epilogue_backward_" + _sfx).argtypes = [_p] * 7 + [_z] + [_i] * 6 + [_p]

_lib.dwconv2d_general_backward_workspace_bytes.restype = _z
_lib.dwconv2d_general_backward_workspace_bytes.argtypes = [_i] * 14
for _sfx in ("f32", "f64", "f16", "bf16"):
    getattr(_lib, "dwconv2d_general_" + _sfx).restype = _i
    getattr(_lib, "dwconv2d_general_" + _sfx).argtypes = [_p, _p, _p] + [_i] * 13 + [_p]
    getattr(_lib, "dwconv2d_general_backward_" + _sfx).restype = _i
    getattr(_lib, "dwconv2d_general_backward_" + _sfx).argtypes = [_p, _p, _p, _p, _p, _p, _z] + [_i] * 15 + [_p]

ACTIVATIONS = {None: 0, "none": 0, "relu": 1, "relu6": 2, "silu": 3}

_SUFFIX = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16"}


def version():
    return _lib.dwconv_version().decode()


def last_variant():
    """Name of the kernel variant the last call on this thread launched."""
    return _lib.dwconv_last_variant().decode()


def _check_cuda(t, name):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def _suffix(*tensors):
    dtype = tensors[0].dtype
    if dtype not in _SUFFIX:
        raise RuntimeError(f"torch_dwconv supports float32, float64, float16 and bfloat16 tensors, got {dtype}")
    for t in tensors[1:]:
        if t.dtype != dtype:
            raise RuntimeError(f"torch_dwconv needs tensors of one dtype, got {dtype} and {t.dtype}")
        if t.device != tensors[0].device:
            raise RuntimeError(f"torch_dwconv needs tensors on one device, got {tensors[0].device} and {t.device}")
    return _SUFFIX[dtype]


def _check_shapes(input, kernel):
    if input.dim() != 4 or kernel.dim() != 4:
        raise RuntimeError("torch_dwconv expects a 4-D input (N,C,H,W) and a 4-D kernel (C,1,KH,KW)")
    if kernel.shape[0] != input.shape[1] or kernel.shape[1] != 1:
        raise RuntimeError(
            f"kernel of shape {tuple(kernel.shape)} does not match an input with {input.shape[1]} channels: "
            "expected (C,1,KH,KW)"
        )


def _raise(status):
    raise RuntimeError(f"libdwconv_hip error {status}: {_lib.dwconv_last_error().decode()}")


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def use_dwconv2d_small(input, kernel, up_h, up_w, down_h, down_w, pad_h, pad_w):
    """torch_dwconv/dwconv_kernel.cu:652-662; pure geometry, no device work."""
    return bool(
        _lib.dwconv_use_dwconv2d_small(
            input.shape[2], input.shape[3], kernel.shape[2], kernel.shape[3],
            up_h, up_w, down_h, down_w, pad_h, pad_w,
        )
    )


def dwconv2d(input, kernel, up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward):
    """torch_dwconv/dwconv.cpp:27-35: up-sample / filter / down-sample of every plane."""
    _check_cuda(input, "input")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    sfx = _suffix(input, kernel)
    x, k = input.contiguous(), kernel.contiguous()
    n, c, h, w = x.shape
    kh, kw = k.shape[2], k.shape[3]
    oh = max(_lib.dwconv_out_size(h, up_h, down_h, pad_h0, pad_h1, kh), 0)
    ow = max(_lib.dwconv_out_size(w, up_w, down_w, pad_w0, pad_w1, kw), 0)
    out = torch.empty((n, c, oh, ow), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_" + sfx)(
            x.data_ptr(), k.data_ptr(), out.data_ptr(), n, c, h, w, kh, kw,
            up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, int(bool(forward)), _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return out


def dwconv2d_small(input, kernel, up_h, up_w, down_h, down_w, pad_h, pad_w, forward):
    """torch_dwconv/dwconv.cpp:37-46: whole-plane stride-1 same-size convolution."""
    _check_cuda(input, "input")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    sfx = _suffix(input, kernel)
    x, k = input.contiguous(), kernel.contiguous()
    n, c, h, w = x.shape
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_small_" + sfx)(
            x.data_ptr(), k.data_ptr(), out.data_ptr(), n, c, h, w, k.shape[2], k.shape[3],
            up_h, up_w, down_h, down_w, pad_h, pad_w, int(bool(forward)), _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return out


def dwconv2d_backward_kernel(input, out_grad, kernel, up_h, up_w, down_h, down_w, pad_h, pad_w):
    """torch_dwconv/dwconv.cpp:48-58: gradient of the filter; `kernel` only lends its shape."""
    _check_cuda(input, "input")
    _check_cuda(out_grad, "out_grad")
    if input.dim() != 4 or out_grad.dim() != 4 or kernel.dim() != 4:
        raise RuntimeError("torch_dwconv expects 4-D tensors")
    if out_grad.shape[:2] != input.shape[:2] or kernel.shape[0] != input.shape[1]:
        raise RuntimeError(
            f"shapes do not belong to one depthwise conv: input {tuple(input.shape)}, "
            f"out_grad {tuple(out_grad.shape)}, kernel {tuple(kernel.shape)}"
        )
    sfx = _suffix(input, out_grad)
    x, gy = input.contiguous(), out_grad.contiguous()
    n, c, h, w = x.shape
    oh, ow = gy.shape[2], gy.shape[3]
    kh, kw = kernel.shape[2], kernel.shape[3]
    gw = torch.empty((c, 1, kh, kw), dtype=x.dtype, device=x.device)
    geom = (n, c, h, w, oh, ow, kh, kw)
    ws_bytes = _lib.dwconv2d_backward_kernel_workspace_bytes(*geom, down_h, down_w, pad_h, pad_w, x.element_size())
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_backward_kernel_" + sfx)(
            x.data_ptr(), gy.data_ptr(), gw.data_ptr(), ws.data_ptr(), ws_bytes, *geom,
            up_h, up_w, down_h, down_w, pad_h, pad_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return gw


def dwconv2d_backward(input, out_grad, kernel, stride_h, stride_w, pad_h, pad_w):
    """Both gradients of ``depthwise_conv2d(input, kernel, stride, pad)`` for float32, float16 or bfloat16 tensors.

    One call for the two the reference's backward makes (torch_dwconv/dwconv.py:56-68); the library reads
    ``out_grad`` once where a fused kernel covers the geometry.  Returns ``(grad_input, grad_kernel)``.
    """
    _check_cuda(input, "input")
    _check_cuda(out_grad, "out_grad")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    if out_grad.dim() != 4 or out_grad.shape[:2] != input.shape[:2]:
        raise RuntimeError(f"out_grad of shape {tuple(out_grad.shape)} does not belong to input {tuple(input.shape)}")
    suffix = _suffix(input, out_grad, kernel)
    if suffix == "f64":
        raise RuntimeError("dwconv2d_backward has no float64 entry point")
    x, gy, k = input.contiguous(), out_grad.contiguous(), kernel.contiguous()
    n, c, h, w = x.shape
    oh, ow = gy.shape[2], gy.shape[3]
    kh, kw = k.shape[2], k.shape[3]
    gx = torch.empty_like(x)
    gw = torch.empty_like(k)
    geom = (n, c, h, w, oh, ow, kh, kw)
    ws_bytes = _lib.dwconv2d_backward_kernel_workspace_bytes(*geom, stride_h, stride_w, pad_h, pad_w, x.element_size())
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_backward_" + suffix)(
            x.data_ptr(), gy.data_ptr(), k.data_ptr(), gx.data_ptr(), gw.data_ptr(), ws.data_ptr(), ws_bytes,
            *geom, stride_h, stride_w, pad_h, pad_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return gx, gw


def dwconv2d_backward_noalloc(input, out_grad, kernel, in_grad, kernel_grad, stride_h, stride_w, pad_h, pad_w):
    """``dwconv2d_backward`` into tensors the caller already owns, with no allocation anywhere: float32, dense NCHW
    tensors only; the library's built-in scratch buffer (``NOALLOC_SCRATCH_BYTES`` per device) stands for the
    workspace.  Calls on one device share that buffer: keep them on one stream.  No counterpart in the reference."""
    for name, t in (("input", input), ("out_grad", out_grad), ("kernel", kernel), ("in_grad", in_grad),
                    ("kernel_grad", kernel_grad)):
        _check_cuda(t, name)
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous float32 tensor")
    _check_shapes(input, kernel)
    if out_grad.dim() != 4 or out_grad.shape[:2] != input.shape[:2]:
        raise RuntimeError(f"out_grad of shape {tuple(out_grad.shape)} does not belong to input {tuple(input.shape)}")
    if in_grad.shape != input.shape or kernel_grad.shape != kernel.shape:
        raise RuntimeError("in_grad / kernel_grad must have the shapes of input / kernel")
    n, c, h, w = input.shape
    with torch.cuda.device(input.device):
        rc = _lib.dwconv2d_backward_noalloc_f32(
            input.data_ptr(), out_grad.data_ptr(), kernel.data_ptr(), in_grad.data_ptr(), kernel_grad.data_ptr(),
            n, c, h, w, out_grad.shape[2], out_grad.shape[3], kernel.shape[2], kernel.shape[3],
            stride_h, stride_w, pad_h, pad_w, _stream(input),
        )
    if rc != 0:
        _raise(rc)


# ---- channels-last tensors -----------------------------------------------------------------------------
def is_channels_last(t):
    """True when ``t`` (logical shape N,C,H,W) is laid out N,H,W,C in memory and not also N,C,H,W."""
    return t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last) and not t.is_contiguous()


def dwconv2d_nhwc(input, kernel, stride_h, stride_w, pad_h, pad_w):
    """Forward convolution of a channels-last ``input`` (logical shape N,C,H,W); the result is channels-last too.

    The reference has no such path: it makes ``input`` NCHW-contiguous first (torch_dwconv/dwconv_kernel.cu:855).
    """
    _check_cuda(input, "input")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    sfx = _suffix(input, kernel)
    x, k = input.contiguous(memory_format=torch.channels_last), kernel.contiguous()
    n, c, h, w = x.shape
    kh, kw = k.shape[2], k.shape[3]
    oh = max(_lib.dwconv_out_size(h, 1, stride_h, pad_h, pad_h, kh), 0)
    ow = max(_lib.dwconv_out_size(w, 1, stride_w, pad_w, pad_w, kw), 0)
    out = torch.empty((n, c, oh, ow), dtype=x.dtype, device=x.device, memory_format=torch.channels_last)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_nhwc_" + sfx)(
            x.data_ptr(), k.data_ptr(), out.data_ptr(), n, c, h, w, kh, kw, stride_h, stride_w, pad_h, pad_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return out


def dwconv2d_backward_nhwc(input, out_grad, kernel, stride_h, stride_w, pad_h, pad_w, need_input_grad=True,
                           need_kernel_grad=True):
    """Both gradients for channels-last ``input`` / ``out_grad``; ``grad_input`` comes back channels-last.  A gradient
    that is not needed is not computed and comes back as ``None``."""
    _check_cuda(input, "input")
    _check_cuda(out_grad, "out_grad")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    if out_grad.dim() != 4 or out_grad.shape[:2] != input.shape[:2]:
        raise RuntimeError(f"out_grad of shape {tuple(out_grad.shape)} does not belong to input {tuple(input.shape)}")
    sfx = _suffix(input, out_grad, kernel)
    x = input.contiguous(memory_format=torch.channels_last)
    gy = out_grad.contiguous(memory_format=torch.channels_last)
    k = kernel.contiguous()
    n, c, h, w = x.shape
    oh, ow = gy.shape[2], gy.shape[3]
    kh, kw = k.shape[2], k.shape[3]
    if not (need_input_grad or need_kernel_grad):
        return None, None
    gx = torch.empty_like(x, memory_format=torch.channels_last) if need_input_grad else None
    gw = torch.empty_like(k) if need_kernel_grad else None
    ws_bytes = _lib.dwconv2d_backward_nhwc_workspace_bytes(n, c, h, w, kh, kw, stride_h, stride_w, pad_h, pad_w,
                                                           x.element_size())
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_backward_nhwc_" + sfx)(
            x.data_ptr(), gy.data_ptr(), k.data_ptr(), gx.data_ptr() if need_input_grad else None,
            gw.data_ptr() if need_kernel_grad else None, ws.data_ptr(), ws_bytes,
            n, c, h, w, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return gx, gw


def dwconv2d_fused(input, kernel, scale, shift, activation, stride_h, stride_w, pad_h, pad_w):
    """``act(conv(input, kernel) * scale[c] + shift[c])`` in one kernel; NCHW or channels-last (kept) input.

    ``scale`` / ``shift``: per-channel tensors or ``None``; ``activation``: ``None``, ``'relu'``, ``'relu6'`` or
    ``'silu'``.  The reference has no such entry point (it rejects a bias, torch_dwconv/dwconv.py:108-109).
    """
    _check_cuda(input, "input")
    _check_cuda(kernel, "kernel")
    _check_shapes(input, kernel)
    sfx = _suffix(input, kernel)
    if activation not in ACTIVATIONS:
        raise ValueError(f"unknown activation {activation!r}; expected one of None, 'relu', 'relu6', 'silu'")
    param_dtype = torch.float64 if input.dtype == torch.float64 else torch.float32
    params = []
    for name, t in (("scale", scale), ("shift", shift)):
        if t is None:
            params.append(None)
            continue
        _check_cuda(t, name)
        if t.numel() != input.shape[1]:
            raise RuntimeError(f"{name} must have one entry per channel ({input.shape[1]}), got {tuple(t.shape)}")
        params.append(t.detach().reshape(-1).to(device=input.device, dtype=param_dtype).contiguous())
    nhwc = is_channels_last(input)
    x = input.contiguous(memory_format=torch.channels_last) if nhwc else input.contiguous()
    k = kernel.contiguous()
    n, c, h, w = x.shape
    kh, kw = k.shape[2], k.shape[3]
    oh = max(_lib.dwconv_out_size(h, 1, stride_h, pad_h, pad_h, kh), 0)
    ow = max(_lib.dwconv_out_size(w, 1, stride_w, pad_w, pad_w, kw), 0)
    out = torch.empty((n, c, oh, ow), dtype=x.dtype, device=x.device,
                      memory_format=torch.channels_last if nhwc else torch.contiguous_format)
    fn = getattr(_lib, ("dwconv2d_fused_nhwc_" if nhwc else "dwconv2d_fused_") + sfx)
    with torch.cuda.device(x.device):
        rc = fn(x.data_ptr(), k.data_ptr(), params[0].data_ptr() if params[0] is not None else None,
                params[1].data_ptr() if params[1] is not None else None, out.data_ptr(), n, c, h, w, kh, kw,
                stride_h, stride_w, pad_h, pad_w, ACTIVATIONS[activation], _stream(x))
    if rc != 0:
        _raise(rc)
    return out


def dwconv2d_epilogue_backward(conv_out, out_grad, scale, shift, activation):
    """Backward of ``act(conv_out * scale[c] + shift[c])`` in one sweep (float32, float16 or bfloat16; NCHW or
    channels-last, taken from ``conv_out``): returns ``(conv_out_grad, scale_grad, shift_grad)``.  ``conv_out`` is
    overwritten with ``conv_out_grad`` (the same tensor comes back); the two parameter gradients are float32
    vectors of ``C`` entries.  No counterpart in the reference."""
    _check_cuda(conv_out, "conv_out")
    _check_cuda(out_grad, "out_grad")
    sfx = _suffix(conv_out, out_grad)
    if sfx == "f64":
        raise RuntimeError("dwconv2d_epilogue_backward has no float64 entry point")
    if activation not in ACTIVATIONS:
        raise ValueError(f"unknown activation {activation!r}; expected one of None, 'relu', 'relu6', 'silu'")
    if conv_out.dim() != 4 or out_grad.shape != conv_out.shape:
        raise RuntimeError(f"out_grad of shape {tuple(out_grad.shape)} does not belong to conv_out {tuple(conv_out.shape)}")
    nhwc = is_channels_last(conv_out)
    fmt = torch.channels_last if nhwc else torch.contiguous_format
    if not conv_out.is_contiguous(memory_format=fmt):
        raise RuntimeError("conv_out must be dense (NCHW or channels-last): it is overwritten in place")
    gy = out_grad.contiguous(memory_format=fmt)
    n, c, oh, ow = conv_out.shape
    params = []
    for name, t in (("scale", scale), ("shift", shift)):
        if t is None:
            params.append(None)
            continue
        _check_cuda(t, name)
        if t.numel() != c:
            raise RuntimeError(f"{name} must have one entry per channel ({c}), got {tuple(t.shape)}")
        params.append(t.detach().reshape(-1).to(device=conv_out.device, dtype=torch.float32).contiguous())
    grads = torch.empty((c, 2), dtype=torch.float32, device=conv_out.device)
    ws_bytes = _lib.dwconv2d_epilogue_backward_workspace_bytes(n, c, oh, ow, int(nhwc))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=conv_out.device)
    with torch.cuda.device(conv_out.device):
        rc = getattr(_lib, "dwconv2d_epilogue_backward_" + sfx)(
            conv_out.data_ptr(), gy.data_ptr(), params[0].data_ptr() if params[0] is not None else None,
            params[1].data_ptr() if params[1] is not None else None, conv_out.data_ptr(), grads.data_ptr(),
            ws.data_ptr(), ws_bytes, n, c, oh, ow, ACTIVATIONS[activation], int(nhwc), _stream(conv_out),
        )
    if rc != 0:
        _raise(rc)
    return conv_out, grads[:, 0], grads[:, 1]


# ---- dilation and depth multiplier -----------------------------------------------------------------------
def _multiplier(input, kernel):
    if input.dim() != 4 or kernel.dim() != 4 or kernel.shape[1] != 1 or input.shape[1] == 0 or \
            kernel.shape[0] % input.shape[1] != 0 or kernel.shape[0] == 0:
        raise RuntimeError(
            f"kernel of shape {tuple(kernel.shape)} does not match an input of shape {tuple(input.shape)}: "
            "expected (C*multiplier,1,KH,KW)"
        )
    return kernel.shape[0] // input.shape[1]


def dwconv2d_general(input, kernel, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w):
    """``F.conv2d(input, kernel, stride, padding, dilation, groups=C)`` for a kernel of shape (C*M,1,KH,KW)."""
    _check_cuda(input, "input")
    _check_cuda(kernel, "kernel")
    m = _multiplier(input, kernel)
    sfx = _suffix(input, kernel)
    x, k = input.contiguous(), kernel.contiguous()
    n, c, h, w = x.shape
    kh, kw = k.shape[2], k.shape[3]
    oh = max((h + 2 * pad_h - dil_h * (kh - 1) - 1) // stride_h + 1, 0) if h + 2 * pad_h - dil_h * (kh - 1) - 1 >= 0 else 0
    ow = max((w + 2 * pad_w - dil_w * (kw - 1) - 1) // stride_w + 1, 0) if w + 2 * pad_w - dil_w * (kw - 1) - 1 >= 0 else 0
    out = torch.empty((n, c * m, oh, ow), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_general_" + sfx)(
            x.data_ptr(), k.data_ptr(), out.data_ptr(), n, c, h, w, m, kh, kw, stride_h, stride_w, pad_h, pad_w,
            dil_h, dil_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return out


def dwconv2d_general_backward(input, out_grad, kernel, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w):
    """Both gradients of ``dwconv2d_general``; returns ``(grad_input, grad_kernel)``."""
    _check_cuda(input, "input")
    _check_cuda(out_grad, "out_grad")
    _check_cuda(kernel, "kernel")
    m = _multiplier(input, kernel)
    sfx = _suffix(input, out_grad, kernel)
    x, gy, k = input.contiguous(), out_grad.contiguous(), kernel.contiguous()
    n, c, h, w = x.shape
    if gy.dim() != 4 or gy.shape[0] != n or gy.shape[1] != c * m:
        raise RuntimeError(f"out_grad of shape {tuple(gy.shape)} does not belong to input {tuple(x.shape)}")
    oh, ow = gy.shape[2], gy.shape[3]
    kh, kw = k.shape[2], k.shape[3]
    gx = torch.empty_like(x)
    gw = torch.empty_like(k)
    ws_bytes = _lib.dwconv2d_general_backward_workspace_bytes(n, c, h, w, m, kh, kw, stride_h, stride_w, pad_h, pad_w,
                                                              dil_h, dil_w, x.element_size())
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = getattr(_lib, "dwconv2d_general_backward_" + sfx)(
            x.data_ptr(), gy.data_ptr(), k.data_ptr(), gx.data_ptr(), gw.data_ptr(), ws.data_ptr(), ws_bytes,
            n, c, h, w, oh, ow, m, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, _stream(x),
        )
    if rc != 0:
        _raise(rc)
    return gx, gw
