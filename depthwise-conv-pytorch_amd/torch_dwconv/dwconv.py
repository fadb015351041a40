"""Python surface of the depthwise conv2d op: same names, argument order and
errors as the reference's torch_dwconv/dwconv.py, on top of the HIP library.

``depthwise_conv2d(input, weight, bias=None, stride=1, padding=0, dilation=1,
groups=None)`` computes what ``F.conv2d(input, weight, stride=stride,
padding=padding, groups=C)`` computes, for GPU tensors in float32, float64,
float16 or bfloat16, NCHW-contiguous or channels-last (the output then is
channels-last as well).

One deliberate difference: the reference hands planes of at most 32x32 that its
small kernel cannot take (stride 2, or a filter too large for the plane) to
``F.conv2d`` (torch_dwconv/dwconv.py:125-128).  Here those go through the HIP
library as well, so nothing inside ``custom=True`` ever leaves it; the values
are the same function either way.
"""
import torch
from torch import nn
from torch.autograd import Function
from torch.nn import functional as F

from . import _C


def make_tuple(value, n_value):
    """Reference: torch_dwconv/dwconv.py:76-91.

    A scalar becomes ``n_value`` copies; a list/tuple that is longer raises
    ``ValueError``; one of exactly that length is returned unchanged; a shorter
    one is repeated ``n_value`` times.
    """
    if isinstance(value, (list, tuple)):
        have = len(value)
        if have > n_value:
            raise ValueError(
                f'Number items does not match with requirements: {have}, expected: {n_value}'
            )
        return value if have == n_value else value * n_value
    return (value,) * n_value


_UNSUPPORTED = (
    # (predicate over the normalised options, message) in the reference's order,
    # torch_dwconv/dwconv.py:99-112
    (lambda o: o['dilation'][0] > 1 or o['dilation'][1] > 1,
     'DepthwiseConv2d does not support dilations > 1'),
    (lambda o: o['groups'] is not None and o['groups'] != o['in_channels'],
     'DepthwiseConv2d does not support groups != in_channels'),
    (lambda o: o['in_channels'] != o['out_channels'],
     'DepthwiseConv2d does not support in_channels != out_channels'),
    (lambda o: bool(o['bias']),
     'DepthwiseConv2d does not support bias'),
    (lambda o: o['padding_mode'] != 'zeros',
     'DepthwiseConv2d does not non-zero paddings'),
)


def check_options(in_channels, out_channels, dilation, groups, bias, padding_mode='zeros'):
    """Reference: torch_dwconv/dwconv.py:94-112. Raises ``ValueError`` on the first unsupported option."""
    options = dict(
        in_channels=in_channels, out_channels=out_channels, dilation=make_tuple(dilation, 2),
        groups=groups, bias=bias, padding_mode=padding_mode,
    )
    for rejected, message in _UNSUPPORTED:
        if rejected(options):
            raise ValueError(message)


def use_dwconv2d_small(input, weight, up, stride, padding):
    """Reference: torch_dwconv/dwconv.py:9-12."""
    return _C.use_dwconv2d_small(input, weight, up[0], up[1], stride[0], stride[1], padding[0], padding[1])


class DepthwiseConv2dFunction(Function):
    """Reference: torch_dwconv/dwconv.py:15-70 (same arguments, same six-value backward)."""

    @staticmethod
    def forward(ctx, input, kernel, stride, pad, small):
        ctx.save_for_backward(input, kernel)
        ctx.stride, ctx.pad, ctx.use_small = stride, pad, small
        # Channels-last activations stay channels-last (the reference converts them to NCHW,
        # torch_dwconv/dwconv_kernel.cu:855): same values, no layout-conversion pass either side of the op.
        ctx.channels_last = _C.is_channels_last(input)
        if ctx.channels_last:
            ctx.g_pad = None
            return _C.dwconv2d_nhwc(input, kernel, stride[0], stride[1], pad[0], pad[1])
        if small:
            out = _C.dwconv2d_small(input, kernel, 1, 1, stride[0], stride[1], pad[0], pad[1], True)
        else:
            out = _C.dwconv2d(input, kernel, 1, 1, stride[0], stride[1], pad[0], pad[0], pad[1], pad[1], True)
        # Padding of the transposed problem (reference :39-44): leading k-1-p zeros, and trailing
        # whatever makes the gradient come out with the input's extent (this also covers the rows
        # and columns a stride leaves unused).
        ctx.g_pad = tuple(
            v
            for axis in (0, 1)
            for v in (
                kernel.shape[2 + axis] - pad[axis] - 1,
                input.shape[2 + axis] - out.shape[2 + axis] * stride[axis] + pad[axis],
            )
        )
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, kernel = ctx.saved_tensors
        stride, pad, g_pad = ctx.stride, ctx.pad, ctx.g_pad
        # The reference always computes both gradients (:48-70).  Here a gradient nobody asked for (a frozen filter, the
        # network's first layer) is skipped: autograd takes None for it.
        need_input, need_kernel = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if ctx.channels_last:
            grad_input, grad_kernel = _C.dwconv2d_backward_nhwc(
                input, grad_output, kernel, stride[0], stride[1], pad[0], pad[1], need_input, need_kernel
            )
            return grad_input, grad_kernel, None, None, None, None
        if input.dtype != torch.float64 and need_input and need_kernel:
            # one library call for the pair of calls below; same values, out_grad read once where fused
            grad_input, grad_kernel = _C.dwconv2d_backward(
                input, grad_output, kernel, stride[0], stride[1], pad[0], pad[1]
            )
            return grad_input, grad_kernel, None, None, None, None
        grad_input = grad_kernel = None
        if need_input and ctx.use_small:
            grad_input = _C.dwconv2d_small(
                grad_output, kernel, stride[0], stride[1], 1, 1, g_pad[0], g_pad[2], False
            )
        elif need_input:
            grad_input = _C.dwconv2d(grad_output, kernel, stride[0], stride[1], 1, 1, *g_pad, False)
        if need_kernel:
            grad_kernel = _C.dwconv2d_backward_kernel(
                input, grad_output, kernel, 1, 1, stride[0], stride[1], pad[0], pad[1]
            )
        return grad_input, grad_kernel, None, None, None, None


depthwise_conv2d_fn = DepthwiseConv2dFunction.apply


def _autocast(input, weight):
    """Inside ``torch.autocast('cuda', dtype)`` both operands are cast to the autocast dtype, as PyTorch does for its own
    convolutions (the casts are differentiable, so ``weight.grad`` keeps the parameter's dtype).  The reference has no
    autocast rule: there a half-precision activation and an fp32 weight do not meet."""
    if input.is_cuda and torch.is_autocast_enabled("cuda"):
        dtype = torch.get_autocast_dtype("cuda")
        return input.to(dtype), weight.to(dtype)
    return input, weight


def depthwise_conv2d(input, weight, bias=None, stride=1, padding=0, dilation=1, groups=None):
    """Reference: torch_dwconv/dwconv.py:115-130."""
    stride = make_tuple(stride, 2)
    padding = make_tuple(padding, 2)
    check_options(input.shape[1], weight.shape[0], dilation, groups, bias)
    input, weight = _autocast(input, weight)
    small = use_dwconv2d_small(input, weight, (1, 1), stride, padding)
    return depthwise_conv2d_fn(input, weight, stride, padding, small)


class DepthwiseConv2dGeneralFunction(Function):
    """Autograd wrapper of the entry points with dilation and depth multiplier (not in the reference)."""

    @staticmethod
    def forward(ctx, input, kernel, stride, pad, dilation):
        ctx.save_for_backward(input, kernel)
        ctx.geometry = (stride[0], stride[1], pad[0], pad[1], dilation[0], dilation[1])
        return _C.dwconv2d_general(input, kernel, *ctx.geometry)

    @staticmethod
    def backward(ctx, grad_output):
        input, kernel = ctx.saved_tensors
        grad_input, grad_kernel = _C.dwconv2d_general_backward(input, grad_output, kernel, *ctx.geometry)
        return grad_input, grad_kernel, None, None, None


def depthwise_conv2d_general(input, weight, stride=1, padding=0, dilation=1):
    """``F.conv2d(input, weight, stride=stride, padding=padding, dilation=dilation, groups=C)`` for a ``weight`` of
    shape ``(C*M, 1, KH, KW)``: the dilation and the depth multiplier ``M`` that ``depthwise_conv2d`` refuses, as the
    reference does (torch_dwconv/dwconv.py:99-106).  With ``M == 1`` and no dilation it runs the same kernels as
    ``depthwise_conv2d``.  Tuned as well: dilation 2 with 3x3 / 5x5 filters at stride 1 and "same" padding, and a depth
    multiplier with square 3x3 / 5x5 / 7x7 filters at stride 1 or 2 on maps from about 46x46 up.  Everything else runs
    per-element kernels (correct for every geometry, not tuned)."""
    stride = make_tuple(stride, 2)
    padding = make_tuple(padding, 2)
    dilation = make_tuple(dilation, 2)
    return DepthwiseConv2dGeneralFunction.apply(input, weight, stride, padding, dilation)


_TORCH_ACTIVATIONS = {None: None, "none": None, "relu": F.relu, "relu6": F.relu6, "silu": F.silu}


class DepthwiseConv2dFusedFunction(Function):
    """Autograd wrapper of the fused forward ``act(conv(x, w) * scale + shift)`` (not in the reference).

    Forward: one kernel; only the inputs are kept for the backward pass (no pre-activation tensor).  Backward:
    the convolution result is recomputed with the plain forward kernel, one sweep turns it and ``grad_output``
    into the gradient of the convolution result plus the gradients of ``scale`` and ``shift``
    (``_C.dwconv2d_epilogue_backward``), and that goes through the ordinary backward kernels.

    Corner behaviour with float16 / bfloat16 tensors and ReLU / ReLU6: the forward kernel applies the activation to
    its fp32 sum, the backward pass takes the mask from the recomputed result after that was rounded to 16 bits.
    An output whose pre-activation lies within one 16-bit rounding step of 0 (or of 6) can therefore get the slope
    of the other side of the corner; no other output is affected (with fp32 tensors the window shrinks to the last
    bit of the fp32 sum)."""

    @staticmethod
    def forward(ctx, input, kernel, scale, shift, activation, stride, pad):
        ctx.save_for_backward(input, kernel, scale, shift)
        ctx.activation, ctx.stride, ctx.pad = activation, stride, pad
        return _C.dwconv2d_fused(input, kernel, scale, shift, activation, stride[0], stride[1], pad[0], pad[1])

    @staticmethod
    def backward(ctx, grad_output):
        input, kernel, scale, shift = ctx.saved_tensors
        stride, pad = ctx.stride, ctx.pad
        need_input, need_kernel, need_scale, need_shift = ctx.needs_input_grad[:4]
        if _C.is_channels_last(input):
            conv = _C.dwconv2d_nhwc(input, kernel, stride[0], stride[1], pad[0], pad[1])
        else:
            conv = _C.dwconv2d(input, kernel, 1, 1, stride[0], stride[1], pad[0], pad[0], pad[1], pad[1], True)
        conv_grad, scale_grad, shift_grad = _C.dwconv2d_epilogue_backward(conv, grad_output, scale, shift, ctx.activation)
        grad_input = grad_kernel = None
        if _C.is_channels_last(input):
            grad_input, grad_kernel = _C.dwconv2d_backward_nhwc(input, conv_grad, kernel, stride[0], stride[1], pad[0],
                                                                pad[1], need_input, need_kernel)
        elif need_input and need_kernel:
            grad_input, grad_kernel = _C.dwconv2d_backward(input, conv_grad, kernel, stride[0], stride[1], pad[0], pad[1])
        elif need_input:
            g_pad = tuple(v for a in (0, 1) for v in (kernel.shape[2 + a] - pad[a] - 1,
                                                      input.shape[2 + a] - conv.shape[2 + a] * stride[a] + pad[a]))
            grad_input = _C.dwconv2d(conv_grad, kernel, stride[0], stride[1], 1, 1, *g_pad, False)
        elif need_kernel:
            grad_kernel = _C.dwconv2d_backward_kernel(input, conv_grad, kernel, 1, 1, stride[0], stride[1], pad[0], pad[1])
        scale_grad = scale_grad.to(scale.dtype).view_as(scale) if need_scale and scale is not None else None
        shift_grad = shift_grad.to(shift.dtype).view_as(shift) if need_shift and shift is not None else None
        return grad_input, grad_kernel, scale_grad, shift_grad, None, None, None


def depthwise_conv2d_fused(input, weight, bias=None, scale=None, activation=None, stride=1, padding=0):
    """``act(depthwise_conv2d(input, weight) * scale[c] + bias[c])``: the convolution together with the step that
    follows it in EfficientNet / MobileNet blocks (bias or folded batch-norm, then ReLU / ReLU6 / SiLU).

    Not in the reference, whose ``check_options`` rejects a bias (torch_dwconv/dwconv.py:108-109).  One kernel in the
    forward pass, with or without gradients.  In training the backward pass recomputes the convolution result instead of
    keeping it (``DepthwiseConv2dFusedFunction``); float64 tensors, which have no such kernels, are composed from
    ``depthwise_conv2d`` and PyTorch's elementwise ops when a gradient is needed.
    """
    if activation not in _TORCH_ACTIVATIONS:
        raise ValueError(f"unknown activation {activation!r}; expected one of None, 'relu', 'relu6', 'silu'")
    stride = make_tuple(stride, 2)
    padding = make_tuple(padding, 2)
    check_options(input.shape[1], weight.shape[0], 1, None, False)
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (input, weight, bias, scale)
    )
    if not needs_grad:
        return _C.dwconv2d_fused(input, weight, scale, bias, activation, stride[0], stride[1], padding[0], padding[1])
    if input.dtype != torch.float64:
        return DepthwiseConv2dFusedFunction.apply(input, weight, scale, bias, activation, stride, padding)
    out = depthwise_conv2d(input, weight, None, stride, padding)
    if scale is not None:
        out = out * scale.view(1, -1, 1, 1).to(out.dtype)
    if bias is not None:
        out = out + bias.view(1, -1, 1, 1).to(out.dtype)
    act = _TORCH_ACTIVATIONS[activation]
    return out if act is None else act(out)


class DepthwiseConv2d(nn.Module):
    """Reference: torch_dwconv/dwconv.py:133-175.

    ``weight`` has the shape and ``state_dict`` key of ``nn.Conv2d(C, C, k, groups=C, bias=False)``;
    ``custom=False`` runs PyTorch's own grouped convolution instead of this library.
    """

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=None, bias=False, padding_mode='zeros', custom=True):
        super().__init__()
        check_options(in_channels, out_channels, dilation, groups, bias, padding_mode)
        self.in_channel = in_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.custom = custom
        self.weight = nn.Parameter(torch.randn(out_channels, 1, kernel_size, kernel_size))

    def forward(self, input):
        if not self.custom:
            return F.conv2d(input, self.weight, stride=self.stride, padding=self.padding,
                            groups=input.shape[1])
        return depthwise_conv2d(input, self.weight, None, self.stride, self.padding)
