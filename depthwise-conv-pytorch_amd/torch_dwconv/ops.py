"""``torch.library`` registration of the depthwise conv2d op.

Not part of the reference (its op is reachable only through ``DepthwiseConv2dFunction``); this is the caller-side
integration that lets the op pass through ``torch.compile`` / ``torch.export`` as one opaque node:

* ``torch.ops.torch_dwconv.depthwise_conv2d(input, weight, stride, padding) -> Tensor``
* ``torch.ops.torch_dwconv.depthwise_conv2d_backward(input, grad_output, weight, stride, padding, output_mask)
  -> (Tensor, Tensor)``

Both carry fake-tensor (meta) implementations whose results have the shapes *and strides* of the real ones, and the
forward op has its autograd formula registered, so ``compiled_depthwise_conv2d`` below is differentiable.  Values and
memory layouts are those of ``torch_dwconv.depthwise_conv2d``: a channels-last input runs the channels-last kernels
and gives channels-last results, anything else is computed NCHW-contiguous.
"""
from typing import List, Tuple

import torch

from . import _C
from .dwconv import _autocast, check_options, make_tuple


def _out_hw(h: int, w: int, kh: int, kw: int, stride: List[int], padding: List[int]) -> Tuple[int, int]:
    return (h + 2 * padding[0] - kh) // stride[0] + 1, (w + 2 * padding[1] - kw) // stride[1] + 1


def _format_of(input):
    """Memory format of the results for this input: channels-last follows channels-last, everything else is dense NCHW."""
    return torch.channels_last if _C.is_channels_last(input) else torch.contiguous_format


@torch.library.custom_op("torch_dwconv::depthwise_conv2d", mutates_args=())
def depthwise_conv2d_op(input: torch.Tensor, weight: torch.Tensor, stride: List[int], padding: List[int]) -> torch.Tensor:
    if _C.is_channels_last(input):
        return _C.dwconv2d_nhwc(input, weight, stride[0], stride[1], padding[0], padding[1])
    return _C.dwconv2d(input, weight, 1, 1, stride[0], stride[1], padding[0], padding[0], padding[1], padding[1], True)


@depthwise_conv2d_op.register_fake
def _(input, weight, stride, padding):
    n, c, h, w = input.shape
    oh, ow = _out_hw(h, w, weight.shape[2], weight.shape[3], stride, padding)
    return torch.empty((n, c, max(oh, 0), max(ow, 0)), dtype=input.dtype, device=input.device,
                       memory_format=_format_of(input))


@torch.library.custom_op("torch_dwconv::depthwise_conv2d_backward", mutates_args=())
def depthwise_conv2d_backward_op(input: torch.Tensor, grad_output: torch.Tensor, weight: torch.Tensor,
                                 stride: List[int], padding: List[int],
                                 output_mask: List[bool]) -> Tuple[torch.Tensor, torch.Tensor]:
    """(grad_input, grad_weight); a gradient whose ``output_mask`` entry is False is not computed and comes back as
    an empty tensor (0 elements), like ``aten::convolution_backward``."""
    need_input, need_weight = output_mask[0], output_mask[1]
    skipped = input.new_empty(0)
    if _C.is_channels_last(input):
        gx, gw = _C.dwconv2d_backward_nhwc(input, grad_output, weight, stride[0], stride[1], padding[0], padding[1],
                                           need_input, need_weight)
        return (gx if need_input else skipped), (gw if need_weight else skipped)
    if need_input and need_weight and input.dtype != torch.float64:
        return _C.dwconv2d_backward(input, grad_output, weight, stride[0], stride[1], padding[0], padding[1])
    gx = gw = skipped
    if need_input:
        kh, kw = weight.shape[2], weight.shape[3]
        g_pad = (kh - padding[0] - 1, input.shape[2] - grad_output.shape[2] * stride[0] + padding[0],
                 kw - padding[1] - 1, input.shape[3] - grad_output.shape[3] * stride[1] + padding[1])
        gx = _C.dwconv2d(grad_output, weight, stride[0], stride[1], 1, 1, *g_pad, False)
    if need_weight:
        gw = _C.dwconv2d_backward_kernel(input, grad_output, weight, 1, 1, stride[0], stride[1], padding[0], padding[1])
    return gx, gw


@depthwise_conv2d_backward_op.register_fake
def _(input, grad_output, weight, stride, padding, output_mask):
    skipped = input.new_empty(0)
    gx = torch.empty(input.shape, dtype=input.dtype, device=input.device, memory_format=_format_of(input))
    gw = torch.empty(weight.shape, dtype=weight.dtype, device=weight.device)
    return (gx if output_mask[0] else skipped), (gw if output_mask[1] else skipped)


def _setup_context(ctx, inputs, output):
    input, weight, stride, padding = inputs
    ctx.save_for_backward(input, weight)
    ctx.stride, ctx.padding = stride, padding


def _backward(ctx, grad_output):
    input, weight = ctx.saved_tensors
    mask = [bool(ctx.needs_input_grad[0]), bool(ctx.needs_input_grad[1])]
    if not any(mask):
        return None, None, None, None
    gx, gw = depthwise_conv2d_backward_op(input, grad_output, weight, ctx.stride, ctx.padding, mask)
    return (gx if mask[0] else None), (gw if mask[1] else None), None, None


depthwise_conv2d_op.register_autograd(_backward, setup_context=_setup_context)


def compiled_depthwise_conv2d(input, weight, bias=None, stride=1, padding=0, dilation=1, groups=None):
    """Same signature, checks and values as ``torch_dwconv.depthwise_conv2d``, routed through the registered op."""
    stride = list(make_tuple(stride, 2))
    padding = list(make_tuple(padding, 2))
    check_options(input.shape[1], weight.shape[0], dilation, groups, bias)
    input, weight = _autocast(input, weight)
    return depthwise_conv2d_op(input, weight, stride, padding)
