"""``torch.library`` registration of the depthwise conv2d op.

Not part of the reference (its op is reachable only through ``DepthwiseConv2dFunction``); this is the caller-side
integration that lets the op pass through ``torch.compile`` / ``torch.export`` as one opaque node:

* ``torch.ops.torch_dwconv.depthwise_conv2d(input, weight, stride, padding) -> Tensor``
* ``torch.ops.torch_dwconv.depthwise_conv2d_backward(input, grad_output, weight, stride, padding) -> (Tensor, Tensor)``

Both carry fake-tensor (meta) implementations, and the forward op has its autograd formula registered, so
``compiled_depthwise_conv2d`` below is differentiable.  Values are those of ``torch_dwconv.depthwise_conv2d``.
"""
from typing import List, Tuple

import torch

from . import _C
from .dwconv import _autocast, check_options, make_tuple


def _out_hw(h: int, w: int, kh: int, kw: int, stride: List[int], padding: List[int]) -> Tuple[int, int]:
    return (h + 2 * padding[0] - kh) // stride[0] + 1, (w + 2 * padding[1] - kw) // stride[1] + 1


@torch.library.custom_op("torch_dwconv::depthwise_conv2d", mutates_args=())
def depthwise_conv2d_op(input: torch.Tensor, weight: torch.Tensor, stride: List[int], padding: List[int]) -> torch.Tensor:
    return _C.dwconv2d(input, weight, 1, 1, stride[0], stride[1], padding[0], padding[0], padding[1], padding[1], True)


@depthwise_conv2d_op.register_fake
def _(input, weight, stride, padding):
    n, c, h, w = input.shape
    oh, ow = _out_hw(h, w, weight.shape[2], weight.shape[3], stride, padding)
    return input.new_empty((n, c, max(oh, 0), max(ow, 0)))


@torch.library.custom_op("torch_dwconv::depthwise_conv2d_backward", mutates_args=())
def depthwise_conv2d_backward_op(input: torch.Tensor, grad_output: torch.Tensor, weight: torch.Tensor,
                                 stride: List[int], padding: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    if input.dtype != torch.float64:
        return _C.dwconv2d_backward(input, grad_output, weight, stride[0], stride[1], padding[0], padding[1])
    kh, kw = weight.shape[2], weight.shape[3]
    g_pad = (kh - padding[0] - 1, input.shape[2] - grad_output.shape[2] * stride[0] + padding[0],
             kw - padding[1] - 1, input.shape[3] - grad_output.shape[3] * stride[1] + padding[1])
    gx = _C.dwconv2d(grad_output, weight, stride[0], stride[1], 1, 1, *g_pad, False)
    gw = _C.dwconv2d_backward_kernel(input, grad_output, weight, 1, 1, stride[0], stride[1], padding[0], padding[1])
    return gx, gw


@depthwise_conv2d_backward_op.register_fake
def _(input, grad_output, weight, stride, padding):
    return torch.empty_like(input), torch.empty_like(weight)


def _setup_context(ctx, inputs, output):
    input, weight, stride, padding = inputs
    ctx.save_for_backward(input, weight)
    ctx.stride, ctx.padding = stride, padding


def _backward(ctx, grad_output):
    input, weight = ctx.saved_tensors
    gx, gw = depthwise_conv2d_backward_op(input, grad_output.contiguous(), weight, ctx.stride, ctx.padding)
    return gx, gw, None, None


depthwise_conv2d_op.register_autograd(_backward, setup_context=_setup_context)


def compiled_depthwise_conv2d(input, weight, bias=None, stride=1, padding=0, dilation=1, groups=None):
    """Same signature, checks and values as ``torch_dwconv.depthwise_conv2d``, routed through the registered op."""
    stride = list(make_tuple(stride, 2))
    padding = list(make_tuple(padding, 2))
    check_options(input.shape[1], weight.shape[0], dilation, groups, bias)
    input, weight = _autocast(input, weight)
    return depthwise_conv2d_op(input, weight, stride, padding)
