"""Swap the depthwise ``nn.Conv2d`` layers of a model for ``DepthwiseConv2d``.

Not part of the reference; it is the one-line way to put this library under an existing network
(EfficientNet, MobileNet, ConvNeXt ...).  ``DepthwiseConv2d.weight`` has the shape and ``state_dict`` key of
``nn.Conv2d(C, C, k, groups=C, bias=False).weight`` (torch_dwconv/dwconv.py:156-158), so the parameter object is
simply moved over: optimizers and checkpoints keep working.
"""
from torch import nn

from .dwconv import DepthwiseConv2d


def _convertible(m):
    if not isinstance(m, nn.Conv2d) or type(m) is not nn.Conv2d:
        return False
    k = m.kernel_size
    return (
        m.groups == m.in_channels == m.out_channels
        and m.bias is None
        and m.dilation == (1, 1)
        and m.padding_mode == "zeros"
        and not isinstance(m.padding, str)
        and k[0] == k[1]
    )


def convert_model(module, custom=True):
    """Replaces, in place and recursively, every square-filter, bias-free, undilated depthwise ``nn.Conv2d``.

    Returns ``(module, number_of_layers_replaced)``.  Layers with a bias, a dilation, string padding or a
    non-square filter are left alone (``DepthwiseConv2d`` rejects those options, torch_dwconv/dwconv.py:94-112).
    """
    replaced = 0
    for name, child in list(module.named_children()):
        if _convertible(child):
            new = DepthwiseConv2d(child.in_channels, child.out_channels, child.kernel_size[0], stride=child.stride,
                                  padding=child.padding, custom=custom)
            new.weight = child.weight  # same Parameter object
            new.train(child.training)
            setattr(module, name, new)
            replaced += 1
        else:
            replaced += convert_model(child, custom)[1]
    return module, replaced
