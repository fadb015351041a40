"""Depthwise conv2d for AMD MI355X behind the ``torch_dwconv`` API.

Public surface of the reference package (torch_dwconv/__init__.py:1).
"""
from .dwconv import (  # noqa: F401
    depthwise_conv2d,
    depthwise_conv2d_fused,
    depthwise_conv2d_general,
    DepthwiseConv2d,
)
