"""Restatement of the reference's pure-Python argument handling.

TEST INFRASTRUCTURE ONLY -- written as lookup-style logic, independent of the
shipped ``torch_dwconv/dwconv.py``, so that the two can be compared.
"""

# torch_dwconv/dwconv.py:99-112: the five rejections, in the order the reference tests them.
REJECTIONS = (
    "dilation",       # :99-100   any dilation component > 1
    "groups",         # :102-103  groups given and != in_channels
    "channels",       # :105-106  in_channels != out_channels
    "bias",           # :108-109  truthy bias
    "padding_mode",   # :111-112  anything but 'zeros'
)


def expand(value, n):
    """torch_dwconv/dwconv.py:76-91 (make_tuple).

    scalar -> n copies; sequence longer than n -> ValueError; sequence of
    exactly n -> itself; shorter sequence -> repeated n times (so a 1-element
    list becomes n elements; an empty one stays empty).
    """
    if not isinstance(value, (list, tuple)):
        return tuple([value] * n)
    if len(value) > n:
        raise ValueError("too many items")
    if len(value) == n:
        return value
    return value * n


def first_rejection(in_channels, out_channels, dilation, groups, bias, padding_mode="zeros"):
    """Name of the first failing check of dwconv.py:94-112, or None."""
    d = expand(dilation, 2)
    if d[0] > 1 or d[1] > 1:
        return "dilation"
    if groups is not None and groups != in_channels:
        return "groups"
    if in_channels != out_channels:
        return "channels"
    if bias:
        return "bias"
    if padding_mode != "zeros":
        return "padding_mode"
    return None


def g_pad(in_hw, out_hw, kernel_hw, stride, pad):
    """torch_dwconv/dwconv.py:39-44."""
    return (
        kernel_hw[0] - pad[0] - 1,
        in_hw[0] - out_hw[0] * stride[0] + pad[0],
        kernel_hw[1] - pad[1] - 1,
        in_hw[1] - out_hw[1] * stride[1] + pad[1],
    )


def route(in_hw, kernel_hw, stride, pad, small):
    """torch_dwconv/dwconv.py:123-130: which of the three paths the reference takes."""
    if not small and in_hw[0] <= 32 and in_hw[1] <= 32:
        return "native_conv2d"
    return "small" if small else "large"
