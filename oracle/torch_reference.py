"""The oracle the reference's own tests use: PyTorch's grouped conv on the CPU.

test/test_forward.py:14 compares against ``F.conv2d(x, k, stride, padding,
groups=C)``; test/test_grad.py:23-39 checks the gradients in fp64.  Here both
are done in fp64 on the CPU.  TEST INFRASTRUCTURE ONLY.
"""
import time

import torch
from torch.nn import functional as F


def torch_reference(x, w, gy=None, stride=1, padding=0):
    """fp64 CPU forward (and, given gy, both gradients). Returns (y, gx, gw)."""
    xd = x.detach().to("cpu", torch.float64).requires_grad_(gy is not None)
    wd = w.detach().to("cpu", torch.float64).requires_grad_(gy is not None)
    y = F.conv2d(xd, wd, stride=stride, padding=padding, groups=xd.shape[1])
    if gy is None:
        return y.detach(), None, None
    gx, gw = torch.autograd.grad(y, (xd, wd), gy.detach().to("cpu", torch.float64))
    return y.detach(), gx, gw


def torch_reference_general(x, w, gy=None, stride=1, padding=0, dilation=1):
    """fp64 CPU ``F.conv2d(x, w, stride, padding, dilation, groups=C)`` for a weight of shape (C*M,1,KH,KW) and, given
    gy, both gradients: the options the reference's check_options refuses (torch_dwconv/dwconv.py:99-106)."""
    xd = x.detach().to("cpu", torch.float64).requires_grad_(gy is not None)
    wd = w.detach().to("cpu", torch.float64).requires_grad_(gy is not None)
    y = F.conv2d(xd, wd, stride=stride, padding=padding, dilation=dilation, groups=xd.shape[1])
    if gy is None:
        return y.detach(), None, None
    gx, gw = torch.autograd.grad(y, (xd, wd), gy.detach().to("cpu", torch.float64))
    return y.detach(), gx, gw


def shift_add_reference(x, w, gy, stride, padding):
    """(y, gx, gw) in fp64 on whatever device ``x`` lives on, from the closed forms alone: one strided slice of the
    zero-padded input per tap, multiplied and added (no convolution routine of any library is involved).

        y [n,c,oy,ox] = sum_{i,j} xpad[n,c, oy*s+i, ox*s+j] * w[c,i,j]
        gxpad[n,c, oy*s+i, ox*s+j] += gy[n,c,oy,ox] * w[c,i,j]          (then the padding is cut off)
        gw[c,i,j]     = sum_{n,oy,ox} gy[n,c,oy,ox] * xpad[n,c, oy*s+i, ox*s+j]

    which is what torch_dwconv/dwconv_kernel.cu:148-178 and :269-297 evaluate per output.  Used for whole-tensor
    checks at sizes where the C oracle would take minutes; pinned against it in tests/test_oracle.py."""
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    ph, pw = (padding, padding) if isinstance(padding, int) else padding
    xd, wd, gd = x.detach().double(), w.detach().double(), gy.detach().double()
    n, c, h, wid = xd.shape
    kh, kw = wd.shape[2:]
    oh, ow = gd.shape[2:]
    xpad = F.pad(xd, (pw, pw, ph, ph))
    y = torch.zeros_like(gd)
    gxpad = torch.zeros_like(xpad)
    gw = torch.zeros_like(wd)
    for i in range(kh):
        for j in range(kw):
            # rows i, i+s, ... (oh of them) and columns j, j+s, ... (ow of them) of the padded plane
            window = xpad[:, :, i:i + (oh - 1) * sh + 1:sh, j:j + (ow - 1) * sw + 1:sw]
            tap = wd[:, 0, i, j].view(1, c, 1, 1)
            y += window * tap
            gxpad[:, :, i:i + (oh - 1) * sh + 1:sh, j:j + (ow - 1) * sw + 1:sw] += gd * tap
            gw[:, 0, i, j] = (gd * window).sum(dim=(0, 2, 3))
    gx = gxpad[:, :, ph:ph + h, pw:pw + wid].contiguous()
    return y, gx, gw


_ACTIVATIONS = {None: lambda v: v, "none": lambda v: v, "relu": F.relu, "relu6": F.relu6, "silu": F.silu}


def torch_reference_fused(x, w, scale=None, shift=None, activation=None, stride=1, padding=0):
    """fp64 CPU value of ``act(conv(x, w) * scale[c] + shift[c])``: PyTorch's conv followed by PyTorch's own
    elementwise functions (the fused forward entry points have no counterpart in the reference)."""
    y, _, _ = torch_reference(x, w, None, stride, padding)
    if scale is not None:
        y = y * scale.detach().to("cpu", torch.float64).view(1, -1, 1, 1)
    if shift is not None:
        y = y + shift.detach().to("cpu", torch.float64).view(1, -1, 1, 1)
    return _ACTIVATIONS[activation](y)


def torch_cpu_fp32_step(x, w, gy, stride, padding, iters=3, threads=None, all_times=False):
    """Time fp32 ``F.conv2d(groups=C)`` forward + both gradients on the host cores.

    Baseline only (never the correctness oracle).  Returns (median seconds, threads), or with ``all_times`` the list
    of the ``iters`` timings in run order (after one untimed warm-up pass) instead of their median.
    """
    if threads:
        torch.set_num_threads(threads)
    x = x.detach().to("cpu", torch.float32).requires_grad_(True)
    w = w.detach().to("cpu", torch.float32).requires_grad_(True)
    gy = gy.detach().to("cpu", torch.float32)
    times = []
    for _ in range(iters + 1):
        t0 = time.perf_counter()
        y = F.conv2d(x, w, stride=stride, padding=padding, groups=x.shape[1])
        torch.autograd.grad(y, (x, w), gy)
        times.append(time.perf_counter() - t0)
    if all_times:
        return times[1:], torch.get_num_threads()
    times = sorted(times[1:])
    return times[len(times) // 2], torch.get_num_threads()
