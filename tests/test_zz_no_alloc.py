"""The entry point that allocates nothing (dwconv2d_backward_noalloc_f32) against dwconv2d_backward_f32.

Both run the same kernels with the same plan, so the results must be equal bit for bit.  Two calls in a row on one
device, the second on a smaller problem: the built-in scratch buffer keeps the first call's partial sums, and the
second call must not see them."""
import ctypes

import pytest
import torch

import shapes
from torch_dwconv import _C

pytestmark = pytest.mark.gpu

# every kernel family behind dwconv2d_backward_f32: fused tiled stride 1, fused stride 2, fused whole-plane,
# the two separate passes (pad 0), the per-element kernels (rectangular filter)
PAIRS = [
    ((16, 48, 56, 56, 3, 1, 1), (4, 24, 28, 28, 5, 2, 2)),
    ((32, 96, 14, 14, 5, 1, 2), (3, 10, 7, 7, 3, 1, 1)),
    ((8, 32, 64, 64, 5, 2, 2), (8, 32, 33, 35, 3, 1, 0)),
    ((64, 128, 7, 7, 7, 1, 3), (2, 5, 19, 23, 7, 1, 3)),
]


def _reference(x, gy, w, s, p):
    """dwconv2d_backward_f32 through the C ABI with a workspace from torch."""
    n, c, h, wd = x.shape
    oh, ow = gy.shape[2:]
    kh, kw = w.shape[2:]
    need = _C._lib.dwconv2d_backward_kernel_workspace_bytes(n, c, h, wd, oh, ow, kh, kw, s, s, p, p, 4)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    gx = torch.full_like(x, float("nan"))
    gw = torch.full_like(w, float("nan"))
    rc = _C._lib.dwconv2d_backward_f32(x.data_ptr(), gy.data_ptr(), w.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                       ws.data_ptr(), need, n, c, h, wd, oh, ow, kh, kw, s, s, p, p,
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _C._lib.dwconv_last_error().decode()
    return gx, gw, need, _C.last_variant()


def _noalloc(x, gy, w, s, p):
    n, c, h, wd = x.shape
    oh, ow = gy.shape[2:]
    kh, kw = w.shape[2:]
    gx = torch.full_like(x, float("nan"))
    gw = torch.full_like(w, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = _C._lib.dwconv2d_backward_noalloc_f32(x.data_ptr(), gy.data_ptr(), w.data_ptr(), gx.data_ptr(),
                                               gw.data_ptr(), n, c, h, wd, oh, ow, kh, kw, s, s, p, p,
                                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _C._lib.dwconv_last_error().decode()
    assert torch.cuda.memory_allocated() == before
    return gx, gw, _C.last_variant()


@pytest.mark.parametrize("first,second", PAIRS, ids=lambda s: shapes.shape_id(s))
def test_noalloc_matches_backward_two_calls_in_a_row(first, second):
    dev = torch.device("cuda:0")
    for shape in (first, second):  # second call: smaller problem, same scratch buffer
        x, w, gy = (t.to(dev) for t in shapes.make_inputs(shape, seed=7))
        s, p = shape[5], shape[6]
        gx, gw, variant = _noalloc(x, gy, w, s, p)
        gx_ref, gw_ref, need, variant_ref = _reference(x, gy, w, s, p)
        torch.cuda.synchronize()
        assert need <= _C.NOALLOC_SCRATCH_BYTES
        assert variant == variant_ref
        assert not torch.isnan(gx).any() and not torch.isnan(gw).any()
        assert torch.equal(gx, gx_ref), f"{shapes.shape_id(shape)} [{variant}] in_grad differs"
        assert torch.equal(gw, gw_ref), f"{shapes.shape_id(shape)} [{variant}] kernel_grad differs"


def test_noalloc_wrapper_and_oracle():
    """The Python wrapper, checked against the CPU oracle as well (1e-5 / 1e-4 bounds as everywhere)."""
    import numpy as np

    import oracle

    dev = torch.device("cuda:0")
    shape = (6, 40, 28, 28, 3, 2, 1)
    x, w, gy = shapes.make_inputs(shape, seed=3)
    xg, wg, gyg = x.to(dev), w.to(dev), gy.to(dev)
    gx = torch.full_like(xg, float("nan"))
    gw = torch.full_like(wg, float("nan"))
    _C.dwconv2d_backward_noalloc(xg, gyg, wg, gx, gw, 2, 2, 1, 1)
    gx_ref = oracle.grad_input(gy.numpy(), w.numpy(), (28, 28), 2, 1)
    gw_ref = oracle.grad_weight(x.numpy(), gy.numpy(), w.shape, 2, 1)
    np.testing.assert_allclose(gx.cpu().numpy(), gx_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gw.cpu().numpy(), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())


def test_noalloc_rejects_oversized_geometry():
    """Beyond the built-in buffer the call is refused before anything is launched."""
    n, c, h, k = 2, 65536, 16, 15
    need = _C._lib.dwconv2d_backward_kernel_workspace_bytes(n, c, h, h, h, h, k, k, 1, 1, 7, 7, 4)
    assert need > _C.NOALLOC_SCRATCH_BYTES
    one = torch.zeros(1, device="cuda:0")
    rc = _C._lib.dwconv2d_backward_noalloc_f32(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                               one.data_ptr(), n, c, h, h, h, h, k, k, 1, 1, 7, 7, None)
    assert rc == 3  # DWCONV_ERR_WORKSPACE
    assert "scratch" in _C._lib.dwconv_last_error().decode()


def test_noalloc_inside_a_hip_graph():
    """What the entry point is for: a backward step captured into a HIP graph (no allocation may happen during
    capture).  Every replay, with fresh input values and eager work in between, must equal the eager call bit for bit."""
    dev = torch.device("cuda:0")
    shape = (8, 32, 28, 28, 5, 1, 2)
    n, c, h, wd, k, s, p = shape
    x, w, gy = (t.to(dev) for t in shapes.make_inputs(shape, seed=11))
    gx = torch.empty_like(x)
    gw = torch.empty_like(w)

    def call(stream):
        rc = _C._lib.dwconv2d_backward_noalloc_f32(x.data_ptr(), gy.data_ptr(), w.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                                   n, c, h, wd, gy.shape[2], gy.shape[3], k, k, s, s, p, p,
                                                   ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, _C._lib.dwconv_last_error().decode()

    call(torch.cuda.current_stream())  # first call on the device: looks up the scratch buffer, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream())
    gen = torch.Generator("cpu").manual_seed(13)
    for replay in range(3):
        x.copy_(torch.randn(x.shape, generator=gen))
        gy.copy_(torch.randn(gy.shape, generator=gen))
        gx.fill_(float("nan"))
        gw.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        gx_ref, gw_ref, _, _ = _reference(x, gy, w, s, p)
        torch.cuda.synchronize()
        assert torch.equal(gx, gx_ref) and torch.equal(gw, gw_ref), replay


_FIRST_CALL_UNDER_CAPTURE = r"""
import ctypes, sys
import torch
sys.path[:0] = {paths!r}
from torch_dwconv import _C

hip = ctypes.CDLL("libamdhip64.so")
x = torch.zeros(2, 4, 8, 8, device="cuda:0"); w = torch.zeros(4, 1, 3, 3, device="cuda:0")
gx = torch.empty_like(x); gw = torch.empty_like(w)
side = torch.cuda.Stream()
torch.cuda.synchronize()
stream = ctypes.c_void_p(side.cuda_stream)
assert hip.hipStreamBeginCapture(stream, 2) == 0  # relaxed mode
rc = _C._lib.dwconv2d_backward_noalloc_f32(x.data_ptr(), x.data_ptr(), w.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                           2, 4, 8, 8, 8, 8, 3, 3, 1, 1, 1, 1, stream)
message = _C._lib.dwconv_last_error().decode()
graph = ctypes.c_void_p()
assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
if graph.value:
    hip.hipGraphDestroy(graph)
assert rc == 2, (rc, message)  # DWCONV_ERR_UNSUPPORTED, nothing recorded
assert "outside stream capture" in message, message
# the same call outside capture then works
rc = _C._lib.dwconv2d_backward_noalloc_f32(x.data_ptr(), x.data_ptr(), w.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                           2, 4, 8, 8, 8, 8, 3, 3, 1, 1, 1, 1, stream)
assert rc == 0, _C._lib.dwconv_last_error().decode()
torch.cuda.synchronize()
assert float(gx.abs().sum()) == 0.0
print("ok")
"""


def test_noalloc_first_call_under_capture_is_refused():
    """The scratch buffer's address is looked up on the first call on a device; a first call on a capturing stream
    is refused with a clear error instead of recording the lookup.  Needs a process of its own (first call)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    paths = [root, os.path.join(root, "depthwise-conv-pytorch_amd")]
    out = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE.format(paths=paths)], capture_output=True,
                         text=True, timeout=170)
    assert out.returncode == 0 and "ok" in out.stdout, out.stdout + out.stderr
