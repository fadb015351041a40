"""CPU-only checks of the host side: argument handling, the C-ABI library's
exports and its geometry helpers.  No kernel is launched here."""
import ctypes
import itertools
import os
import re

import pytest
import torch

import oracle
from test_oracle import SMALL_TRUTH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dwconv_hip.h")


@pytest.fixture(scope="module")
def dw():
    import torch_dwconv.dwconv as m

    return m


@pytest.fixture(scope="module")
def lib():
    from torch_dwconv import _C

    return _C._lib


def test_library_exports_every_declared_symbol():
    from torch_dwconv import _C

    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(dwconv\w*)\s*\(", text)
    assert len(set(names)) >= 12
    raw = ctypes.CDLL(_C.LIBRARY_PATH)
    for name in set(names):
        assert hasattr(raw, name), f"{name} is declared in include/dwconv_hip.h but not exported"


def test_version_and_empty_error(lib):
    assert b"gfx950" in lib.dwconv_version()
    assert isinstance(lib.dwconv_last_error(), bytes)


def test_out_size_matches_oracle(lib):
    for h, up, down, p0, p1, k in itertools.product((1, 7, 14, 33, 112), (1, 2), (1, 2, 3), (0, 1, 3), (0, 2), (1, 3, 5, 7)):
        assert lib.dwconv_out_size(h, up, down, p0, p1, k) == oracle.out_size(h, up, down, p0, p1, k)


@pytest.mark.parametrize("geom,expected", SMALL_TRUTH)
def test_small_predicate_truth_table(lib, geom, expected):
    h, w, kh, kw, down, pad = geom
    assert bool(lib.dwconv_use_dwconv2d_small(h, w, kh, kw, 1, 1, down, down, pad, pad)) is expected


def test_small_predicate_sweep_against_oracle(lib):
    for h, w, k, down, pad in itertools.product(range(1, 36, 3), range(1, 36, 4), (1, 3, 5, 7), (1, 2), (0, 1, 2, 3)):
        got = bool(lib.dwconv_use_dwconv2d_small(h, w, k, k, 1, 1, down, down, pad, pad))
        assert got == oracle.use_dwconv2d_small(h, w, k, k, 1, 1, down, down, pad, pad), (h, w, k, down, pad)


def test_workspace_query_needs_no_gpu(lib):
    n = lib.dwconv2d_backward_kernel_workspace_bytes(128, 32, 112, 112, 112, 112, 3, 3, 1, 1, 1, 1, 4)
    assert n > 0
    assert lib.dwconv2d_backward_kernel_workspace_bytes(0, 32, 8, 8, 8, 8, 3, 3, 1, 1, 1, 1, 4) == 0


def test_argument_errors_come_back_as_status_codes(lib):
    # invalid geometry is rejected before anything touches a device
    rc = lib.dwconv2d_f32(None, None, None, 1, 1, 8, 8, 0, 3, 1, 1, 1, 1, 0, 0, 0, 0, 1, None)
    assert rc == 1 and b"kernel extent" in lib.dwconv_last_error()
    rc = lib.dwconv2d_f32(None, None, None, 1, 1, 8, 8, 3, 3, 1, 1, 0, 1, 0, 0, 0, 0, 1, None)
    assert rc == 1
    rc = lib.dwconv2d_f32(None, None, None, 1, 1, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, None)
    assert rc == 1 and b"null" in lib.dwconv_last_error()
    rc = lib.dwconv2d_small_f32(None, None, None, 1, 1, 8, 8, 3, 3, 1, 1, 2, 2, 1, 1, 1, None)
    assert rc == 2
    rc = lib.dwconv2d_small_f32(None, None, None, 1, 1, 40, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, None)
    assert rc == 2
    rc = lib.dwconv2d_backward_kernel_f32(None, None, None, None, 0, 1, 1, 8, 8, 8, 8, 3, 3, 2, 1, 1, 1, 1, 1, None)
    assert rc == 2 and b"up == 1" in lib.dwconv_last_error()
    # empty problems succeed without a device
    assert lib.dwconv2d_f32(None, None, None, 0, 4, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, None) == 0


# ---- python surface ------------------------------------------------------------
def test_noalloc_entry_point_refuses_oversized_geometry_without_a_gpu(lib):
    # the size check comes before anything touches a device, so it can be exercised here
    n, c, h, k = 2, 65536, 16, 15
    need = lib.dwconv2d_backward_kernel_workspace_bytes(n, c, h, h, h, h, k, k, 1, 1, 7, 7, 4)
    assert need > 32 << 20
    lib.dwconv2d_backward_noalloc_f32.restype = ctypes.c_int
    lib.dwconv2d_backward_noalloc_f32.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 12 + [ctypes.c_void_p]
    rc = lib.dwconv2d_backward_noalloc_f32(8, 8, 8, 8, 8, n, c, h, h, h, h, k, k, 1, 1, 7, 7, None)
    assert rc == 3  # DWCONV_ERR_WORKSPACE
    assert b"scratch" in lib.dwconv_last_error()


def test_make_tuple_matches_restatement(dw):
    for v in (1, 3, (1, 2), [2, 1], [4], (5,), []):
        assert dw.make_tuple(v, 2) == oracle.host_logic.expand(v, 2)
    with pytest.raises(ValueError, match="Number items does not match with requirements: 3, expected: 2"):
        dw.make_tuple((1, 2, 3), 2)


MESSAGES = {
    "dilation": "DepthwiseConv2d does not support dilations > 1",
    "groups": "DepthwiseConv2d does not support groups != in_channels",
    "channels": "DepthwiseConv2d does not support in_channels != out_channels",
    "bias": "DepthwiseConv2d does not support bias",
    "padding_mode": "DepthwiseConv2d does not non-zero paddings",
}


def test_check_options_rejections_and_order(dw):
    cases = itertools.product((8,), (8, 16), (1, 2, (1, 3)), (None, 8, 4), (None, False, True), ("zeros", "reflect"))
    for cin, cout, dil, groups, bias, mode in cases:
        want = oracle.host_logic.first_rejection(cin, cout, dil, groups, bias, mode)
        if want is None:
            dw.check_options(cin, cout, dil, groups, bias, mode)
        else:
            with pytest.raises(ValueError) as e:
                dw.check_options(cin, cout, dil, groups, bias, mode)
            assert str(e.value) == MESSAGES[want]


def test_functional_rejects_options_before_touching_the_device(dw):
    x, w = torch.randn(1, 4, 8, 8), torch.randn(4, 1, 3, 3)
    with pytest.raises(ValueError, match="dilations"):
        dw.depthwise_conv2d(x, w, dilation=2)
    with pytest.raises(ValueError, match="bias"):
        dw.depthwise_conv2d(x, w, True)
    # like the reference's `if bias:` (dwconv.py:108), a one-element tensor is tested by its truth value
    with pytest.raises(ValueError, match="bias"):
        dw.depthwise_conv2d(x, w, torch.ones(1))
    with pytest.raises(ValueError, match="in_channels != out_channels"):
        dw.depthwise_conv2d(x, torch.randn(8, 1, 3, 3))
    with pytest.raises(ValueError, match="groups"):
        dw.depthwise_conv2d(x, w, groups=2)
    with pytest.raises(ValueError, match="Number items"):
        dw.depthwise_conv2d(x, w, stride=(1, 1, 1))


def test_cpu_tensors_are_refused_not_computed(dw):
    # torch_dwconv/dwconv.cpp:24-25: the extension only takes GPU tensors; there is no CPU path.
    x, w = torch.randn(1, 4, 40, 40), torch.randn(4, 1, 3, 3)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        dw.depthwise_conv2d(x, w, padding=1)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        dw.depthwise_conv2d(torch.randn(1, 4, 8, 8), w, padding=1)


def test_module_surface(dw):
    m = dw.DepthwiseConv2d(6, 6, 5, stride=2, padding=2)
    assert tuple(m.weight.shape) == (6, 1, 5, 5)
    assert list(m.state_dict().keys()) == ["weight"]
    ref = torch.nn.Conv2d(6, 6, 5, stride=2, padding=2, groups=6, bias=False)
    ref.load_state_dict(m.state_dict())  # interchangeable checkpoints
    assert (m.stride, m.padding, m.in_channel, m.kernel_size, m.custom) == (2, 2, 6, 5, True)
    with pytest.raises(ValueError, match="bias"):
        dw.DepthwiseConv2d(6, 6, 3, bias=True)
    with pytest.raises(ValueError, match="non-zero paddings"):
        dw.DepthwiseConv2d(6, 6, 3, padding_mode="circular")
    # custom=False is PyTorch's own conv and runs anywhere
    plain = dw.DepthwiseConv2d(6, 6, 3, padding=1, custom=False)
    x = torch.randn(2, 6, 9, 9)
    torch.testing.assert_close(plain(x), torch.nn.functional.conv2d(x, plain.weight, padding=1, groups=6))


def test_package_exports():
    import torch_dwconv

    assert callable(torch_dwconv.depthwise_conv2d) and issubclass(torch_dwconv.DepthwiseConv2d, torch.nn.Module)
    from torch_dwconv.dwconv import DepthwiseConv2dFunction, depthwise_conv2d_fn, use_dwconv2d_small  # noqa: F401


def test_product_code_never_reaches_for_the_oracle_or_working_files():
    """The package under depthwise-conv-pytorch_amd/ is the product: it must not import the CPU oracle (test
    infrastructure) or anything from the builder's working folder; bench.py may use the oracle only in its
    cpu_baseline leg and the entry script only in smoke()."""
    import re

    pkg = os.path.join(ROOT, "depthwise-conv-pytorch_amd")
    offenders = []
    for folder, _, files in os.walk(pkg):
        for name in files:
            if not name.endswith((".py", ".hip", ".hpp", ".h", "Makefile")):
                continue
            text = open(os.path.join(folder, name), encoding="utf-8").read()
            if re.search(r"^\s*(import|from)\s+oracle\b", text, re.M) or "_work/" in text or "oracle/" in text:
                offenders.append(os.path.join(folder, name))
    assert offenders == []
    tracked = ["bench.py", "__graft_entry__.py", "include/dwconv_hip.h"]
    for rel in tracked:
        assert "_work/" not in open(os.path.join(ROOT, rel), encoding="utf-8").read(), rel
    bench = open(os.path.join(ROOT, "bench.py"), encoding="utf-8").read()
    uses = [m.start() for m in re.finditer(r"(import|from)\s+oracle\b", bench)]
    start = bench.index("def cpu_baseline")
    end = bench.index("\ndef ", start + 1)
    assert uses and all(start < u < end for u in uses), "bench.py touches the oracle outside cpu_baseline()"
