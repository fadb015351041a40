"""Caller-side integration: torch.library registration and the model converter (neither exists in the reference)."""
import pytest
import torch
from torch import nn


def _toy():
    return nn.Sequential(
        nn.Conv2d(8, 8, 3, padding=1, groups=8, bias=False), nn.ReLU(),
        nn.Conv2d(8, 16, 1),
        nn.Sequential(nn.Conv2d(16, 16, 5, stride=2, padding=2, groups=16, bias=False),
                      nn.Conv2d(16, 16, 3, groups=16),                       # has a bias: left alone
                      nn.Conv2d(16, 16, 3, dilation=2, groups=16, bias=False)),  # dilated: left alone
    )


def test_convert_model_swaps_only_what_the_op_supports():
    from torch_dwconv import DepthwiseConv2d
    from torch_dwconv.convert import convert_model

    m = _toy()
    keys = list(m.state_dict().keys())
    w0 = m[0].weight
    m, n = convert_model(m)
    assert n == 2
    assert isinstance(m[0], DepthwiseConv2d) and m[0].weight is w0
    assert isinstance(m[3][0], DepthwiseConv2d) and (m[3][0].stride, m[3][0].padding) == ((2, 2), (2, 2))
    assert type(m[3][1]) is nn.Conv2d and type(m[3][2]) is nn.Conv2d and type(m[2]) is nn.Conv2d
    assert list(m.state_dict().keys()) == keys  # checkpoints interchange
    # custom=False keeps PyTorch's conv underneath: the converted model still runs on the CPU and matches
    ref = _toy()
    ref.load_state_dict(m.state_dict())
    m2, _ = convert_model(_toy(), custom=False)
    m2.load_state_dict(m.state_dict())
    x = torch.randn(2, 8, 20, 20)
    torch.testing.assert_close(m2(x), ref(x))


def test_registered_ops_have_fake_implementations():
    from torch._subclasses.fake_tensor import FakeTensorMode

    import torch_dwconv.ops  # noqa: F401  (registers the ops)

    with FakeTensorMode():
        x, w = torch.empty(2, 8, 17, 19), torch.empty(8, 1, 5, 5)
        y = torch.ops.torch_dwconv.depthwise_conv2d(x, w, [2, 2], [2, 2])
        assert tuple(y.shape) == (2, 8, 9, 10)
        assert y.is_contiguous()
        gx, gw = torch.ops.torch_dwconv.depthwise_conv2d_backward(x, y, w, [2, 2], [2, 2], [True, True])
        assert gx.shape == x.shape and gw.shape == w.shape and gx.is_contiguous()
        gx, gw = torch.ops.torch_dwconv.depthwise_conv2d_backward(x, y, w, [2, 2], [2, 2], [False, True])
        assert gx.numel() == 0 and gw.shape == w.shape
        # channels-last in, channels-last out (strides as the real kernels produce them)
        xc = x.contiguous(memory_format=torch.channels_last)
        yc = torch.ops.torch_dwconv.depthwise_conv2d(xc, w, [2, 2], [2, 2])
        assert yc.is_contiguous(memory_format=torch.channels_last) and not yc.is_contiguous()
        gx, _ = torch.ops.torch_dwconv.depthwise_conv2d_backward(xc, yc, w, [2, 2], [2, 2], [True, False])
        assert gx.stride() == xc.stride()
        # an input that is neither dense NCHW nor channels-last is computed (and returned) dense NCHW
        xs = torch.empty(2, 8, 17, 38)[:, :, :, ::2]
        gx, _ = torch.ops.torch_dwconv.depthwise_conv2d_backward(xs, y, w, [2, 2], [2, 2], [True, True])
        assert gx.is_contiguous()


def test_compiled_entry_keeps_the_option_checks():
    from torch_dwconv.ops import compiled_depthwise_conv2d

    x, w = torch.randn(1, 4, 8, 8), torch.randn(4, 1, 3, 3)
    with pytest.raises(ValueError, match="dilations"):
        compiled_depthwise_conv2d(x, w, dilation=2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        compiled_depthwise_conv2d(x, w, padding=1)


@pytest.mark.gpu
def test_registered_op_values_gradients_and_compile(gpu):
    from torch_dwconv import depthwise_conv2d
    from torch_dwconv.ops import compiled_depthwise_conv2d

    g = torch.Generator("cpu").manual_seed(3)
    for (c, h, k, s) in [(6, 28, 3, 1), (5, 30, 5, 2), (4, 57, 3, 2)]:
        x = torch.randn(2, c, h, h, generator=g).to(gpu).requires_grad_(True)
        w = (torch.randn(c, 1, k, k, generator=g) / k).to(gpu).requires_grad_(True)
        y_ref = depthwise_conv2d(x, w, stride=s, padding=k // 2)
        gy = torch.randn_like(y_ref)
        gx_ref, gw_ref = torch.autograd.grad(y_ref, (x, w), gy)
        y = compiled_depthwise_conv2d(x, w, stride=s, padding=k // 2)
        gx, gw = torch.autograd.grad(y, (x, w), gy)
        assert torch.equal(y, y_ref) and torch.equal(gx, gx_ref) and torch.equal(gw, gw_ref)
        # through torch.compile without a code generator: the op stays one opaque node
        fn = torch.compile(lambda a, b: compiled_depthwise_conv2d(a, b, stride=s, padding=k // 2) * 2.0, backend="aot_eager")
        torch.testing.assert_close(fn(x, w), y_ref * 2.0)


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
def test_registered_op_backward_through_compile(gpu, layout):
    """Forward and backward traced by torch.compile (AOT autograd, fake tensors first): values, memory layouts and the
    skipping of a gradient nobody wants, for dense NCHW and channels-last inputs, against the eager autograd Function
    and against the fp64 oracle."""
    import numpy as np

    import oracle
    from torch_dwconv import _C, depthwise_conv2d
    from torch_dwconv.ops import compiled_depthwise_conv2d

    fmt = torch.channels_last if layout == "nhwc" else torch.contiguous_format
    g = torch.Generator("cpu").manual_seed(5)
    for (c, h, k, s) in [(8, 28, 3, 1), (12, 30, 5, 2)]:
        p = k // 2
        x0 = torch.randn(3, c, h, h, generator=g)
        w0 = torch.randn(c, 1, k, k, generator=g) / k
        x = x0.to(gpu).contiguous(memory_format=fmt).requires_grad_(True)
        w = w0.to(gpu).requires_grad_(True)
        fn = torch.compile(lambda a, b: compiled_depthwise_conv2d(a, b, stride=s, padding=p), backend="aot_eager")
        y = fn(x, w)
        assert y.is_contiguous(memory_format=fmt)
        gy0 = torch.randn(y.shape, generator=g)
        gy = gy0.to(gpu).contiguous(memory_format=fmt)
        gx, gw = torch.autograd.grad(y, (x, w), gy)
        assert gx.is_contiguous(memory_format=fmt) and gw.is_contiguous()
        variant = _C.last_variant()
        assert variant.startswith("nhwc_") == (layout == "nhwc"), variant
        y_e = depthwise_conv2d(x, w, stride=s, padding=p)
        gx_e, gw_e = torch.autograd.grad(y_e, (x, w), gy)
        assert torch.equal(y, y_e) and torch.equal(gx, gx_e) and torch.equal(gw, gw_e)
        np.testing.assert_allclose(y.detach().cpu().numpy(), oracle.forward(x0.numpy(), w0.numpy(), s, p), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gx.cpu().numpy(), oracle.grad_input(gy0.numpy(), w0.numpy(), (h, h), s, p), rtol=1e-5, atol=1e-5)
        gw_ref = oracle.grad_weight(x0.numpy(), gy0.numpy(), w0.shape, s, p)
        np.testing.assert_allclose(gw.cpu().numpy(), gw_ref, rtol=1e-4, atol=1e-4 * np.abs(gw_ref).max())
        # a frozen filter: only grad-input is computed (one kernel, no grad-weight variant in the name)
        xf = x.detach().clone().requires_grad_(True)
        fn(xf, w.detach()).backward(gy)
        # (a single gradient takes the separate kernels, which add in another order than the fused one: same bounds
        # as against the oracle, not the same bits)
        torch.testing.assert_close(xf.grad, gx_e, rtol=1e-5, atol=1e-5)
        assert "wgrad" not in _C.last_variant() and "bwd" not in _C.last_variant(), _C.last_variant()
        # a frozen input: only grad-weight
        wf = w.detach().clone().requires_grad_(True)
        fn(x.detach(), wf).backward(gy)
        torch.testing.assert_close(wf.grad, gw_e, rtol=1e-4, atol=1e-4 * float(gw_e.abs().max()))


@pytest.mark.gpu
def test_converted_model_trains_like_the_original(gpu):
    from torch_dwconv.convert import convert_model

    torch.manual_seed(0)
    ref = _toy().to(gpu)
    new, n = convert_model(_toy())
    new = new.to(gpu)
    new.load_state_dict(ref.state_dict())
    x = torch.randn(3, 8, 40, 40, device=gpu)
    out_ref, out_new = ref(x), new(x)
    torch.testing.assert_close(out_new, out_ref, rtol=1e-4, atol=1e-5)
    out_ref.square().mean().backward()
    out_new.square().mean().backward()
    for (name, p), (_, q) in zip(ref.named_parameters(), new.named_parameters()):
        torch.testing.assert_close(q.grad, p.grad, rtol=1e-3, atol=1e-5, msg=name)
