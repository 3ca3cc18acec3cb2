"""Parity of the drop-in modules as the reference composes them: ``SimpleGate`` stand-alone
(pyramid_dwconv/conv_block.py:6-22), ``OptimizedDepthwiseConv2d`` as a module
(dwconv_triton.py:389-426) and ``ConvBlock`` with non-default ``scales`` / ``inter_ratio``
(conv_block.py:26-34), all against the float64 oracle."""
import numpy as np
import pytest
import torch

from parity import assert_close, randn

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scale_factor", [1.0, 0.5])
@pytest.mark.parametrize("shape,k", [((2, 16, 24, 32), 7), ((3, 13, 17, 24), 5), ((1, 57, 61, 16), 9)])
def test_simple_gate_module(oracle, dtype, scale_factor, shape, k):
    """pool -> conv -> gate -> bilinear through the module's own forward and autograd, even and odd extents."""
    import pyramidconvblock_amd as P

    B, H, W, I = shape
    torch.manual_seed(11)
    gate = P.SimpleGate(I, kernel_size=k, scale_factor=scale_factor).to(dtype)
    gen = torch.Generator().manual_seed(11)
    a = randn(gen, *shape).to(dtype)
    g = randn(gen, B, H, W, I // 2).to(dtype)
    w = gate.conv_spatial.weight.detach().double().numpy()
    yo, cache = oracle.simple_gate_fwd(a.double().numpy(), w, scale_factor)
    dao, dwo = oracle.simple_gate_bwd(cache, g.double().numpy())
    gate = gate.cuda()
    ad = a.cuda().requires_grad_()
    y = gate(ad)
    assert y.dtype == dtype and tuple(y.shape) == (B, H, W, I // 2)
    assert_close(y, yo, dtype, "y")
    torch.autograd.backward(y, g.cuda())
    assert_close(ad.grad, dao, dtype, "da")
    assert_close(gate.conv_spatial.weight.grad, dwo, dtype, "dw")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", [
    ((2, 20, 28, 32), 13, 1, 6, 1),      # the geometry SimpleGate builds
    ((2, 9, 11, 24), 3, 1, 0, 1),        # no padding: the output shrinks
    ((1, 15, 18, 8), 5, 2, 2, 1),        # strided
    ((2, 12, 12, 16), 3, 1, 2, 2),       # dilated
])
def test_depthwise_module(oracle, dtype, case):
    """OptimizedDepthwiseConv2d.forward and its autograd backward on the device."""
    import pyramidconvblock_amd as P

    shape, k, stride, pad, dil = case
    B, H, W, C = shape
    torch.manual_seed(5)
    conv = P.OptimizedDepthwiseConv2d(C, k, stride=stride, padding=pad, dilation=dil)
    assert conv.weight.dtype == torch.float16
    conv = conv.to(dtype)
    gen = torch.Generator().manual_seed(5)
    x = randn(gen, *shape).to(dtype)
    w = conv.weight.detach().double().numpy()
    yo = oracle.dwconv_fwd(x.double().numpy(), w, stride, pad, dil)
    g = randn(gen, *yo.shape).to(dtype)
    dxo = oracle.dwconv_dgrad(g.double().numpy(), w, (H, W), stride, pad, dil)
    dwo = oracle.dwconv_wgrad(x.double().numpy(), g.double().numpy(), (k, k), stride, pad, dil)
    conv = conv.cuda()
    xd = x.cuda().requires_grad_()
    y = conv(xd)
    assert y.dtype == dtype and tuple(y.shape) == yo.shape
    assert_close(y, yo, dtype, "y")
    torch.autograd.backward(y, g.cuda())
    assert_close(xd.grad, dxo, dtype, "dx")
    assert_close(conv.weight.grad, dwo, dtype, "dw")
    assert conv.weight.grad.dtype == dtype and xd.grad.dtype == dtype


def _block(oracle, dim, k, shape, dtype, seed=0, **kw):
    import pyramid_dwconv

    torch.manual_seed(seed)
    m = pyramid_dwconv.ConvBlock(dim=dim, kernel_size=k, **kw)
    scales = tuple(float(s) for s in kw.get("scales", (1., 0.5)))
    gen = torch.Generator().manual_seed(seed)
    x, g = randn(gen, *shape).to(dtype), randn(gen, *shape).to(dtype)
    m = m.to(dtype)
    params = {n: p.detach().double().numpy() for n, p in m.state_dict().items()}
    yo, cache = oracle.convblock_fwd(x.double().numpy(), params, scales=scales)
    dxo, go = oracle.convblock_bwd(cache, g.double().numpy())
    m = m.cuda()
    xd = x.cuda().requires_grad_()
    y = m(xd)
    assert y.dtype == dtype and y.shape == xd.shape
    assert_close(y, yo, dtype, "y")
    torch.autograd.backward(y, g.cuda())
    assert_close(xd.grad, dxo, dtype, "dx")
    names = [n for n, _ in m.named_parameters()]
    assert sorted(names) == sorted(go.keys())
    for n, p in m.named_parameters():
        assert p.grad is not None, n
        assert_close(p.grad, go[n], dtype, "grad " + n)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scales", [(1.,), (0.5,), (1., 0.5, 0.25), (0.5, 1.), (1., 1.), (1., 0.75)])
@pytest.mark.parametrize("shape", [(2, 16, 24, 64), (2, 13, 18, 64)])
def test_block_scales(oracle, dtype, scales, shape):
    """Every combination of scales the constructor accepts runs the single-branch launches of the block
    (one gate per branch, pooled gradients accumulated into the full-resolution one)."""
    _block(oracle, 64, 7, shape, dtype, scales=scales)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter_ratio,dim", [(0.25, 128), (1.0, 32), (0.75, 64)])
def test_block_inter_ratio(oracle, dtype, inter_ratio, dim):
    _block(oracle, dim, 5, (2, 12, 16, dim), dtype, inter_ratio=inter_ratio)


def test_block_bias_and_three_scales(oracle):
    _block(oracle, 128, 9, (2, 24, 24, 128), torch.bfloat16, bias=True, out_bias=False, scales=(1., 0.5, 0.25))
