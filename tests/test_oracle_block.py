"""Pins the float64 block oracle (oracle/cpu_oracle.py convblock_fwd/bwd) against torch
autograd through the library operators, including BASELINE config 1 (CPU plumbing)."""
import math

import numpy as np
import pytest
import torch

from oracle import torch_path


def _np(P):
    return {k: v.double().numpy() for k, v in P.items()}


def _check_block(oracle, dim, k, shape, seed, dist="normal", bias=False, scales=(1.0, 0.5), inter_ratio=0.5):
    torch.manual_seed(seed)
    P = torch_path.default_params(dim, k, bias=bias, scales=scales, inter_ratio=inter_ratio)
    x = torch.randn(*shape) if dist == "normal" else torch.rand(*shape) * 4 - 2
    g = torch.randn(*shape)
    Pd = {k_: v.double().requires_grad_() for k_, v in P.items()}
    xd = x.double().requires_grad_()
    yt = torch_path.convblock(xd, Pd, scales=scales)
    grads = torch.autograd.grad(yt, [xd] + list(Pd.values()), g.double())
    y, cache = oracle.convblock_fwd(x.numpy(), _np(P), scales=scales)
    np.testing.assert_allclose(y, yt.detach().numpy(), atol=1e-11)
    dx, gr = oracle.convblock_bwd(cache, g.numpy())
    np.testing.assert_allclose(dx, grads[0].numpy(), atol=1e-10)
    for name, gt in zip(Pd.keys(), grads[1:]):
        scale = max(1.0, float(gt.abs().max()))
        np.testing.assert_allclose(gr[name], gt.numpy(), atol=1e-10 * scale, err_msg=name)
    return P


def test_config1_cpu_plumbing(oracle):
    """ConvBlock(dim=64, kernel_size=7), x [2,32,32,64] ~ N(0,1), seed 0, fp32 values."""
    P = _check_block(oracle, 64, 7, (2, 32, 32, 64), 0)
    # the depthwise conv runs on inter_dim = 32 channels
    assert tuple(P["gates.0.conv_spatial.weight"].shape) == (7, 7, 32)
    assert P["gates.0.conv_spatial.weight"].dtype == torch.float16
    assert list(P.keys()) == ["conv_up.weight", "gates.0.conv_spatial.weight", "gates.1.conv_spatial.weight",
                              "conv_out.weight", "conv_out.bias", "conv_pool.weight", "conv_pool.bias"]


@pytest.mark.parametrize("k", [9, 15])
def test_ragged_config5_small_batch(oracle, k):
    """Config 5 geometry (57x61, C=200 -> 100 conv channels, odd pool bins) at B=1."""
    _check_block(oracle, 200, k, (1, 57, 61, 200), 0, dist="uniform")


@pytest.mark.parametrize("shape", [(2, 16, 16, 64), (2, 13, 19, 64)])
@pytest.mark.parametrize("scales", [(1.,), (0.5,), (1., 0.5, 0.25), (0.5, 1.), (1., 1.), (1., 0.75)])
def test_block_scales(oracle, scales, shape):
    """The oracle's block with every non-default ``scales`` tuple the GPU tests use it for as their checker,
    against autograd through torch's library operators in float64 (pooled extents int(H * s), conv_block.py:16;
    one gate per scale, concatenated in order, conv_block.py:41-44)."""
    _check_block(oracle, 64, 7, shape, 11, scales=scales)


@pytest.mark.parametrize("inter_ratio", [0.25, 0.75, 1.0])
def test_block_inter_ratio(oracle, inter_ratio):
    _check_block(oracle, 64, 5, (2, 10, 12, 64), 12, inter_ratio=inter_ratio)


def test_block_with_up_bias(oracle):
    _check_block(oracle, 16, 3, (2, 6, 10, 16), 3, bias=True)


def test_depthwise_init_closed_form():
    torch.manual_seed(0)
    P = torch_path.default_params(64, 7)
    b = torch_path.dw_init_bound(7, 32)
    assert math.isclose(b, math.sqrt(6 / (7 * 32)))
    w = P["gates.0.conv_spatial.weight"].float()
    assert w.abs().max() <= b * (1 + 1e-3) and w.abs().max() > 0.95 * b
    assert abs(float(w.mean())) < 0.02 * b * 3 and math.isclose(float(w.std()), b / math.sqrt(3), rel_tol=0.05)
