"""Pins the float64 pool / bilinear / gate oracle against torch's CPU operators (the
third-party routines the reference calls at conv_block.py:16 and conv_block.py:21) and
against closed forms."""
import numpy as np
import pytest
import torch

from oracle import torch_path

POOL = [((8, 10), (4, 5)), ((57, 61), (28, 30)), ((9, 7), (4, 3)), ((5, 5), (5, 5)), ((7, 9), (1, 1)), ((6, 6), (4, 4))]
UP = [((4, 5), (8, 10)), ((28, 30), (57, 61)), ((3, 4), (7, 9)), ((5, 5), (5, 5)), ((1, 1), (4, 3)), ((8, 8), (5, 6))]


@pytest.mark.parametrize("hw,out", POOL)
def test_avgpool_matches_torch(oracle, hw, out):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, *hw, 3))
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch_path.avgpool_nhwc(xt, out)
    np.testing.assert_allclose(oracle.avgpool_fwd(x, out), yt.detach().numpy(), atol=1e-14)
    g = rng.standard_normal(tuple(yt.shape))
    (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(g))
    np.testing.assert_allclose(oracle.avgpool_bwd(g, hw), gx.numpy(), atol=1e-14)


def test_avgpool_closed_forms(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 8, 6, 2))
    ref = x.reshape(1, 4, 2, 3, 2, 2).mean(axis=(2, 4))  # exact 2x2 mean for even sizes
    np.testing.assert_allclose(oracle.avgpool_fwd(x, (4, 3)), ref, atol=1e-15)
    # 57 -> 28: every bin is 3 wide and starts at floor(i*57/28)
    ramp = np.arange(57, dtype=float).reshape(1, 57, 1, 1)
    y = oracle.avgpool_fwd(ramp, (28, 1))[0, :, 0, 0]
    np.testing.assert_allclose(y, [(i * 57) // 28 + 1.0 for i in range(28)], atol=1e-13)
    # constants are preserved; gradient of a constant cotangent sums to the same mass
    assert np.allclose(oracle.avgpool_fwd(np.full((1, 7, 5, 1), 2.5), (3, 2)), 2.5)
    g = rng.standard_normal((1, 3, 2, 1))
    assert np.isclose(oracle.avgpool_bwd(g, (7, 5)).sum(), g.sum())


@pytest.mark.parametrize("hw,out", UP)
def test_bilinear_matches_torch(oracle, hw, out):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, *hw, 3))
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch_path.bilinear_nhwc(xt, out)
    np.testing.assert_allclose(oracle.bilinear_fwd(x, out), yt.detach().numpy(), atol=1e-13)
    g = rng.standard_normal(tuple(yt.shape))
    (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(g))
    np.testing.assert_allclose(oracle.bilinear_bwd(g, hw), gx.numpy(), atol=1e-13)


def test_bilinear_closed_forms(oracle):
    # exact 2x: output 2m+1 = .75 x[m] + .25 x[m+1], output 2m+2 = .25 x[m] + .75 x[m+1]; borders clamp
    x = np.array([1.0, 5.0, 2.0, 8.0]).reshape(1, 1, 4, 1)
    y = oracle.bilinear_fwd(x, (1, 8))[0, 0, :, 0]
    ref = [1.0, 0.75 * 1 + 0.25 * 5, 0.25 * 1 + 0.75 * 5, 0.75 * 5 + 0.25 * 2, 0.25 * 5 + 0.75 * 2,
           0.75 * 2 + 0.25 * 8, 0.25 * 2 + 0.75 * 8, 8.0]
    np.testing.assert_allclose(y, ref, atol=1e-15)
    assert np.allclose(oracle.bilinear_fwd(np.full((1, 3, 4, 2), -1.5), (7, 9)), -1.5)
    # a linear ramp is reproduced away from the clamped border: out(i) = (i+.5)*in/out - .5
    ramp = np.arange(6, dtype=float).reshape(1, 6, 1, 1)
    y = oracle.bilinear_fwd(ramp, (13, 1))[0, :, 0, 0]
    src = (np.arange(13) + 0.5) * 6 / 13 - 0.5
    inner = (src >= 0) & (src <= 5)
    np.testing.assert_allclose(y[inner], src[inner], atol=1e-13)
    # adjoint identity
    rng = np.random.default_rng(3)
    a, g = rng.standard_normal((2, 5, 6, 3)), rng.standard_normal((2, 11, 13, 3))
    assert np.isclose(np.sum(oracle.bilinear_fwd(a, (11, 13)) * g), np.sum(a * oracle.bilinear_bwd(g, (5, 6))))


def test_gate(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 3, 4, 10))
    y = oracle.gate_fwd(x)
    np.testing.assert_allclose(y, x[..., :5] * x[..., 5:] * np.sqrt(5.0), rtol=1e-14)
    xt = torch.from_numpy(x).requires_grad_()
    yt = torch_path.gate(xt)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-14)
    g = rng.standard_normal(y.shape)
    (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(g))
    np.testing.assert_allclose(oracle.gate_bwd(x, g), gx.numpy(), rtol=1e-13)
