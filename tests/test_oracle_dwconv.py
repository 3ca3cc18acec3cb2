"""Pins the float64 depthwise-conv oracle (oracle/pdw_oracle.c) without the reference:
library routine (F.conv2d + autograd, float64), brute force, closed forms, adjoint
identities and finite differences."""
import itertools

import numpy as np
import pytest
import torch

from oracle import torch_path

CASES = [
    # B, H, W, C, KH, KW, stride, padding, dilation
    (2, 9, 11, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 12, 10, 7, 7, 7, (1, 1), (3, 3), (1, 1)),
    (2, 8, 13, 4, 5, 3, (1, 1), (2, 1), (1, 1)),
    (1, 14, 15, 3, 3, 5, (2, 1), (0, 2), (1, 2)),
    (2, 11, 11, 6, 4, 2, (2, 3), (2, 1), (2, 1)),
    (1, 6, 6, 2, 9, 9, (1, 1), (4, 4), (1, 1)),  # kernel larger than the image
]


def _rand(rng, *shape):
    return rng.standard_normal(shape)


@pytest.mark.parametrize("case", CASES)
def test_fwd_dgrad_wgrad_match_torch_float64(oracle, case):
    B, H, W, C, KH, KW, s, p, d = case
    rng = np.random.default_rng(1)
    x, w = _rand(rng, B, H, W, C), _rand(rng, KH, KW, C)
    xt = torch.from_numpy(x).requires_grad_()
    wt = torch.from_numpy(w).requires_grad_()
    yt = torch_path.dwconv_nhwc(xt, wt, s, p, d)
    y = oracle.dwconv_fwd(x, w, s, p, d)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=0, atol=1e-12)
    gy = _rand(rng, *y.shape)
    gx_t, gw_t = torch.autograd.grad(yt, (xt, wt), torch.from_numpy(gy))
    np.testing.assert_allclose(oracle.dwconv_dgrad(gy, w, (H, W), s, p, d), gx_t.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(oracle.dwconv_wgrad(x, gy, (KH, KW), s, p, d), gw_t.numpy(), rtol=0, atol=1e-11)


def test_brute_force_python_loops(oracle):
    rng = np.random.default_rng(2)
    B, H, W, C, K, P = 1, 5, 6, 2, 3, 1
    x, w = _rand(rng, B, H, W, C), _rand(rng, K, K, C)
    ref = np.zeros((B, H, W, C))
    for b, i, j, c, kh, kw in itertools.product(range(B), range(H), range(W), range(C), range(K), range(K)):
        ih, iw = i - P + kh, j - P + kw
        if 0 <= ih < H and 0 <= iw < W:
            ref[b, i, j, c] += x[b, ih, iw, c] * w[kh, kw, c]
    np.testing.assert_allclose(oracle.dwconv_fwd(x, w, 1, P, 1), ref, atol=1e-13)


def test_closed_forms(oracle):
    rng = np.random.default_rng(3)
    x = _rand(rng, 2, 10, 9, 4)
    # delta kernel -> identity; off-centre delta -> shift with zero fill
    k = 7
    w = np.zeros((k, k, 4))
    w[k // 2, k // 2] = 1.0
    np.testing.assert_array_equal(oracle.dwconv_fwd(x, w, 1, k // 2, 1), x)
    w = np.zeros((k, k, 4))
    w[k // 2 + 2, k // 2 - 1] = 1.0  # y[i,j] = x[i+2, j-1]
    y = oracle.dwconv_fwd(x, w, 1, k // 2, 1)
    np.testing.assert_array_equal(y[:, :-2, 1:], x[:, 2:, :-1])
    assert np.all(y[:, -2:] == 0) and np.all(y[:, :, 0] == 0)
    # k=1 -> per-channel scale
    s = _rand(rng, 1, 1, 4)
    np.testing.assert_allclose(oracle.dwconv_fwd(x, s, 1, 0, 1), x * s[0, 0], atol=1e-15)
    # all ones -> area of the window clipped at the border
    H, W, k = 8, 11, 5
    y = oracle.dwconv_fwd(np.ones((1, H, W, 1)), np.ones((k, k, 1)), 1, k // 2, 1)[0, :, :, 0]
    cnt = lambda n, i: min(n - 1, i + k // 2) - max(0, i - k // 2) + 1
    ref = np.array([[cnt(H, i) * cnt(W, j) for j in range(W)] for i in range(H)], dtype=float)
    np.testing.assert_array_equal(y, ref)


@pytest.mark.parametrize("case", CASES)
def test_adjoint_identities(oracle, case):
    B, H, W, C, KH, KW, s, p, d = case
    rng = np.random.default_rng(4)
    x, w = _rand(rng, B, H, W, C), _rand(rng, KH, KW, C)
    y = oracle.dwconv_fwd(x, w, s, p, d)
    g = _rand(rng, *y.shape)
    lhs = np.sum(y * g)
    assert np.isclose(lhs, np.sum(x * oracle.dwconv_dgrad(g, w, (H, W), s, p, d)), rtol=1e-11)
    assert np.isclose(lhs, np.sum(w * oracle.dwconv_wgrad(x, g, (KH, KW), s, p, d)), rtol=1e-11)


@pytest.mark.parametrize("k", [3, 7, 9, 13])
def test_reference_flipped_dgrad_equals_adjoint_for_same_padding(oracle, k):
    """dwconv_triton.py:154-185 is the true input gradient iff stride 1 and 2*pad == k-1."""
    rng = np.random.default_rng(5)
    g, w = _rand(rng, 2, 10, 12, 3), _rand(rng, k, k, 3)
    a = oracle.dwconv_dgrad(g, w, (10, 12), 1, k // 2, 1)
    b = oracle.dwconv_dgrad_flipped(g, w, k // 2)
    np.testing.assert_allclose(a, b, atol=1e-12)
    # and it is the forward op applied with the 180-degree rotated filter
    np.testing.assert_allclose(a, oracle.dwconv_fwd(g, w[::-1, ::-1].copy(), 1, k // 2, 1), atol=1e-12)


def test_flipped_dgrad_is_wrong_for_other_padding(oracle):
    rng = np.random.default_rng(6)
    g, w = _rand(rng, 1, 8, 8, 2), _rand(rng, 3, 3, 2)
    x_hw = (6, 6)  # padding 2 with k=3 grows the map: 6 -> 8
    exact = oracle.dwconv_dgrad(g, w, x_hw, 1, 2, 1)
    assert exact.shape == (1, 6, 6, 2)
    assert not np.allclose(oracle.dwconv_dgrad_flipped(g, w, 2)[:, :6, :6], exact)


def test_finite_differences(oracle):
    rng = np.random.default_rng(7)
    x, w = _rand(rng, 1, 6, 7, 2), _rand(rng, 5, 5, 2)
    g = _rand(rng, 1, 6, 7, 2)
    f = lambda xx, ww: np.sum(oracle.dwconv_fwd(xx, ww, 1, 2, 1) * g)
    dx, dw = oracle.dwconv_dgrad(g, w, (6, 7), 1, 2, 1), oracle.dwconv_wgrad(x, g, (5, 5), 1, 2, 1)
    eps = 1e-6
    for idx in [(0, 0, 0, 0), (0, 3, 4, 1), (0, 5, 6, 0)]:
        e = np.zeros_like(x)
        e[idx] = eps
        assert np.isclose((f(x + e, w) - f(x - e, w)) / (2 * eps), dx[idx], rtol=1e-6, atol=1e-8)
    for idx in [(0, 0, 0), (2, 2, 1), (4, 1, 0)]:
        e = np.zeros_like(w)
        e[idx] = eps
        assert np.isclose((f(x, w + e) - f(x, w - e)) / (2 * eps), dw[idx], rtol=1e-6, atol=1e-8)


def test_output_size_formula(oracle):
    for n, k, s, p, d in [(56, 13, 1, 6, 1), (57, 9, 1, 4, 1), (32, 7, 2, 3, 1), (20, 3, 1, 0, 2), (5, 9, 1, 0, 1)]:
        t = torch.zeros(1, 1, n, n)
        try:
            ref = torch.nn.functional.conv2d(t, torch.zeros(1, 1, k, k), None, s, p, d).shape[-1]
        except RuntimeError:
            ref = 0
        assert oracle.out_size(n, k, s, p, d) == ref
