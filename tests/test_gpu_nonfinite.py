"""The non-finite contract of the depthwise convolution (include/pdw.h, "Non-finite inputs").

The reference masks its loads (dwconv_triton.py:55-86): an Inf or NaN pixel reaches exactly the K x K footprint of
the filter around it.  The kernels here multiply a window somewhat larger than the filter by zero-padded filter
operands, so the value may also turn nearby outputs into NaN (0 * Inf), by at most PDW_NONFINITE_REACH pixels in
every direction.  These tests pin that: every output further away, and every other channel, must equal the
float64 oracle of the clean input to the usual tolerance; every output the reference makes non-finite must be
non-finite here as well.
"""
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from parity import TOL, randn

pytestmark = pytest.mark.gpu

REACH = int(re.search(r"#define\s+PDW_NONFINITE_REACH\s+(\d+)", (Path(__file__).resolve().parents[1] / "include" / "pdw.h").read_text()).group(1))


def _box(shape_hw, pix, k, pad, reach):
    """Mask [H, W] of the outputs a value at input pixel `pix` reaches through a k x k 'same' filter, dilated."""
    H, W = shape_hw
    m = np.zeros((H, W), dtype=bool)
    i, j = pix
    # output (oi, oj) reads input (oi - pad + u, oj - pad + v), 0 <= u, v < k
    lo_i, hi_i = i + pad - (k - 1) - reach, i + pad + reach
    lo_j, hi_j = j + pad - (k - 1) - reach, j + pad + reach
    m[max(lo_i, 0):max(min(hi_i, H - 1) + 1, 0), max(lo_j, 0):max(min(hi_j, W - 1) + 1, 0)] = True
    return m


CASES = [
    # shape, k, dtype, planted (b, i, j, c, value)
    ((2, 40, 44, 64), 13, torch.bfloat16),   # matrix-core kernels, 16 patches per image row
    ((2, 40, 44, 64), 7, torch.float16),
    ((4, 28, 28, 64), 13, torch.bfloat16),   # two images side by side in one instruction
    ((2, 57, 61, 24), 9, torch.bfloat16),
    ((2, 30, 33, 100), 9, torch.bfloat16),   # C % 8 != 0: vector kernel, 16-bit dot products
    ((2, 30, 33, 20), 13, torch.float32),    # fp32, small tensor: matrix-core kernel
    ((2, 40, 44, 8), 17, torch.float32),     # fp32 matrix-core kernel
    ((2, 30, 33, 20), 7, torch.float32),     # fp32 vector kernel
    ((1, 24, 25, 16), 17, torch.float16),
]
PLANTS = [(0, 17, 19, 5, float("inf")), (1, 2, 1, 3, float("nan")), (0, 23, 0, 7, float("-inf"))]


@pytest.mark.parametrize("shape,k,dtype", CASES)
def test_forward_and_input_gradient_footprint(oracle, shape, k, dtype):
    from pyramidconvblock_amd.dwconv import dwconv_dgrad, dwconv_forward

    B, H, W, C = shape
    pad = k // 2
    gen = torch.Generator().manual_seed(k + C)
    x = randn(gen, B, H, W, C).to(dtype)
    w = (randn(gen, k, k, C) / k).to(dtype)
    geo = ((1, 1), (pad, pad), (1, 1))
    clean_fwd = oracle.dwconv_fwd(x.double().numpy(), w.double().numpy(), 1, (pad, pad), 1)
    clean_dg = oracle.dwconv_dgrad(x.double().numpy(), w.double().numpy(), (H, W), 1, (pad, pad), 1)
    xp = x.clone()
    plants = [p for p in PLANTS if p[0] < B and p[1] < H and p[2] < W and p[3] < C]
    for (b, i, j, c, v) in plants:
        xp[b, i, j, c] = v
    bad_fwd = oracle.dwconv_fwd(xp.double().numpy(), w.double().numpy(), 1, (pad, pad), 1)
    bad_dg = oracle.dwconv_dgrad(xp.double().numpy(), w.double().numpy(), (H, W), 1, (pad, pad), 1)
    for name, got, clean, bad, flip in (
        ("forward", dwconv_forward(xp.cuda(), w.cuda(), *geo), clean_fwd, bad_fwd, False),
        ("input gradient", dwconv_dgrad(xp.cuda(), w.cuda(), (B, H, W, C), *geo), clean_dg, bad_dg, True),
    ):
        got = got.float().cpu().numpy().astype(np.float64)
        may = np.zeros((B, H, W, C), dtype=bool)
        for (b, i, j, c, _) in plants:
            # forward: output o reads input o - pad + u; the input gradient is the same with the filter rotated
            # (pad' = k - 1 - pad = pad for odd k), so the box is the same
            may[b, :, :, c] |= _box((H, W), (i, j), k, pad, REACH)
        # 1. away from the planted values: finite and equal to the clean oracle
        far = ~may
        assert np.isfinite(got[far]).all(), f"{name}: non-finite output beyond the stated reach"
        scale = np.abs(clean).max()
        err = np.abs(got[far] - clean[far]).max() / scale
        assert err <= TOL[dtype], f"{name}: outputs outside the reach differ from the clean oracle: {err}"
        # 2. where the reference's masked loads give a non-finite result, so does the kernel
        ref_bad = ~np.isfinite(bad)
        assert ref_bad.any()
        assert (~np.isfinite(got[ref_bad])).all(), f"{name}: a non-finite reference output came out finite"
        assert not (ref_bad & far).any()


@pytest.mark.parametrize("shape,k,dtype", CASES[:5])
def test_weight_gradient_other_channels_unaffected(oracle, shape, k, dtype):
    """A non-finite value in x or gy may make any tap of ITS channel non-finite (the reference: the taps whose shifted
    position falls inside the image, which is nearly all of them); the other channels must be untouched."""
    from pyramidconvblock_amd.dwconv import dwconv_wgrad

    B, H, W, C = shape
    pad = k // 2
    gen = torch.Generator().manual_seed(3 * k + C)
    x = randn(gen, B, H, W, C).to(dtype)
    g = randn(gen, B, H, W, C).to(dtype)
    geo = ((1, 1), (pad, pad), (1, 1))
    clean = oracle.dwconv_wgrad(x.double().numpy(), g.double().numpy(), (k, k), 1, (pad, pad), 1)
    xp, gp = x.clone(), g.clone()
    xp[0, 5, 6, 5] = float("inf")
    gp[B - 1, 3, 2, 9] = float("nan")
    bad = oracle.dwconv_wgrad(xp.double().numpy(), gp.double().numpy(), (k, k), 1, (pad, pad), 1)
    got = dwconv_wgrad(xp.cuda(), gp.cuda(), (k, k, C), *geo).float().cpu().numpy().astype(np.float64)
    others = np.ones(C, dtype=bool)
    others[[5, 9]] = False
    assert np.isfinite(got[:, :, others]).all()
    err = np.abs(got[:, :, others] - clean[:, :, others]).max() / np.abs(clean).max()
    assert err <= TOL[dtype], err
    ref_bad = ~np.isfinite(bad)
    assert ref_bad[:, :, [5, 9]].any() and not ref_bad[:, :, others].any()
    assert (~np.isfinite(got[ref_bad])).all()
