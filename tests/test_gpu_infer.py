"""The inference form of the block: the convolution with the gate applied in its store (pdw_dwconv_fwd_gate) and the
whole forward without a saved convolution output (pdw_convblock_infer, which ConvBlock.forward uses when nothing
requires a gradient), against the float64 oracle and against the training forward."""
import ctypes

import numpy as np
import pytest
import torch

from parity import TOL, assert_close, randn

pytestmark = pytest.mark.gpu

DT = {torch.float16: 1, torch.bfloat16: 2, torch.float32: 0}


def _gate_conv(x, w, ldy, ych, pool, dtype):
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    B, H, W, C = x.shape
    K = w.shape[0]
    y = torch.full((B, H, W, ldy), 7.0, device="cuda", dtype=dtype)
    xp = torch.empty((B, H // 2, W // 2, C), device="cuda", dtype=dtype) if pool else None
    rc = L.pdw_dwconv_fwd_gate(x.data_ptr(), w.data_ptr(), y.data_ptr(), xp.data_ptr() if pool else None, B, H, W, C, K,
                               K // 2, ldy, ych, DT[dtype], ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return rc, y, xp


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,k,ldy,ych,pool", [
    ((2, 24, 28, 32), 13, 16, 0, False),
    ((2, 24, 28, 32), 13, 32, 16, True),
    ((3, 20, 22, 64), 9, 64, 0, True),
    ((3, 20, 22, 64), 7, 64, 0, False),
    ((4, 28, 28, 64), 13, 32, 0, False),     # two images side by side in one instruction
    ((2, 57, 61, 48), 9, 24, 0, False),      # odd extents
    ((1, 8, 8, 16), 5, 8, 0, True),
    ((2, 30, 26, 96), 11, 104, 56, False),
    ((2, 16, 16, 32), 3, 16, 0, False),
    ((2, 24, 28, 32), 17, 16, 0, False),     # 8 channels per workgroup: 4 of each half of C
    ((3, 40, 36, 64), 15, 64, 32, False),
    ((8, 56, 56, 48), 17, 24, 0, False),     # (C = 48: three 16-channel gate groups over six slices)
    ((1, 57, 33, 96), 15, 48, 0, False),
])
def test_conv_gate_matches_oracle(oracle, shape, k, ldy, ych, pool, dtype):
    B, H, W, C = shape
    gen = torch.Generator().manual_seed(k + C)
    x = randn(gen, B, H, W, C).to(dtype)
    w = (randn(gen, k, k, C) / k).to(dtype)
    rc, y, xp = _gate_conv(x.cuda(), w.cuda(), ldy, ych, pool, dtype)
    assert rc == 0
    conv = oracle.dwconv_fwd(x.double().numpy(), w.double().numpy(), 1, (k // 2, k // 2), 1)
    want = oracle.gate_fwd(conv)
    assert_close(y[..., ych:ych + C // 2], want, dtype, "gated conv")
    # channels of the strided output that are not the gate's are untouched
    rest = torch.ones(ldy, dtype=torch.bool)
    rest[ych:ych + C // 2] = False
    assert torch.all(y[..., rest.cuda()] == 7.0)
    if pool:
        assert_close(xp, oracle.avgpool_fwd(x.double().numpy(), (H // 2, W // 2)), dtype, "pooled input")


def test_conv_gate_equals_separate_kernels_bitwise():
    """Same arithmetic as pdw_dwconv_fwd followed by pdw_gate_fwd (the gate multiplies the rounded outputs)."""
    from pyramidconvblock_amd import ops
    from pyramidconvblock_amd.dwconv import dwconv_forward

    gen = torch.Generator().manual_seed(5)
    x = randn(gen, 4, 28, 28, 64).to(torch.bfloat16).cuda()
    w = (randn(gen, 13, 13, 64) / 13).to(torch.bfloat16).cuda()
    rc, y, _ = _gate_conv(x, w, 32, 0, False, torch.bfloat16)
    assert rc == 0
    c = dwconv_forward(x, w, (1, 1), (6, 6), (1, 1))
    ref = torch.empty(4, 28, 28, 32, device="cuda", dtype=torch.bfloat16)
    ops.gate_forward(c, out=ref)
    assert torch.equal(y, ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,k", [((32, 56, 56, 64), 13), ((2, 40, 36, 32), 9), ((3, 34, 70, 16), 3),
                                     ((1, 36, 40, 48), 5), ((2, 40, 48, 32), 15), ((2, 20, 24, 32), 9),
                                     ((32, 56, 56, 64), 9), ((32, 56, 56, 64), 17), ((64, 56, 56, 64), 13),
                                     ((128, 56, 56, 64), 13)])
def test_two_scale_conv_gate_is_the_two_calls(shape, k, dtype):
    """pdw_dwconv_fwd2_gate (the gated convolutions of both scales in one launch, into strided outputs) gives bitwise
    the results of two pdw_dwconv_fwd_gate calls, and status 3 where it does not cover the case."""
    from pyramidconvblock_amd import _lib

    L = _lib.lib()
    B, H, W, C = shape
    G = C // 2
    gen = torch.Generator().manual_seed(k + H)
    x0 = randn(gen, B, H, W, C).to(dtype).cuda()
    x1 = randn(gen, B, H // 2, W // 2, C).to(dtype).cuda()
    w0, w1 = ((randn(gen, k, k, C) / k).to(dtype).cuda() for _ in range(2))
    y0 = torch.full((B, H, W, C), 7.0, device="cuda", dtype=dtype)           # the gate's G channels from channel G on
    y1 = torch.full((B, H // 2, W // 2, G), 7.0, device="cuda", dtype=dtype)
    rc = L.pdw_dwconv_fwd2_gate(x0.data_ptr(), w0.data_ptr(), y0.data_ptr(), C, G, x1.data_ptr(), w1.data_ptr(),
                                y1.data_ptr(), G, 0, B, H, W, C, k, DT[dtype],
                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    wide = -(-W // 64) * 64 * B <= -(-W // 32) * 32 * (-(-B // 2) * 2)
    covered = dtype != torch.float32 and C % 16 == 0 and wide
    assert rc == (0 if covered else 3)
    if not covered:
        return
    r0, want0, _ = _gate_conv(x0, w0, C, G, False, dtype)
    r1, want1, _ = _gate_conv(x1, w1, G, 0, False, dtype)
    assert r0 == 0 and r1 == 0
    assert torch.equal(y0, want0) and torch.equal(y1, want1)


def test_conv_gate_not_covered_returns_3():
    x = torch.zeros(1, 8, 8, 32, device="cuda")
    w = torch.zeros(5, 5, 32, device="cuda")
    rc, _, _ = _gate_conv(x, w, 16, 0, False, torch.float32)       # fp32
    assert rc == 3
    xb, wb = x.bfloat16(), torch.zeros(17, 17, 32, device="cuda", dtype=torch.bfloat16)
    rc, _, _ = _gate_conv(xb, wb, 16, 0, True, torch.bfloat16)      # pooled output from 8 channels per workgroup
    assert rc == 3
    x24 = torch.zeros(1, 8, 8, 24, device="cuda", dtype=torch.bfloat16)
    rc, _, _ = _gate_conv(x24, torch.zeros(5, 5, 24, device="cuda", dtype=torch.bfloat16), 12, 0, False, torch.bfloat16)
    assert rc == 3                                                   # C % 16 != 0
    x32 = torch.zeros(1, 8, 8, 32, device="cuda", dtype=torch.bfloat16)
    rc, _, _ = _gate_conv(x32, torch.zeros(7, 7, 32, device="cuda", dtype=torch.bfloat16), 16, 0, True, torch.bfloat16)
    assert rc == 3                                                   # pooled output with odd padding


@pytest.mark.parametrize("dim,k,shape,dtype", [
    (128, 13, (32, 56, 56, 128), torch.bfloat16),    # headline workload
    (128, 9, (4, 56, 56, 128), torch.float16),
    (128, 17, (4, 56, 56, 128), torch.bfloat16),     # 8 channels per convolution workgroup
    (128, 15, (2, 24, 40, 128), torch.float16),
    (64, 7, (3, 16, 24, 64), torch.bfloat16),
    (128, 13, (1, 8, 8, 128), torch.bfloat16),
])
def test_block_inference_forward(oracle, dim, k, shape, dtype):
    import pyramid_dwconv
    from pyramidconvblock_amd import conv_block

    torch.manual_seed(1)
    m = pyramid_dwconv.ConvBlock(dim=dim, kernel_size=k).to(dtype)
    gen = torch.Generator().manual_seed(1)
    x = randn(gen, *shape).to(dtype)
    params = {n: p.detach().double().numpy() for n, p in m.state_dict().items()}
    yo, _ = oracle.convblock_fwd(x.double().numpy(), params)
    m = m.cuda()
    calls = []
    orig = conv_block.convblock_infer
    conv_block.convblock_infer = lambda *a, **kw: (calls.append(1), orig(*a, **kw))[1]
    try:
        with torch.no_grad():
            y = m(x.cuda())
    finally:
        conv_block.convblock_infer = orig
    assert calls, "the inference entry point was not used"
    assert_close(y, yo, dtype, "y (inference)")
    # and it agrees with the training forward to rounding of the half-resolution gate
    yt = m(x.cuda().requires_grad_())
    scale = yt.detach().float().abs().max().item()
    assert (y.float() - yt.detach().float()).abs().max().item() <= TOL[dtype] * scale


@pytest.mark.parametrize("dim,kw", [(112, {}), (128, {"bias": True}), (64, {"scales": (1., 0.5, 0.25)})])
def test_block_inference_other_shapes_use_the_stepwise_path(oracle, dim, kw):
    """What the library's single call does not cover (an inner width of 56, a bias on conv_up, three scales) still
    gives the right forward under no_grad, through the operator's launches one by one."""
    import pyramid_dwconv
    from pyramidconvblock_amd import conv_block

    torch.manual_seed(2)
    m = pyramid_dwconv.ConvBlock(dim=dim, kernel_size=9, **kw).to(torch.float16)
    gen = torch.Generator().manual_seed(2)
    x = randn(gen, 2, 24, 20, dim).to(torch.float16)
    params = {n: p.detach().double().numpy() for n, p in m.state_dict().items()}
    yo, _ = oracle.convblock_fwd(x.double().numpy(), params, scales=tuple(kw.get("scales", (1., 0.5))))
    calls = []
    orig = conv_block.convblock_infer
    conv_block.convblock_infer = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        with torch.no_grad():
            y = m.cuda()(x.cuda())
    finally:
        conv_block.convblock_infer = orig
    assert not calls, "the single-call inference entry point was taken for a configuration it does not cover"
    assert_close(y, yo, torch.float16, "y")
