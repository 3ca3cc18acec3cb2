"""Parity of the HIP depthwise conv (fwd, dgrad, wgrad) with the float64 oracle, called
through the C ABI of libpdw.so via the operator mirror."""
import numpy as np
import pytest
import torch

from parity import TOL, assert_close, randn, rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _run(oracle, shape, k, dtype, stride=1, padding=None, dilation=1, seed=0, dist="normal", wscale=None):
    import pyramidconvblock_amd as P

    B, H, W, C = shape
    kh, kw = (k, k) if isinstance(k, int) else k
    pad = (kh // 2, kw // 2) if padding is None else padding
    gen = torch.Generator().manual_seed(seed)
    x = randn(gen, B, H, W, C) if dist == "normal" else torch.rand(B, H, W, C, generator=gen) * 4 - 2
    w = randn(gen, kh, kw, C) * (wscale if wscale is not None else 1.0 / max(kh, kw))
    xr, wr = x.to(dtype), w.to(dtype)
    xd = xr.cuda().requires_grad_()
    wd = wr.cuda().requires_grad_()
    y = P.DepthwiseConv2DFunction.apply(xd, wd, stride, pad, dilation, dtype)
    yo = oracle.dwconv_fwd(xr.double().numpy(), wr.double().numpy(), stride, pad, dilation)
    assert y.dtype == dtype and tuple(y.shape) == yo.shape
    errs = [assert_close(y, yo, dtype, "y")]
    g = randn(gen, *y.shape).to(dtype)
    y.backward(g.cuda())
    go = g.double().numpy()
    errs.append(assert_close(xd.grad, oracle.dwconv_dgrad(go, wr.double().numpy(), (H, W), stride, pad, dilation), dtype, "dx"))
    errs.append(assert_close(wd.grad, oracle.dwconv_wgrad(xr.double().numpy(), go, (kh, kw), stride, pad, dilation), dtype, "dW"))
    assert xd.grad.dtype == dtype and wd.grad.dtype == dtype and wd.grad.shape == wd.shape
    return errs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [3, 5, 7, 9, 11, 13, 15, 17])
def test_same_padding_small(oracle, dtype, k):
    _run(oracle, (2, 20, 23, 24), k, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [1, 3, 10, 50, 100, 136])
def test_channel_counts_and_vector_widths(oracle, dtype, C):
    _run(oracle, (2, 11, 9, C), 5, dtype, seed=C)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [
    dict(k=(3, 5), stride=(2, 1), padding=(0, 2), dilation=(1, 2)),
    dict(k=(4, 2), stride=(2, 3), padding=(2, 1), dilation=(2, 1)),
    dict(k=(5, 5), stride=1, padding=(0, 0)),
    dict(k=(5, 7), stride=1, padding=(4, 1)),
    dict(k=(9, 9), stride=1, padding=(4, 4)),
])
def test_general_stride_padding_dilation(oracle, dtype, geom):
    _run(oracle, (2, 14, 15, 12), dtype=dtype, **geom)


def test_kernel_larger_than_image(oracle):
    _run(oracle, (1, 6, 5, 8), 13, torch.float32)
    _run(oracle, (1, 6, 5, 8), 13, torch.bfloat16)


@pytest.mark.parametrize("case", [((3, 57, 61, 100), 15, None), ((2, 40, 70, 12), 17, None), ((1, 33, 35, 4), 11, None),
                                  ((2, 24, 64, 20), 13, None), ((3, 20, 90, 36), 17, (8, 8)), ((2, 37, 41, 8), 17, (3, 11)),
                                  ((1, 70, 130, 16), 13, (0, 6)), ((2, 56, 56, 128), 17, None)])
def test_fp32_matrix_core_forward_and_input_gradient(oracle, case):
    """Shapes on which the fp32 forward / input gradient take the fp32 matrix-core kernel (the largest filter on
    images wider than 32 columns, filters from 11 on small tensors): ragged channel counts, extents off the 16 x 64
    tiles, paddings other than k // 2 (the input gradient then runs at padding k - 1 - p), against the oracle."""
    shape, k, pad = case
    _run(oracle, shape, k, torch.float32, padding=pad, seed=k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [9, 15])
def test_config5_ragged(oracle, dtype, k):
    """[3,57,61,100] is the conv the ragged ConvBlock(200) runs; U(-2,2) input."""
    _run(oracle, (3, 57, 61, 100), k, dtype, dist="uniform")
    _run(oracle, (3, 28, 30, 100), k, dtype, dist="uniform")


@pytest.mark.parametrize("k", [9, 13, 17])
def test_config2_full_size_bf16(oracle, k):
    """x [32,56,56,128] ~ N(0,1), w ~ N(0, 1/k^2), bf16 (forward is the benchmarked op; grads checked too)."""
    _run(oracle, (32, 56, 56, 128), k, torch.bfloat16)


def test_config4_conv_fp16(oracle):
    _run(oracle, (8, 112, 112, 48), 17, torch.float16)


def test_empty_batch_and_empty_output():
    import pyramidconvblock_amd as P

    w = torch.randn(3, 3, 8, device="cuda")
    y = P.DepthwiseConv2DFunction.apply(torch.zeros(0, 5, 5, 8, device="cuda"), w, 1, 1, 1, torch.float32)
    assert tuple(y.shape) == (0, 5, 5, 8)
    x = torch.randn(2, 2, 2, 8, device="cuda", requires_grad=True)
    wp = w.clone().requires_grad_()
    y = P.DepthwiseConv2DFunction.apply(x, wp, 1, 0, 1, torch.float32)  # 3x3 valid conv on 2x2: empty
    assert tuple(y.shape) == (2, 0, 0, 8)
    y.sum().backward()
    assert torch.all(x.grad == 0) and torch.all(wp.grad == 0)


def test_wgrad_is_deterministic():
    import pyramidconvblock_amd as P

    gen = torch.Generator().manual_seed(1)
    x = randn(gen, 4, 33, 31, 40).to(torch.bfloat16).cuda()
    g = randn(gen, 4, 33, 31, 40).to(torch.bfloat16).cuda()
    from pyramidconvblock_amd.dwconv import dwconv_wgrad
    a = dwconv_wgrad(x, g, (9, 9, 40), (1, 1), (4, 4), (1, 1))
    b = dwconv_wgrad(x, g, (9, 9, 40), (1, 1), (4, 4), (1, 1))
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", [(32, 56, 56, 28, 28, 64, 13), (2, 20, 24, 10, 12, 40, 9), (3, 9, 11, 17, 5, 8, 3),
                                  (1, 30, 30, 15, 15, 16, 17)])
def test_wgrad_pair_is_the_two_separate_calls(dtype, case):
    """pdw_dwconv_wgrad_pair (two problems in one launch for 16-bit types, two launches otherwise) gives bitwise
    the results of two pdw_dwconv_wgrad calls, immediately and with the summations deferred."""
    from pyramidconvblock_amd import _lib
    from pyramidconvblock_amd.dwconv import dwconv_wgrad, dwconv_wgrad_pair

    B, H0, W0, H1, W1, C, k = case
    gen = torch.Generator().manual_seed(7)
    t = [randn(gen, B, H, W, C).to(dtype).cuda() for H, W in ((H0, W0), (H0, W0), (H1, W1), (H1, W1))]
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    want = [dwconv_wgrad(t[0], t[1], (k, k, C), *geo), dwconv_wgrad(t[2], t[3], (k, k, C), *geo)]
    got = dwconv_wgrad_pair(t[0], t[1], t[2], t[3], (k, k, C))
    with _lib.deferred_reductions(t[0].device):
        later = dwconv_wgrad_pair(t[0], t[1], t[2], t[3], (k, k, C))
    torch.cuda.synchronize()
    for w, g, l in zip(want, got, later):
        assert torch.equal(w, g) and torch.equal(w, l)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", [(32, 56, 56, 64, 13), (8, 112, 112, 48, 17), (2, 40, 36, 32, 9), (3, 34, 70, 16, 3),
                                  (1, 36, 40, 48, 15), (2, 20, 24, 40, 9), (4, 56, 56, 64, 7), (5, 58, 66, 24, 5),
                                  (64, 56, 56, 64, 11), (1, 130, 72, 16, 13), (32, 56, 56, 64, 9),
                                  (32, 56, 56, 64, 17), (64, 56, 56, 64, 13), (128, 56, 56, 64, 13)])
def test_fwd2_is_the_two_separate_calls(dtype, case):
    """pdw_dwconv_fwd2 (the convolutions of a block's two scales in one launch, with band heights of its own) gives
    bitwise the results of the two separate calls; pdw_dwconv_fwd2_supported says beforehand whether it takes the
    shape."""
    from pyramidconvblock_amd import _lib
    from pyramidconvblock_amd.dwconv import dwconv_forward, dwconv_forward2

    B, H, W, C, k = case
    gen = torch.Generator().manual_seed(17)
    x0 = randn(gen, B, H, W, C).to(dtype).cuda()
    x1 = randn(gen, B, H // 2, W // 2, C).to(dtype).cuda()
    w0, w1 = ((randn(gen, k, k, C) / k).to(dtype).cuda() for _ in range(2))
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    got = dwconv_forward2(x0, w0, x1, w1)
    # the full scale must be a shape for which the kernel's 64-column tile wastes no more than its 32-column one
    wide = -(-W // 64) * 64 * B <= -(-W // 32) * 32 * (-(-B // 2) * 2)
    covered = dtype != torch.float32 and C % 8 == 0 and wide
    assert bool(_lib.lib().pdw_dwconv_fwd2_supported(B, H, W, C, k, _lib.dtype_code(dtype))) == covered
    assert (got is not None) == covered
    if got is None:
        return
    want = [dwconv_forward(x0, w0, *geo), dwconv_forward(x1, w1, *geo)]
    torch.cuda.synchronize()
    for w, g in zip(want, got):
        assert torch.equal(w, g)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("case", [(32, 56, 56, 64, 13), (8, 112, 112, 48, 17), (2, 40, 36, 32, 9), (3, 34, 70, 16, 3),
                                  (1, 36, 40, 48, 15), (2, 20, 24, 40, 9), (4, 56, 56, 64, 7), (32, 56, 56, 64, 9),
                                  (32, 56, 56, 64, 17), (64, 56, 56, 64, 13), (128, 56, 56, 64, 13),
                                  (128, 4, 64, 64, 3), (128, 6, 64, 64, 13), (96, 2, 34, 16, 5)])
def test_bwd3_is_the_three_separate_calls(dtype, case):
    """pdw_dwconv_bwd3 (the full scale's input gradient with the pooled branch's added and the weight gradients of
    both scales in one launch) gives the results of the three separate calls: the input gradient bitwise, the weight
    gradients up to the order of the fp32 summation (the launch cuts the images into fewer, taller bands, so its
    partial sums are other ones: a difference of one rounding of the result at most), and bitwise the same whether the
    summations run at once or deferred; where the fused kernel does not cover the case it says so and launches
    nothing."""
    from pyramidconvblock_amd import _lib
    from pyramidconvblock_amd.dwconv import dwconv_bwd3, dwconv_dgrad, dwconv_wgrad

    B, H, W, C, k = case
    gen = torch.Generator().manual_seed(13)
    gy0, x0 = (randn(gen, B, H, W, C).to(dtype).cuda() for _ in range(2))
    gp, x1, gy1 = (randn(gen, B, H // 2, W // 2, C).to(dtype).cuda() for _ in range(3))
    w0 = (randn(gen, k, k, C) / k).to(dtype).cuda()
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    got = dwconv_bwd3(gy0, w0, gp, x0, x1, gy1)
    covered = dtype != torch.float32 and C % 16 == 0 and W > 32
    assert (got is not None) == covered
    if got is None:
        return
    want = [dwconv_dgrad(gy0, w0, x0.shape, *geo, pooled_grad=gp), dwconv_wgrad(x0, gy0, (k, k, C), *geo),
            dwconv_wgrad(x1, gy1, (k, k, C), *geo)]
    with _lib.deferred_reductions(gy0.device):
        later = dwconv_bwd3(gy0, w0, gp, x0, x1, gy1)
    torch.cuda.synchronize()
    assert torch.equal(want[0], got[0])
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    for w, g, l in zip(want, got, later):
        assert torch.equal(g, l)
        w, g = w.float(), g.float()
        # one unit in the last place of the larger value, plus the fp32 rounding of sums of B * H * W products
        tol = 2 * ulp * torch.maximum(w.abs(), g.abs()) + 1e-5 * (B * H * W) ** 0.5
        assert bool(((w - g).abs() <= tol).all()), float((w - g).abs().max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_full_size_properties(dtype):
    """Size-independent checks at the benchmark shape: delta kernel = identity, linearity in w,
    and the adjoint identity <conv(x,w), g> = <x, dgrad(g,w)> = <w, wgrad(x,g)>."""
    from pyramidconvblock_amd.dwconv import dwconv_dgrad, dwconv_forward, dwconv_wgrad

    B, H, W, C, k = 32, 56, 56, 128, 13
    gen = torch.Generator().manual_seed(3)
    x = randn(gen, B, H, W, C).to(dtype).cuda()
    g = randn(gen, B, H, W, C).to(dtype).cuda()
    w = (randn(gen, k, k, C) / k).to(dtype).cuda()
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    delta = torch.zeros(k, k, C, dtype=dtype, device="cuda")
    delta[k // 2, k // 2] = 1
    assert torch.equal(dwconv_forward(x, delta, *geo), x)
    y = dwconv_forward(x, w, *geo)
    y2 = dwconv_forward(x, (2 * w), *geo)
    assert rel_err(y2, 2 * y.double().cpu().numpy()) <= TOL[dtype]
    lhs = float((y.double() * g.double()).sum())
    dx = dwconv_dgrad(g, w, x.shape, *geo)
    dw = dwconv_wgrad(x, g, w.shape, *geo)
    tol = 5e-3 if dtype != torch.float32 else 1e-4
    assert abs(float((dx.double() * x.double()).sum()) - lhs) <= tol * abs(lhs)
    assert abs(float((dw.double() * w.double()).sum()) - lhs) <= tol * abs(lhs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 16, 24, 32, 13, (8, 12)), (1, 56, 56, 24, 9, (28, 28)), (2, 12, 10, 8, 3, (6, 5)),
                                   (2, 14, 18, 16, 5, (5, 7)), (1, 40, 36, 12, 7, (20, 18)), (3, 9, 9, 8, 5, (4, 4))])
def test_dgrad_with_pooled_gradient(oracle, dtype, shape):
    """Input gradient plus the gradient of an average pool of the same tensor: the fused kernel (exact
    halving, 16-bit, C % 8 == 0) and the two-kernel path behind the same entry point."""
    from pyramidconvblock_amd.dwconv import dwconv_dgrad

    B, H, W, C, k, hw = shape
    gen = torch.Generator().manual_seed(H * W + k)
    g = randn(gen, B, H, W, C).to(dtype)
    w = (randn(gen, k, k, C) / k).to(dtype)
    gp = randn(gen, B, *hw, C).to(dtype)
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    dx = dwconv_dgrad(g.cuda(), w.cuda(), (B, H, W, C), *geo, pooled_grad=gp.cuda())
    ref = (oracle.dwconv_dgrad(g.double().numpy(), w.double().numpy(), (H, W), 1, k // 2, 1)
           + oracle.avgpool_bwd(gp.double().numpy(), (H, W)))
    assert_close(dx, ref, dtype, "dgrad + pooled gradient")


def test_deferred_reductions_match_immediate_ones():
    """Weight gradients whose summation kernels are recorded and run as one launch are bit-identical to the
    ones computed call by call (more jobs than the table holds included)."""
    from pyramidconvblock_amd import _lib, ops
    from pyramidconvblock_amd.dwconv import dwconv_wgrad

    gen = torch.Generator().manual_seed(11)
    cases = []
    for (B, H, W, C, k, dt) in [(2, 20, 24, 32, 13, torch.bfloat16), (1, 9, 11, 5, 3, torch.float32),
                                (2, 16, 16, 16, 9, torch.float16), (1, 30, 30, 8, 5, torch.bfloat16)]:
        x = randn(gen, B, H, W, C).to(dt).cuda()
        g = randn(gen, B, H, W, C).to(dt).cuda()
        cases.append((x, g, (k, k, C), ((1, 1), (k // 2, k // 2), (1, 1))))
    a = randn(gen, 4096, 64).to(torch.bfloat16).cuda()
    b = randn(gen, 4096, 128).to(torch.bfloat16).cuda()
    ref = [dwconv_wgrad(x, g, ws, *geo) for (x, g, ws, geo) in cases] + [ops.dense_wgrad(a, b)]
    for reps in (1, 3):   # 5 jobs, then 15: beyond the 8 the table holds
        with _lib.deferred_reductions(a.device):
            got = []
            for _ in range(reps):
                got += [dwconv_wgrad(x, g, ws, *geo) for (x, g, ws, geo) in cases] + [ops.dense_wgrad(a, b)]
        torch.cuda.synchronize()
        for i, t in enumerate(got):
            assert torch.equal(t, ref[i % len(ref)]), i
    with pytest.raises(RuntimeError):
        _lib.check(_lib.lib().pdw_reduce_defer_flush(None), "flush without begin")


def test_deferred_reductions_ride_on_a_dense_layer():
    """The recorded summations executed inside later launches (the conv's inside the dense weight gradient's, that
    one's inside a dense layer's) give the same weight gradients, and the dense result is unchanged."""
    from pyramidconvblock_amd import _lib, ops
    from pyramidconvblock_amd.dwconv import dwconv_wgrad

    gen = torch.Generator().manual_seed(12)
    x = randn(gen, 2, 20, 24, 32).to(torch.bfloat16).cuda()
    g = randn(gen, 2, 20, 24, 32).to(torch.bfloat16).cuda()
    a = randn(gen, 960, 64).to(torch.bfloat16).cuda()
    b = randn(gen, 960, 128).to(torch.bfloat16).cuda()
    w = (randn(gen, 128, 64) / 8).to(torch.bfloat16).cuda()
    geo = ((1, 1), (6, 6), (1, 1))
    ref = (dwconv_wgrad(x, g, (13, 13, 32), *geo), ops.dense_wgrad(a, b), ops.dense_forward(a, w))
    for kmajor in (False, True):
        wk = w.t().contiguous() if kmajor else w
        with _lib.deferred_reductions(a.device):
            d0 = dwconv_wgrad(x, g, (13, 13, 32), *geo)
            d1 = ops.dense_wgrad(a, b)
            y = ops.dense_forward(a, wk, w_kmajor=kmajor, flush_reductions=True)
        torch.cuda.synchronize()
        assert torch.equal(d0, ref[0]) and torch.equal(d1, ref[1]) and torch.equal(y, ref[2])
    y = ops.dense_forward(a, w, flush_reductions=True)   # nothing recorded: a plain dense layer
    assert torch.equal(y, ref[2])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 16, 24, 32, 13, (8, 12)), (1, 56, 56, 24, 9, (28, 28)), (2, 12, 10, 8, 3, (6, 5)),
                                   (2, 14, 18, 16, 5, (5, 7)), (1, 40, 36, 12, 7, (20, 18)), (2, 60, 64, 16, 13, (30, 32)),
                                   (1, 20, 20, 16, 11, (10, 10))])
def test_forward_with_pooled_input(oracle, dtype, shape):
    """Conv output plus the average pool of the conv's input from one entry point: the fused kernel (exact
    halving, even padding, 16-bit, C % 8 == 0) and the two-kernel path behind it."""
    from pyramidconvblock_amd.dwconv import dwconv_forward

    B, H, W, C, k, hw = shape
    gen = torch.Generator().manual_seed(H + W + k)
    x = randn(gen, B, H, W, C).to(dtype)
    w = (randn(gen, k, k, C) / k).to(dtype)
    geo = ((1, 1), (k // 2, k // 2), (1, 1))
    y, xp = dwconv_forward(x.cuda(), w.cuda(), *geo, pool_to=hw)
    assert_close(y, oracle.dwconv_fwd(x.double().numpy(), w.double().numpy(), 1, k // 2, 1), dtype, "y")
    assert_close(xp, oracle.avgpool_fwd(x.double().numpy(), hw), dtype, "pooled input")


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_matrix_core_kernels(oracle, seed):
    """Random extents, batch sizes, channel counts (multiples of 8) and filter sizes through the 16-bit stride-1
    kernels: ragged bands and column tiles, one or two images per instruction, one to many channel slices."""
    rng = np.random.default_rng(100 + seed)
    k = int(rng.choice([3, 5, 7, 9, 11, 13, 15, 17]))
    B = int(rng.integers(1, 6))
    H = int(rng.integers(max(4, k // 2 + 1), 75))
    W = int(rng.integers(max(4, k // 2 + 1), 75))
    C = 8 * int(rng.integers(1, 10))
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    _run(oracle, (B, H, W, C), k, dtype, seed=seed)
