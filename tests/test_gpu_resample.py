"""Parity of the HIP adaptive average pool, bilinear resize and gate (forward and
backward) with the float64 oracle, through the C ABI."""
import pytest
import torch

from parity import assert_close, randn

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.float16, torch.bfloat16]

POOL = [((8, 10), (4, 5), 16), ((57, 61), (28, 30), 100), ((9, 7), (4, 3), 3), ((5, 5), (5, 5), 8), ((7, 9), (1, 1), 6),
        ((6, 6), (4, 4), 2), ((56, 56), (28, 28), 64), ((4, 5), (9, 11), 4), ((2, 2), (1, 1), 8), ((2, 6), (1, 3), 5)]
UP = [((4, 5), (8, 10), 16), ((28, 30), (57, 61), 50), ((3, 4), (7, 9), 3), ((5, 5), (5, 5), 8), ((1, 1), (4, 3), 6),
      ((8, 8), (5, 6), 2), ((28, 28), (56, 56), 32), ((56, 56), (112, 112), 24), ((1, 1), (2, 2), 8), ((1, 3), (2, 6), 5),
      ((2, 1), (4, 2), 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hw,out,C", POOL)
def test_avgpool(oracle, dtype, hw, out, C):
    import pyramidconvblock_amd as P

    gen = torch.Generator().manual_seed(C)
    x = randn(gen, 3, *hw, C).to(dtype)
    xd = x.cuda().requires_grad_()
    y = P.AdaptiveAvgPool2dFunction.apply(xd, out)
    assert_close(y, oracle.avgpool_fwd(x.double().numpy(), out), dtype, "pool y")
    g = randn(gen, *y.shape).to(dtype)
    y.backward(g.cuda())
    assert_close(xd.grad, oracle.avgpool_bwd(g.double().numpy(), hw), dtype, "pool dx")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hw,out,C", UP)
def test_bilinear(oracle, dtype, hw, out, C):
    import pyramidconvblock_amd as P

    gen = torch.Generator().manual_seed(C + 100)
    x = randn(gen, 2, *hw, C).to(dtype)
    xd = x.cuda().requires_grad_()
    y = P.BilinearInterp2dFunction.apply(xd, out)
    assert_close(y, oracle.bilinear_fwd(x.double().numpy(), out), dtype, "bilinear y")
    g = randn(gen, *y.shape).to(dtype)
    y.backward(g.cuda())
    assert_close(xd.grad, oracle.bilinear_bwd(g.double().numpy(), hw), dtype, "bilinear dx")


def test_bilinear_exact_2x_is_exact_in_fp32():
    """At exact 2x the weights are 0.25/0.75 (and 1 at the border), representable exactly."""
    import pyramidconvblock_amd as P

    x = torch.tensor([1.0, 5.0, 2.0, 8.0]).reshape(1, 1, 4, 1).repeat(1, 1, 1, 4).cuda()
    y = P.OptimizedBilinearInterp2d((1, 8))(x)[0, 0, :, 0].cpu()
    ref = torch.tensor([1.0, 2.0, 4.0, 4.25, 2.75, 3.5, 6.5, 8.0])
    assert torch.equal(y, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("I", [2, 6, 32, 64, 100, 48])
def test_gate(oracle, dtype, I):
    import pyramidconvblock_amd as P

    gen = torch.Generator().manual_seed(I)
    x = randn(gen, 2, 5, 7, I).to(dtype)
    xd = x.cuda().requires_grad_()
    y = P.GateFunction.apply(xd)
    assert_close(y, oracle.gate_fwd(x.double().numpy()), dtype, "gate y")
    g = randn(gen, *y.shape).to(dtype)
    y.backward(g.cuda())
    assert_close(xd.grad, oracle.gate_bwd(x.double().numpy(), g.double().numpy()), dtype, "gate dx")


def test_modules_and_empty():
    import pyramidconvblock_amd as P

    x = torch.randn(2, 8, 8, 16, device="cuda")
    assert tuple(P.OptimizedAdaptiveAvgPool2d(4)(x).shape) == (2, 4, 4, 16)
    assert tuple(P.OptimizedBilinearInterp2d(12)(x).shape) == (2, 12, 12, 16)
    e = torch.zeros(0, 8, 8, 16, device="cuda")
    assert tuple(P.OptimizedAdaptiveAvgPool2d((3, 2))(e).shape) == (0, 3, 2, 16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_strided_outputs_and_accumulate(oracle, dtype):
    """Gate / bilinear results written into (and gradients read from) a channel slice of a wider
    buffer, and the pool gradient accumulated in place: the pieces the fused block uses."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(7)
    B, H, W, I = 2, 10, 12, 24
    G = I // 2
    x = randn(gen, B, H, W, I).to(dtype)
    wide = torch.full((B, H, W, 3 * G), 7.0, dtype=dtype, device="cuda")
    ops.gate_forward(x.cuda(), out=wide[..., G:2 * G])
    assert_close(wide[..., G:2 * G], oracle.gate_fwd(x.double().numpy()), dtype, "gate into slice")
    assert torch.all(wide[..., :G] == 7) and torch.all(wide[..., 2 * G:] == 7)
    small = randn(gen, B, 5, 6, G).to(dtype)
    ops.bilinear_forward(small.cuda(), (H, W), out=wide[..., 2 * G:])
    assert_close(wide[..., 2 * G:], oracle.bilinear_fwd(small.double().numpy(), (H, W)), dtype, "bilinear into slice")
    assert torch.all(wide[..., :G] == 7)
    gwide = randn(gen, B, H, W, 3 * G).to(dtype)
    gd = gwide.cuda()
    assert_close(ops.gate_backward(x.cuda(), gd[..., G:2 * G]),
                 oracle.gate_bwd(x.double().numpy(), gwide[..., G:2 * G].double().numpy()), dtype, "gate bwd from slice")
    assert_close(ops.bilinear_backward(gd[..., 2 * G:], (5, 6)),
                 oracle.bilinear_bwd(gwide[..., 2 * G:].double().numpy(), (5, 6)), dtype, "bilinear bwd from slice")
    base = randn(gen, B, H, W, G).to(dtype)
    gp = randn(gen, B, 5, 6, G).to(dtype)
    acc = base.cuda().clone()
    ops.avgpool_backward(gp.cuda(), (H, W), out=acc, accumulate=True)
    assert_close(acc, base.double().numpy() + oracle.avgpool_bwd(gp.double().numpy(), (H, W)), dtype, "pool bwd accumulate")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hw,out,I", [((5, 6), (10, 12), 24), ((28, 28), (56, 56), 64), ((4, 5), (9, 11), 6),
                                      ((14, 14), (28, 28), 256), ((2, 2), (4, 4), 2), ((3, 7), (6, 14), 20)])
def test_gate_bilinear_fused(oracle, dtype, hw, out, I):
    """The one-kernel gate+resize pair (forward into a channel slice, backward out of one) against the
    oracle's gate and bilinear applied in turn, and against the two separate kernels."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(I + hw[0])
    B, G = 2, I // 2
    x = randn(gen, B, *hw, I).to(dtype)
    xd = x.cuda()
    wide = torch.full((B, *out, 2 * G + 8), 3.0, dtype=dtype, device="cuda")
    dst = wide[..., 8:8 + G]
    ops.gate_bilinear_forward(xd, out, out=dst)
    ref = oracle.bilinear_fwd(oracle.gate_fwd(x.double().numpy()), out)
    assert_close(dst, ref, dtype, "gate+bilinear y")
    assert torch.all(wide[..., :8] == 3) and torch.all(wide[..., 8 + G:] == 3)
    two = ops.bilinear_forward(ops.gate_forward(xd), out)
    assert_close(dst, two.double().cpu().numpy(), dtype, "gate+bilinear y vs separate kernels")
    g = randn(gen, B, *out, 2 * G + 8).to(dtype)
    gs = g.cuda()[..., 8:8 + G]
    gx = ops.bilinear_gate_backward(xd, gs)
    gref = oracle.gate_bwd(x.double().numpy(), oracle.bilinear_bwd(g[..., 8:8 + G].double().numpy(), hw))
    assert_close(gx, gref, dtype, "gate+bilinear dx")
    gtwo = ops.gate_backward(xd, ops.bilinear_backward(gs, hw))
    assert_close(gx, gtwo.double().cpu().numpy(), dtype, "gate+bilinear dx vs separate kernels")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hw,out,I", [((5, 6), (10, 12), 24), ((28, 28), (56, 56), 64), ((4, 5), (9, 11), 6),
                                      ((2, 2), (4, 4), 2), ((3, 7), (6, 14), 20), ((28, 30), (57, 61), 100),
                                      ((1, 1), (3, 2), 8), ((7, 9), (7, 9), 16)])
def test_gate_pair(oracle, dtype, hw, out, I):
    """Both gates of a two-scale block written into the concatenated tensor by one launch, and their gradients
    taken from it by one launch, against the oracle's gate / bilinear applied branch by branch."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(I + out[0])
    B, G = 2, I // 2
    xf = randn(gen, B, *out, I).to(dtype)
    xh = randn(gen, B, *hw, I).to(dtype)
    wide = torch.full((B, *out, I + 8), 3.0, dtype=dtype, device="cuda")
    cat = wide[..., 8:]
    ops.gate_pair_forward(xf.cuda(), xh.cuda(), cat)
    assert_close(cat[..., :G], oracle.gate_fwd(xf.double().numpy()), dtype, "pair: full-resolution gate")
    assert_close(cat[..., G:], oracle.bilinear_fwd(oracle.gate_fwd(xh.double().numpy()), out), dtype,
                 "pair: pooled gate")
    assert torch.all(wide[..., :8] == 3)
    g = randn(gen, B, *out, I + 8).to(dtype)
    gs = g.cuda()[..., 8:]
    gxf, gxh = ops.gate_pair_backward(xf.cuda(), xh.cuda(), gs)
    assert_close(gxf, oracle.gate_bwd(xf.double().numpy(), g[..., 8:8 + G].double().numpy()), dtype, "pair: d full")
    assert_close(gxh, oracle.gate_bwd(xh.double().numpy(), oracle.bilinear_bwd(g[..., 8 + G:].double().numpy(), hw)),
                 dtype, "pair: d pooled")
    # the same bits as the single-branch kernels, whatever the ratio of the extents
    assert torch.equal(gxf, ops.gate_backward(xf.cuda(), gs[..., :G]))
    assert torch.equal(gxh, ops.gate_backward(xh.cuda(), ops.bilinear_backward(gs[..., G:], hw)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(3, 7, 9, 20), (32, 56, 56, 128), (2, 57, 61, 200), (1, 1, 1, 4), (5, 33, 2, 3)])
def test_spatial_sum_and_rowbias(dtype, shape):
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(11)
    x = randn(gen, *shape).to(dtype)
    s = ops.spatial_sum(x.cuda())
    ref = x.double().sum(dim=(1, 2)).numpy()
    assert s.dtype == torch.float32
    assert_close(s, ref, torch.float32, "spatial sum", scale=4.0)  # fp32 accumulation of up to 3136 terms
    v = randn(gen, shape[0], shape[3])
    y = x.cuda().clone()
    ops.add_rowbias_(y, v.cuda())
    assert_close(y, x.double().numpy() + v.double().numpy()[:, None, None, :], dtype, "rowbias")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K,NO", [(128, 64), (64, 128), (96, 48), (48, 96), (64, 32), (32, 64), (8, 8), (120, 104), (16, 24)])
@pytest.mark.parametrize("N,P", [(3 * 35, 35), (1, 1), (4 * 3136, 3136), (100, 33), (50, 7), (96, 32)])
def test_dense_layers(dtype, K, NO, N, P):
    """Matrix-core dense kernels against float64: forward in both weight layouts with bias and per-image
    row bias (images that end inside a 32-row tile, images shorter than a tile, a last image cut short), and
    the weight gradient."""
    from pyramidconvblock_amd import ops

    if not (ops.dense_supported(K, NO, dtype) and ops.dense_supported(NO, K, dtype)):
        pytest.skip("shape not covered by the dense kernels in both directions")
    gen = torch.Generator().manual_seed(K * 1000 + NO + N)
    x = randn(gen, N, K).to(dtype)
    w = (randn(gen, NO, K) / K ** 0.5).to(dtype)
    b = randn(gen, NO).to(dtype)
    rb = randn(gen, (N + P - 1) // P, NO)
    ref = x.double() @ w.double().t() + b.double() + rb.double().repeat_interleave(P, 0)[:N]
    y = ops.dense_forward(x.cuda(), w.cuda(), bias=b.cuda(), rowbias=rb.cuda(), rows_per_image=P)
    assert_close(y, ref.numpy(), dtype, "dense fwd")
    g = randn(gen, N, NO).to(dtype)
    dx = ops.dense_forward(g.cuda(), w.cuda(), w_kmajor=True)         # g @ w : [N,NO] x [NO,K]
    assert_close(dx, (g.double() @ w.double()).numpy(), dtype, "dense dgrad")
    dw = ops.dense_wgrad(g.cuda(), x.cuda())                           # g^T @ x : [NO, K]
    assert_close(dw, (g.double().t() @ x.double()).numpy(), dtype, "dense wgrad")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("K,NO", [(200, 100), (100, 200), (128, 64), (64, 128), (256, 132), (4, 4), (36, 52), (12, 256)])
@pytest.mark.parametrize("N,P", [(3 * 35, 35), (1, 1), (3 * 3477, 3477), (100, 33), (50, 7), (96, 32), (130, 64)])
def test_dense_layers_any_width_and_fp32(dtype, K, NO, N, P):
    """The dense entry points on fp32 and on widths the tiled kernels do not take (multiples of 4, wider than 128: the
    ragged block's 200 / 100), against float64: forward in both weight layouts with bias and per-image rows (images
    that end inside a 32-row tile, images shorter than a tile, a last image cut short) and the weight gradient."""
    from pyramidconvblock_amd import ops

    assert ops.dense_supported(K, NO, dtype) and ops.dense_supported(NO, K, dtype)
    gen = torch.Generator().manual_seed(K * 1000 + NO + N)
    x = randn(gen, N, K).to(dtype)
    w = (randn(gen, NO, K) / K ** 0.5).to(dtype)
    b = randn(gen, NO).to(dtype)
    rb = randn(gen, (N + P - 1) // P, NO)
    ref = x.double() @ w.double().t() + b.double() + rb.double().repeat_interleave(P, 0)[:N]
    y = ops.dense_forward(x.cuda(), w.cuda(), bias=b.cuda(), rowbias=rb.cuda(), rows_per_image=P)
    assert_close(y, ref.numpy(), dtype, "dense fwd")
    y0 = ops.dense_forward(x.cuda(), w.cuda())
    assert_close(y0, (x.double() @ w.double().t()).numpy(), dtype, "dense fwd, no bias")
    g = randn(gen, N, NO).to(dtype)
    dx = ops.dense_forward(g.cuda(), w.cuda(), w_kmajor=True)         # g @ w : [N,NO] x [NO,K]
    assert_close(dx, (g.double() @ w.double()).numpy(), dtype, "dense dgrad")
    dw = ops.dense_wgrad(g.cuda(), x.cuda())                           # g^T @ x : [NO, K]
    assert_close(dw, (g.double().t() @ x.double()).numpy(), dtype, "dense wgrad")
    assert not ops.dense_supported(K + 2, NO, dtype) and not ops.dense_supported(260, NO, torch.float32)


def test_dense_fp32_rows_beyond_two_gigabytes():
    """x of more than 2^31 bytes in fp32 (32-bit byte offsets would wrap at row 4 194 304): rows at the start, around
    that row and at the end against float64."""
    from pyramidconvblock_amd import ops

    K, NO, N = 128, 64, 4_300_000
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(N, K, device="cuda", generator=gen)
    w = torch.randn(NO, K, device="cuda", generator=gen) / K ** 0.5
    y = ops.dense_forward(x, w)
    torch.cuda.synchronize()
    for lo in (0, (1 << 31) // (K * 4) - 40, N - 70):
        sl = slice(lo, lo + 70)
        ref = x[sl].double().cpu() @ w.double().cpu().t()
        assert_close(y[sl], ref.numpy(), torch.float32, f"rows from {lo}")
    del x, y


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("K,NO", [(200, 100), (128, 64)])
def test_dense_layers_on_no_rows(dtype, K, NO):
    """An empty batch: the forward returns an empty tensor, the weight gradient zeros."""
    from pyramidconvblock_amd import ops

    x = torch.zeros(0, K, dtype=dtype, device="cuda")
    g = torch.zeros(0, NO, dtype=dtype, device="cuda")
    w = torch.ones(NO, K, dtype=dtype, device="cuda")
    assert tuple(ops.dense_forward(x, w).shape) == (0, NO)
    dw = ops.dense_wgrad(g, x)
    torch.cuda.synchronize()
    assert tuple(dw.shape) == (NO, K) and not dw.any()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 9, 7, 24), (32, 56, 56, 128), (3, 57, 61, 200)])
def test_pool_branch(dtype, shape):
    """Global-mean branch (conv_block.py:46-47) forward and backward against float64."""
    from pyramidconvblock_amd import ops

    B, H, W, D = shape
    gen = torch.Generator().manual_seed(D)
    x = randn(gen, *shape).to(dtype)
    wp = (randn(gen, D, D) / D ** 0.5).to(dtype)
    bp, bo = randn(gen, D).to(dtype), randn(gen, D).to(dtype)
    m, rb = ops.pool_branch_forward(x.cuda(), wp.cuda(), bp.cuda(), bo.cuda())
    m_ref = x.double().mean(dim=(1, 2))
    assert_close(m, m_ref.numpy(), dtype, "mean")
    rb_ref = m.double().cpu() @ wp.double().t() + bp.double() + bo.double()   # from the rounded mean, as computed
    assert_close(rb, rb_ref.numpy(), torch.float32, "rowbias", scale=2.0)
    gy = randn(gen, *shape).to(dtype)
    gbias, gwp, dmean = ops.pool_branch_backward(gy.cuda(), m, wp.cuda())
    gs = gy.double().sum(dim=(1, 2))
    assert_close(gbias[0], gs.sum(0).numpy(), dtype, "bias grad")
    assert torch.equal(gbias[0], gbias[1])
    assert_close(gwp, (gs.t() @ m.double().cpu()).numpy(), dtype, "w_pool grad")
    assert_close(dmean, ((gs @ wp.double()) / (H * W)).numpy(), torch.float32, "dmean", scale=8.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,P,K,NO,kmajor", [(3, 64, 128, 64, False), (2, 96, 64, 128, True), (32, 3136, 128, 64, False),
                                             (1, 32, 128, 8, True), (3, 160, 96, 48, False), (8, 12544, 96, 48, False),
                                             (5, 96, 64, 32, False)])
def test_dense_colsum_feeds_pool_branch(dtype, B, P, K, NO, kmajor):
    """The dense kernel's by-product (sums of x over groups of 32 rows) against a float64 sum, and the mean branch
    computed from it against the one that reads x itself."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(P + K)
    x = randn(gen, B, P, K).to(dtype).cuda()
    w = (randn(gen, K, NO) if kmajor else randn(gen, NO, K)).to(dtype).cuda() / 8
    assert ops.dense_colsum_supported(K, NO, dtype, P)
    y, parts = ops.dense_forward(x, w, w_kmajor=kmajor, colsum=True)
    assert torch.equal(y, ops.dense_forward(x, w, w_kmajor=kmajor))
    R = ops.dense_colsum_rows()
    ref = x.double().view(B * P // R, R, K).sum(1)
    assert (parts.double() - ref).abs().max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
    wp = (randn(gen, K, K) / 11).to(dtype).cuda()
    bp = randn(gen, K).to(dtype).cuda()
    m0, rb0 = ops.pool_branch_forward(x, wp, bp, None)
    m1, rb1 = ops.pool_branch_forward(x, wp, bp, None, parts=parts)
    assert_close(m1, m0.double().cpu().numpy(), dtype, "mean from parts")
    assert (rb1 - rb0).abs().max().item() <= 2e-2 * max(1.0, rb0.abs().max().item())
    g0 = ops.pool_branch_backward(x, m0, wp)
    g1 = ops.pool_branch_backward(x, m0, wp, parts=parts)
    for a, b, what in zip(g1, g0, ("bias grad", "pool weight grad", "mean grad")):
        assert_close(a, b.double().cpu().numpy(), dtype, what + " from parts")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", [(32, 56, 56, 128, 64), (3, 8, 16, 128, 64), (1, 4, 8, 128, 64), (2, 12, 40, 128, 64),
                                  (2, 10, 16, 128, 64), (2, 8, 12, 128, 64), (2, 8, 16, 64, 32), (5, 36, 24, 128, 64),
                                  (8, 112, 112, 96, 48), (1, 4, 8, 96, 48), (3, 12, 40, 96, 48), (2, 8, 12, 96, 48),
                                  (3, 20, 24, 64, 32), (16, 56, 56, 64, 32), (2, 8, 16, 32, 16)])
def test_dense_forward_pool_is_the_layer_then_the_pool(dtype, case):
    """pdw_dense_fwd_colsum_pool: the layer's result bitwise that of pdw_dense_fwd, its 2x2 average pool bitwise that of
    pdw_avgpool_fwd on it, and per-image sums of x from the tile sums (tiles of 4 rows x 8 columns) equal to a float64
    sum; where the kernel does not cover the case (other widths, extents off 4 x 8, fp32) it says so."""
    from pyramidconvblock_amd import ops

    B, H, W, K, NO = case
    gen = torch.Generator().manual_seed(H + W)
    x = randn(gen, B, H, W, K).to(dtype).cuda()
    w = (randn(gen, NO, K) / 8).to(dtype).cuda()
    got = ops.dense_forward_pool(x, w)
    covered = dtype != torch.float32 and (K, NO) in ((128, 64), (96, 48), (64, 32)) and H % 4 == 0 and W % 8 == 0
    assert (got is not None) == covered
    if got is None:
        return
    y, parts, pool = got
    assert torch.equal(y, ops.dense_forward(x, w))
    assert torch.equal(pool, ops.avgpool_forward(y, (H // 2, W // 2)))
    assert parts.shape == (B * H * W // 32, K)
    ref = x.double().view(B, H * W, K).sum(1)
    mine = parts.double().view(B, H * W // 32, K).sum(1)
    assert (mine - ref).abs().max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
    blocks = x.double().view(B, H // 4, 4, W // 8, 8, K).sum((2, 4)).reshape(-1, K)
    assert (parts.double() - blocks).abs().max().item() <= 1e-5 * max(1.0, blocks.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,hw,I,D", [(2, (8, 12), 32, 64), (3, (28, 28), 64, 128), (1, (4, 8), 16, 128)])
def test_block_mid_matches_separate_launches(dtype, B, hw, I, D):
    """Gate pair + mean branch in one launch, forward and backward, against the separate entry points (which
    have their own oracle tests)."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(B + I)
    h, w = hw
    H, W = 2 * h, 2 * w
    P = H * W
    xf = randn(gen, B, H, W, I).to(dtype).cuda()
    xh = randn(gen, B, h, w, I).to(dtype).cuda()
    x = randn(gen, B, P, D).to(dtype).cuda()
    wd = (randn(gen, 64, D) / 8).to(dtype).cuda()
    _, parts = ops.dense_forward(x, wd, colsum=True)
    wp = (randn(gen, D, D) / 11).to(dtype).cuda()
    bp, bo = randn(gen, D).to(dtype).cuda(), randn(gen, D).to(dtype).cuda()
    cat0 = torch.zeros(B, H, W, I, dtype=dtype, device="cuda")
    cat1 = torch.zeros_like(cat0)
    ops.gate_pair_forward(xf, xh, cat0)
    m0, rb0 = ops.pool_branch_forward(x, wp, bp, bo, parts=parts)
    m1, rb1 = ops.block_mid_forward(xf, xh, cat1, parts, P, wp, bp, bo)
    def same(t0, t1):   # two instantiations of the same arithmetic: at most a last-bit difference
        d = (t0.double() - t1.double()).abs().max().item()
        return d <= 2e-3 * max(1.0, t0.double().abs().max().item())

    assert same(cat0, cat1) and torch.equal(m0, m1) and same(rb0, rb1)
    g = randn(gen, B, H, W, I).to(dtype).cuda()
    a0 = ops.gate_pair_backward(xf, xh, g)
    b0 = ops.pool_branch_backward(x, m0, wp, parts=parts)
    r1 = ops.block_mid_backward(xf, xh, g, parts, P, m0, wp)
    for t0, t1 in zip(tuple(a0) + tuple(b0), r1):
        assert same(t0, t1)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [1, 70, 96 * 7, 32 * 56 * 56])
@pytest.mark.parametrize("widths", [(128, 64), (64, 32), (96, 48), (48, 24), (104, 40)])
def test_dense_backward_pair_matches_separate_launches(dtype, N, widths):
    """Input gradient (with column sums) and weight gradient of an I -> O layer from one launch: the same bits
    as the two launches it replaces, and the same with the summation deferred."""
    from pyramidconvblock_amd import _lib, ops

    O, I = widths
    assert ops.dense_backward_pair_supported(O, I, dtype) and not ops.dense_backward_pair_supported(120, 104, dtype)
    gen = torch.Generator().manual_seed(N)
    gy = randn(gen, N, O).to(dtype).cuda()
    x = randn(gen, N, I).to(dtype).cuda()
    w = (randn(gen, O, I) / 8).to(dtype).cuda()
    colsum = N % ops.dense_colsum_rows() == 0 and widths in ((128, 64), (64, 32), (96, 48))   # tile sums: the blocks' shapes only
    if colsum:
        dx0, parts0 = ops.dense_forward(gy, w, w_kmajor=True, colsum=True)
    else:
        dx0, parts0 = ops.dense_forward(gy, w, w_kmajor=True), None
    dw0 = ops.dense_wgrad(gy, x)
    dx1, parts1, dw1 = ops.dense_backward_pair(gy, w, x, colsum=colsum)
    assert torch.equal(dx1, dx0) and torch.equal(dw1, dw0)
    assert (parts1 is None) == (parts0 is None) and (parts0 is None or torch.equal(parts1, parts0))
    assert_close(dw1, (gy.double().t() @ x.double()).cpu().numpy(), dtype, "pair wgrad")
    with _lib.deferred_reductions(gy.device):
        dx2, _, dw2 = ops.dense_backward_pair(gy, w, x, colsum=colsum)
    torch.cuda.synchronize()
    assert torch.equal(dx2, dx0) and torch.equal(dw2, dw0)
    # the other covered shape (128 -> 64 layer), with a per-image term on the input gradient
    if N >= 64:
        P = 32 if N % 32 == 0 else N
        rb = randn(gen, (N + P - 1) // P, O).cuda()
        w2 = (randn(gen, I, O) / 8).to(dtype).cuda()
        assert ops.dense_backward_pair_supported(I, O, dtype, P)
        dxa = ops.dense_forward(x, w2, w_kmajor=True, rowbias=rb, rows_per_image=P)
        dwa = ops.dense_wgrad(x, gy)
        dxb, _, dwb = ops.dense_backward_pair(x, w2, gy, rowbias=rb, rows_per_image=P)
        assert torch.equal(dxb, dxa) and torch.equal(dwb, dwa)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 7), (37, 200, 100), (183, 100, 200), (256, 3, 5), (5, 1)])
def test_sum_parts_is_the_fp32_sum_rounded_once(shape, dtype):
    """pdw_sum_parts (the slab summation of the operator's fallback weight gradient): the sum over the leading
    dimension, against a float64 sum; 16-bit outputs within half an ulp of it plus the fp32 summation error."""
    from pyramidconvblock_amd import ops

    gen = torch.Generator().manual_seed(11)
    parts = torch.randn(*shape, generator=gen, dtype=torch.float32)
    out = ops.sum_parts(parts.cuda(), dtype)
    torch.cuda.synchronize()
    assert out.dtype == dtype and tuple(out.shape) == tuple(shape[1:])
    ref = parts.double().sum(0)
    eps = {torch.float32: 2.0 ** -24, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    tol = eps * ref.abs() + shape[0] * 2.0 ** -24 * parts.abs().double().sum(0) + 1e-7
    assert bool(((out.double().cpu() - ref).abs() <= tol).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_cat", [True, False])
@pytest.mark.parametrize("case", [(32, 56, 56, 64, 128), (1, 4, 8, 64, 128), (3, 8, 16, 64, 128), (2, 12, 40, 64, 128),
                                  (2, 64, 8, 64, 128), (5, 36, 24, 64, 128), (2, 10, 16, 64, 128), (2, 8, 16, 32, 64),
                                  (70, 8, 8, 64, 128), (8, 112, 112, 48, 96), (3, 8, 24, 16, 32), (2, 12, 16, 64, 96),
                                  (2, 8, 8, 32, 128), (2, 8, 8, 48, 56), (2, 8, 8, 96, 128), (2, 8, 8, 24, 48),
                                  (16, 56, 56, 32, 64), (3, 12, 24, 48, 96)])
def test_dense_forward_gated_is_the_gates_then_the_layer(oracle, dtype, with_cat, case):
    """pdw_dense_fwd_gated (the block's output layer on rows it makes from the two convolution outputs: both gates and
    the resize where the tile is staged) gives bitwise what the gate launch followed by the plain layer gives, with
    and without writing the rows out, and the oracle's values; where the kernel does not cover the case (other widths,
    extents off 4 x 8, fp32) it says so and launches nothing."""
    from pyramidconvblock_amd import ops

    B, H, W, I, D = case
    gen = torch.Generator().manual_seed(H * W + B)
    cf = randn(gen, B, H, W, I).to(dtype).cuda()
    ch = randn(gen, B, H // 2, W // 2, I).to(dtype).cuda()
    w = (randn(gen, D, I) / 8).to(dtype).cuda()
    rowbias = randn(gen, B, D).cuda()
    cat = torch.full((B, H, W, I), 5.0, device="cuda", dtype=dtype) if with_cat else None
    y = ops.dense_forward_gated(cf, ch, w, rowbias=rowbias, cat=cat)
    # the inner width a multiple of 16 up to 64, the outer one a multiple of 8 up to 128 and wide enough for the half
    # scale's patch beside a tile's rows (D + 8 >= 1.5 I)
    covered = (dtype != torch.float32 and I % 16 == 0 and I <= 64 and D % 8 == 0 and D <= 128 and 3 * I // 2 <= max(I, D) + 8
               and H % 4 == 0 and W % 8 == 0)
    assert (y is not None) == covered
    from pyramidconvblock_amd import _lib
    assert bool(_lib.lib().pdw_dense_fwd_gated_supported(H, W, I, D, _lib.dtype_code(dtype))) == covered
    if y is None:
        return
    want_cat = torch.empty((B, H, W, I), device="cuda", dtype=dtype)
    ops.gate_pair_forward(cf, ch, want_cat)
    want = ops.dense_forward(want_cat, w, rowbias=rowbias, rows_per_image=H * W)
    torch.cuda.synchronize()
    if with_cat:
        assert torch.equal(cat, want_cat)
    assert torch.equal(y, want)
    if B * H * W <= 4096 or (I, D) == (48, 96):   # and against the oracle, directly
        g0 = oracle.gate_fwd(cf.double().cpu().numpy())
        g1 = oracle.bilinear_fwd(oracle.gate_fwd(ch.double().cpu().numpy()), (H, W))
        rows = torch.cat([torch.from_numpy(g0), torch.from_numpy(g1)], -1)
        yo = rows @ w.double().cpu().t() + rowbias.double().cpu()[:, None, None, :]
        assert_close(y, yo.numpy(), dtype, "y")
    y2 = ops.dense_forward_gated(cf, ch, w)   # no per-image rows
    assert torch.equal(y2, ops.dense_forward(want_cat, w))
    # both scales arriving gated (the inference forward): the full scale compact or as a slice of a wider tensor
    G = I // 2
    g1 = torch.empty((B, H // 2, W // 2, G), device="cuda", dtype=dtype)
    ops.gate_forward(ch, out=g1)
    wide = torch.full((B, H, W, I + 8), 3.0, device="cuda", dtype=dtype)
    wide[..., 8:8 + G] = want_cat[..., :G]
    for g0 in (want_cat[..., :G].contiguous(), wide[..., 8:8 + G]):
        y3 = ops.dense_forward_gated(g0, g1, w, rowbias=rowbias, gated=True)
        assert y3 is not None and torch.equal(y3, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [(32, 56, 56, 64, 13, 128), (2, 40, 36, 32, 9, 64), (64, 56, 56, 64, 11, 128),
                                  (3, 34, 70, 16, 3, 24), (1, 36, 40, 48, 15, 96), (2, 20, 24, 40, 9, 80),
                                  (4, 56, 56, 64, 7, 136)])
@pytest.mark.parametrize("biases", [(True, True), (False, False)])
def test_fwd2_mean_is_the_convolutions_and_the_mean_branch(dtype, case, biases):
    """pdw_dwconv_fwd2_mean (both convolutions and the block's mean branch in one launch) gives bitwise the results of
    pdw_dwconv_fwd2 and pdw_pool_branch_fwd_parts; status 3 where either part is not covered."""
    from pyramidconvblock_amd import ops
    from pyramidconvblock_amd.dwconv import dwconv_forward2, dwconv_forward2_mean

    B, H, W, C, k, D = case
    gen = torch.Generator().manual_seed(B + k)
    x0 = randn(gen, B, H, W, C).to(dtype).cuda()
    x1 = randn(gen, B, H // 2, W // 2, C).to(dtype).cuda()
    w0, w1 = ((randn(gen, k, k, C) / k).to(dtype).cuda() for _ in range(2))
    nparts = 5
    parts = randn(gen, B * nparts, D).cuda()
    wp = (randn(gen, D, D) / 8).to(dtype).cuda()
    bp, bo = ((randn(gen, D).to(dtype).cuda() if b else None) for b in biases)
    got = dwconv_forward2_mean(x0, w0, x1, w1, parts, H * W, wp, bp, bo)
    convs = dwconv_forward2(x0, w0, x1, w1)
    covered = convs is not None and D % 8 == 0 and D <= 128
    assert (got is not None) == covered
    if got is None:
        return
    x = torch.empty(B, H * W, D, device="cuda", dtype=dtype)   # (only its shape is used when parts are given)
    m, rowbias = ops.pool_branch_forward(x, wp, bp, bo, parts=parts)
    torch.cuda.synchronize()
    assert torch.equal(got[0], convs[0]) and torch.equal(got[1], convs[1])
    assert torch.equal(got[2], m) and torch.equal(got[3], rowbias)
    # the same with the gates in the convolutions' stores (the inference forward's launch)
    import ctypes

    from pyramidconvblock_amd import _lib

    L, G = _lib.lib(), C // 2
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ya, yb = (torch.full((B, H, W, G), 7.0, device="cuda", dtype=dtype) for _ in range(2))
    za, zb = (torch.full((B, H // 2, W // 2, G), 7.0, device="cuda", dtype=dtype) for _ in range(2))
    m2, rb2 = torch.zeros_like(m), torch.zeros_like(rowbias)
    rc = L.pdw_dwconv_fwd2_mean(x0.data_ptr(), w0.data_ptr(), ya.data_ptr(), G, 0, x1.data_ptr(), w1.data_ptr(), za.data_ptr(),
                                G, 0, B, H, W, C, k, parts.data_ptr(), nparts, wp.data_ptr(),
                                bp.data_ptr() if bp is not None else None, bo.data_ptr() if bo is not None else None,
                                m2.data_ptr(), rb2.data_ptr(), H * W, D, _lib.dtype_code(dtype), st)
    rg = L.pdw_dwconv_fwd2_gate(x0.data_ptr(), w0.data_ptr(), yb.data_ptr(), G, 0, x1.data_ptr(), w1.data_ptr(), zb.data_ptr(),
                                G, 0, B, H, W, C, k, _lib.dtype_code(dtype), st)
    torch.cuda.synchronize()
    assert rc == rg and rc == (0 if C % 16 == 0 else 3)
    if rc == 0:
        assert torch.equal(ya, yb) and torch.equal(za, zb) and torch.equal(m2, m) and torch.equal(rb2, rowbias)
        assert torch.equal(ya, ops.gate_forward(convs[0])) and torch.equal(za, ops.gate_forward(convs[1]))
