"""Parity of the full ConvBlock (forward, dx and every parameter gradient) with the float64
block oracle at the BASELINE configurations."""
import pytest
import torch

from parity import assert_close, randn

pytestmark = pytest.mark.gpu


def _block_case(oracle, dim, k, shape, dtype, dist="normal", seed=0, scale=1.0):
    import pyramid_dwconv

    torch.manual_seed(seed)  # module first, then x, then grad (the order the configs state)
    m = pyramid_dwconv.ConvBlock(dim=dim, kernel_size=k)
    gen = torch.Generator().manual_seed(seed)
    x = randn(gen, *shape) if dist == "normal" else torch.rand(*shape, generator=gen) * 4 - 2
    g = randn(gen, *shape)
    m = m.to(dtype)
    params = {n: p.detach().double().numpy() for n, p in m.state_dict().items()}
    xr, gr = x.to(dtype), g.to(dtype)
    yo, cache = oracle.convblock_fwd(xr.double().numpy(), params)
    dxo, go = oracle.convblock_bwd(cache, gr.double().numpy())
    m = m.cuda()
    xd = xr.cuda().requires_grad_()
    y = m(xd)
    assert y.dtype == dtype and y.shape == xd.shape
    errs = {"y": assert_close(y, yo, dtype, "y", scale)}
    torch.autograd.backward(y, gr.cuda())
    errs["dx"] = assert_close(xd.grad, dxo, dtype, "dx", scale)
    for n, p in m.named_parameters():
        errs[n] = assert_close(p.grad, go[n], dtype, "grad " + n, scale)
    return errs


def test_config1_fp32(oracle):
    _block_case(oracle, 64, 7, (2, 32, 32, 64), torch.float32)


def test_config3_bf16(oracle):
    _block_case(oracle, 128, 13, (32, 56, 56, 128), torch.bfloat16)


@pytest.mark.parametrize("k", [9, 17])
def test_metric_sweep_bf16(oracle, k):
    _block_case(oracle, 128, k, (8, 56, 56, 128), torch.bfloat16)


@pytest.mark.parametrize("k", [9, 17])
def test_metric_sweep_bf16_full_batch(oracle, k):
    """The k = 9 / 17 rows of the metric at the shape they are timed on (the shared conv launches choose their band
    heights and grid order from the shape)."""
    _block_case(oracle, 128, k, (32, 56, 56, 128), torch.bfloat16)


def test_batch_sweep_b64_bf16(oracle):
    """A larger batch than the headline's: the launch plans with more whole-image bands than compute units."""
    _block_case(oracle, 128, 13, (64, 56, 56, 128), torch.bfloat16)


def test_config4_fp16(oracle):
    _block_case(oracle, 96, 17, (8, 112, 112, 96), torch.float16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [9, 15])
def test_config5_ragged(oracle, dtype, k):
    _block_case(oracle, 200, k, (3, 57, 61, 200), dtype, dist="uniform")


@pytest.mark.parametrize("case", [
    (128, 13, (1, 8, 8, 128), torch.bfloat16),     # one image, a few rows per dense launch
    (128, 9, (3, 10, 14, 128), torch.float16),     # extents not multiples of 4
    (128, 3, (2, 4, 6, 128), torch.bfloat16),      # pooled map of 2 x 3
    (128, 13, (2, 58, 62, 128), torch.bfloat16),   # wider than a conv tile
    (64, 7, (5, 12, 12, 64), torch.bfloat16),      # layer widths without the paired dense launch
    (256, 5, (2, 8, 8, 256), torch.bfloat16),      # layer widths the dense kernels leave to the BLAS library
    (128, 11, (2, 16, 16, 128), torch.float32),
    (64, 7, (3, 8, 16, 64), torch.float16),        # narrow block through the single library call per direction
    (128, 17, (2, 24, 32, 128), torch.float16),
    (32, 7, (3, 8, 8, 32), torch.bfloat16),        # widths 32/16, 96/48, 112/... through the generic-extent dense pair
    (96, 9, (2, 16, 16, 96), torch.float16),
    (96, 13, (4, 28, 32, 96), torch.bfloat16),
    (112, 5, (2, 8, 12, 112), torch.bfloat16),     # inner width 56: not a multiple of 16, the launches one by one
])
def test_small_and_odd_even_extents(oracle, case):
    """Even extents take the fused two-scale path (paired launches, deferred summations); small and unusual
    sizes exercise its tails, partial tiles and fallbacks."""
    dim, k, shape, dtype = case
    _block_case(oracle, dim, k, shape, dtype)


@pytest.mark.parametrize("bias", [(True, True), (True, False), (False, False)])
def test_bias_combinations(oracle, bias):
    import pyramid_dwconv

    torch.manual_seed(3)
    dtype = torch.bfloat16
    m = pyramid_dwconv.ConvBlock(dim=128, bias=bias[0], out_bias=bias[1], kernel_size=9)
    with torch.no_grad():
        for n, p in m.named_parameters():
            if n.endswith("bias"):
                p.normal_(0, 0.5)   # the default initialisation leaves some of them at zero
    gen = torch.Generator().manual_seed(3)
    shape = (3, 12, 16, 128)
    x, g = randn(gen, *shape).to(dtype), randn(gen, *shape).to(dtype)
    m = m.to(dtype)
    params = {n: p.detach().double().numpy() for n, p in m.state_dict().items()}
    yo, cache = oracle.convblock_fwd(x.double().numpy(), params)
    dxo, go = oracle.convblock_bwd(cache, g.double().numpy())
    m = m.cuda()
    xd = x.cuda().requires_grad_()
    y = m(xd)
    assert_close(y, yo, dtype, "y")
    torch.autograd.backward(y, g.cuda())
    assert_close(xd.grad, dxo, dtype, "dx")
    for n, p in m.named_parameters():
        assert p.grad is not None, n
        assert_close(p.grad, go[n], dtype, "grad " + n)


@pytest.mark.parametrize("case", [(128, 13, (4, 56, 56, 128), torch.bfloat16), (128, 9, (3, 8, 16, 128), torch.float16),
                                  (128, 3, (1, 4, 8, 128), torch.bfloat16), (64, 7, (5, 12, 16, 64), torch.bfloat16)])
@pytest.mark.parametrize("out_bias", [True, False])
def test_single_call_block_is_the_stepwise_block(case, out_bias, monkeypatch):
    """pdw_convblock_fwd / _bwd (the block's launch sequence as one library call each way) give bitwise the results
    of the operator making the same launches one by one."""
    import pyramid_dwconv
    from pyramidconvblock_amd import _lib

    dim, k, shape, dtype = case
    B, H, W, D = shape
    assert _lib.lib().pdw_convblock_supported(B, H, W, D, D // 2, k, _lib.dtype_code(dtype)) == 1
    torch.manual_seed(5)
    m = pyramid_dwconv.ConvBlock(dim=dim, kernel_size=k, out_bias=out_bias).to(dtype).cuda()
    gen = torch.Generator().manual_seed(5)
    x = randn(gen, *shape).to(dtype).cuda()
    g = randn(gen, *shape).to(dtype).cuda()

    def run():
        for p in m.parameters():
            p.grad = None
        xi = x.clone().requires_grad_()
        y = m(xi)
        torch.autograd.backward(y, g)
        torch.cuda.synchronize()
        return [y.detach(), xi.grad] + [p.grad for p in m.parameters()]

    single = run()
    from pyramidconvblock_amd import conv_block
    monkeypatch.setattr(conv_block, "FORCE_STEPWISE", True)
    stepwise = run()
    assert len(single) == len(stepwise)
    for i, (s, t) in enumerate(zip(single, stepwise)):
        assert s is not None and torch.equal(s, t), f"result {i} differs"


@pytest.mark.parametrize("seed", range(24))
def test_random_two_scale_blocks(oracle, seed):
    """Seeded random blocks over the widths, extents and filter sizes of the fused forward (conv_up with or without its
    pooling variant, the convolutions with the mean branch in their launch, conv_out on rows it makes itself with the
    extents as constants or as arguments) and its fallbacks (extents off the 4 x 8 tiles, inner widths beyond 64)."""
    import random

    rng = random.Random(1000 + seed)
    dim = rng.choice([32, 64, 96, 128, 128, 160, 192])
    k = rng.choice([3, 5, 7, 9, 11, 13, 15, 17])
    B = rng.choice([1, 2, 3, 5, 9])
    H = rng.choice([4, 8, 12, 16, 20, 28, 6, 10])
    W = rng.choice([8, 16, 24, 40, 56, 12, 36])
    dtype = rng.choice([torch.float16, torch.bfloat16])
    _block_case(oracle, dim, k, (B, H, W, dim), dtype, seed=seed)
