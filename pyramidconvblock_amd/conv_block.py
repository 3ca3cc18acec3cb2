"""``SimpleGate`` and ``ConvBlock`` with the reference's constructor signatures, sub-module
names, parameter shapes and ``[B,H,W,C]`` in/out contract
(pyramid_dwconv/conv_block.py:6-49), running on the gfx950 kernels of libpdw.so.

``state_dict`` keys match the reference: ``conv_up.weight``, ``gates.{i}.conv_spatial.weight``
(``[k,k,inter_dim]``), ``conv_out.{weight,bias}``, ``conv_pool.{weight,bias}``.

``ConvBlock.forward`` runs as ONE autograd node (``ConvBlockFunction``): the pooling, depthwise
convolutions, gates and upsampling go through libpdw.so, the gate outputs are written straight
into the halves of the concatenated buffer (no ``torch.cat``), the pooled branch is added in
place, and the backward reuses one per-image column sum for both bias gradients and the
gradient of the mean.  The dense layers run on the matrix-core kernels of libpdw.so (bias /
broadcast add fused into the store, deterministic split reduction for the weight gradients):
16-bit layers up to 128 wide in the tiled kernels, fp32 and other widths that are multiples of
4 (inner width up to 256) one result tile per wavefront; anything else uses library GEMMs, with
the weight gradients as a batched split-K product.
"""
from __future__ import annotations

import torch
from torch import nn
from torch.nn import functional as F

from . import _lib, ops
from .dwconv import (OptimizedDepthwiseConv2d, dwconv_bwd3, dwconv_dgrad, dwconv_forward, dwconv_forward2,
                     dwconv_forward2_mean,
                     dwconv_wgrad, dwconv_wgrad_pair)


class GateFunction(torch.autograd.Function):
    """y = x[..., :G] * x[..., G:] * sqrt(G), G = I/2   (conv_block.py:10,18-19)."""

    @staticmethod
    def forward(ctx, x):
        x = x.detach().contiguous()
        ctx.save_for_backward(x)
        return ops.gate_forward(x)

    @staticmethod
    def backward(ctx, gy):
        (x,) = ctx.saved_tensors
        return ops.gate_backward(x, gy.contiguous())


class SimpleGate(nn.Module):
    """pool (scale != 1) -> depthwise conv -> gate -> bilinear back to (H, W)   (conv_block.py:6-22).
    ``bias`` is accepted and ignored, as in the reference."""

    def __init__(self, dim: int, kernel_size=13, scale_factor=1., bias=False):
        super().__init__()
        self.scale_factor = scale_factor
        self.scale = (dim / 2) ** -0.5
        self.conv_spatial = OptimizedDepthwiseConv2d(dim, kernel_size=kernel_size, padding=kernel_size // 2)

    def forward(self, x):
        from .avgpool import AdaptiveAvgPool2dFunction
        from .up import BilinearInterp2dFunction

        B, H, W, C = x.shape
        if self.scale_factor != 1.:
            x = AdaptiveAvgPool2dFunction.apply(x, (int(H * self.scale_factor), int(W * self.scale_factor)))
        x = GateFunction.apply(self.conv_spatial(x))
        if self.scale_factor != 1.:
            x = BilinearInterp2dFunction.apply(x, (H, W))
        return x


_BMM_FP32_OUT = [True]

# Test hooks (module attributes, never read from the environment): run the block as one Python-level call per
# launch instead of the library's single call per direction / run conv_up's two gradients as separate launches.
FORCE_STEPWISE = False
NO_UP_PAIR = False


def _weight_grad(g2d: torch.Tensor, x2d: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """g2d[N,O]^T @ x2d[N,I] -> [O,I]: a batched product over S slabs of L = N // S rows (16-bit operands: with
    fp32 accumulation and output), summed in fp32 (the slabs give the library GEMM enough independent tiles; a single
    product over N rows runs on a handful of workgroups), plus the N - S*L left-over rows in fp32.  Without left-over
    rows the slabs are summed by the library's own fixed-order summation (ops.sum_parts), straight into `out_dtype`;
    otherwise the result is fp32."""
    N = g2d.shape[0]
    if N == 0:
        return g2d.new_zeros((g2d.shape[1], x2d.shape[1]), dtype=torch.float32)
    # slabs: a divisor of N (no left-over rows) if one gives 32..256 slabs of at least 48 rows, else a power of two
    S = max((d for d in range(32, 257) if N % d == 0 and N // d >= 48), default=0)
    if S == 0:
        S = 1
        while S < 256 and N // (2 * S) >= 128:
            S *= 2
    L = N // S
    a = g2d[:S * L].view(S, L, -1).transpose(1, 2)
    b = x2d[:S * L].view(S, L, -1)
    out = None
    parts = None
    if g2d.dtype == torch.float32:
        parts = torch.bmm(a, b)
    elif _BMM_FP32_OUT[0]:
        try:
            parts = torch.bmm(a, b, out_dtype=torch.float32)
        except (TypeError, RuntimeError):
            _BMM_FP32_OUT[0] = False
    if parts is not None:
        if S * L == N and g2d.is_cuda:
            return ops.sum_parts(parts, out_dtype)
        out = parts.sum(0)
    if out is None:
        out = torch.bmm(a, b).float().sum(0) if S > 1 else a[0].float() @ b[0].float()
    if S * L < N:
        out = out + g2d[S * L:].float().t() @ x2d[S * L:].float()
    return out


def _block_call_ok(x, scales, w_up, b_up, w_out, b_out, w_pool, b_pool, w_dw) -> bool:
    """Whether pdw_convblock_fwd / _bwd cover this call: scales (1, 1/2), no conv_up bias, everything contiguous and
    of x's 16-bit dtype, one odd square depthwise filter shape, and shapes the library accepts."""
    if FORCE_STEPWISE or b_up is not None or tuple(scales) != (1., 0.5) or x.dim() != 4:
        return False
    dt = x.dtype
    tensors = [w_up, w_out, w_pool, *w_dw] + [b for b in (b_out, b_pool) if b is not None]
    if len(w_dw) != 2 or any(t.dtype != dt or not t.is_contiguous() or t.device != x.device for t in tensors):
        return False
    B, H, W, D = x.shape
    I, K = w_up.shape[0], w_dw[0].shape[0]
    if (dt not in (torch.float16, torch.bfloat16) or tuple(w_up.shape) != (I, D) or tuple(w_out.shape) != (D, I)
            or tuple(w_pool.shape) != (D, D) or any(tuple(w.shape) != (K, K, I) for w in w_dw)):
        return False
    return bool(_lib.lib().pdw_convblock_supported(B, H, W, D, I, K, _lib.dtype_code(dt)))


def convblock_infer(x, w_up, w_out, b_out, w_pool, b_pool, w_dw):
    """Inference forward through pdw_convblock_infer: y only, neither convolution output written to HBM where the
    fused convolution + gate covers the filter (conv_block.py:36-49 under no_grad).  The caller has checked
    ``_block_call_ok``."""
    dev = _lib.require_device(x)
    B, H, W, D = x.shape
    I, K = w_up.shape[0], w_dw[0].shape[0]
    L, code = _lib.lib(), _lib.dtype_code(x.dtype)
    y = torch.empty((B, H, W, D), device=dev, dtype=x.dtype)
    ws = torch.empty(L.pdw_convblock_infer_workspace_bytes(B, H, W, D, I, K, code) // 4 + 1, device=dev,
                     dtype=torch.float32)
    _lib.check(L.pdw_convblock_infer(x.data_ptr(), w_up.data_ptr(), w_dw[0].data_ptr(), w_dw[1].data_ptr(),
                                     w_pool.data_ptr(), b_pool.data_ptr() if b_pool is not None else None,
                                     w_out.data_ptr(), b_out.data_ptr() if b_out is not None else None, y.data_ptr(),
                                     ws.data_ptr(), ws.numel() * 4, B, H, W, D, I, K, code, _lib.stream_ptr(dev)),
               "pdw_convblock_infer")
    return y


def _is_pair(scales) -> bool:
    return len(scales) == 2 and scales[0] == 1. and scales[1] != 1.


class ConvBlockFunction(torch.autograd.Function):
    """The whole block of conv_block.py:36-49 as one differentiable op.

    apply(x, scales, kernel_sizes, w_up, b_up, w_out, b_out, w_pool, b_pool, *dw_weights)"""

    @staticmethod
    def forward(ctx, x, scales, w_up, b_up, w_out, b_out, w_pool, b_pool, *w_dw):
        with _lib.launch_scope(_lib.require_device(x)):  # one device and stream look-up for all launches
            return ConvBlockFunction._forward(ctx, x, scales, w_up, b_up, w_out, b_out, w_pool, b_pool, *w_dw)

    @staticmethod
    def backward(ctx, gy):
        with _lib.launch_scope(_lib.require_device(gy)):
            return ConvBlockFunction._backward(ctx, gy)

    @staticmethod
    def _forward(ctx, x, scales, w_up, b_up, w_out, b_out, w_pool, b_pool, *w_dw):
        dev = _lib.require_device(x)
        x = x.detach().contiguous()
        B, H, W, D = x.shape
        dt = x.dtype
        I = w_up.shape[0]
        ctx.block_call = None
        if _block_call_ok(x, scales, w_up, b_up, w_out, b_out, w_pool, b_pool, w_dw):
            # the whole launch sequence below as one call of the library (same kernels, same order, same results)
            K = w_dw[0].shape[0]
            L, code = _lib.lib(), _lib.dtype_code(dt)
            new = lambda *shape: torch.empty(shape, device=dev, dtype=dt)
            a, c0, cat = new(B, H, W, I), new(B, H, W, I), new(B, H, W, I)
            xp, c1 = new(B, H // 2, W // 2, I), new(B, H // 2, W // 2, I)
            m, y = new(B, D), new(B, H, W, D)
            ws = torch.empty(L.pdw_convblock_fwd_workspace_bytes(B, H, W, D, I, K, code) // 4 + 1, device=dev,
                             dtype=torch.float32)
            _lib.check(L.pdw_convblock_fwd(x.data_ptr(), w_up.data_ptr(), w_dw[0].data_ptr(), w_dw[1].data_ptr(),
                                           w_pool.data_ptr(), b_pool.data_ptr() if b_pool is not None else None,
                                           w_out.data_ptr(), b_out.data_ptr() if b_out is not None else None,
                                           a.data_ptr(), c0.data_ptr(), xp.data_ptr(), c1.data_ptr(), cat.data_ptr(),
                                           m.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel() * 4, B, H, W, D, I, K,
                                           code, _lib.stream_ptr(dev)), "pdw_convblock_fwd")
            ctx.block_call = (B, H, W, D, I, K, code)
            ctx.fast = (True, True)
            ctx.scales = tuple(scales)
            ctx.has_bias = (False, b_out is not None, b_pool is not None)
            ctx.save_for_backward(x, a, cat, m, w_up, w_out, w_pool, *w_dw, c0, c1, xp)
            return y
        fast_up = (ops.dense_supported(D, I, dt) and ops.dense_supported(I, D, dt) and w_up.dtype == dt
                   and (b_up is None or b_up.dtype == dt))
        same_dt = w_pool.dtype == dt and all(b is None or b.dtype == dt for b in (b_pool, b_out))
        # the per-image sums of x that the mean branch needs are taken by conv_up's kernel while it reads x
        xparts = None
        xp_ready = None   # the second scale's input, where conv_up's kernel pools its own result
        two = (_is_pair(scales) and B > 0 and scales[1] == 0.5 and H % 2 == 0 and W % 2 == 0 and len(w_dw) == 2
               and w_dw[0].shape == w_dw[1].shape and w_dw[0].shape[0] == w_dw[0].shape[1] and x.is_cuda
               and dt != torch.float32
               and bool(_lib.lib().pdw_dwconv_fwd2_supported(B, H, W, I, w_dw[0].shape[0], _lib.dtype_code(dt))))
        fused_up = ops.dense_forward_pool(x, w_up.detach().contiguous(), bias=b_up) if (
            two and fast_up and same_dt and b_up is None) else None
        if fused_up is not None:
            a, xparts, xp_ready = fused_up
        elif fast_up and same_dt and B > 0 and ops.dense_colsum_supported(D, I, dt, H * W):
            a, xparts = ops.dense_forward(x, w_up.detach().contiguous(), bias=b_up, colsum=True)
        else:
            a = ops.dense_forward(x, w_up.detach().contiguous(), bias=b_up) if fast_up else F.linear(x, w_up, b_up)
        G = I // 2
        ns = len(scales)
        cat = torch.empty((B, H, W, G * ns), device=dev, dtype=dt)
        convs, pooled = [], []
        pair = _is_pair(scales)           # scales (1, s): both gates go into cat in one launch
        ready = None                      # pooled input already produced by the full-resolution conv's kernel
        both = None
        mean_done = None                  # (m, yp) where the mean branch ran in the convolutions' launch
        if two:
            # the launches of pdw_convblock_fwd: the second scale's input, then both convolutions as one launch
            ws = [w.detach().to(dt).contiguous() for w in w_dw]
            xp = xp_ready if xp_ready is not None else ops.avgpool_forward(a, (H // 2, W // 2))
            # where conv_up left the tile sums of x, the mean branch rides in the convolutions' launch
            if xparts is not None and same_dt:
                both = dwconv_forward2_mean(a, ws[0], xp, ws[1], xparts, H * W, w_pool.detach().contiguous(), b_pool,
                                            b_out)
                if both is not None:
                    mean_done, both = both[2:], both[:2]
            if both is None:
                both = dwconv_forward2(a, ws[0], xp, ws[1])
            if both is not None:
                convs, pooled = [both[0], both[1]], [None, xp]
            else:
                ready = xp
        for i, s in enumerate(scales if both is None else ()):
            w = w_dw[i].detach().to(dt).contiguous()
            k1, k2 = w.shape[0], w.shape[1]
            geo = ((1, 1), (k1 // 2, k2 // 2), (1, 1))
            dst = cat[..., i * G:(i + 1) * G]
            if s != 1.:
                hw = (int(H * s), int(W * s))
                p = ready if ready is not None and tuple(ready.shape[1:3]) == hw else ops.avgpool_forward(a, hw)
                c = dwconv_forward(p, w, *geo)
                if not pair:
                    ops.gate_bilinear_forward(c, (H, W), out=dst)
            else:
                p = None
                if pair and B > 0 and ready is None:   # the conv reads `a` anyway: it also writes the next scale's pooled input
                    c, ready = dwconv_forward(a, w, *geo, pool_to=(int(H * scales[1]), int(W * scales[1])))
                else:
                    c = dwconv_forward(a, w, *geo)
                if not pair:
                    ops.gate_forward(c, out=dst)
            convs.append(c)
            pooled.append(p)
        y = None
        if mean_done is not None:
            # the mean branch is done: conv_out makes its rows (both gates, the resize) where it multiplies them and
            # writes them to cat for the backward pass; where that kernel does not cover the widths, the gates' launch
            m, yp = mean_done
            if w_out.dtype == dt:
                y = ops.dense_forward_gated(convs[0], convs[1], w_out.detach().contiguous(), rowbias=yp, cat=cat)
            if y is None:
                ops.gate_pair_forward(convs[0], convs[1], cat)
        elif pair and xparts is not None:
            # both gates and the mean branch (mean -> conv_pool, plus conv_out's bias: one fp32 row per image) in
            # one launch
            m, yp = ops.block_mid_forward(convs[0], convs[1], cat, xparts, H * W, w_pool.detach().contiguous(),
                                          b_pool, b_out)
        elif pair:
            ops.gate_pair_forward(convs[0], convs[1], cat)
        if mean_done is not None or (pair and xparts is not None):
            pass
        elif same_dt and B > 0:
            # mean over positions -> conv_pool, plus conv_out's bias: one fp32 row per image
            m, yp = ops.pool_branch_forward(x, w_pool.detach().contiguous(), b_pool, b_out, parts=xparts)
        else:
            m = (ops.spatial_sum(x) / float(H * W)).to(dt)
            yp = F.linear(m, w_pool, b_pool).float()
            if b_out is not None:
                yp = yp + b_out.float()
            yp = yp.contiguous()
        fast_out = ops.dense_supported(G * ns, D, dt) and ops.dense_supported(D, G * ns, dt) and w_out.dtype == dt
        if y is not None:
            pass
        elif fast_out:
            y = ops.dense_forward(cat, w_out.detach().contiguous(), rowbias=yp, rows_per_image=H * W)
        else:
            y = ops.add_rowbias_(F.linear(cat, w_out), yp)
        ctx.fast = (fast_up, fast_out)
        ctx.scales = tuple(scales)
        ctx.has_bias = (b_up is not None, b_out is not None, b_pool is not None)
        ctx.save_for_backward(x, a, cat, m, w_up, w_out, w_pool, *w_dw, *convs, *[p for p in pooled if p is not None])
        return y

    @staticmethod
    def _backward(ctx, gy):
        scales = ctx.scales
        ns = len(scales)
        saved = ctx.saved_tensors
        x, a, cat, m, w_up, w_out, w_pool = saved[:7]
        w_dw = saved[7:7 + ns]
        convs = saved[7 + ns:7 + 2 * ns]
        pooled_it = iter(saved[7 + 2 * ns:])
        pooled = [next(pooled_it) if s != 1. else None for s in scales]
        B, H, W, D = x.shape
        dt = x.dtype
        I = a.shape[-1]
        G = I // 2
        N = B * H * W
        gy = gy.to(dt).contiguous()
        g2d = gy.view(N, D)
        if ctx.block_call is not None:
            dev = gy.device
            L = _lib.lib()
            shape = ctx.block_call
            like = lambda t: torch.empty_like(t, memory_format=torch.contiguous_format)
            dx, gw_up, gw_out, gw_pool = like(x), like(w_up), like(w_out), like(w_pool)
            gw_dw = [like(w_dw[0]), like(w_dw[1])]
            gb_out = torch.empty(D, device=dev, dtype=dt) if ctx.has_bias[1] else None
            gb_pool = torch.empty(D, device=dev, dtype=dt) if ctx.has_bias[2] else None
            ws = torch.empty(L.pdw_convblock_bwd_workspace_bytes(*shape) // 4 + 1, device=dev, dtype=torch.float32)
            _lib.check(L.pdw_convblock_bwd(gy.data_ptr(), x.data_ptr(), a.data_ptr(), convs[0].data_ptr(),
                                           pooled[1].data_ptr(), convs[1].data_ptr(), cat.data_ptr(), m.data_ptr(),
                                           w_up.data_ptr(), w_dw[0].data_ptr(), w_dw[1].data_ptr(), w_pool.data_ptr(),
                                           w_out.data_ptr(), dx.data_ptr(), gw_up.data_ptr(), gw_dw[0].data_ptr(),
                                           gw_dw[1].data_ptr(), gw_pool.data_ptr(),
                                           gb_pool.data_ptr() if gb_pool is not None else None, gw_out.data_ptr(),
                                           gb_out.data_ptr() if gb_out is not None else None, ws.data_ptr(),
                                           ws.numel() * 4, *shape, _lib.stream_ptr(dev)), "pdw_convblock_bwd")
            return (dx, None, gw_up, None, gw_out, gb_out, gw_pool, gb_pool, *gw_dw)

        fast_up, fast_out = ctx.fast
        pool_fast = w_pool.dtype == dt and B > 0
        # the four weight gradients end in a small summation kernel each: they are run as one launch at the end
        with _lib.deferred_reductions(gy.device):
            gparts = None
            want = pool_fast and ops.dense_colsum_supported(D, G * ns, dt, H * W)
            pair_out = fast_out and N > 0 and cat.dtype == dt
            if pair_out and want and not ops.dense_backward_pair_supported(D, G * ns, dt, colsum=True):
                want = False   # the pair without the tile sums (the mean branch then sums gy itself) beats two launches
            if pair_out and ops.dense_backward_pair_supported(D, G * ns, dt, colsum=bool(want)):
                # both products that read gy share one launch
                dcat, gparts, grad_w_out = ops.dense_backward_pair(gy, w_out.detach().contiguous(),
                                                                   cat.contiguous(), colsum=want)
            elif fast_out:
                if pool_fast and ops.dense_colsum_supported(D, G * ns, dt, H * W):
                    # the per-image sums of gy for the mean branch come out of the kernel that reads gy anyway
                    dcat, gparts = ops.dense_forward(gy, w_out.detach().contiguous(), w_kmajor=True, colsum=True)
                else:
                    dcat = ops.dense_forward(gy, w_out.detach().contiguous(), w_kmajor=True)
                grad_w_out = ops.dense_wgrad(gy, cat)
            else:
                dcat = torch.matmul(g2d, w_out).view(B, H, W, G * ns)
                grad_w_out = _weight_grad(g2d, cat.view(N, G * ns), w_out.dtype)

            gcs = None
            if (pool_fast and gparts is not None and _is_pair(scales) and H == 2 * convs[1].shape[1]
                    and W == 2 * convs[1].shape[2] and convs[1].shape[1] >= 2 and convs[1].shape[2] >= 2):
                # the gradients of both gates and the mean branch's backward in one launch
                gcf, gch, gbias, grad_w_pool, dmean = ops.block_mid_backward(convs[0], convs[1], dcat, gparts, H * W, m,
                                                                             w_pool.detach().contiguous())
                gcs = (gcf, gch)
            elif pool_fast:
                gbias, grad_w_pool, dmean = ops.pool_branch_backward(gy, m, w_pool.detach().contiguous(), parts=gparts)
            else:
                gs = ops.spatial_sum(gy)                             # [B, D] fp32: column sums per image
                gbias = gs.sum(0).unsqueeze(0).repeat(2, 1)
                grad_w_pool = (gs.t() @ m.float()).to(w_pool.dtype)
                dmean = ((gs @ w_pool.float()) / float(H * W)).contiguous()   # gradient of the per-image mean
            grad_b_out = gbias[0].to(w_out.dtype) if ctx.has_bias[1] else None    # a tensor of its own for each
            grad_b_pool = gbias[1].to(w_pool.dtype) if ctx.has_bias[2] else None  # bias: autograd copies a shared one

            da = None
            grad_w_dw = [None] * ns
            # pooled branches first: the gradient of one of them is added inside the input-gradient kernel of the
            # first full-resolution branch, the others are accumulated into its result
            order = sorted(range(ns), key=lambda i: scales[i] == 1.)
            waiting = []                                               # pooled gradients not yet added to da
            if gcs is None and _is_pair(scales):
                gcs = ops.gate_pair_backward(convs[0], convs[1], dcat)
            srcs = [pooled[i] if scales[i] != 1. else a for i in range(ns)]
            if (gcs is not None and ns == 2 and w_dw[0].shape == w_dw[1].shape and w_dw[0].shape[0] == w_dw[0].shape[1]
                    and w_dw[0].shape[0] % 2 == 1 and all(t.is_contiguous() and t.dtype == dt for t in (*srcs, *gcs))):
                k = w_dw[0].shape[0]
                fused = None
                if tuple(srcs[1].shape) == (B, H // 2, W // 2, I) and H % 2 == 0 and W % 2 == 0 and scales[0] == 1.:
                    # the launches of pdw_convblock_bwd: the half scale's input gradient, then the full scale's (which
                    # adds it) and both weight gradients as one launch
                    geo = ((1, 1), (k // 2, k // 2), (1, 1))
                    ws = [w.detach().to(dt).contiguous() for w in w_dw]
                    dxp = dwconv_dgrad(gcs[1], ws[1], srcs[1].shape, *geo)
                    fused = dwconv_bwd3(gcs[0], ws[0], dxp, srcs[0], srcs[1], gcs[1])
                    if fused is None:
                        waiting.append(dxp)
                        order = [i for i in order if i != 1]
                if fused is not None:
                    da, grad_w_dw[0], grad_w_dw[1] = fused
                    order = []
                else:
                    # the weight gradients of both scales in one launch (the smaller problem fills the larger one's tail)
                    grad_w_dw[0], grad_w_dw[1] = dwconv_wgrad_pair(srcs[0], gcs[0], srcs[1], gcs[1], w_dw[0].shape)
            for i in order:
                s = scales[i]
                w = w_dw[i].detach().to(dt).contiguous()
                k1, k2 = w.shape[0], w.shape[1]
                geo = ((1, 1), (k1 // 2, k2 // 2), (1, 1))
                dslice = dcat[..., i * G:(i + 1) * G]
                c = convs[i]
                src = pooled[i] if s != 1. else a
                if gcs is not None:
                    gc = gcs[i]
                elif s != 1.:
                    gc = ops.bilinear_gate_backward(c, dslice)
                else:
                    gc = ops.gate_backward(c, dslice)
                if grad_w_dw[i] is None:
                    grad_w_dw[i] = dwconv_wgrad(src, gc, w.shape, *geo)
                if s != 1.:
                    waiting.append(dwconv_dgrad(gc, w, src.shape, *geo))
                elif da is None:
                    da = dwconv_dgrad(gc, w, src.shape, *geo, pooled_grad=waiting.pop() if waiting else None)
                else:
                    da.add_(dwconv_dgrad(gc, w, src.shape, *geo))
            for dp in waiting:
                if da is None:
                    da = ops.avgpool_backward(dp, (H, W))
                else:
                    ops.avgpool_backward(dp, (H, W), out=da, accumulate=True)
            a2d = da.view(N, I)
            grad_b_up = a2d.float().sum(0).to(w_up.dtype) if ctx.has_bias[0] else None
            dx = None
            if (fast_up and ctx.needs_input_grad[0] and N > 0 and x.dtype == dt and dmean is not None
                    and ops.dense_backward_pair_supported(I, D, dt, H * W) and not NO_UP_PAIR):
                # both products that read da share the pass's last large launch; the summations recorded on the
                # way run as one small launch when the block of deferred work closes
                dx, _, grad_w_up = ops.dense_backward_pair(da, w_up.detach().contiguous(), x.contiguous(),
                                                           rowbias=dmean, rows_per_image=H * W)
            elif fast_up:
                grad_w_up = ops.dense_wgrad(da, x)
                if ctx.needs_input_grad[0]:
                    # the last kernel of the pass: the recorded summations ride in its grid
                    dx = ops.dense_forward(da, w_up.detach().contiguous(), w_kmajor=True, rowbias=dmean,
                                           rows_per_image=H * W, flush_reductions=True)
            else:
                grad_w_up = _weight_grad(a2d, x.view(N, D), w_up.dtype)
                if ctx.needs_input_grad[0]:
                    dx = ops.add_rowbias_(torch.matmul(a2d, w_up).view(B, H, W, D), dmean)
        grad_w_out = grad_w_out.to(w_out.dtype)
        grad_w_up = grad_w_up.to(w_up.dtype)
        grad_w_dw = [g.to(w_dw[i].dtype) for i, g in enumerate(grad_w_dw)]
        return (dx, None, grad_w_up, grad_b_up, grad_w_out, grad_b_out, grad_w_pool, grad_b_pool, *grad_w_dw)


class ConvBlock(nn.Module):
    """Linear(dim -> inter) -> gates at each scale -> cat -> Linear(-> dim), plus a global-mean
    branch Linear(dim -> dim) added over all positions   (conv_block.py:25-49)."""

    def __init__(self, dim: int, bias=False, out_bias=True, kernel_size=9, scales=(1., 1 / 2), inter_ratio=0.5):
        super().__init__()
        inter_dim = int(dim * inter_ratio)
        self.conv_up = nn.Linear(dim, inter_dim, bias=bias)
        self.gates = nn.ModuleList([SimpleGate(inter_dim, kernel_size=kernel_size, scale_factor=scale, bias=bias)
                                    for scale in scales])
        self.conv_out = nn.Linear(inter_dim // 2 * len(scales), dim, bias=out_bias)
        self.conv_pool = nn.Linear(dim, dim, bias=out_bias)

    def forward(self, x):
        _lib.require_device(x)
        if x.dim() != 4 or x.shape[3] != self.conv_up.in_features:
            raise ValueError(f"expected [B,H,W,{self.conv_up.in_features}] input, got {tuple(x.shape)}")
        scales = tuple(float(g.scale_factor) for g in self.gates)
        if not (torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))):
            # nothing to save for a backward: the inference form of the block, where the library covers the shape
            xc = x.detach().contiguous()
            args = (self.conv_up.weight.detach(), self.conv_up.bias, self.conv_out.weight.detach(),
                    None if self.conv_out.bias is None else self.conv_out.bias.detach(), self.conv_pool.weight.detach(),
                    None if self.conv_pool.bias is None else self.conv_pool.bias.detach(),
                    [g.conv_spatial.weight.detach() for g in self.gates])
            if _block_call_ok(xc, scales, *args):
                with _lib.launch_scope(_lib.require_device(xc)):
                    return convblock_infer(xc, args[0], args[2], args[3], args[4], args[5], args[6])
        return ConvBlockFunction.apply(x, scales, self.conv_up.weight, self.conv_up.bias, self.conv_out.weight,
                                       self.conv_out.bias, self.conv_pool.weight, self.conv_pool.bias,
                                       *[g.conv_spatial.weight for g in self.gates])
