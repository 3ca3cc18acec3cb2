"""Depthwise conv2d on channels-last tensors, backed by libpdw.so.

Mirrors the reference operator API: ``DepthwiseConv2DFunction``
(pyramid_dwconv/dwconv_triton.py:299-387) and ``OptimizedDepthwiseConv2d``
(pyramid_dwconv/dwconv_triton.py:389-426).  Same call signatures, parameter name, weight
layout ``[k1,k2,C]`` and default initialisation.  Differences, all in the direction of
correctness: inputs are made contiguous and moved to the weight dtype, arguments are
checked, the backward is the exact adjoint for every stride/padding/dilation, and the
weight gradient is accumulated in fp32 without atomics (bit-reproducible).
"""
from __future__ import annotations

import torch

from . import _lib


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def _conv_args(x_shape, w_shape, stride, padding, dilation):
    B, H, W, C = x_shape
    KH, KW = w_shape[0], w_shape[1]
    return (B, H, W, C, KH, KW, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1])


def dwconv_forward(x, weight, stride, padding, dilation, pool_to=None):
    """y[B,OH,OW,C] = depthwise cross-correlation of x[B,H,W,C] with weight[k1,k2,C].  With pool_to = (h, w)
    the result is (y, xp): xp[B,h,w,C] the adaptive average pool of x, from the same kernel when it can be."""
    dev = _lib.require_device(x, weight)
    L = _lib.lib()
    args = _conv_args(x.shape, weight.shape, stride, padding, dilation)
    OH = L.pdw_conv_out_size(args[1], args[4], stride[0], padding[0], dilation[0])
    OW = L.pdw_conv_out_size(args[2], args[5], stride[1], padding[1], dilation[1])
    y = torch.empty((x.shape[0], OH, OW, x.shape[3]), device=dev, dtype=x.dtype)
    if pool_to is not None:
        h, w = int(pool_to[0]), int(pool_to[1])
        xp = torch.empty((x.shape[0], h, w, x.shape[3]), device=dev, dtype=x.dtype)
        if y.numel() and xp.numel():
            with _lib.on_device(dev):
                _lib.check(L.pdw_dwconv_fwd_pool(x.data_ptr(), weight.data_ptr(), y.data_ptr(), xp.data_ptr(), *args,
                                                 h, w, _lib.dtype_code(x.dtype), _lib.stream_ptr(dev)),
                           "pdw_dwconv_fwd_pool")
            return y, xp
        from . import ops
        return dwconv_forward(x, weight, stride, padding, dilation), ops.avgpool_forward(x, (h, w))
    if y.numel():
        with _lib.on_device(dev):
            _lib.check(L.pdw_dwconv_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), *args,
                                        _lib.dtype_code(x.dtype), _lib.stream_ptr(dev)), "pdw_dwconv_fwd")
    return y


def dwconv_dgrad(gy, weight, in_shape, stride, padding, dilation, pooled_grad=None):
    """dx[in_shape]; with pooled_grad [B,h,w,C] the gradient of an adaptive average pool of the same
    tensor to (h, w) is added to it."""
    dev = _lib.require_device(gy, weight)
    L = _lib.lib()
    dx = torch.empty(in_shape, device=dev, dtype=gy.dtype)
    if dx.numel():
        if gy.numel() == 0:
            dx.zero_()
            if pooled_grad is not None and pooled_grad.numel():
                from . import ops
                ops.avgpool_backward(pooled_grad, (in_shape[1], in_shape[2]), out=dx, accumulate=True)
            return dx
        args = _conv_args(in_shape, weight.shape, stride, padding, dilation)
        with _lib.on_device(dev):
            if pooled_grad is None:
                _lib.check(L.pdw_dwconv_dgrad(gy.data_ptr(), weight.data_ptr(), dx.data_ptr(), *args,
                                              _lib.dtype_code(gy.dtype), _lib.stream_ptr(dev)), "pdw_dwconv_dgrad")
            else:
                gp = pooled_grad.contiguous()
                _lib.check(L.pdw_dwconv_dgrad_addpool(gy.data_ptr(), weight.data_ptr(), gp.data_ptr(), dx.data_ptr(),
                                                      *args, gp.shape[1], gp.shape[2], _lib.dtype_code(gy.dtype),
                                                      _lib.stream_ptr(dev)), "pdw_dwconv_dgrad_addpool")
    return dx


def dwconv_wgrad(x, gy, w_shape, stride, padding, dilation):
    dev = _lib.require_device(x, gy)
    L = _lib.lib()
    dw = torch.empty(tuple(w_shape), device=dev, dtype=x.dtype)
    if x.numel() == 0 or gy.numel() == 0:
        return dw.zero_()
    args = _conv_args(x.shape, w_shape, stride, padding, dilation)
    code = _lib.dtype_code(x.dtype)
    nbytes = L.pdw_dwconv_wgrad_workspace_bytes(*args, code)
    ws = torch.empty(max(nbytes, 4) // 4 + 1, device=dev, dtype=torch.float32)
    with _lib.on_device(dev):
        _lib.check(L.pdw_dwconv_wgrad(x.data_ptr(), gy.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws.numel() * 4,
                                      *args, code, _lib.stream_ptr(dev)), "pdw_dwconv_wgrad")
    _lib.keep_until_flush(ws)
    return dw


def dwconv_wgrad_pair(x0, gy0, x1, gy1, w_shape):
    """The weight gradients of two 'same' convolutions (stride 1, padding k // 2) with filters of one odd square
    shape `w_shape` on tensors of different extents, as one call of the library: (dw0, dw1)."""
    dev = _lib.require_device(x0, gy0, x1, gy1)
    L = _lib.lib()
    K, C = int(w_shape[0]), int(w_shape[2])
    B = x0.shape[0]
    if (w_shape[0] != w_shape[1] or K % 2 == 0 or x0.shape != gy0.shape or x1.shape != gy1.shape or x1.shape[0] != B
            or x0.shape[3] != C or x1.shape[3] != C or x1.dtype != x0.dtype):
        raise ValueError("dwconv_wgrad_pair: two same-padded convolutions with one odd square filter shape needed")
    dws = [torch.empty(tuple(w_shape), device=dev, dtype=x0.dtype) for _ in range(2)]
    if x0.numel() == 0 or x1.numel() == 0:
        geo = ((1, 1), (K // 2, K // 2), (1, 1))
        return dwconv_wgrad(x0, gy0, w_shape, *geo), dwconv_wgrad(x1, gy1, w_shape, *geo)
    code = _lib.dtype_code(x0.dtype)
    wss = []
    for x in (x0, x1):
        nbytes = L.pdw_dwconv_wgrad_workspace_bytes(B, x.shape[1], x.shape[2], C, K, K, 1, 1, K // 2, K // 2, 1, 1, code)
        wss.append(torch.empty(max(nbytes, 4) // 4 + 1, device=dev, dtype=torch.float32))
    with _lib.on_device(dev):
        _lib.check(L.pdw_dwconv_wgrad_pair(x0.data_ptr(), gy0.data_ptr(), dws[0].data_ptr(), wss[0].data_ptr(),
                                           wss[0].numel() * 4, x0.shape[1], x0.shape[2], x1.data_ptr(), gy1.data_ptr(),
                                           dws[1].data_ptr(), wss[1].data_ptr(), wss[1].numel() * 4, x1.shape[1],
                                           x1.shape[2], B, C, K, code, _lib.stream_ptr(dev)), "pdw_dwconv_wgrad_pair")
    for ws in wss:
        _lib.keep_until_flush(ws)
    return dws[0], dws[1]


def dwconv_forward2(x0, w0, x1, w1):
    """The 'same' convolutions of a two-scale block's two scales as one call of the library (pdw_dwconv_fwd2):
    (conv(x0, w0), conv(x1, w1)) with one odd square filter shape and x1 at exactly half the extents of x0; None when
    the fused kernel does not cover the case (the caller then makes the two calls)."""
    dev = _lib.require_device(x0, w0, x1, w1)
    L = _lib.lib()
    K, C = int(w0.shape[0]), int(w0.shape[2])
    B, H, W = x0.shape[0], x0.shape[1], x0.shape[2]
    if (w0.shape[0] != w0.shape[1] or K % 2 == 0 or w1.shape != w0.shape or tuple(x1.shape) != (B, H // 2, W // 2, C)
            or H % 2 or W % 2 or x0.shape[3] != C or any(t.dtype != x0.dtype for t in (w0, x1, w1)) or B == 0):
        return None
    args = [t.contiguous() for t in (x0, w0, x1, w1)]
    y0, y1 = torch.empty_like(args[0]), torch.empty_like(args[2])
    with _lib.on_device(dev):
        st = L.pdw_dwconv_fwd2(args[0].data_ptr(), args[1].data_ptr(), y0.data_ptr(), args[2].data_ptr(), args[3].data_ptr(),
                               y1.data_ptr(), B, H, W, C, K, _lib.dtype_code(x0.dtype), _lib.stream_ptr(dev))
    if st == 3:
        return None
    _lib.check(st, "pdw_dwconv_fwd2")
    return y0, y1


def dwconv_forward2_mean(x0, w0, x1, w1, parts, P, w_pool, b_pool=None, b_out=None):
    """dwconv_forward2 with the block's mean branch in the same launch (pdw_dwconv_fwd2_mean): returns
    (conv(x0, w0), conv(x1, w1), m, rowbias) with m [B, D] the per-image mean of the block's input (from the fp32
    sums `parts` [B * nparts, D] over groups of positions, P positions per image) and rowbias fp32 [B, D] =
    m w_pool^T + b_pool + b_out; None when the launch does not cover the case."""
    dev = _lib.require_device(x0, w0, x1, w1, parts, w_pool)
    L = _lib.lib()
    K, C = int(w0.shape[0]), int(w0.shape[2])
    B, H, W = x0.shape[0], x0.shape[1], x0.shape[2]
    D = int(w_pool.shape[0])
    dt = x0.dtype
    if (w0.shape[0] != w0.shape[1] or K % 2 == 0 or w1.shape != w0.shape or tuple(x1.shape) != (B, H // 2, W // 2, C)
            or H % 2 or W % 2 or x0.shape[3] != C or B == 0 or parts.dtype != torch.float32 or parts.shape[0] % B
            or tuple(w_pool.shape) != (D, D) or parts.shape[1] != D
            or any(t is not None and t.dtype != dt for t in (w0, x1, w1, w_pool, b_pool, b_out))):
        return None
    args = [t.contiguous() for t in (x0, w0, x1, w1, parts, w_pool)]
    y0, y1 = torch.empty_like(args[0]), torch.empty_like(args[2])
    m = torch.empty((B, D), device=dev, dtype=dt)
    rowbias = torch.empty((B, D), device=dev, dtype=torch.float32)
    with _lib.on_device(dev):
        st = L.pdw_dwconv_fwd2_mean(args[0].data_ptr(), args[1].data_ptr(), y0.data_ptr(), 0, 0, args[2].data_ptr(),
                                    args[3].data_ptr(), y1.data_ptr(), 0, 0, B, H, W, C, K, args[4].data_ptr(),
                                    parts.shape[0] // B, args[5].data_ptr(),
                                    b_pool.data_ptr() if b_pool is not None else None,
                                    b_out.data_ptr() if b_out is not None else None, m.data_ptr(), rowbias.data_ptr(),
                                    int(P), D, _lib.dtype_code(dt), _lib.stream_ptr(dev))
    if st == 3:
        return None
    _lib.check(st, "pdw_dwconv_fwd2_mean")
    return y0, y1, m, rowbias


def dwconv_bwd3(gy0, w0, gp, x0, x1, gy1):
    """The end of a two-scale block's backward pass as one call of the library (pdw_dwconv_bwd3): returns
    (dx, dw0, dw1) = (dwconv_dgrad(gy0, w0, pooled_grad=gp), dwconv_wgrad(x0, gy0), dwconv_wgrad(x1, gy1)) for 'same'
    convolutions with one odd square filter shape, x1 / gy1 / gp at exactly half the extents of x0 / gy0; None when
    the fused kernel does not cover the case (the caller then makes the three calls)."""
    dev = _lib.require_device(gy0, w0, gp, x0, x1, gy1)
    L = _lib.lib()
    K, C = int(w0.shape[0]), int(w0.shape[2])
    B, H, W = x0.shape[0], x0.shape[1], x0.shape[2]
    if (w0.shape[0] != w0.shape[1] or K % 2 == 0 or x0.shape != gy0.shape or x1.shape != gy1.shape or gp.shape != x1.shape
            or tuple(x1.shape) != (B, H // 2, W // 2, C) or H % 2 or W % 2 or x0.shape[3] != C
            or any(t.dtype != x0.dtype for t in (gy0, w0, gp, x1, gy1)) or B == 0):
        return None
    code = _lib.dtype_code(x0.dtype)
    dx = torch.empty_like(x0)
    dws = [torch.empty(tuple(w0.shape), device=dev, dtype=x0.dtype) for _ in range(2)]
    wss = []
    for x in (x0, x1):
        nbytes = L.pdw_dwconv_wgrad_workspace_bytes(B, x.shape[1], x.shape[2], C, K, K, 1, 1, K // 2, K // 2, 1, 1, code)
        wss.append(torch.empty(max(nbytes, 4) // 4 + 1, device=dev, dtype=torch.float32))
    args = [t.contiguous() for t in (gy0, w0, gp, x0, x1, gy1)]
    with _lib.on_device(dev):
        st = L.pdw_dwconv_bwd3(args[0].data_ptr(), args[1].data_ptr(), args[2].data_ptr(), dx.data_ptr(), args[3].data_ptr(),
                               dws[0].data_ptr(), wss[0].data_ptr(), wss[0].numel() * 4, args[4].data_ptr(),
                               args[5].data_ptr(), dws[1].data_ptr(), wss[1].data_ptr(), wss[1].numel() * 4, B, H, W, C, K,
                               code, _lib.stream_ptr(dev))
    if st == 3:
        return None
    _lib.check(st, "pdw_dwconv_bwd3")
    for ws in wss:
        _lib.keep_until_flush(ws)
    return dx, dws[0], dws[1]


class DepthwiseConv2DFunction(torch.autograd.Function):
    """apply(input[B,H,W,C], weight[k1,k2,C], stride, padding, dilation, dtype) -> output[B,OH,OW,C] of `dtype`.

    backward returns (grad_input like input, grad_weight like weight, None, None, None, None),
    as dwconv_triton.py:387 does.
    """

    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation, dtype):
        stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
        if input.dim() != 4 or weight.dim() != 3 or input.shape[3] != weight.shape[2]:
            raise ValueError(f"expected input [B,H,W,C] and weight [k1,k2,C], got {tuple(input.shape)} and "
                             f"{tuple(weight.shape)}")
        dtype = dtype if dtype is not None else weight.dtype
        ctx.stride, ctx.padding, ctx.dilation = stride, padding, dilation
        ctx.in_dtype, ctx.w_dtype = input.dtype, weight.dtype
        x = input.detach().to(dtype).contiguous()
        w = weight.detach().to(dtype).contiguous()
        y = dwconv_forward(x, w, stride, padding, dilation)
        ctx.save_for_backward(x, w)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, w = ctx.saved_tensors
        gy = grad_output.to(x.dtype).contiguous()
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = dwconv_dgrad(gy, w, x.shape, ctx.stride, ctx.padding, ctx.dilation).to(ctx.in_dtype)
        if ctx.needs_input_grad[1]:
            dw = dwconv_wgrad(x, gy, w.shape, ctx.stride, ctx.padding, ctx.dilation).to(ctx.w_dtype)
        return dx, dw, None, None, None, None


class OptimizedDepthwiseConv2d(torch.nn.Module):
    """Depthwise conv layer with weight ``[k1,k2,C]`` on ``[B,H,W,C]`` input.

    As in the reference (dwconv_triton.py:390-416) the ``dtype`` argument is accepted and
    ignored: the weight is created in float16 and filled by ``kaiming_uniform_``; callers move
    the module with ``.to(dtype)``.  There is no bias.
    """

    def __init__(self, channels, kernel_size, stride=1, padding=0, dilation=1, dtype=None):
        super().__init__()
        self.channels = channels
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.weight = torch.nn.Parameter(torch.empty(self.kernel_size[0], self.kernel_size[1], channels,
                                                     dtype=torch.float16))
        torch.nn.init.kaiming_uniform_(self.weight)

    def forward(self, x):
        assert x.dim() == 4 and x.shape[3] == self.channels, "input must be [B,H,W,C] with matching channels"
        return DepthwiseConv2DFunction.apply(x, self.weight, self.stride, self.padding, self.dilation,
                                             self.weight.dtype)

    def extra_repr(self):
        return (f"channels={self.channels}, kernel_size={self.kernel_size}, stride={self.stride}, "
                f"padding={self.padding}, dilation={self.dilation}")
