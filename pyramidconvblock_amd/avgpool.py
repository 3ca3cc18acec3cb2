"""Adaptive average pooling on channels-last tensors, backed by libpdw.so.

Operator shape of the reference's stand-alone NHWC pool (pyramid_dwconv/avgpool_triton.py:205-268);
bins are computed with exact integer arithmetic and the gradient is a gather (no atomics).
"""
from __future__ import annotations

import torch

from . import _lib


def _pool_call(fn_name, src, dst, B, H, W, C, h, w):
    dev = _lib.require_device(src, dst)
    if src.numel() and dst.numel():
        with _lib.on_device(dev):
            fn = getattr(_lib.lib(), fn_name)
            _lib.check(fn(src.data_ptr(), dst.data_ptr(), B, H, W, C, h, w, _lib.dtype_code(src.dtype),
                          _lib.stream_ptr(dev)), fn_name)
    return dst


def avgpool_forward(x, out_hw):
    B, H, W, C = x.shape
    h, w = int(out_hw[0]), int(out_hw[1])
    return _pool_call("pdw_avgpool_fwd", x, torch.empty((B, h, w, C), device=x.device, dtype=x.dtype), B, H, W, C, h, w)


def avgpool_backward(gy, in_hw):
    B, h, w, C = gy.shape
    H, W = int(in_hw[0]), int(in_hw[1])
    return _pool_call("pdw_avgpool_bwd", gy, torch.empty((B, H, W, C), device=gy.device, dtype=gy.dtype), B, H, W, C, h, w)


class AdaptiveAvgPool2dFunction(torch.autograd.Function):
    """apply(input[B,H,W,C], output_size=(h,w)) -> [B,h,w,C]   (avgpool_triton.py:207-257)."""

    @staticmethod
    def forward(ctx, input, output_size):
        if input.dim() != 4:
            raise ValueError("input must be [B,H,W,C]")
        ctx.in_hw = (input.shape[1], input.shape[2])
        return avgpool_forward(input.detach().contiguous(), output_size)

    @staticmethod
    def backward(ctx, grad_output):
        return avgpool_backward(grad_output.contiguous(), ctx.in_hw), None


class OptimizedAdaptiveAvgPool2d(torch.nn.Module):
    def __init__(self, output_size):
        super().__init__()
        self.output_size = (output_size, output_size) if isinstance(output_size, int) else tuple(output_size)

    def forward(self, x):
        assert x.dim() == 4, "input must be a 4-D [B,H,W,C] tensor"
        return AdaptiveAvgPool2dFunction.apply(x, self.output_size)
