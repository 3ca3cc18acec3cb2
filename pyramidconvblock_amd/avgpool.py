"""Adaptive average pooling on channels-last tensors, backed by libpdw.so.

Operator shape of the reference's stand-alone NHWC pool (pyramid_dwconv/avgpool_triton.py:205-268);
bins are computed with exact integer arithmetic and the gradient is a gather (no atomics).
"""
from __future__ import annotations

import torch

from .ops import avgpool_backward, avgpool_forward  # noqa: F401  (re-exported)


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
