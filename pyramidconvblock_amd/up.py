"""Bilinear resize (align_corners=False) on channels-last tensors, backed by libpdw.so.

Operator shape of the reference's stand-alone NHWC interpolation module
(pyramid_dwconv/up_triton.py:127-162).  Unlike the reference module this one is
differentiable: the backward is the exact transpose of the forward.
"""
from __future__ import annotations

import torch

from .ops import bilinear_backward, bilinear_forward  # noqa: F401  (re-exported)


class BilinearInterp2dFunction(torch.autograd.Function):
    """apply(input[B,h,w,C], output_size=(H,W)) -> [B,H,W,C]."""

    @staticmethod
    def forward(ctx, input, output_size):
        if input.dim() != 4:
            raise ValueError("input must be [B,H,W,C]")
        ctx.in_hw = (input.shape[1], input.shape[2])
        return bilinear_forward(input.detach().contiguous(), output_size)

    @staticmethod
    def backward(ctx, grad_output):
        return bilinear_backward(grad_output.contiguous(), ctx.in_hw), None


class OptimizedBilinearInterp2d(torch.nn.Module):
    """``align_corners`` is stored and, as in the reference (up_triton.py:131), not used:
    the kernel always implements align_corners=False."""

    def __init__(self, output_size, align_corners=False):
        super().__init__()
        self.output_size = output_size
        self.align_corners = align_corners

    def forward(self, x):
        assert x.dim() == 4, "input must be a 4-D [B,H,W,C] tensor"
        size = (self.output_size, self.output_size) if isinstance(self.output_size, int) else tuple(self.output_size)
        return BilinearInterp2dFunction.apply(x, size)
