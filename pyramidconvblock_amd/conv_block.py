"""``SimpleGate`` and ``ConvBlock`` with the reference's constructor signatures, sub-module
names, parameter shapes and ``[B,H,W,C]`` in/out contract
(pyramid_dwconv/conv_block.py:6-49), running on the gfx950 kernels of libpdw.so.

``state_dict`` keys match the reference: ``conv_up.weight``, ``gates.{i}.conv_spatial.weight``
(``[k,k,inter_dim]``), ``conv_out.{weight,bias}``, ``conv_pool.{weight,bias}``.
"""
from __future__ import annotations

import torch
from torch import nn

from . import _lib
from .avgpool import AdaptiveAvgPool2dFunction
from .dwconv import OptimizedDepthwiseConv2d
from .up import BilinearInterp2dFunction


class GateFunction(torch.autograd.Function):
    """y = x[..., :G] * x[..., G:] * sqrt(G), G = I/2   (conv_block.py:10,18-19)."""

    @staticmethod
    def forward(ctx, x):
        x = x.detach().contiguous()
        dev = _lib.require_device(x)
        I = x.shape[-1]
        if I % 2:
            raise ValueError("gate needs an even channel count")
        y = torch.empty(x.shape[:-1] + (I // 2,), device=dev, dtype=x.dtype)
        if y.numel():
            with _lib.on_device(dev):
                _lib.check(_lib.lib().pdw_gate_fwd(x.data_ptr(), y.data_ptr(), x.numel() // I, I,
                                                   _lib.dtype_code(x.dtype), _lib.stream_ptr(dev)), "pdw_gate_fwd")
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, gy):
        (x,) = ctx.saved_tensors
        gy = gy.contiguous()
        dev = x.device
        I = x.shape[-1]
        gx = torch.empty_like(x)
        if gx.numel():
            with _lib.on_device(dev):
                _lib.check(_lib.lib().pdw_gate_bwd(x.data_ptr(), gy.data_ptr(), gx.data_ptr(), x.numel() // I, I,
                                                   _lib.dtype_code(x.dtype), _lib.stream_ptr(dev)), "pdw_gate_bwd")
        return gx


class SimpleGate(nn.Module):
    """pool (scale != 1) -> depthwise conv -> gate -> bilinear back to (H, W)   (conv_block.py:6-22).
    ``bias`` is accepted and ignored, as in the reference."""

    def __init__(self, dim: int, kernel_size=13, scale_factor=1., bias=False):
        super().__init__()
        self.scale_factor = scale_factor
        self.scale = (dim / 2) ** -0.5
        self.conv_spatial = OptimizedDepthwiseConv2d(dim, kernel_size=kernel_size, padding=kernel_size // 2)

    def forward(self, x):
        B, H, W, C = x.shape
        if self.scale_factor != 1.:
            x = AdaptiveAvgPool2dFunction.apply(x, (int(H * self.scale_factor), int(W * self.scale_factor)))
        x = GateFunction.apply(self.conv_spatial(x))
        if self.scale_factor != 1.:
            x = BilinearInterp2dFunction.apply(x, (H, W))
        return x


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
        x_conv = self.conv_up(x)
        x_conv = torch.cat([gate(x_conv) for gate in self.gates], dim=-1)
        x_conv = self.conv_out(x_conv)
        x_pool = self.conv_pool(x.mean(dim=(1, 2), keepdim=True))
        return x_conv + x_pool
