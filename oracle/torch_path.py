"""The reference's "PyTorch path" restated with torch library operators.  TEST INFRASTRUCTURE ONLY.

Used (a) to pin ``cpu_oracle`` against library routines in float64 and (b) as the CPU
baseline that the bench times next to the GPU path.  The op set is the one the reference's
pure-torch twin uses (``pyramid_dwconv/conv_block.py:52-97``): ``F.conv2d(groups=C)``,
``F.adaptive_avg_pool2d``, ``F.interpolate(mode='bilinear', align_corners=False)`` and linear
layers, composed in the order of ``conv_block.py:13-22`` and ``conv_block.py:36-49``.  The
weight layout map ``[k1,k2,C] -> [C,1,k1,k2]`` is the reference's (``dwconv_triton.py:457``).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def dwconv_nhwc(x, w, stride=1, padding=0, dilation=1):
    """x [B,H,W,C], w [k1,k2,C] -> [B,OH,OW,C] through F.conv2d on an NCHW view."""
    C = x.shape[-1]
    y = F.conv2d(x.permute(0, 3, 1, 2), w.permute(2, 0, 1).unsqueeze(1), None, stride, padding, dilation, C)
    return y.permute(0, 2, 3, 1)


def avgpool_nhwc(x, out_hw):
    return F.adaptive_avg_pool2d(x.permute(0, 3, 1, 2), out_hw).permute(0, 2, 3, 1)


def bilinear_nhwc(x, out_hw):
    return F.interpolate(x.permute(0, 3, 1, 2), size=out_hw, mode="bilinear", align_corners=False).permute(0, 2, 3, 1)


def gate(x):
    I = x.shape[-1]
    scale = (I / 2) ** -0.5
    x1, x2 = x.chunk(2, dim=-1)
    return x1 * (x2 / scale)


def simple_gate(a, w, scale_factor):
    B, H, W, I = a.shape
    k = w.shape[0]
    if scale_factor != 1.0:
        a = avgpool_nhwc(a, (int(H * scale_factor), int(W * scale_factor)))
    y = gate(dwconv_nhwc(a, w, 1, k // 2, 1))
    if scale_factor != 1.0:
        y = bilinear_nhwc(y, (H, W))
    return y


def convblock(x, params, scales=(1.0, 0.5)):
    """x [B,H,W,D]; params keyed like the reference's state_dict."""
    a = F.linear(x, params["conv_up.weight"], params.get("conv_up.bias"))
    ys = [simple_gate(a, params[f"gates.{i}.conv_spatial.weight"], s) for i, s in enumerate(scales)]
    y = F.linear(torch.cat(ys, dim=-1), params["conv_out.weight"], params.get("conv_out.bias"))
    m = x.mean(dim=(1, 2), keepdim=True)
    return y + F.linear(m, params["conv_pool.weight"], params.get("conv_pool.bias"))


def default_params(dim, kernel_size=9, bias=False, out_bias=True, scales=(1.0, 0.5), inter_ratio=0.5):
    """Default-initialised parameters drawn in the reference's construction order
    (conv_block.py:29-34): conv_up, one depthwise weight per gate, conv_out, conv_pool.
    Linear layers use torch's nn.Linear initialiser; each depthwise weight is an fp16
    [k,k,I] tensor filled by kaiming_uniform_ (dwconv_triton.py:410-416), i.e.
    U(-b, b) with b = sqrt(6 / (k * I))."""
    inter = int(dim * inter_ratio)
    P = {}
    lin = torch.nn.Linear(dim, inter, bias=bias)
    P["conv_up.weight"] = lin.weight.detach()
    if bias:
        P["conv_up.bias"] = lin.bias.detach()
    for i, _ in enumerate(scales):
        w = torch.empty(kernel_size, kernel_size, inter, dtype=torch.float16)
        torch.nn.init.kaiming_uniform_(w)
        P[f"gates.{i}.conv_spatial.weight"] = w
    lin = torch.nn.Linear(inter // 2 * len(scales), dim, bias=out_bias)
    P["conv_out.weight"] = lin.weight.detach()
    if out_bias:
        P["conv_out.bias"] = lin.bias.detach()
    lin = torch.nn.Linear(dim, dim, bias=out_bias)
    P["conv_pool.weight"] = lin.weight.detach()
    if out_bias:
        P["conv_pool.bias"] = lin.bias.detach()
    return P


def dw_init_bound(k2, channels):
    """Closed form of kaiming_uniform_(a=0) on a [k1,k2,C] tensor: fan_in = k2*C."""
    return math.sqrt(6.0 / (k2 * channels))
