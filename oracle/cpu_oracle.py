"""CPU oracle for the pyramid depthwise-conv hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the cpu_baseline leg of the bench may import this
module; the product package never does and has no CPU fallback.

Two layers:

* thin numpy/ctypes wrappers over ``libpdw_oracle.so`` (``pdw_oracle.c``), float64 NHWC;
* a float64 restatement of the block dataflow with a hand-written backward:
  ``simple_gate_*`` follows ``pyramid_dwconv/conv_block.py:13-22`` and ``convblock_*``
  follows ``pyramid_dwconv/conv_block.py:36-49`` of the reference.  Parameter names and
  shapes are those of the reference's ``state_dict`` (``conv_block.py:30-34``,
  ``dwconv_triton.py:413``).

Parity status: the reference has no golden vectors; these functions are pinned in
tests/ against torch's CPU library operators (float64 autograd), closed forms and
adjoint identities.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libpdw_oracle.so")


def build(force: bool = False) -> str:
    """Compile pdw_oracle.c with the Makefile beside it (gcc, OpenMP)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f64(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _pair(v):
    return (int(v), int(v)) if np.isscalar(v) else (int(v[0]), int(v[1]))


def out_size(n, k, s, p, d):
    """dwconv_triton.py:311-312."""
    return int(lib().pdwo_out_size(int(n), int(k), int(s), int(p), int(d)))


def _conv_args(B, H, W, C, KH, KW, stride, padding, dilation):
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    return [ctypes.c_int(v) for v in (B, H, W, C, KH, KW, s[0], s[1], p[0], p[1], d[0], d[1])], s, p, d


def dwconv_fwd(x, w, stride=1, padding=0, dilation=1):
    x, w = _f64(x), _f64(w)
    B, H, W, C = x.shape
    KH, KW, Cw = w.shape
    assert Cw == C
    args, s, p, d = _conv_args(B, H, W, C, KH, KW, stride, padding, dilation)
    OH, OW = out_size(H, KH, s[0], p[0], d[0]), out_size(W, KW, s[1], p[1], d[1])
    y = np.empty((B, OH, OW, C), dtype=np.float64)
    lib().pdwo_dwconv_fwd(_p(x), _p(w), _p(y), *args)
    return y


def dwconv_dgrad(gy, w, in_hw, stride=1, padding=0, dilation=1):
    gy, w = _f64(gy), _f64(w)
    B, OH, OW, C = gy.shape
    KH, KW, _ = w.shape
    H, W = in_hw
    args, s, p, d = _conv_args(B, H, W, C, KH, KW, stride, padding, dilation)
    assert (OH, OW) == (out_size(H, KH, s[0], p[0], d[0]), out_size(W, KW, s[1], p[1], d[1]))
    dx = np.empty((B, H, W, C), dtype=np.float64)
    lib().pdwo_dwconv_dgrad(_p(gy), _p(w), _p(dx), *args)
    return dx


def dwconv_dgrad_flipped(gy, w, padding):
    """The reference's own dgrad formula (dwconv_triton.py:154-185)."""
    gy, w = _f64(gy), _f64(w)
    B, H, W, C = gy.shape
    KH, KW, _ = w.shape
    p = _pair(padding)
    dx = np.empty_like(gy)
    lib().pdwo_dwconv_dgrad_flipped(_p(gy), _p(w), _p(dx), *[ctypes.c_int(v) for v in (B, H, W, C, KH, KW, p[0], p[1])])
    return dx


def dwconv_wgrad(x, gy, kernel_hw, stride=1, padding=0, dilation=1):
    x, gy = _f64(x), _f64(gy)
    B, H, W, C = x.shape
    KH, KW = kernel_hw
    args, s, p, d = _conv_args(B, H, W, C, KH, KW, stride, padding, dilation)
    assert gy.shape == (B, out_size(H, KH, s[0], p[0], d[0]), out_size(W, KW, s[1], p[1], d[1]), C)
    dw = np.empty((KH, KW, C), dtype=np.float64)
    lib().pdwo_dwconv_wgrad(_p(x), _p(gy), _p(dw), *args)
    return dw


def avgpool_fwd(x, out_hw):
    x = _f64(x)
    B, H, W, C = x.shape
    h, w = out_hw
    y = np.empty((B, h, w, C), dtype=np.float64)
    lib().pdwo_avgpool_fwd(_p(x), _p(y), *[ctypes.c_int(v) for v in (B, H, W, C, h, w)])
    return y


def avgpool_bwd(gy, in_hw):
    gy = _f64(gy)
    B, h, w, C = gy.shape
    H, W = in_hw
    gx = np.empty((B, H, W, C), dtype=np.float64)
    lib().pdwo_avgpool_bwd(_p(gy), _p(gx), *[ctypes.c_int(v) for v in (B, H, W, C, h, w)])
    return gx


def bilinear_fwd(x, out_hw):
    x = _f64(x)
    B, h, w, C = x.shape
    H, W = out_hw
    y = np.empty((B, H, W, C), dtype=np.float64)
    lib().pdwo_bilinear_fwd(_p(x), _p(y), *[ctypes.c_int(v) for v in (B, h, w, C, H, W)])
    return y


def bilinear_bwd(gy, in_hw):
    gy = _f64(gy)
    B, H, W, C = gy.shape
    h, w = in_hw
    gx = np.empty((B, h, w, C), dtype=np.float64)
    lib().pdwo_bilinear_bwd(_p(gy), _p(gx), *[ctypes.c_int(v) for v in (B, h, w, C, H, W)])
    return gx


def gate_fwd(x):
    x = _f64(x)
    I = x.shape[-1]
    M = x.size // I
    y = np.empty(x.shape[:-1] + (I // 2,), dtype=np.float64)
    lib().pdwo_gate_fwd(_p(x), _p(y), ctypes.c_longlong(M), ctypes.c_int(I))
    return y


def gate_bwd(x, gy):
    x, gy = _f64(x), _f64(gy)
    I = x.shape[-1]
    M = x.size // I
    gx = np.empty_like(x)
    lib().pdwo_gate_bwd(_p(x), _p(gy), _p(gx), ctypes.c_longlong(M), ctypes.c_int(I))
    return gx


# ----------------------------------------------------------------------------------------------
# Block dataflow (float64, explicit backward)
# ----------------------------------------------------------------------------------------------

def simple_gate_fwd(a, w, scale_factor):
    """conv_block.py:13-22.  a [B,H,W,I], w [k,k,I] -> ([B,H,W,I/2], cache)."""
    B, H, W, I = a.shape
    k = w.shape[0]
    if scale_factor != 1.0:
        hw = (int(H * scale_factor), int(W * scale_factor))  # conv_block.py:16
        p = avgpool_fwd(a, hw)
    else:
        hw = (H, W)
        p = _f64(a)
    c = dwconv_fwd(p, w, 1, k // 2, 1)  # conv_block.py:11 (padding=k//2, stride 1)
    g = gate_fwd(c)
    y = bilinear_fwd(g, (H, W)) if scale_factor != 1.0 else g
    return y, dict(p=p, c=c, hw=hw, HW=(H, W), scale_factor=scale_factor, w=_f64(w))


def simple_gate_bwd(cache, gy):
    """Returns (d a, d w)."""
    sf, k = cache["scale_factor"], cache["w"].shape[0]
    gg = bilinear_bwd(gy, cache["hw"]) if sf != 1.0 else _f64(gy)
    gc = gate_bwd(cache["c"], gg)
    dw = dwconv_wgrad(cache["p"], gc, (k, cache["w"].shape[1]), 1, k // 2, 1)
    dp = dwconv_dgrad(gc, cache["w"], cache["hw"], 1, k // 2, 1)
    da = avgpool_bwd(dp, cache["HW"]) if sf != 1.0 else dp
    return da, dw


def convblock_fwd(x, params, scales=(1.0, 0.5)):
    """conv_block.py:36-49.  params uses the reference's state_dict keys."""
    x = _f64(x)
    P = {k: _f64(v) for k, v in params.items()}
    a = x @ P["conv_up.weight"].T
    if "conv_up.bias" in P:
        a = a + P["conv_up.bias"]
    outs, caches = [], []
    for i, s in enumerate(scales):
        y, c = simple_gate_fwd(a, P[f"gates.{i}.conv_spatial.weight"], s)
        outs.append(y)
        caches.append(c)
    cat = np.concatenate(outs, axis=-1)
    y = cat @ P["conv_out.weight"].T
    if "conv_out.bias" in P:
        y = y + P["conv_out.bias"]
    m = x.mean(axis=(1, 2), keepdims=True)
    yp = m @ P["conv_pool.weight"].T
    if "conv_pool.bias" in P:
        yp = yp + P["conv_pool.bias"]
    return y + yp, dict(x=x, a=a, cat=cat, m=m, caches=caches, P=P, scales=scales)


def convblock_bwd(cache, gy):
    """Returns (dx, dict of parameter gradients keyed like the state_dict)."""
    gy = _f64(gy)
    P, x = cache["P"], cache["x"]
    B, H, W, D = x.shape
    grads = {}
    g2 = gy.reshape(-1, D)
    # pooled branch
    gp = gy.sum(axis=(1, 2), keepdims=True)  # broadcast add
    grads["conv_pool.weight"] = gp.reshape(-1, D).T @ cache["m"].reshape(-1, D)
    if "conv_pool.bias" in P:
        grads["conv_pool.bias"] = gp.reshape(-1, D).sum(0)
    dm = gp @ P["conv_pool.weight"]
    dx = np.broadcast_to(dm / (H * W), x.shape).copy()
    # conv branch
    cat = cache["cat"]
    grads["conv_out.weight"] = g2.T @ cat.reshape(-1, cat.shape[-1])
    if "conv_out.bias" in P:
        grads["conv_out.bias"] = g2.sum(0)
    dcat = gy @ P["conv_out.weight"]
    G = cat.shape[-1] // len(cache["scales"])
    da = np.zeros_like(cache["a"])
    for i, c in enumerate(cache["caches"]):
        dai, dwi = simple_gate_bwd(c, dcat[..., i * G:(i + 1) * G])
        da += dai
        grads[f"gates.{i}.conv_spatial.weight"] = dwi
    I = da.shape[-1]
    grads["conv_up.weight"] = da.reshape(-1, I).T @ x.reshape(-1, D)
    if "conv_up.bias" in P:
        grads["conv_up.bias"] = da.reshape(-1, I).sum(0)
    dx += da @ P["conv_up.weight"]
    return dx, grads
