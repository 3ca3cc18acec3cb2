"""Thin tensor-level wrappers over the C ABI of libpdw.so (one call = one or two kernel
launches on torch's current stream).  Outputs may be channel slices of wider tensors: a
destination whose last dimension is contiguous and whose pixels are a fixed stride apart is
passed to the kernels as (pointer, leading dimension)."""
from __future__ import annotations

import torch

from . import _lib


def _pixel_stride(t: torch.Tensor) -> int:
    """Element stride between consecutive pixels of a [..., C] tensor whose leading dims are
    laid out densely over a (possibly wider) channels-last buffer."""
    if t.stride(-1) != 1 and t.shape[-1] != 1:
        raise ValueError("last dimension must be contiguous")
    ld = t.stride(-2)
    exp = ld
    for d in range(t.dim() - 2, -1, -1):
        if t.shape[d] != 1 and t.stride(d) != exp:
            raise ValueError("tensor is not a channel slice of a dense channels-last buffer")
        exp *= t.shape[d]
    return ld


def _aligned(t):
    """The dense matrix-core kernels move 16-byte pieces: a view whose storage offset is not a multiple of 16
    bytes (a slice of a larger parameter buffer, say) is copied to a fresh, aligned allocation."""
    return t if t is None or t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)


def _launch(name, dev, *args):
    with _lib.on_device(dev):
        _lib.check(getattr(_lib.lib(), name)(*args, _lib.stream_ptr(dev)), name)


def avgpool_forward(x, out_hw):
    dev = _lib.require_device(x)
    B, H, W, C = x.shape
    h, w = int(out_hw[0]), int(out_hw[1])
    y = torch.empty((B, h, w, C), device=dev, dtype=x.dtype)
    if x.numel() and y.numel():
        _launch("pdw_avgpool_fwd", dev, x.data_ptr(), y.data_ptr(), B, H, W, C, h, w, _lib.dtype_code(x.dtype))
    return y


def avgpool_backward(gy, in_hw, out=None, accumulate=False):
    """gx[B,H,W,C] = transpose of the pool applied to gy[B,h,w,C]; with `out` and accumulate the
    result is added to `out` in place."""
    dev = _lib.require_device(gy)
    B, h, w, C = gy.shape
    H, W = int(in_hw[0]), int(in_hw[1])
    if out is None:
        out = torch.empty((B, H, W, C), device=dev, dtype=gy.dtype)
        accumulate = False
    if gy.numel() and out.numel():
        _launch("pdw_avgpool_bwd", dev, gy.data_ptr(), out.data_ptr(), B, H, W, C, h, w, 1 if accumulate else 0,
                _lib.dtype_code(gy.dtype))
    return out


def bilinear_forward(x, out_hw, out=None):
    dev = _lib.require_device(x)
    B, h, w, C = x.shape
    H, W = int(out_hw[0]), int(out_hw[1])
    if out is None:
        out = torch.empty((B, H, W, C), device=dev, dtype=x.dtype)
    if x.numel() and out.numel():
        _launch("pdw_bilinear_fwd", dev, x.data_ptr(), out.data_ptr(), B, h, w, C, H, W, _pixel_stride(out),
                _lib.dtype_code(x.dtype))
    return out


def bilinear_backward(gy, in_hw):
    """gy may be a channel slice of a wider [B,H,W,*] tensor."""
    dev = _lib.require_device(gy)
    B, H, W, C = gy.shape
    h, w = int(in_hw[0]), int(in_hw[1])
    gx = torch.empty((B, h, w, C), device=dev, dtype=gy.dtype)
    if gy.numel() and gx.numel():
        _launch("pdw_bilinear_bwd", dev, gy.data_ptr(), gx.data_ptr(), B, h, w, C, H, W, _pixel_stride(gy),
                _lib.dtype_code(gy.dtype))
    return gx


def gate_forward(x, out=None):
    dev = _lib.require_device(x)
    I = x.shape[-1]
    if I % 2:
        raise ValueError("gate needs an even channel count")
    if out is None:
        out = torch.empty(x.shape[:-1] + (I // 2,), device=dev, dtype=x.dtype)
    if out.numel():
        _launch("pdw_gate_fwd", dev, x.data_ptr(), out.data_ptr(), x.numel() // I, I, _pixel_stride(out),
                _lib.dtype_code(x.dtype))
    return out


def gate_backward(x, gy):
    """gy may be a channel slice of a wider tensor."""
    dev = _lib.require_device(x, gy)
    I = x.shape[-1]
    gx = torch.empty_like(x)
    if gx.numel():
        _launch("pdw_gate_bwd", dev, x.data_ptr(), gy.data_ptr(), gx.data_ptr(), x.numel() // I, I, _pixel_stride(gy),
                _lib.dtype_code(x.dtype))
    return gx


def gate_bilinear_forward(x, out_hw, out=None):
    """gate then bilinear resize to out_hw in one kernel; x [B,h,w,I] -> [B,H,W,I/2] (conv_block.py:18-21)."""
    dev = _lib.require_device(x)
    B, h, w, I = x.shape
    if I % 2:
        raise ValueError("gate needs an even channel count")
    H, W = int(out_hw[0]), int(out_hw[1])
    if out is None:
        out = torch.empty((B, H, W, I // 2), device=dev, dtype=x.dtype)
    if x.numel() and out.numel():
        _launch("pdw_gate_bilinear_fwd", dev, x.data_ptr(), out.data_ptr(), B, h, w, I, H, W, _pixel_stride(out),
                _lib.dtype_code(x.dtype))
    return out


def bilinear_gate_backward(x, gy):
    """Gradient of gate_bilinear_forward w.r.t. x; gy [B,H,W,I/2] may be a channel slice of a wider tensor.
    One kernel when the extents are exactly doubled, the two separate ones otherwise."""
    dev = _lib.require_device(x, gy)
    B, h, w, I = x.shape
    H, W = gy.shape[1], gy.shape[2]
    if H == 2 * h and W == 2 * w and h >= 2 and w >= 2:
        gx = torch.empty_like(x)
        if gx.numel():
            _launch("pdw_bilinear_gate_bwd", dev, gy.data_ptr(), x.data_ptr(), gx.data_ptr(), B, h, w, I, H, W,
                    _pixel_stride(gy), _lib.dtype_code(x.dtype))
        return gx
    return gate_backward(x, bilinear_backward(gy, (h, w)))


def gate_pair_forward(xf, xh, out):
    """out[..., :G] = gate(xf), out[..., G:2G] = bilinear(gate(xh)) to xf's extents, one launch; out [B,H,W,>=2G]
    may be a channel slice of a wider tensor."""
    dev = _lib.require_device(xf, xh, out)
    B, H, W, I = xf.shape
    h, w = xh.shape[1], xh.shape[2]
    if I % 2 or xh.shape[3] != I or out.shape[3] != I:
        raise ValueError("gate pair: xf, xh need the same even channel count I and out I channels")
    if xf.numel():
        _launch("pdw_gate_pair_fwd", dev, xf.data_ptr(), xh.data_ptr(), out.data_ptr(), B, H, W, h, w, I,
                _pixel_stride(out), _lib.dtype_code(xf.dtype))
    return out


def gate_pair_backward(xf, xh, gy):
    """Gradients (gxf, gxh) of gate_pair_forward; gy [B,H,W,2G] may be a channel slice.  One launch
    (pdw_gate_pair_bwd), whatever the ratio of the extents."""
    dev = _lib.require_device(xf, xh, gy)
    B, H, W, I = xf.shape
    h, w = xh.shape[1], xh.shape[2]
    G = I // 2
    if xf.numel() and xh.numel():
        gxf, gxh = torch.empty_like(xf), torch.empty_like(xh)
        if xf.numel():
            _launch("pdw_gate_pair_bwd", dev, gy.data_ptr(), xf.data_ptr(), xh.data_ptr(), gxf.data_ptr(),
                    gxh.data_ptr(), B, H, W, h, w, I, _pixel_stride(gy), _lib.dtype_code(xf.dtype))
        return gxf, gxh
    return gate_backward(xf, gy[..., :G]), bilinear_gate_backward(xh, gy[..., G:2 * G])


def block_mid_forward(xf, xh, out, parts, P, w_pool, b_pool=None, b_out=None):
    """gate_pair_forward(xf, xh, out) and pool_branch_forward(parts=...) as one launch -> (m, rowbias)."""
    dev = _lib.require_device(xf, xh, out, w_pool)
    B, H, W, I = xf.shape
    h, w = xh.shape[1], xh.shape[2]
    D = w_pool.shape[0]
    if I % 2 or xh.shape[3] != I or out.shape[3] != I:
        raise ValueError("gate pair: xf, xh need the same even channel count I and out I channels")
    m = torch.empty((B, D), device=dev, dtype=xf.dtype)
    rowbias = torch.empty((B, D), device=dev, dtype=torch.float32)
    _launch("pdw_block_mid_fwd", dev, xf.data_ptr(), xh.data_ptr(), out.data_ptr(), B, H, W, h, w, I, _pixel_stride(out),
            parts.data_ptr(), parts.shape[0] // B, w_pool.data_ptr(), b_pool.data_ptr() if b_pool is not None else None,
            b_out.data_ptr() if b_out is not None else None, m.data_ptr(), rowbias.data_ptr(), int(P), D,
            _lib.dtype_code(xf.dtype))
    return m, rowbias


def block_mid_backward(xf, xh, gy, parts, P, m, w_pool):
    """gate_pair_backward and pool_branch_backward(parts=...) as one launch (exactly doubled extents only)
    -> (gxf, gxh, gbias [2, D], gw_pool, dmean)."""
    dev = _lib.require_device(xf, xh, gy, m, w_pool)
    B, H, W, I = xf.shape
    h, w = xh.shape[1], xh.shape[2]
    D = w_pool.shape[0]
    gxf, gxh = torch.empty_like(xf), torch.empty_like(xh)
    gbias = torch.empty((2, D), device=dev, dtype=xf.dtype)
    gwp = torch.empty((D, D), device=dev, dtype=xf.dtype)
    dmean = torch.empty((B, D), device=dev, dtype=torch.float32)
    ws = _pool_ws(B, int(P), D, dev)
    _launch("pdw_block_mid_bwd", dev, gy.data_ptr(), xf.data_ptr(), xh.data_ptr(), gxf.data_ptr(), gxh.data_ptr(), B, H, W,
            h, w, I, _pixel_stride(gy), parts.data_ptr(), parts.shape[0] // B, m.data_ptr(), w_pool.data_ptr(),
            gbias[0].data_ptr(), gbias[1].data_ptr(), gwp.data_ptr(), dmean.data_ptr(), ws.data_ptr(), ws.numel() * 4,
            int(P), D, _lib.dtype_code(xf.dtype))
    _lib.keep_until_flush(ws)  # inside deferred_reductions gbias and gw_pool are summed from it at the flush
    return gxf, gxh, gbias, gwp, dmean


def spatial_sum(x):
    """x [B, ..., C] -> fp32 [B, C]: sum over all middle dimensions."""
    dev = _lib.require_device(x)
    B, C = x.shape[0], x.shape[-1]
    P = x.numel() // max(B * C, 1)
    out = torch.empty((B, C), device=dev, dtype=torch.float32)
    if B == 0:
        return out
    if P == 0:
        return out.zero_()
    nbytes = _lib.lib().pdw_spatial_sum_workspace_bytes(B, P, C)
    ws = torch.empty(nbytes // 4 + 1, device=dev, dtype=torch.float32)
    _launch("pdw_spatial_sum", dev, x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel() * 4, B, P, C,
            _lib.dtype_code(x.dtype))
    return out


def add_rowbias_(y, v):
    """In place y[b, ..., c] += v[b, c] with v fp32 [B, C]."""
    dev = _lib.require_device(y, v)
    B, C = y.shape[0], y.shape[-1]
    P = y.numel() // max(B * C, 1)
    assert v.dtype == torch.float32 and v.is_contiguous() and tuple(v.shape) == (B, C)
    if y.numel():
        _launch("pdw_add_rowbias", dev, y.data_ptr(), v.data_ptr(), B, P, C, _lib.dtype_code(y.dtype))
    return y


def dense_supported(K, NO, dtype):
    """True when the matrix-core dense kernels cover an inner size K, output size NO layer of this dtype (forward,
    input gradient and weight gradient): 16-bit layers up to 128 wide in the tiled kernels, and fp32 or other widths
    (multiples of 4, inner width up to 256) one result tile per wavefront."""
    if dtype not in _lib._DTYPES:
        return False
    return bool(_lib.lib().pdw_dense_supported(int(K), int(NO), _lib.dtype_code(dtype)))


def dense_colsum_rows() -> int:
    """Rows per chunk sum of dense_forward(..., colsum=True): the row tile of the dense kernel."""
    return int(_lib.lib().pdw_dense_colsum_rows())


def dense_colsum_supported(K, NO, dtype, rows_per_image) -> bool:
    """Whether dense_forward(..., colsum=True) can deliver per-image chunk sums for this shape."""
    return (dtype in _lib._DTYPES and rows_per_image % dense_colsum_rows() == 0
            and bool(_lib.lib().pdw_dense_colsum_supported(int(K), int(NO), _lib.dtype_code(dtype))))


def dense_forward(x, w, w_kmajor=False, bias=None, rowbias=None, rows_per_image=1, colsum=False,
                  flush_reductions=False):
    """y[..., o] = sum_k x[..., k] * W(o, k) + bias[o] + rowbias[image][o].

    w is [NO, K] (nn.Linear layout) or, with w_kmajor, [K, NO].  rowbias is fp32 [B, NO], one row per
    `rows_per_image` consecutive rows of x.  With colsum (see dense_colsum_supported) the result is
    (y, parts): parts fp32 [N / R, K], the sums of x over each group of R = dense_colsum_rows() consecutive rows.  With
    flush_reductions, inside _lib.deferred_reductions, the summations recorded so far run in this launch."""
    dev = _lib.require_device(x, w)
    x, w, bias, rowbias = _aligned(x), _aligned(w), _aligned(bias), _aligned(rowbias)
    K = x.shape[-1]
    NO = w.shape[1] if w_kmajor else w.shape[0]
    assert (w.shape[0] if w_kmajor else w.shape[1]) == K and x.is_contiguous() and w.is_contiguous()
    N = x.numel() // K
    y = torch.empty(x.shape[:-1] + (NO,), device=dev, dtype=x.dtype)
    if colsum:
        R = dense_colsum_rows()
        parts = torch.empty(((N + R - 1) // R, K), device=dev, dtype=torch.float32)
        if N:
            _launch("pdw_dense_fwd_colsum", dev, x.data_ptr(), w.data_ptr(), 1 if w_kmajor else 0,
                    bias.data_ptr() if bias is not None else None, rowbias.data_ptr() if rowbias is not None else None,
                    y.data_ptr(), parts.data_ptr(), N, K, NO, int(rows_per_image), _lib.dtype_code(x.dtype))
        return y, parts
    if N:
        _launch("pdw_dense_fwd_flush" if flush_reductions else "pdw_dense_fwd", dev, x.data_ptr(), w.data_ptr(),
                1 if w_kmajor else 0, bias.data_ptr() if bias is not None else None,
                rowbias.data_ptr() if rowbias is not None else None, y.data_ptr(), N, K, NO, int(rows_per_image),
                _lib.dtype_code(x.dtype))
    return y


def dense_forward_gated(cf, ch, w, rowbias=None, bias=None, cat=None, gated=False):
    """The output layer of a two-scale block on rows made in the kernel (pdw_dense_fwd_gated): y = [gate(cf) |
    resize(gate(ch))] W^T + bias + rowbias[image] for the convolution outputs cf [B,H,W,I], ch [B,H/2,W/2,I] of the
    two scales; `cat` ([B,H,W,I], optional) receives the rows.  With `gated` the scales arrive gated (cf [B,H,W,I/2],
    possibly a channel slice of a wider tensor, ch [B,H/2,W/2,I/2]) and only the resize is left to do.  None where the
    kernel does not cover the case."""
    dev = _lib.require_device(cf, ch, w)
    if cf.dim() != 4 or not (ch.is_contiguous() and w.is_contiguous()):
        return None
    B, H, W, C = cf.shape
    I = 2 * C if gated else C
    D = w.shape[0]
    dt = cf.dtype
    ldf = _pixel_stride(cf) if gated else 0
    if not gated and not cf.is_contiguous():
        return None
    if (B == 0 or H % 2 or W % 2 or tuple(ch.shape) != (B, H // 2, W // 2, C) or w.shape[1] != I
            or any(t is not None and t.dtype != dt for t in (ch, w, bias, cat))
            or (rowbias is not None and (rowbias.dtype != torch.float32 or tuple(rowbias.shape) != (B, D)
                                         or not rowbias.is_contiguous()))
            or (cat is not None and (gated or tuple(cat.shape) != (B, H, W, I) or not cat.is_contiguous()))):
        return None
    y = torch.empty((B, H, W, D), device=dev, dtype=dt)
    with _lib.on_device(dev):
        st = _lib.lib().pdw_dense_fwd_gated(cf.data_ptr(), ch.data_ptr(), cat.data_ptr() if cat is not None else None,
                                            w.data_ptr(), bias.data_ptr() if bias is not None else None,
                                            rowbias.data_ptr() if rowbias is not None else None, y.data_ptr(), B, H, W,
                                            I, D, ldf, _lib.dtype_code(dt), _lib.stream_ptr(dev))
    if st == 3:
        return None
    _lib.check(st, "pdw_dense_fwd_gated")
    return y


def dense_forward_pool(x, w, bias=None):
    """x[B, H, W, K] -> (y, parts, pool): y = x W^T (+ bias), parts the fp32 sums of x over the kernel's 32-pixel tiles
    (H * W / 32 per image) and pool the 2x2 average pool of y, in one launch (pdw_dense_fwd_colsum_pool); None where
    the kernel does not cover the case."""
    dev = _lib.require_device(x, w)
    x, w, bias = _aligned(x), _aligned(w), _aligned(bias)
    if x.dim() != 4 or not x.is_contiguous() or not w.is_contiguous() or w.dtype != x.dtype:
        return None
    B, H, W, K = x.shape
    NO = w.shape[0]
    if w.shape[1] != K or B == 0 or H % 2 or W % 2 or (bias is not None and bias.dtype != x.dtype):
        return None
    y = torch.empty((B, H, W, NO), device=dev, dtype=x.dtype)
    parts = torch.empty((B * H * W // 32, K), device=dev, dtype=torch.float32)
    pool = torch.empty((B, H // 2, W // 2, NO), device=dev, dtype=x.dtype)
    with _lib.on_device(dev):
        st = _lib.lib().pdw_dense_fwd_colsum_pool(x.data_ptr(), w.data_ptr(), bias.data_ptr() if bias is not None else None,
                                                  y.data_ptr(), parts.data_ptr(), pool.data_ptr(), B, H, W, K, NO,
                                                  _lib.dtype_code(x.dtype), _lib.stream_ptr(dev))
    if st == 3:
        return None
    _lib.check(st, "pdw_dense_fwd_colsum_pool")
    return y, parts, pool


def dense_wgrad(a, b):
    """dw[m, o] = sum_n a[n, m] * b[n, o] over all leading dimensions; returns [M, NO] in a's dtype."""
    dev = _lib.require_device(a, b)
    a, b = _aligned(a), _aligned(b)
    M, NO = a.shape[-1], b.shape[-1]
    N = a.numel() // M
    assert b.numel() // NO == N and a.is_contiguous() and b.is_contiguous()
    dw = torch.empty((M, NO), device=dev, dtype=a.dtype)
    nbytes = _lib.lib().pdw_dense_wgrad_workspace_bytes(N, M, NO)
    ws = torch.empty(nbytes // 4 + 1, device=dev, dtype=torch.float32)
    _launch("pdw_dense_wgrad", dev, a.data_ptr(), b.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws.numel() * 4, N, M, NO,
            _lib.dtype_code(a.dtype))
    _lib.keep_until_flush(ws)
    return dw


def sum_parts(parts, dtype):
    """parts[S, ...] (fp32) -> their sum over S, added in fp32 in a fixed order and rounded once to `dtype`
    (pdw_sum_parts; inside a deferral the summation joins the pass's single reduction launch)."""
    dev = _lib.require_device(parts)
    assert parts.dtype == torch.float32 and parts.dim() >= 2
    parts = parts.contiguous()
    out = torch.empty(parts.shape[1:], device=dev, dtype=dtype)
    _launch("pdw_sum_parts", dev, parts.data_ptr(), out.data_ptr(), parts.shape[0], out.numel(), _lib.dtype_code(dtype))
    _lib.keep_until_flush(parts)
    return out


def dense_backward_pair_supported(O, I, dtype, rows_per_image=None, colsum=False) -> bool:
    """Whether dense_backward_pair covers a layer with weight [O, I] (and a per-image term over images of
    rows_per_image rows; with `colsum`, the tile sums of gy as well)."""
    if dtype not in _lib._DTYPES or (rows_per_image is not None and rows_per_image < 32):
        return False
    fn = _lib.lib().pdw_dense_bwd_pair_colsum_supported if colsum else _lib.lib().pdw_dense_bwd_pair_supported
    return bool(fn(int(O), int(I), _lib.dtype_code(dtype)))


def dense_backward_pair(gy, w, x, colsum=False, rowbias=None, rows_per_image=1):
    """Both gradients of y = x W^T that need gy, one launch: (dx [..., I], parts or None, dw [O, I]) with
    dx = gy W + rowbias[image] (rowbias fp32 [B, I] or None), dw = gy^T x and, with colsum, parts as in
    dense_forward(gy, ..., colsum=True)."""
    dev = _lib.require_device(gy, w, x)
    gy, w, x, rowbias = _aligned(gy), _aligned(w), _aligned(x), _aligned(rowbias)
    O, I = w.shape
    N = gy.numel() // O
    assert gy.shape[-1] == O and x.shape[-1] == I and x.numel() // I == N
    assert gy.is_contiguous() and w.is_contiguous() and x.is_contiguous()
    dx = torch.empty(gy.shape[:-1] + (I,), device=dev, dtype=gy.dtype)
    dw = torch.empty((O, I), device=dev, dtype=gy.dtype)
    parts = None
    if colsum:
        R = dense_colsum_rows()
        parts = torch.empty(((N + R - 1) // R, O), device=dev, dtype=torch.float32)
    nbytes = _lib.lib().pdw_dense_wgrad_workspace_bytes(N, O, I)
    ws = torch.empty(nbytes // 4 + 1, device=dev, dtype=torch.float32)
    _launch("pdw_dense_bwd_pair", dev, gy.data_ptr(), w.data_ptr(), x.data_ptr(), dx.data_ptr(),
            parts.data_ptr() if parts is not None else None, dw.data_ptr(), ws.data_ptr(), ws.numel() * 4,
            rowbias.data_ptr() if rowbias is not None else None, int(rows_per_image), N, O, I,
            _lib.dtype_code(gy.dtype))
    _lib.keep_until_flush(ws)
    return dx, parts, dw


def _pool_ws(B, P, D, dev):
    nbytes = _lib.lib().pdw_pool_branch_workspace_bytes(B, P, D)
    return torch.empty(nbytes // 4 + 1, device=dev, dtype=torch.float32)


def pool_branch_forward(x, w_pool, b_pool=None, b_out=None, parts=None):
    """x [B, ..., D] -> (m [B, D] in x's dtype: the per-image mean; rowbias fp32 [B, D] = m @ w_pool^T + b_pool + b_out).
    parts (fp32 [B * n, D], n equal-sized chunk sums per image, from dense_forward(colsum=True)) replaces the
    pass over x."""
    dev = _lib.require_device(x, w_pool)
    B, D = x.shape[0], x.shape[-1]
    P = x.numel() // max(B * D, 1)
    m = torch.empty((B, D), device=dev, dtype=x.dtype)
    rowbias = torch.empty((B, D), device=dev, dtype=torch.float32)
    if B and P and parts is not None:
        _launch("pdw_pool_branch_fwd_parts", dev, parts.data_ptr(), parts.shape[0] // B, w_pool.data_ptr(),
                b_pool.data_ptr() if b_pool is not None else None, b_out.data_ptr() if b_out is not None else None,
                m.data_ptr(), rowbias.data_ptr(), B, P, D, _lib.dtype_code(x.dtype))
    elif B and P:
        ws = _pool_ws(B, P, D, dev)
        _launch("pdw_pool_branch_fwd", dev, x.data_ptr(), w_pool.data_ptr(),
                b_pool.data_ptr() if b_pool is not None else None, b_out.data_ptr() if b_out is not None else None,
                m.data_ptr(), rowbias.data_ptr(), ws.data_ptr(), ws.numel() * 4, B, P, D, _lib.dtype_code(x.dtype))
    return m, rowbias


def pool_branch_backward(gy, m, w_pool, parts=None):
    """-> (gbias [2, D]: the same sums twice, one tensor row for each bias; gw_pool [D, D] in gy's dtype;
    dmean fp32 [B, D]).  parts: chunk sums of gy as in pool_branch_forward."""
    dev = _lib.require_device(gy, m, w_pool)
    B, D = gy.shape[0], gy.shape[-1]
    P = gy.numel() // max(B * D, 1)
    gbias = torch.empty((2, D), device=dev, dtype=gy.dtype)
    gwp = torch.empty((D, D), device=dev, dtype=gy.dtype)
    dmean = torch.empty((B, D), device=dev, dtype=torch.float32)
    ws = _pool_ws(B, P, D, dev)
    if parts is not None:
        _launch("pdw_pool_branch_bwd_parts", dev, parts.data_ptr(), parts.shape[0] // B, m.data_ptr(), w_pool.data_ptr(),
                gbias[0].data_ptr(), gbias[1].data_ptr(), gwp.data_ptr(), dmean.data_ptr(), ws.data_ptr(),
                ws.numel() * 4, B, P, D, _lib.dtype_code(gy.dtype))
        return gbias, gwp, dmean
    _launch("pdw_pool_branch_bwd", dev, gy.data_ptr(), m.data_ptr(), w_pool.data_ptr(), gbias[0].data_ptr(),
            gbias[1].data_ptr(), gwp.data_ptr(), dmean.data_ptr(), ws.data_ptr(), ws.numel() * 4, B, P, D,
            _lib.dtype_code(gy.dtype))
    return gbias, gwp, dmean
