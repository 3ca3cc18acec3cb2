// The pyramid block of conv_block.py:25-49 as one host call each way: the launch sequence that the Python operator
// makes through the single entry points (3 or 4 launches forward, 6 backward), for callers that cannot afford an
// interpreter between launches.  Host code only: every step is one of the library's own entry points, in the order
// and with the arguments of pyramidconvblock_amd/conv_block.py, so the results are bitwise the same.
#include <stdint.h>

#include "../../include/pdw.h"
#include "common.h"
#include "kernels.h"

namespace {

using namespace pdw;

size_t up256(size_t b) { return (b + 255) & ~(size_t)255; }

// Hands out 256-byte aligned pieces of the caller's workspace.
struct Carver {
    char* p;
    size_t left;
    bool ok = true;
    void* take(size_t bytes) {
        bytes = up256(bytes);
        if (bytes > left) {
            ok = false;
            return nullptr;
        }
        void* r = p;
        p += bytes, left -= bytes;
        return r;
    }
};

struct Shape {
    int B, H, W, D, I, K, dtype;
    int h, w, P, R, es;
    long long N, nt;  // rows of the dense layers, row tiles (chunk sums)
};

Shape shape_of(int B, int H, int W, int D, int I, int K, int dtype) {
    Shape s{B, H, W, D, I, K, dtype, H / 2, W / 2, H * W, pdw_dense_colsum_rows(), 2, 0, 0};
    s.N = (long long)B * H * W;
    s.nt = (s.N + s.R - 1) / s.R;
    return s;
}

}  // namespace

extern "C" {

int pdw_convblock_supported(int B, int H, int W, int D, int I, int K, int dtype) {
    if (dtype != kF16 && dtype != kBF16) return 0;
    if (B < 1 || H < 4 || W < 4 || (H & 1) || (W & 1) || K < 1 || !(K & 1) || D < 8 || I < 16 || (I & 15)) return 0;
    if ((long long)B * H * W * (D > I ? D : I) > 0x7fffffffLL) return 0;
    if ((H * W) % pdw_dense_colsum_rows()) return 0;
    return pdw_dense_supported(D, I, dtype) && pdw_dense_supported(I, D, dtype) && pdw_dense_colsum_supported(D, I, dtype) &&
           pdw_dense_bwd_pair_colsum_supported(D, I, dtype) && pdw_dense_bwd_pair_supported(I, D, dtype);
}

size_t pdw_convblock_fwd_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype)) return 0;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    return up256((size_t)s.nt * D * 4) + up256((size_t)B * D * 4);
}

int pdw_convblock_fwd(const void* x, const void* w_up, const void* w_dw0, const void* w_dw1, const void* w_pool,
                      const void* b_pool, const void* w_out, const void* b_out, void* a, void* c0, void* xp, void* c1,
                      void* cat, void* m, void* y, void* workspace, size_t workspace_bytes, int B, int H, int W, int D,
                      int I, int K, int dtype, void* stream) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype))
        return set_error("pdw_convblock_fwd: shape not covered (B=%d H=%d W=%d D=%d I=%d K=%d dtype=%d)", B, H, W, D, I, K,
                         dtype), 1;
    for (const void* ptr : {x, w_up, w_dw0, w_dw1, w_pool, w_out, (const void*)a, (const void*)c0, (const void*)xp,
                            (const void*)c1, (const void*)cat, (const void*)m, (const void*)y, (const void*)workspace})
        if (!ptr) return set_error("pdw_convblock_fwd: null pointer"), 1;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    if (workspace_bytes < pdw_convblock_fwd_workspace_bytes(B, H, W, D, I, K, dtype))
        return set_error("pdw_convblock_fwd: workspace of %zu bytes given, %zu needed", workspace_bytes,
                         pdw_convblock_fwd_workspace_bytes(B, H, W, D, I, K, dtype)), 1;
    Carver ws{(char*)workspace, workspace_bytes};
    float* xparts = (float*)ws.take((size_t)s.nt * D * 4);  // sums of x over each row tile
    float* yp = (float*)ws.take((size_t)B * D * 4);         // mean branch: one row per image
    const int pad = K / 2;
    // conv_up, with the tile sums of x for the mean branch                                   (conv_block.py:37, 46)
    // (where the layer's kernel can also pool its result for the second scale, the convolutions need no pooling launch)
    const bool two = pdw_dwconv_fwd2_supported(B, H, W, I, K, dtype) != 0;
    int pooled = 3;
    if (two) {
        pooled = pdw_dense_fwd_colsum_pool(x, w_up, nullptr, a, xparts, xp, B, H, W, D, I, dtype, stream);
        if (pooled != 0 && pooled != 3) return pooled;
    }
    if (pooled == 3)
        if (int e = pdw_dense_fwd_colsum(x, w_up, 0, nullptr, nullptr, a, xparts, s.N, D, I, s.P, dtype, stream)) return e;
    // the second scale's input, then the convolutions of both scales as one launch; where that launch does not take the
    // shape, the full-resolution conv also pools its input and the second scale's follows   (conv_block.py:14-16)
    int both = 3;
    bool mean_done = false;
    if (two) {
        if (pooled == 3)
            if (int e = pdw_avgpool_fwd(a, xp, B, H, W, I, s.h, s.w, dtype, stream)) return e;
        // (with the mean branch in the same launch where that is covered: mean -> conv_pool (+ both biases) into yp)
        both = pdw_dwconv_fwd2_mean(a, w_dw0, c0, 0, 0, xp, w_dw1, c1, 0, 0, B, H, W, I, K, xparts, (int)(s.nt / B), w_pool,
                                    b_pool, b_out, m, yp, s.P, D, dtype, stream);
        if (both != 0 && both != 3) return both;
        mean_done = both == 0;
        if (both == 3) both = pdw_dwconv_fwd2(a, w_dw0, c0, xp, w_dw1, c1, B, H, W, I, K, dtype, stream);
        if (both != 0 && both != 3) return both;
        if (both == 3)
            if (int e = pdw_dwconv_fwd(a, w_dw0, c0, B, H, W, I, K, K, 1, 1, pad, pad, 1, 1, dtype, stream)) return e;
    } else if (int e = pdw_dwconv_fwd_pool(a, w_dw0, c0, xp, B, H, W, I, K, K, 1, 1, pad, pad, 1, 1, s.h, s.w, dtype, stream)) {
        return e;
    }
    if (both == 3)
        if (int e = pdw_dwconv_fwd(xp, w_dw1, c1, B, s.h, s.w, I, K, K, 1, 1, pad, pad, 1, 1, dtype, stream)) return e;
    if (mean_done) {
        // conv_out on rows it makes itself (both gates, the resize), written to cat for the backward; where its kernel
        // does not cover the widths, the gates' launch and the plain layer                   (conv_block.py:40-44, 49)
        const int r = pdw_dense_fwd_gated(c0, c1, cat, w_out, nullptr, yp, y, B, H, W, I, D, 0, dtype, stream);
        if (r != 3) return r;
        if (int e = pdw_gate_pair_fwd(c0, c1, cat, B, H, W, s.h, s.w, I, I, dtype, stream)) return e;
        return pdw_dense_fwd(cat, w_out, 0, nullptr, yp, y, s.N, I, D, s.P, dtype, stream);
    }
    // both gates into cat, mean -> conv_pool (+ both biases) into yp                          (conv_block.py:40-49)
    if (int e = pdw_block_mid_fwd(c0, c1, cat, B, H, W, s.h, s.w, I, I, xparts, (int)(s.nt / B), w_pool, b_pool, b_out, m,
                                  yp, s.P, D, dtype, stream))
        return e;
    // conv_out plus the per-image row                                                        (conv_block.py:44, 49)
    return pdw_dense_fwd(cat, w_out, 0, nullptr, yp, y, s.N, I, D, s.P, dtype, stream);
}

// The convolution with the gate in its store, for the widths conv_out's made-rows kernel does not cover: images small
// enough for the kernel's 32-bit offsets (two images side by side), and filters up to 13 (with the 8-channel slices of
// larger filters the gated store's 8-byte loads cost more than they save: 62.6 against 54.7 us for the forward at
// [8,112,112,96], K = 17, so those run the training forward's launches on workspace tensors).
static bool infer_fused(int H, int W, int I, int K) { return K <= 13 && (long long)H * W * I * 2 <= 0x1fffffffLL; }
// conv_out on rows it makes itself from the convolution outputs (pdw_dense_fwd_gated), after the convolutions of both
// scales as one launch: every odd K.
static bool infer_made_rows(int B, int H, int W, int D, int I, int K, int dtype) {
    return pdw_dense_fwd_gated_supported(H, W, I, D, dtype) != 0 && pdw_dwconv_fwd2_supported(B, H, W, I, K, dtype) != 0;
}

size_t pdw_convblock_infer_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype)) return 0;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    const size_t full = (size_t)s.N * I * s.es, half = (size_t)B * s.h * s.w * I * s.es;
    size_t b = up256(full) /* a */ + up256(half) /* xp */ + up256(full) /* cat */ + up256((size_t)B * D * s.es) /* m */ +
               up256((size_t)s.nt * D * 4) + up256((size_t)B * D * 4);
    if (infer_made_rows(B, H, W, D, I, K, dtype) || infer_fused(H, W, I, K))
        b += up256(half);  // the gated half-resolution scale, or the half scale's convolution output
    else
        b += up256(full) + up256(half);  // c0, c1
    return b;
}

int pdw_convblock_infer(const void* x, const void* w_up, const void* w_dw0, const void* w_dw1, const void* w_pool,
                        const void* b_pool, const void* w_out, const void* b_out, void* y, void* workspace,
                        size_t workspace_bytes, int B, int H, int W, int D, int I, int K, int dtype, void* stream) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype))
        return set_error("pdw_convblock_infer: shape not covered (B=%d H=%d W=%d D=%d I=%d K=%d dtype=%d)", B, H, W, D, I,
                         K, dtype), 1;
    for (const void* ptr : {x, w_up, w_dw0, w_dw1, w_pool, w_out, (const void*)y, (const void*)workspace})
        if (!ptr) return set_error("pdw_convblock_infer: null pointer"), 1;
    const size_t need = pdw_convblock_infer_workspace_bytes(B, H, W, D, I, K, dtype);
    if (workspace_bytes < need)
        return set_error("pdw_convblock_infer: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    const size_t full = (size_t)s.N * I * s.es, half = (size_t)B * s.h * s.w * I * s.es;
    Carver ws{(char*)workspace, workspace_bytes};
    void* a = ws.take(full);
    void* xp = ws.take(half);
    void* cat = ws.take(full);
    void* m = ws.take((size_t)B * D * s.es);
    float* xparts = (float*)ws.take((size_t)s.nt * D * 4);
    float* yp = (float*)ws.take((size_t)B * D * 4);
    const int pad = K / 2, G = I / 2;
    if (infer_made_rows(B, H, W, D, I, K, dtype) && !(reinterpret_cast<uintptr_t>(w_out) & 15)) {
        // three launches (four where conv_up's kernel does not pool): conv_up (with the tile sums of x and the pool of its result), the convolutions of both scales
        // with the mean branch, conv_out on rows made from their outputs, which pass through the workspace (measured:
        // as fast as gating them in the convolutions' stores at K <= 13, 2 us faster at K = 17)   (conv_block.py:36-49)
        void* c0 = cat;
        void* c1 = ws.take(half);
        int r = pdw_dense_fwd_colsum_pool(x, w_up, nullptr, a, xparts, xp, B, H, W, D, I, dtype, stream);
        if (r == 3) {   // (widths whose conv_up kernel does not pool: the layer with its tile sums, then the pool)
            if ((r = pdw_dense_fwd_colsum(x, w_up, 0, nullptr, nullptr, a, xparts, s.N, D, I, s.P, dtype, stream))) return r;
            r = pdw_avgpool_fwd(a, xp, B, H, W, I, s.h, s.w, dtype, stream);
        }
        if (r) return r;
        r = pdw_dwconv_fwd2_mean(a, w_dw0, c0, 0, 0, xp, w_dw1, c1, 0, 0, B, H, W, I, K, xparts, (int)(s.nt / B), w_pool,
                                     b_pool, b_out, m, yp, s.P, D, dtype, stream);
        if (r == 3) {   // (a mean branch the riding form does not cover, e.g. an unaligned conv_pool weight)
            if ((r = pdw_dwconv_fwd2(a, w_dw0, c0, xp, w_dw1, c1, B, H, W, I, K, dtype, stream))) return r;
            r = pdw_pool_branch_fwd_parts(xparts, (int)(s.nt / B), w_pool, b_pool, b_out, m, yp, B, s.P, D, dtype, stream);
        }
        if (r) return r;
        return pdw_dense_fwd_gated(c0, c1, nullptr, w_out, nullptr, yp, y, B, H, W, I, D, 0, dtype, stream);
    }
    if (!infer_fused(H, W, I, K)) {
        void* c0 = ws.take(full);
        void* c1 = ws.take(half);
        // the forward's own launches; its workspace is xparts and yp, which lie next to each other
        return pdw_convblock_fwd(x, w_up, w_dw0, w_dw1, w_pool, b_pool, w_out, b_out, a, c0, xp, c1, cat, m, y, xparts,
                                 up256((size_t)s.nt * D * 4) + up256((size_t)B * D * 4), B, H, W, D, I, K, dtype, stream);
    }
    void* g1 = ws.take(half);
    // conv_up; where its kernel can also pool its result, the gated convolutions of both scales follow as one launch
    // (scale 1 into cat[..., :G], scale 1/2 into g1)                                        (conv_block.py:14-19, 37)
    int both = 3;
    if (pdw_dwconv_fwd2_supported(B, H, W, I, K, dtype)) {
        const int pooled = pdw_dense_fwd_colsum_pool(x, w_up, nullptr, a, xparts, xp, B, H, W, D, I, dtype, stream);
        if (pooled != 0 && pooled != 3) return pooled;
        if (pooled == 0) {
            both = pdw_dwconv_fwd2_gate(a, w_dw0, cat, I, 0, xp, w_dw1, g1, G, 0, B, H, W, I, K, dtype, stream);
            if (both != 0 && both != 3) return both;
        } else if (int e = pdw_dense_fwd_colsum(x, w_up, 0, nullptr, nullptr, a, xparts, s.N, D, I, s.P, dtype, stream)) {
            return e;
        }
        if (both == 3 && pooled == 0) {   // the pool is there: the two gated convolutions one after the other
            if (int e = pdw_dwconv_fwd_gate(a, w_dw0, cat, nullptr, B, H, W, I, K, pad, I, 0, dtype, stream)) return e;
            if (int e = pdw_dwconv_fwd_gate(xp, w_dw1, g1, nullptr, B, s.h, s.w, I, K, pad, G, 0, dtype, stream)) return e;
            both = 0;
        }
    } else if (int e = pdw_dense_fwd_colsum(x, w_up, 0, nullptr, nullptr, a, xparts, s.N, D, I, s.P, dtype, stream)) {
        return e;
    }
    if (both == 3) {
        // scale 1: conv + gate into cat[..., :G], and the pooled input of scale 1/2            (conv_block.py:14-19)
        // (the convolution's staging threads hold whole pool windows only when the padding is even)
        const bool pool_fused = (pad & 1) == 0 && K <= 13;   // (with 16 channels per workgroup only)
        if (int e = pdw_dwconv_fwd_gate(a, w_dw0, cat, pool_fused ? xp : nullptr, B, H, W, I, K, pad, I, 0, dtype, stream))
            return e;
        if (!pool_fused)
            if (int e = pdw_avgpool_fwd(a, xp, B, H, W, I, s.h, s.w, dtype, stream)) return e;
        // scale 1/2: conv + gate, upsampled into cat[..., G:]                                   (conv_block.py:17-21)
        if (int e = pdw_dwconv_fwd_gate(xp, w_dw1, g1, nullptr, B, s.h, s.w, I, K, pad, G, 0, dtype, stream)) return e;
    }
    // ... together with mean -> conv_pool (+ both biases) into yp                             (conv_block.py:46-49)
    if (int e = pdw_block_mid_infer(g1, (char*)cat + (size_t)G * s.es, B, H, W, s.h, s.w, G, I, xparts, (int)(s.nt / B),
                                    w_pool, b_pool, b_out, m, yp, s.P, D, dtype, stream))
        return e;
    return pdw_dense_fwd(cat, w_out, 0, nullptr, yp, y, s.N, I, D, s.P, dtype, stream);
}

size_t pdw_convblock_bwd_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype)) return 0;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    const int pad = K / 2;
    const size_t full = (size_t)s.N * I * s.es, half = (size_t)B * s.h * s.w * I * s.es;
    return up256(full) /* dcat */ + up256((size_t)s.nt * D * 4) /* gparts */ +
           up256(pdw_dense_wgrad_workspace_bytes(s.N, D, I)) + up256(full) /* gcf */ + up256(half) /* gch */ +
           up256((size_t)2 * D * s.es) /* gbias */ + up256((size_t)B * D * 4) /* dmean */ +
           up256(pdw_pool_branch_workspace_bytes(B, s.P, D)) +
           up256(pdw_dwconv_wgrad_workspace_bytes(B, H, W, I, K, K, 1, 1, pad, pad, 1, 1, dtype)) +
           up256(pdw_dwconv_wgrad_workspace_bytes(B, s.h, s.w, I, K, K, 1, 1, pad, pad, 1, 1, dtype)) +
           up256(half) /* dxp */ + up256(full) /* da */ + up256(pdw_dense_wgrad_workspace_bytes(s.N, I, D));
}

int pdw_convblock_bwd(const void* gy, const void* x, const void* a, const void* c0, const void* xp, const void* c1,
                      const void* cat, const void* m, const void* w_up, const void* w_dw0, const void* w_dw1,
                      const void* w_pool, const void* w_out, void* dx, void* gw_up, void* gw_dw0, void* gw_dw1,
                      void* gw_pool, void* gb_pool, void* gw_out, void* gb_out, void* workspace, size_t workspace_bytes,
                      int B, int H, int W, int D, int I, int K, int dtype, void* stream) {
    if (!pdw_convblock_supported(B, H, W, D, I, K, dtype))
        return set_error("pdw_convblock_bwd: shape not covered (B=%d H=%d W=%d D=%d I=%d K=%d dtype=%d)", B, H, W, D, I, K,
                         dtype), 1;
    for (const void* ptr : {gy, x, a, c0, xp, c1, cat, m, w_up, w_dw0, w_dw1, w_pool, w_out, (const void*)dx,
                            (const void*)gw_up, (const void*)gw_dw0, (const void*)gw_dw1, (const void*)gw_pool,
                            (const void*)gw_out, (const void*)workspace})
        if (!ptr) return set_error("pdw_convblock_bwd: null pointer"), 1;
    const size_t need = pdw_convblock_bwd_workspace_bytes(B, H, W, D, I, K, dtype);
    if (workspace_bytes < need)
        return set_error("pdw_convblock_bwd: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    const Shape s = shape_of(B, H, W, D, I, K, dtype);
    const int pad = K / 2;
    const size_t full = (size_t)s.N * I * s.es, half = (size_t)B * s.h * s.w * I * s.es;
    Carver ws{(char*)workspace, workspace_bytes};
    void* dcat = ws.take(full);
    float* gparts = (float*)ws.take((size_t)s.nt * D * 4);
    const size_t b_po = pdw_dense_wgrad_workspace_bytes(s.N, D, I);
    void* ws_po = ws.take(b_po);
    void* gcf = ws.take(full);
    void* gch = ws.take(half);
    char* gbias = (char*)ws.take((size_t)2 * D * s.es);
    float* dmean = (float*)ws.take((size_t)B * D * 4);
    const size_t b_pool_ws = pdw_pool_branch_workspace_bytes(B, s.P, D);
    void* ws_pool = ws.take(b_pool_ws);
    const size_t b_w0 = pdw_dwconv_wgrad_workspace_bytes(B, H, W, I, K, K, 1, 1, pad, pad, 1, 1, dtype);
    const size_t b_w1 = pdw_dwconv_wgrad_workspace_bytes(B, s.h, s.w, I, K, K, 1, 1, pad, pad, 1, 1, dtype);
    void* ws_w0 = ws.take(b_w0);
    void* ws_w1 = ws.take(b_w1);
    void* dxp = ws.take(half);
    void* da = ws.take(full);
    const size_t b_pu = pdw_dense_wgrad_workspace_bytes(s.N, I, D);
    void* ws_pu = ws.take(b_pu);
    if (!ws.ok) return set_error("pdw_convblock_bwd: workspace layout exceeds %zu bytes", workspace_bytes), 1;

    // the final summations of all weight gradients run as one launch at the end
    if (int e = pdw_reduce_defer_begin()) return e;
    int e = 0;
    do {
        // conv_out: gradient of cat, weight gradient, and the tile sums of gy for the mean branch   (conv_block.py:44)
        if ((e = pdw_dense_bwd_pair(gy, w_out, cat, dcat, gparts, gw_out, ws_po, up256(b_po), nullptr, 1, s.N, D, I,
                                    dtype, stream)))
            break;
        // both gates and the mean branch                                                            (conv_block.py:40-49)
        if ((e = pdw_block_mid_bwd(dcat, c0, c1, gcf, gch, B, H, W, s.h, s.w, I, I, gparts, (int)(s.nt / B), m, w_pool,
                                   gb_out ? gb_out : (void*)gbias, gb_pool ? gb_pool : (void*)(gbias + (size_t)D * s.es),
                                   gw_pool, dmean, ws_pool, up256(b_pool_ws), s.P, D, dtype, stream)))
            break;
        // depthwise convs: the pooled scale's input gradient, then the full scale's (which adds it) together with the
        // weight gradients of both scales in one launch where that is covered
        {
            if ((e = pdw_dwconv_dgrad(gch, w_dw1, dxp, B, s.h, s.w, I, K, K, 1, 1, pad, pad, 1, 1, dtype, stream))) break;
            const int r = pdw_dwconv_bwd3(gcf, w_dw0, dxp, da, a, gw_dw0, ws_w0, up256(b_w0), xp, gch, gw_dw1, ws_w1,
                                          up256(b_w1), B, H, W, I, K, dtype, stream);
            if (r != 0 && r != 3) {
                e = r;
                break;
            }
            if (r == 0) {
                e = pdw_dense_bwd_pair(da, w_up, x, dx, nullptr, gw_up, ws_pu, up256(b_pu), dmean, s.P, s.N, I, D, dtype, stream);
                break;
            }
        }
        // otherwise: weight gradients of both scales, then the full scale's input gradient
        if ((e = pdw_dwconv_wgrad_pair(a, gcf, gw_dw0, ws_w0, up256(b_w0), H, W, xp, gch, gw_dw1, ws_w1, up256(b_w1), s.h,
                                       s.w, B, I, K, dtype, stream)))
            break;
        if ((e = pdw_dwconv_dgrad_addpool(gcf, w_dw0, dxp, da, B, H, W, I, K, K, 1, 1, pad, pad, 1, 1, s.h, s.w, dtype,
                                          stream)))
            break;
        // conv_up: input gradient (plus the mean branch's per-image term) and weight gradient        (conv_block.py:37)
        e = pdw_dense_bwd_pair(da, w_up, x, dx, nullptr, gw_up, ws_pu, up256(b_pu), dmean, s.P, s.N, I, D, dtype, stream);
    } while (false);
    const int f = pdw_reduce_defer_flush(stream);  // also ends the deferral after an error
    return e ? e : f;
}

}  // extern "C"
