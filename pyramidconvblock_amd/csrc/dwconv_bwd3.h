// The three convolution launches at the end of a two-scale block's backward pass that do not depend on one another
// (the full-scale input gradient with the pooled branch's gradient added, and the weight gradients of both scales) as
// one launch: on a compute unit a band of each runs back to back, without two drains and launch gaps in between.
// The kernel template and its per-filter-size launcher; dwconv_bwd3_k<K>.hip instantiate it, one file per size.
#pragma once
#include "dwconv_tz.h"
#include "dwconv_wgrad_tz.h"
#include "reduce_parts.h"

namespace pdw {

struct Bwd3Args {
    const void *gy, *w, *add;   // input gradient: dx = conv^T(gy, w) + add / 4 (2x2 blocks)
    void* dx;
    const void *x0, *gy0, *x1, *gy1;   // weight gradients
    float *part0, *part1;
    TzGeom gd;
    WgTzGeom g0, g1;
    int nd, n1;
};

// The input gradient's workgroups come first in the grid, then the half scale's weight gradient, then the full scale's.
template <typename T, int K, int CS, int NGA, int NCB1, int NB>
__global__ __launch_bounds__(512, 1) void dwconv_bwd3_k(const Bwd3Args a) {
    const int blk = blockIdx.x;
    if (blk < a.nd)
        dwconv_tz_body<T, K, 16, CS, 1>((const T*)a.gy, (const T*)a.w, (const T*)a.add, nullptr, (T*)a.dx, a.gd, blk, a.nd);
    else if (blk < a.nd + a.n1)
        dwconv_wgrad_tz_body<T, NGA, NCB1, NB>((const T*)a.x1, (const T*)a.gy1, a.part1, a.g1, blk - a.nd, a.n1);
    else
        dwconv_wgrad_tz_body<T, NGA, 8, NB>((const T*)a.x0, (const T*)a.gy0, a.part0, a.g0, blk - a.nd - a.n1,
                                            (int)gridDim.x - a.nd - a.n1);
}

// -1: not covered (the caller makes the three launches).  16-bit types, C % 16 == 0, padding K / 2, the second scale
// exactly half the first, the full scale in the wide tiles of both kernels.
template <int K>
static int launch_bwd3(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0,
                       const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int dtype,
                       hipStream_t s) {
    constexpr int CS = (2 * 4 * TzShape<K, 16, 16>::NM + 2 * 4 * TzShape<K, 16, 16>::RING) <= 160 ? 16 : 8;
    constexpr int NGA0 = (4 + 2 * ((K - 1) / 2) + 3) / 4, NGA = NGA0 < 2 ? 2 : NGA0, NB = K == 17 ? 3 : 2;
    if (dtype == kF32 || C % 16 != 0 || (H & 1) || (W & 1) || B < 1) return -1;
    const int P = K / 2, h = H / 2, wd = W / 2;
    for (const void* p : {gyf, w0, addp, (const void*)dx, x0, (const void*)ws0, x1, gy1, (const void*)ws1})
        if (!p || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    const long long pad16 = (long long)cdiv(W, 64) * 64 * B, pad8 = (long long)cdiv(W, 32) * 32 * cdiv(B, 2) * 2;
    if (pad16 > pad8) return -1;   // the input gradient's wide tile only
    Bwd3Args a;
    long long nd;
    if (!tz_make_geom<K, 16, CS>(a.gd, nd, true, B, H, W, C, K - 1 - P, K - 1 - P, true, nullptr)) return -1;
    const WgTzPlan p0 = wgrad_tz_plan(B, H, W, C, K, P, P), p1 = wgrad_tz_plan(B, h, wd, C, K, P, P);
    if (!p0.ok || !p1.ok || p0.ncb != 8 || wgrad_tz_nga(K) != NGA) return -1;
    if (nd + p0.nblocks + p1.nblocks > 0x7fffffffLL) return -1;
    a.gy = gyf, a.w = w0, a.add = addp, a.dx = dx;
    a.x0 = x0, a.gy0 = gyf, a.x1 = x1, a.gy1 = gy1, a.part0 = (float*)ws0, a.part1 = (float*)ws1;
    a.g0 = p0.g, a.g1 = p1.g, a.nd = (int)nd, a.n1 = (int)p1.nblocks;
    size_t lds = TzShape<K, 16, CS>::lds_bytes;
    if (WgTzShape<NGA, 8, NB>::lds_bytes > lds) lds = WgTzShape<NGA, 8, NB>::lds_bytes;
    if (WgTzShape<NGA, 5, NB>::lds_bytes > lds) lds = WgTzShape<NGA, 5, NB>::lds_bytes;
    const unsigned grid = (unsigned)(nd + p0.nblocks + p1.nblocks);
    static std::once_flag once[4];
#define PDW_BWD3_GO(T, NCB1, SLOT)                                                                                        \
    {                                                                                                                     \
        auto kern = dwconv_bwd3_k<T, K, CS, NGA, NCB1, NB>;                                                               \
        std::call_once(once[SLOT], [&] {                                                                                  \
            (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);         \
        });                                                                                                               \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, s, a);                                                       \
    }
    if (dtype == kF16) {
        if (p1.ncb == 8) PDW_BWD3_GO(f16_t, 8, 0) else PDW_BWD3_GO(f16_t, 5, 1)
    } else {
        if (p1.ncb == 8) PDW_BWD3_GO(bf16_t, 8, 2) else PDW_BWD3_GO(bf16_t, 5, 3)
    }
#undef PDW_BWD3_GO
    if (int e = check_launch("dwconv_bwd3")) return e;
    const int n0 = B * p0.g.nbands * p0.g.ncolt, n1 = B * p1.g.nbands * p1.g.ncolt;
    if (dtype == kF16) {
        if (int e = wgrad_reduce_launch<f16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
        return wgrad_reduce_launch<f16_t>((const float*)ws1, dw1, n1, K * K * C, s);
    }
    if (int e = wgrad_reduce_launch<bf16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
    return wgrad_reduce_launch<bf16_t>((const float*)ws1, dw1, n1, K * K * C, s);
}

}  // namespace pdw
