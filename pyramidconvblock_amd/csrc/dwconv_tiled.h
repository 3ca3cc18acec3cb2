// LDS-tiled depthwise convolution for stride 1, dilation 1, odd kernel width: forward and
// input gradient (the same kernel run on gy with the 180-degree rotated filter and padding
// k-1-p).
//
// Mapping.  A workgroup of 4 wavefronts owns a TH x TW tile of output pixels for a slice of
// CS channels.  A lane is a channel: lane l works on channel l % CS of patch group l / CS, so
// every LDS read of a wavefront is a run of consecutive dwords (no bank conflicts) and the
// staging copy from channels-last global memory is a straight 16-byte-vector copy.  Each
// lane computes a patch of Q rows x R columns of outputs with a register sliding window:
// one LDS read of a row segment feeds R * KW multiply-adds.
//
// 16-bit types.  Pixels are staged in LDS as column pairs, dword (x[.., 2m], x[.., 2m+1]) per
// channel, and the filter row as tap pairs, so one v_dot2_f32_{bf16,f16} does two taps with
// fp32 accumulation (products of 16-bit values are exact in fp32).  Even output columns use
// tap pairs (w0,w1),(w2,w3),..,(w_{K-1},0); odd output columns use the same pixel pairs with
// (0,w0),(w1,w2),..,(w_{K-2},w_{K-1}), built from the former with one v_alignbit each.
// fp32 uses the same structure with single columns and v_fma_f32.
//
// A zero tap multiplies the pixel one column outside the window, so a non-finite value there
// would leak into the output (0 * inf); finite inputs are unaffected.
#pragma once
#include <stdlib.h>

#include "common.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

struct TiledGeom {
    int H, W, C;      // input extents
    int OH, OW;       // output extents
    int KH;           // filter rows (filter columns are the template parameter)
    int PH, PW;       // padding
    int NRG, NST;     // tile = (Q*NRG) rows x (R*NST) columns of outputs
    int tiles_h, tiles_w, slices, batch;
    int CPn;          // LDS column units per staged row
    int rows_in;      // staged rows = Q*NRG + KH - 1
    int flip;         // 1: use the 180-degree rotated filter (input gradient)
    int ulog;         // log2 of the staging threads laid along a row of LDS units
};

template <typename T, int KW, int R, int Q, int CS, int V>
__global__ __launch_bounds__(256) void dwconv_tiled_k(const T* __restrict__ x, const T* __restrict__ w,
                                                      T* __restrict__ y, const TiledGeom g) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int NP = (KW + PK - 1) / PK;  // filter units per row (tap pairs or taps)
    constexpr int RU = R / PK;              // output units per patch row
    constexpr int XU = RU + NP - 1;         // staged units read per patch row
    constexpr int NG = 64 / CS;
    static_assert(R % 2 == 0 && 64 % CS == 0 && CS % V == 0, "bad tile parameters");
    extern __shared__ uint32_t smem[];
    uint32_t* xl = smem;                                  // [rows_in][CPn][CS]
    uint32_t* wl = smem + g.rows_in * g.CPn * CS;         // [KH][NP][CS]

    int item = xcd_remap(blockIdx.x, gridDim.x);
    const int tw = item % g.tiles_w;
    item /= g.tiles_w;
    const int th = item % g.tiles_h;
    item /= g.tiles_h;
    const int sl = item % g.slices;
    const int b = item / g.slices;
    const int c0 = sl * CS;
    const int orow0 = th * (Q * g.NRG), ocol0 = tw * (R * g.NST);
    const int irow0 = orow0 - g.PH, icol0 = ocol0 - g.PW;
    const int tid = threadIdx.x;

    // ---- stage the filter slice: wl[kh][m][c] = unit m of (rotated) filter row kh.
    // Thread (c, mt) walks the filter rows; SU rows are loaded (clamped, always valid addresses)
    // before the first LDS write waits, so the global latency is paid once per batch.
    {
        constexpr int MT = 256 / CS;
        constexpr int SU = 4;
        const int c = tid % CS, mt = tid / CS;
        const int ch = min(c0 + c, g.C - 1);
        const bool chok = c0 + c < g.C;
        for (int m = mt; m < NP; m += MT) {
            int s0, s1;
            if constexpr (PK == 2) {
                const int k0 = 2 * m, k1 = min(2 * m + 1, KW - 1);
                s0 = g.flip ? KW - 1 - k0 : k0, s1 = g.flip ? KW - 1 - k1 : k1;
            } else {
                s0 = g.flip ? KW - 1 - m : m, s1 = s0;
            }
            const bool hi_ok = PK == 2 && 2 * m + 1 < KW;
            for (int kb = 0; kb < g.KH; kb += SU) {
                uint32_t lo[SU], hi[SU];
#pragma unroll
                for (int s = 0; s < SU; ++s) {
                    const int kh = min(kb + s, g.KH - 1);
                    const int skh = g.flip ? g.KH - 1 - kh : kh;
                    const T* wr = w + (skh * KW) * g.C + ch;
                    if constexpr (PK == 2) {
                        lo[s] = bits16(wr[s0 * g.C]);
                        hi[s] = bits16(wr[s1 * g.C]);
                    } else {
                        lo[s] = __builtin_bit_cast(uint32_t, wr[s0 * g.C]);
                        hi[s] = 0;
                    }
                }
#pragma unroll
                for (int s = 0; s < SU; ++s) {
                    if (kb + s < g.KH) {
                        const uint32_t v = lo[s] | ((hi_ok ? hi[s] : 0u) << 16);
                        wl[((kb + s) * NP + m) * CS + c] = chok ? v : 0u;
                    }
                }
            }
        }
    }

    // ---- stage the input tile with its halo (zeros outside the image / channel range)
    stage_tile<T, CS, V>(xl, x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, irow0, icol0, g.rows_in, g.CPn,
                         g.ulog, c0, tid);
    __syncthreads();

    // ---- compute: each (wave, lane group) slot walks the tile's patches
    const int lane = tid & 63, wv = tid >> 6;
    const int c = lane % CS, grp = lane / CS;
    const int slot = wv * NG + grp;
    const int npatch = g.NRG * g.NST;
    const int rowstride = g.CPn * CS;
    for (int p0 = 0; p0 < npatch; p0 += 4 * NG) {
        const bool valid = p0 + slot < npatch;
        const int p = valid ? p0 + slot : npatch - 1;
        const int rg = p / g.NST, st = p % g.NST;
        float acc[Q][R];
#pragma unroll
        for (int q = 0; q < Q; ++q)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[q][r] = 0.f;
        const uint32_t* xbase = xl + (rg * Q) * rowstride + (st * RU) * CS + c;
        const uint32_t* wbase = wl + c;
#pragma unroll 1
        for (int kh = 0; kh < g.KH; ++kh) {
            uint32_t wa[NP];
#pragma unroll
            for (int m = 0; m < NP; ++m) wa[m] = wbase[(kh * NP + m) * CS];
            if constexpr (PK == 2) {
                uint32_t wb[NP];
                wb[0] = wa[0] << 16;
#pragma unroll
                for (int m = 1; m < NP; ++m) wb[m] = __builtin_amdgcn_alignbit(wa[m], wa[m - 1], 16);
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const uint32_t* xr = xbase + (kh + q) * rowstride;
                    uint32_t xp[XU];
#pragma unroll
                    for (int i = 0; i < XU; ++i) xp[i] = xr[i * CS];
#pragma unroll
                    for (int t = 0; t < RU; ++t)
#pragma unroll
                        for (int m = 0; m < NP; ++m) {
                            acc[q][2 * t] = dot2acc(xp[t + m], wa[m], acc[q][2 * t], T());
                            acc[q][2 * t + 1] = dot2acc(xp[t + m], wb[m], acc[q][2 * t + 1], T());
                        }
                }
            } else {
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const uint32_t* xr = xbase + (kh + q) * rowstride;
                    float xp[XU];
#pragma unroll
                    for (int i = 0; i < XU; ++i) xp[i] = __builtin_bit_cast(float, xr[i * CS]);
#pragma unroll
                    for (int t = 0; t < R; ++t)
#pragma unroll
                        for (int m = 0; m < NP; ++m)
                            acc[q][t] = fmaf(xp[t + m], __builtin_bit_cast(float, wa[m]), acc[q][t]);
                }
            }
        }
        // ---- store (one rounding to T)
        const int ch = c0 + c;
        if (valid && ch < g.C) {
            const int orow_b = orow0 + rg * Q, ocol_b = ocol0 + st * R;
            T* yp = y + (((long long)b * g.OH + orow_b) * g.OW + ocol_b) * g.C + ch;
            if (orow_b + Q <= g.OH && ocol_b + R <= g.OW) {
#pragma unroll
                for (int q = 0; q < Q; ++q)
#pragma unroll
                    for (int r = 0; r < R; ++r) yp[(q * g.OW + r) * g.C] = from_f32<T>(acc[q][r]);
            } else {
#pragma unroll
                for (int q = 0; q < Q; ++q)
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        if (orow_b + q < g.OH && ocol_b + r < g.OW) yp[(q * g.OW + r) * g.C] = from_f32<T>(acc[q][r]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Host side: tile selection and launch

struct TiledPlan {
    double cost = -1;  // estimated wave-instructions, < 0: no tile fits
    int nrg = 1, nst = 1;
};

template <typename T, int KW, int R, int Q, int CS>
static TiledPlan plan_tiled(int OH, int OW, int KH) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int NP = (KW + PK - 1) / PK;
    // Estimated wave-instructions per workgroup (compute rounds + staging) times the number of
    // workgroups; ragged edges show up as extra workgroups, halo re-reads as staging.
    const int slots = 4 * (64 / CS);
    TiledPlan best;
    for (int nrg = 1; nrg <= 32; ++nrg)
        for (int nst = 1; nst <= 16; ++nst) {
            const int np = nrg * nst;
            if (np > 4 * slots) continue;
            const int th = Q * nrg, tw = R * nst;
            if ((th >= 2 * OH && nrg > 1) || (tw >= 2 * OW && nst > 1)) continue;
            const int rows_in = th + KH - 1, cpn = (tw + KW - 1 + PK - 1) / PK;
            const long long lds = ((long long)rows_in * cpn + (long long)KH * NP) * CS * 4;
            if (lds > 72 * 1024) continue;
            const double nt = (double)cdiv(OH, th) * cdiv(OW, tw);
            const int rounds = cdiv(np, slots);
            const double compute =
                4.0 * rounds * (KH * (Q * R * NP + NP) * (PK == 2 ? 1.06 : 1.0) + 6.0 * Q * R + 60);
            const double stage = rows_in * cpn * (CS / 8) / 64.0 * 40.0 + KH * NP * CS / 64.0 * 14.0 + 150;
            const double cost = nt * (compute + stage);
            if (best.cost < 0 || cost < best.cost) best.cost = cost, best.nrg = nrg, best.nst = nst;
        }
    return best;
}

template <typename T, int KW, int R, int Q, int CS>
static int launch_tiled(const TiledPlan& plan, const void* x, const void* w, void* y, int B, int H, int W, int C,
                        int KH, int PH, int PW, bool flip, hipStream_t s) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int NP = (KW + PK - 1) / PK;
    TiledGeom g;
    g.H = H, g.W = W, g.C = C;
    g.OH = H + 2 * PH - KH + 1, g.OW = W + 2 * PW - KW + 1;
    g.KH = KH, g.PH = PH, g.PW = PW, g.flip = flip ? 1 : 0;
    g.slices = cdiv(C, CS), g.batch = B;
    g.NRG = plan.nrg, g.NST = plan.nst;
    g.tiles_h = cdiv(g.OH, Q * g.NRG), g.tiles_w = cdiv(g.OW, R * g.NST);
    g.rows_in = Q * g.NRG + KH - 1;
    g.CPn = (R * g.NST + KW - 1 + PK - 1) / PK;
    g.ulog = 0;
    const size_t lds = ((size_t)g.rows_in * g.CPn + (size_t)KH * NP) * CS * 4;
    const long long nblocks = (long long)g.tiles_h * g.tiles_w * g.slices * B;
    if (nblocks > 0x7fffffffLL || (long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL)
        return -1;
    const void* ptrs[1] = {x};
    const int vec = pick_vec(C, sizeof(T), ptrs, 1);
#define PDW_GO(V)                                                                                            \
    {                                                                                                        \
        auto kern = dwconv_tiled_k<T, KW, R, Q, CS, V>;                                                      \
        g.ulog = stage_ulog(g.CPn, CS, V);                                                                   \
        static bool attr_done = false;                                                                       \
        if (!attr_done) {                                                                                    \
            (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            attr_done = true;                                                                                \
        }                                                                                                    \
        hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), lds, s, (const T*)x, (const T*)w, (T*)y, g); \
    }
    if constexpr (sizeof(T) == 2) {
        if (vec >= 8) PDW_GO(8) else if (vec >= 4) PDW_GO(4) else PDW_GO(1)
    } else {
        if (vec >= 4) PDW_GO(4) else PDW_GO(1)
    }
#undef PDW_GO
    return check_launch("dwconv_tiled");
}

// Picks the patch shape (R columns x Q rows per lane) with the lowest estimated cost and launches.
template <typename T, int KW>
static int launch_best(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                       bool flip, hipStream_t s) {
    const int OH = H + 2 * PH - KH + 1, OW = W + 2 * PW - KW + 1;
    const TiledPlan p0 = plan_tiled<T, KW, 8, 2, 32>(OH, OW, KH);
    const TiledPlan p1 = plan_tiled<T, KW, 14, 1, 32>(OH, OW, KH);
    const TiledPlan p2 = plan_tiled<T, KW, 14, 2, 32>(OH, OW, KH);
    int pick = -1;
    double best = -1;
    const TiledPlan* ps[3] = {&p0, &p1, &p2};
    for (int i = 0; i < 3; ++i)
        if (ps[i]->cost >= 0 && (best < 0 || ps[i]->cost < best)) best = ps[i]->cost, pick = i;
    const char* force = getenv("PDW_PATCH");
    if (force) pick = atoi(force);
    TiledPlan p = pick >= 0 ? *ps[pick] : p0;
    if (pick < 0 || p.cost < 0) return -1;
    if (getenv("PDW_NRG") && getenv("PDW_NST")) p.nrg = atoi(getenv("PDW_NRG")), p.nst = atoi(getenv("PDW_NST"));
    switch (pick) {
        case 0: return launch_tiled<T, KW, 8, 2, 32>(p, x, w, y, B, H, W, C, KH, PH, PW, flip, s);
        case 1: return launch_tiled<T, KW, 14, 1, 32>(p, x, w, y, B, H, W, C, KH, PH, PW, flip, s);
        default: return launch_tiled<T, KW, 14, 2, 32>(p, x, w, y, B, H, W, C, KH, PH, PW, flip, s);
    }
}

template <int KW>
static int launch_dtype(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                        bool flip, int dtype, hipStream_t s) {
    switch (dtype) {
        case kF32: return launch_best<float, KW>(x, w, y, B, H, W, C, KH, PH, PW, flip, s);
        case kF16: return launch_best<f16_t, KW>(x, w, y, B, H, W, C, KH, PH, PW, flip, s);
        default: return launch_best<bf16_t, KW>(x, w, y, B, H, W, C, KH, PH, PW, flip, s);
    }
}

}  // namespace pdw
