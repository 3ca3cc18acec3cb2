// Device helpers shared by the LDS-tiled depthwise-convolution kernels: the 16-bit pair
// packing, the dot2 wrappers, the XCD-aware work order and the tile staging routine.
#pragma once
#include "common.h"

namespace pdw {

template <typename T>
struct PackOf {
    static constexpr int PK = 2;
};
template <>
struct PackOf<float> {
    static constexpr int PK = 1;
};

__device__ __forceinline__ float dot2acc(uint32_t a, uint32_t b, float c, bf16_t) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
}
__device__ __forceinline__ float dot2acc(uint32_t a, uint32_t b, float c, f16_t) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
}

__device__ __forceinline__ uint32_t bits16(bf16_t v) { return (uint32_t)__builtin_bit_cast(unsigned short, v); }
__device__ __forceinline__ uint32_t bits16(f16_t v) { return (uint32_t)__builtin_bit_cast(unsigned short, v); }

// XCD-aware work order: consecutive workgroup ids go to the 8 XCDs round-robin, so give each
// XCD a contiguous range of work items (neighbouring tiles of one image share an L2).
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
    const int per = nblocks >> 3;
    if (bid >= (per << 3)) return bid;  // tail that does not fill all 8
    return (bid & 7) * per + (bid >> 3);
}

// Copies a (rows x CPn units) window of one channels-last image into LDS as xl[row][unit][CS]
// dwords, zero outside the image or channel range.  For 16-bit types a unit is a pair of
// adjacent columns packed into one dword per channel (low half = even column); for fp32 a
// unit is one column.  Window origin (row0, col0) may be negative.  All 256 threads take part:
// thread (cv, u, rs) copies channel vector cv of unit u in rows rs, rs+RS, ..., with SU rows of
// loads (clamped, always valid addresses) in flight before the first LDS write.  `ulog` is log2
// of the threads laid along a row of units (a power of two >= CPn when there are enough threads).
template <typename T, int CS, int V, int SU = 4>
__device__ __forceinline__ void stage_tile(uint32_t* __restrict__ xl, const T* __restrict__ img, int H, int W, int C,
                                           int row0, int col0, int rows, int CPn, int ulog, int c0, int tid) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int CV = CS / V;
    constexpr int UT = 256 / CV;
    constexpr int NL = PK;  // pixels loaded per LDS unit
    const int cv = tid % CV, tu = tid / CV;
    const int u0 = tu & ((1 << ulog) - 1), rs = tu >> ulog;
    const int US = 1 << ulog, RS = UT >> ulog;
    const int ch = c0 + cv * V;
    const bool chok = ch < C;
    const int chc = chok ? ch : 0;
    for (int u = u0; u < CPn; u += US) {
        int coff[NL];
        bool cok[NL];
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            const int iw = col0 + NL * u + l;
            cok[l] = chok && iw >= 0 && iw < W;
            coff[l] = min(max(iw, 0), W - 1) * C + chc;
        }
        for (int rb = rs; rb < rows; rb += RS * SU) {
            ChanVec<T, V> ld[SU][NL];
#pragma unroll
            for (int s = 0; s < SU; ++s) {
                const int ih = min(max(row0 + rb + s * RS, 0), H - 1);
                const T* xr = img + (long long)ih * W * C;
#pragma unroll
                for (int l = 0; l < NL; ++l) ld[s][l] = *reinterpret_cast<const ChanVec<T, V>*>(xr + coff[l]);
            }
#pragma unroll
            for (int s = 0; s < SU; ++s) {
                const int r = rb + s * RS;
                if (r < rows) {
                    const int ih = row0 + r;
                    const bool rok = ih >= 0 && ih < H;
                    uint32_t out[V];
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        if constexpr (PK == 2)
                            out[i] = ((rok && cok[0]) ? bits16(ld[s][0].v[i]) : 0u) |
                                     (((rok && cok[NL - 1]) ? bits16(ld[s][NL - 1].v[i]) : 0u) << 16);
                        else
                            out[i] = (rok && cok[0]) ? __builtin_bit_cast(uint32_t, ld[s][0].v[i]) : 0u;
                    }
                    uint32_t* dst = xl + (r * CPn + u) * CS + cv * V;
                    if constexpr (V % 4 == 0) {
#pragma unroll
                        for (int i = 0; i < V; i += 4)
                            *reinterpret_cast<uint4*>(dst + i) = make_uint4(out[i], out[i + 1], out[i + 2], out[i + 3]);
                    } else {
#pragma unroll
                        for (int i = 0; i < V; ++i) dst[i] = out[i];
                    }
                }
            }
        }
    }
}

// Number of persistent workgroups per channel slice for `ntiles` equal tiles, all resident at once
// (at most `max_resident` per CU over 256 CUs): minimises the estimated makespan
// rounds * (1 + 0.15 * (workgroups sharing a CU - 1)), preferring more workgroups on ties.  Returns the
// makespan in units of one tile's stand-alone time through *cost.
inline int pick_chunks(long long ntiles, int slices, int max_resident, double* cost) {
    int best_n = 1;
    double best = -1;
    long long hi = (256LL * max_resident) / slices;
    if (hi < 1) hi = 1;
    if (hi > ntiles) hi = ntiles;
    for (long long cand = 1; cand <= hi; ++cand) {
        const long long per_cu = (cand * slices + 255) / 256;
        const double t = (double)((ntiles + cand - 1) / cand) * (1.0 + 0.15 * (per_cu - 1));
        if (best < 0 || t <= best + 1e-9) best = t, best_n = (int)cand;
    }
    if (cost) *cost = best;
    return best_n;
}

// log2 of the staging threads laid along a row of CPn units (see stage_tile).
inline int stage_ulog(int CPn, int CS, int V) {
    const int ut = 256 / (CS / V);
    int ulog = 0;
    while ((1 << ulog) < CPn && (2 << ulog) <= ut) ++ulog;
    return ulog;
}

}  // namespace pdw
