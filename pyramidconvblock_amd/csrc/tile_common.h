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

// Interleaves two pixels (adjacent columns a, b; V channels each) into V dwords (low half = a's channel,
// high half = b's), then clears the halves whose pixel lies outside the image: `mask` has 0xffff in the low
// half if a is inside and 0xffff0000 if b is.  Two byte-permutes per channel pair instead of shifts and selects.
template <typename T, int V>
__device__ __forceinline__ void pack_pairs(const ChanVec<T, V>& a, const ChanVec<T, V>& b, uint32_t mask, uint32_t* out) {
    static_assert(sizeof(T) == 2, "16-bit element types only");
    if constexpr (V % 2 == 0) {
        const uint32_t* aw = reinterpret_cast<const uint32_t*>(&a);
        const uint32_t* bw = reinterpret_cast<const uint32_t*>(&b);
#pragma unroll
        for (int j = 0; j < V / 2; ++j) {
            out[2 * j] = __builtin_amdgcn_perm(bw[j], aw[j], 0x05040100u) & mask;
            out[2 * j + 1] = __builtin_amdgcn_perm(bw[j], aw[j], 0x07060302u) & mask;
        }
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) out[i] = (bits16(a.v[i]) | (bits16(b.v[i]) << 16)) & mask;
    }
}

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
                    if constexpr (PK == 2) {
                        const uint32_t mask = ((rok && cok[0]) ? 0xffffu : 0u) | ((rok && cok[NL - 1]) ? 0xffff0000u : 0u);
                        pack_pairs<T, V>(ld[s][0], ld[s][NL - 1], mask, out);
                    } else {
#pragma unroll
                        for (int i = 0; i < V; ++i)
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

// Software-pipelined form of stage_tile for persistent workgroups: issue() requests the first NPRE staging
// passes of a window (clamped, always valid addresses) and keeps them in registers while the previous tile is
// being computed; commit() packs them into LDS (zeros outside the image / channel range) and stages whatever
// the window has beyond NPRE passes directly.  Thread t owns channel vector t % CV of unit t / CV in pass 0 and
// advances by NTHREADS / CV units per pass, units numbered row-major over the (rows x CPn) window.
// LDS layout: xl[row][unit][CS] (channel fastest), or with CHMAJOR xl[row][channel][pitch] (unit fastest,
// `pitch` >= CPn dwords per channel row), the operand order of the matrix-core kernels.
template <typename T, int CS, int V, int NPRE, bool CHMAJOR = false, int NTHREADS = 256>
struct TileStager {
    static constexpr int PK = PackOf<T>::PK;
    static constexpr int NL = PK;          // pixels loaded per LDS unit
    static constexpr int CV = CS / V;      // channel vectors per unit
    static constexpr int UPP = NTHREADS / CV;  // units per pass of the workgroup
    int scv, sr0, su0, step_r, step_u, CPn, rows, chc, pitch, rpitch;
    bool chok;
    ChanVec<T, V> pre[NPRE][NL];

    // pitch_: dwords per channel row, rpitch_: dwords per staged row (default CS * pitch_), CHMAJOR only
    __device__ __forceinline__ void init(int tid, int c0, int C, int rows_, int CPn_, int pitch_ = 0, int rpitch_ = 0) {
        scv = tid % CV;
        const int tu = tid / CV;
        CPn = CPn_, rows = rows_, pitch = pitch_, rpitch = rpitch_ > 0 ? rpitch_ : CS * pitch_;
        sr0 = tu / CPn, su0 = tu - sr0 * CPn;
        step_r = UPP / CPn, step_u = UPP - step_r * CPn;
        const int ch = c0 + scv * V;
        chok = ch < C;
        chc = chok ? ch : 0;
    }

    // Requests the first NPRE passes of a window.  For 16-bit types the address is the (uniform) image pointer plus
    // an unsigned 32-bit byte offset, which the load takes as it is (no 64-bit arithmetic per load; the callers
    // guard H * W * C < 2^31): the request phase is pure address arithmetic, and everything behind it waits for the
    // data.
    __device__ __forceinline__ void issue(const T* __restrict__ img, int H, int W, int C, int row0, int col0) {
        const char* base = reinterpret_cast<const char*>(img);
        const int WC = W * C;
        int r = sr0, u = su0;
#pragma unroll
        for (int it = 0; it < NPRE; ++it) {
            const int ih = min(max(row0 + min(r, rows - 1), 0), H - 1);
            const int rowoff = ih * WC + chc;
#pragma unroll
            for (int l = 0; l < NL; ++l) {
                const int iw = min(max(col0 + NL * u + l, 0), W - 1);
                if constexpr (sizeof(T) == 2) {  // < 2^31 elements: the byte offset fits 32 bits
                    const unsigned off = (unsigned)(rowoff + iw * C) * 2u;
                    pre[it][l] = *reinterpret_cast<const ChanVec<T, V>*>(base + off);
                } else {
                    pre[it][l] = *reinterpret_cast<const ChanVec<T, V>*>(img + (rowoff + iw * C));
                }
            }
            r += step_r, u += step_u;
            if (u >= CPn) u -= CPn, ++r;
        }
    }

    __device__ __forceinline__ void put(uint32_t* __restrict__ xl, const ChanVec<T, V>* ld, int r, int u, int H, int W,
                                        int row0, int col0) const {
        const int ih = row0 + r;
        const bool rok = chok && ih >= 0 && ih < H;
        const int iw0 = col0 + NL * u;
        const bool ok0 = rok && iw0 >= 0 && iw0 < W;
        const bool ok1 = rok && iw0 + 1 >= 0 && iw0 + 1 < W;
        uint32_t out[V];
        if constexpr (PK == 2) {
            pack_pairs<T, V>(ld[0], ld[NL - 1], (ok0 ? 0xffffu : 0u) | (ok1 ? 0xffff0000u : 0u), out);
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) out[i] = ok0 ? __builtin_bit_cast(uint32_t, ld[0].v[i]) : 0u;
        }
        if constexpr (CHMAJOR) {
            uint32_t* dst = xl + r * rpitch + scv * V * pitch + u;
#pragma unroll
            for (int i = 0; i < V; ++i) dst[i * pitch] = out[i];
        } else {
            uint32_t* dst = xl + (r * CPn + u) * CS + scv * V;
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

    // One prefetched pass at a time, for callers that spread the LDS writes over their compute loop:
    // commit_begin(), then commit_next(.., it, ..) for it = 0 .. NPRE-1 in order.
    int cr, cu;
    __device__ __forceinline__ void commit_begin() { cr = sr0, cu = su0; }
    __device__ __forceinline__ void commit_next(uint32_t* __restrict__ xl, int it, int H, int W, int row0, int col0) {
        if (cr < rows) put(xl, pre[it], cr, cu, H, W, row0, col0);
        cr += step_r, cu += step_u;
        if (cu >= CPn) cu -= CPn, ++cr;
    }

    __device__ __forceinline__ void commit(uint32_t* __restrict__ xl, const T* __restrict__ img, int H, int W, int C,
                                           int row0, int col0) {
        int r = sr0, u = su0;
#pragma unroll
        for (int it = 0; it < NPRE; ++it) {
            if (r < rows) put(xl, pre[it], r, u, H, W, row0, col0);
            r += step_r, u += step_u;
            if (u >= CPn) u -= CPn, ++r;
        }
        if (NPRE * UPP < rows * CPn) {  // window larger than the prefetch depth (uniform branch)
            const T* xb = img + chc;
            while (r < rows) {
                ChanVec<T, V> ld[NL];
                const int ih = min(max(row0 + r, 0), H - 1);
#pragma unroll
                for (int l = 0; l < NL; ++l) {
                    const int iw = min(max(col0 + NL * u + l, 0), W - 1);
                    ld[l] = *reinterpret_cast<const ChanVec<T, V>*>(xb + (ih * W + iw) * C);
                }
                put(xl, ld, r, u, H, W, row0, col0);
                r += step_r, u += step_u;
                if (u >= CPn) u -= CPn, ++r;
            }
        }
    }
};

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
