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
#include <mutex>
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
    int ntiles;       // tiles per channel slice = batch * tiles_h * tiles_w
    int nchunks;      // workgroups per channel slice; workgroup q walks tiles q, q+nchunks, ...
    int step_r, step_u;  // (row, unit) advance of a thread's staging item per pass of 256 threads
};

// Staging passes whose global loads are issued one tile ahead and held in registers while the
// current tile is computed (software pipelining across the persistent tile loop).
constexpr int kPrefetchPasses = 8;

template <typename T, int KW, int R, int Q, int CS, int V>
__global__ __launch_bounds__(256) void dwconv_tiled_k(const T* __restrict__ x, const T* __restrict__ w,
                                                      T* __restrict__ y, const TiledGeom g) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int NP = (KW + PK - 1) / PK;  // filter units per row (tap pairs or taps)
    constexpr int RU = R / PK;              // output units per patch row
    constexpr int XU = RU + NP - 1;         // staged units read per patch row
    constexpr int NG = 64 / CS;
    constexpr int CV = CS / V;              // channel vectors per LDS unit
    constexpr int UPP = 256 / CV;           // LDS units staged per pass of the workgroup
    constexpr int NL = PK;                  // pixels loaded per LDS unit
    constexpr int MAXIT = kPrefetchPasses;
    static_assert(R % 2 == 0 && 64 % CS == 0 && CS % V == 0, "bad tile parameters");
    extern __shared__ uint32_t smem[];
    uint32_t* xl = smem;                                  // [rows_in][CPn][CS]
    uint32_t* wl = smem + g.rows_in * g.CPn * CS;         // [KH][NP][CS]

    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int sl = bid % g.slices, chunk = bid / g.slices;
    const int c0 = sl * CS;
    const int tid = threadIdx.x;
    const int tiles_per_img = g.tiles_h * g.tiles_w;

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

    // ---- staging map of this thread (the same for every tile): channel vector cv of LDS unit
    // (r, u) in pass 0, advancing by (step_r, step_u) units per pass.
    const int scv = tid % CV;
    const int sr0 = (tid / CV) / g.CPn, su0 = (tid / CV) % g.CPn;
    const int sch = c0 + scv * V;
    const bool schok = sch < g.C;
    const int schc = schok ? sch : 0;
    const int nunits = g.rows_in * g.CPn;
    ChanVec<T, V> pre[MAXIT][NL];

    // Issues the global loads of a tile's first MAXIT staging passes (clamped, always valid addresses).
    auto prefetch = [&](int tile) {
        const int b = tile / tiles_per_img, rem = tile % tiles_per_img;
        const int irow0 = (rem / g.tiles_w) * (Q * g.NRG) - g.PH, icol0 = (rem % g.tiles_w) * (R * g.NST) - g.PW;
        const T* xb = x + (long long)b * g.H * g.W * g.C + schc;
        int r = sr0, u = su0;
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            const int ih = min(max(irow0 + min(r, g.rows_in - 1), 0), g.H - 1);
#pragma unroll
            for (int l = 0; l < NL; ++l) {
                const int iw = min(max(icol0 + NL * u + l, 0), g.W - 1);
                pre[it][l] = *reinterpret_cast<const ChanVec<T, V>*>(xb + (ih * g.W + iw) * g.C);
            }
            r += g.step_r, u += g.step_u;
            if (u >= g.CPn) u -= g.CPn, ++r;
        }
    };

    // Packs one staged unit (zeros outside the image / channel range) and writes it to LDS.
    auto put = [&](const ChanVec<T, V>* ld, int r, int u, int irow0, int icol0) {
        const int ih = irow0 + r;
        const bool rok = schok && ih >= 0 && ih < g.H;
        const int iw0 = icol0 + NL * u;
        const bool ok0 = rok && iw0 >= 0 && iw0 < g.W;
        const bool ok1 = rok && iw0 + 1 >= 0 && iw0 + 1 < g.W;
        uint32_t out[V];
        if constexpr (PK == 2) {
            pack_pairs<T, V>(ld[0], ld[NL - 1], (ok0 ? 0xffffu : 0u) | (ok1 ? 0xffff0000u : 0u), out);
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) out[i] = ok0 ? __builtin_bit_cast(uint32_t, ld[0].v[i]) : 0u;
        }
        uint32_t* dst = xl + (r * g.CPn + u) * CS + scv * V;
        if constexpr (V % 4 == 0) {
#pragma unroll
            for (int i = 0; i < V; i += 4)
                *reinterpret_cast<uint4*>(dst + i) = make_uint4(out[i], out[i + 1], out[i + 2], out[i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) dst[i] = out[i];
        }
    };

    // Writes the prefetched passes to LDS and stages any remaining passes directly.
    auto commit = [&](int tile) {
        const int b = tile / tiles_per_img, rem = tile % tiles_per_img;
        const int irow0 = (rem / g.tiles_w) * (Q * g.NRG) - g.PH, icol0 = (rem % g.tiles_w) * (R * g.NST) - g.PW;
        int r = sr0, u = su0;
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if (r < g.rows_in) put(pre[it], r, u, irow0, icol0);
            r += g.step_r, u += g.step_u;
            if (u >= g.CPn) u -= g.CPn, ++r;
        }
        if (MAXIT * UPP < nunits) {  // tiles larger than the prefetch window (uniform branch)
            const T* xb = x + (long long)b * g.H * g.W * g.C + schc;
            for (; r < g.rows_in;) {
                ChanVec<T, V> ld[NL];
                const int ih = min(max(irow0 + r, 0), g.H - 1);
#pragma unroll
                for (int l = 0; l < NL; ++l) {
                    const int iw = min(max(icol0 + NL * u + l, 0), g.W - 1);
                    ld[l] = *reinterpret_cast<const ChanVec<T, V>*>(xb + (ih * g.W + iw) * g.C);
                }
                put(ld, r, u, irow0, icol0);
                r += g.step_r, u += g.step_u;
                if (u >= g.CPn) u -= g.CPn, ++r;
            }
        }
    };

    const int lane = tid & 63, wv = tid >> 6;
    const int c = lane % CS, grp = lane / CS;
    const int slot = wv * NG + grp;
    const int npatch = g.NRG * g.NST;
    const int rowstride = g.CPn * CS;

    int tile = chunk;
    if (tile < g.ntiles) prefetch(tile);
    for (; tile < g.ntiles; tile += g.nchunks) {
    __syncthreads();  // the previous tile is fully consumed (and, first time, the filter is staged)
    commit(tile);
    __syncthreads();
    if (tile + g.nchunks < g.ntiles) prefetch(tile + g.nchunks);  // in flight during the compute below
    const int b = tile / tiles_per_img, rem = tile % tiles_per_img;
    const int orow0 = (rem / g.tiles_w) * (Q * g.NRG), ocol0 = (rem % g.tiles_w) * (R * g.NST);

    // ---- compute: each (wave, lane group) slot walks the tile's patches
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
        if (g.KH == KW) {
            // Square filter: walk the KW+Q-1 staged rows once, fully unrolled.  Row j feeds output row q
            // through filter row j-q, so every LDS row segment is read once per patch and the
            // scheduler is free to issue a row's reads while the previous row's dot products run.
            uint32_t wa[KW][NP], wb[KW][NP];
#pragma unroll
            for (int j = 0; j < KW + Q - 1; ++j) {
                if (j < KW) {
#pragma unroll
                    for (int m = 0; m < NP; ++m) wa[j][m] = wbase[(j * NP + m) * CS];
                    if constexpr (PK == 2) {
                        wb[j][0] = wa[j][0] << 16;
#pragma unroll
                        for (int m = 1; m < NP; ++m) wb[j][m] = __builtin_amdgcn_alignbit(wa[j][m], wa[j][m - 1], 16);
                    }
                }
                const uint32_t* xr = xbase + j * rowstride;
                uint32_t xp[XU];
#pragma unroll
                for (int i = 0; i < XU; ++i) xp[i] = xr[i * CS];
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const int kh = j - q;
                    if (kh >= 0 && kh < KW) {
                        if constexpr (PK == 2) {
#pragma unroll
                            for (int t = 0; t < RU; ++t)
#pragma unroll
                                for (int m = 0; m < NP; ++m) {
                                    acc[q][2 * t] = dot2acc(xp[t + m], wa[kh][m], acc[q][2 * t], T());
                                    acc[q][2 * t + 1] = dot2acc(xp[t + m], wb[kh][m], acc[q][2 * t + 1], T());
                                }
                        } else {
#pragma unroll
                            for (int t = 0; t < R; ++t)
#pragma unroll
                                for (int m = 0; m < NP; ++m)
                                    acc[q][t] = fmaf(__builtin_bit_cast(float, xp[t + m]),
                                                     __builtin_bit_cast(float, wa[kh][m]), acc[q][t]);
                        }
                    }
                }
            }
        } else {
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
        }  // filter-shape branch
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
    }  // tile loop
}

// ------------------------------------------------------------------------------------------------
// Host side: tile selection and launch

struct TiledPlan {
    double cost = -1;  // estimated wave-instructions, < 0: no tile fits
    int nrg = 1, nst = 1;
};

template <typename T, int KW, int R, int Q, int CS>
static TiledPlan plan_tiled(int OH, int OW, int KH, int B, int C) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int NP = (KW + PK - 1) / PK;
    // Estimated wave-instructions per tile (compute rounds + staging) times the makespan, in tiles, of
    // spreading the tiles over the chip (pick_chunks); ragged edges show up as extra tiles, halo re-reads
    // as staging, too few tiles as idle CUs.
    const int slots = 4 * (64 / CS);
    const int slices = cdiv(C, CS);
    TiledPlan best;
    // tiles that leave room for two workgroups per compute unit; where none fits (wide fp32 filters: the filter
    // slice alone is KH * KW * 128 bytes), any tile that fits at all.  fp32 filters from 13 x 13 on choose among all
    // tiles: the ones that leave room for a second workgroup are the 8-column patches, measured half as fast as a
    // 14-column patch with the compute unit to itself (253 against 130 us at [32,56,56,128]; at 9 x 9 the other way)
    const bool fp32_big = sizeof(T) == 4 && (tune_env("PDW_FP32_BIG") ? atoi(tune_env("PDW_FP32_BIG")) != 0 : KH * KW >= 169);
    for (long long lds_cap : {72LL * 1024, 156LL * 1024}) {
        if (best.cost >= 0 && !fp32_big) break;
    for (int nrg = 1; nrg <= 32; ++nrg)
        for (int nst = 1; nst <= 16; ++nst) {
            const int np = nrg * nst;
            if (np > 4 * slots) continue;
            const int th = Q * nrg, tw = R * nst;
            if ((th >= 2 * OH && nrg > 1) || (tw >= 2 * OW && nst > 1)) continue;
            const int rows_in = th + KH - 1, cpn = (tw + KW - 1 + PK - 1) / PK;
            const long long lds = ((long long)rows_in * cpn + (long long)KH * NP) * CS * 4;
            if (lds > lds_cap) continue;
            const long long nt = (long long)B * cdiv(OH, th) * cdiv(OW, tw);
            int occ = (int)((160 * 1024) / (lds + 512));
            occ = occ < 1 ? 1 : (occ > 3 ? 3 : occ);
            double span;
            pick_chunks(nt, slices, occ, &span);
            const int rounds = cdiv(np, slots);
            const double compute =
                4.0 * rounds * (KH * (Q * R * NP + NP) * (PK == 2 ? 1.06 : 1.0) + 6.0 * Q * R + 60);
            const double stage = rows_in * cpn * (CS / 8) / 64.0 * 40.0 + KH * NP * CS / 64.0 * 14.0 + 150;
            // Plenty of tiles: minimise total work.  Fewer workgroups than CUs: minimise the makespan.
            const double cost = (nt * slices >= 512 ? (double)nt * slices / 512.0 : span) * (compute + stage);
            if (best.cost < 0 || cost < best.cost) best.cost = cost, best.nrg = nrg, best.nst = nst;
        }
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
    const size_t lds = ((size_t)g.rows_in * g.CPn + (size_t)KH * NP) * CS * 4;
    const long long ntiles = (long long)g.tiles_h * g.tiles_w * B;
    if (ntiles > 0x7fffffffLL || (long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL)
        return -1;
    g.ntiles = (int)ntiles;
    // Persistent workgroups: as many as fit on the chip at once (LDS allows `occ` per CU, at most 3), then
    // trimmed so the tiles divide as evenly as possible among them.
    int occ = (int)((160 * 1024) / (lds + 512));
    const int occ_max = tune_env("PDW_OCC") ? atoi(tune_env("PDW_OCC")) : 3;
    occ = occ < 1 ? 1 : (occ > occ_max ? occ_max : occ);
    const int target = (256 * occ) / g.slices > 1 ? (256 * occ) / g.slices : 1;
    int nch = (int)(ntiles < target ? ntiles : target);
    {
        double beste = -1;
        for (int cand = (target + 1) / 2; cand <= target && cand <= ntiles; ++cand) {
            const double rounds = (double)cdiv(ntiles, cand);
            const long long blocks = (long long)cand * g.slices;
            const double eff = ntiles / (rounds * cand) * blocks / (double)(cdiv(blocks, 256) * 256);
            if (eff >= beste) beste = eff, nch = cand;
        }
    }
    if (tune_env("PDW_NCH")) nch = atoi(tune_env("PDW_NCH"));
    g.nchunks = nch < 1 ? 1 : nch;
    const long long nblocks = (long long)g.nchunks * g.slices;
    const void* ptrs[3] = {x, w, y};  // all three are moved with the same channel vectors
    const int vec = pick_vec(C, sizeof(T), ptrs, 3);
#define PDW_GO(V)                                                                                            \
    {                                                                                                        \
        auto kern = dwconv_tiled_k<T, KW, R, Q, CS, V>;                                                      \
        const int upp = 256 / (CS / V);                                                                      \
        g.step_r = upp / g.CPn, g.step_u = upp % g.CPn;                                                      \
        static std::once_flag attr_once;                                                                       \
        std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });                                                                                                    \
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
    const TiledPlan p0 = plan_tiled<T, KW, 8, 2, 32>(OH, OW, KH, B, C);
    const TiledPlan p1 = plan_tiled<T, KW, 14, 1, 32>(OH, OW, KH, B, C);
    const TiledPlan p2 = plan_tiled<T, KW, 14, 2, 32>(OH, OW, KH, B, C);
    int pick = -1;
    double best = -1;
    const TiledPlan* ps[3] = {&p0, &p1, &p2};
    for (int i = 0; i < 3; ++i)
        if (ps[i]->cost >= 0 && (best < 0 || ps[i]->cost < best)) best = ps[i]->cost, pick = i;
    const char* force = tune_env("PDW_PATCH");
    if (force && atoi(force) >= 0 && atoi(force) < 3) pick = atoi(force);
    TiledPlan p = pick >= 0 ? *ps[pick] : p0;
    if (pick < 0 || p.cost < 0) return -1;
    if (tune_env("PDW_NRG") && tune_env("PDW_NST")) p.nrg = atoi(tune_env("PDW_NRG")), p.nst = atoi(tune_env("PDW_NST"));
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
