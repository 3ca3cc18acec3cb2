// Depthwise-convolution weight gradient on the matrix cores (16-bit types, stride 1, dilation 1, odd square
// filters):      dw[u,v,c] = sum_{b,i,j} gy[b,i,j,c] * x[b, i+u-PH, j+v-PW, c].
//
// v_mfma_f32_4x4x4_16b_{bf16,f16} multiplies 16 independent 4x4x4 blocks per instruction; a block is one
// channel.  For the staged input row rr (window coordinates: rr = i + u) and a block of 4 output columns j0..j0+3
//     D[m][n] += sum_k A[m][k] * B[k][n]
//     A[m][k] = gy[rr - 4 ub - m][j0 + k]            filter row u = 4 ub + m   (zero outside the tile's rows)
//     B[k][n] = x[rr][j0 + k + v],  v = 8 vg + 2 n + par
// accumulates dw[4 ub + m][8 vg + 2 n + par] for the 16 channels of the workgroup: 1024 multiply-adds per
// instruction, 66 % of them on real taps at K = 13.  Even v read the input row as aligned column pairs, odd v
// the same pairs shifted by 16 bits (two v_alignbit per operand).  A lane is (channel b = lane / 4, q = lane % 4),
// q being m in the A operand and n in the B operand.
//
// Operand reuse.  With rr = 4 rho + s the A operand of filter-row block ub is G_s[rho - ub], where G_s[c] holds
// gy row 4 c + s - m in lane m: one new operand per input row serves ceil(K/4) consecutive rows, so a wavefront
// that keeps (j0, s) fixed and walks rho reads one gy operand and ceil((K+1)/8) input-row operands from LDS per
// 2 ceil(K/4) ceil((K+1)/8) MFMAs.  The (j0, s) combinations of a tile are dealt out to the wavefronts; every
// wavefront accumulates all taps of its 16 channels in registers, the wavefronts are summed through LDS at the
// end and the workgroup writes one fp32 partial, reduced over the workgroups in a fixed order by
// wgrad_reduce_parts (no atomics: bit-reproducible).
//
// Both windows are staged in LDS channel-major, [row][channel][column pair], as in dwconv_mfma.h.
#pragma once
#include <mutex>
#include <stdlib.h>

#include "common.h"
#include "dwconv_mfma.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

struct WgradMfmaGeom {
    int H, W, C;      // x extents
    int OH, OW;       // gy extents
    int PH, PW;
    int TH, TW;       // tile of gy positions (TW a multiple of 4)
    int tiles_h, tiles_w, ntiles, nchunks, slices;
    int XP, GP;       // LDS dwords per channel row of the x / gy window
    int red_tiles;    // accumulator tiles summed per round of the final cross-wavefront reduction
};

template <int K>
struct WgradMfmaShape {
    static constexpr int CS = 16;
    static constexpr int NUB = (K + 3) / 4;        // filter-row blocks
    static constexpr int NVG = ((K + 1) / 2 + 3) / 4;  // groups of 4 even (or odd) filter columns
    static constexpr int NTILE = NUB * NVG * 2;    // accumulator tiles (4 registers each) per lane
};

// One launch can hold two independent problems of the same filter size (the two resolutions of a pyramid block):
// workgroups from `first1` on work on problem 1.  Its workgroups start as compute units finish their workgroup of
// problem 0, so the second problem fills the first one's tail instead of paying a launch, a ramp and a tail of its
// own.  A single problem is first1 = gridDim.x.
template <typename T, int K, int NWV>
__global__ __launch_bounds__(NWV * 64, 1) void dwconv_wgrad_mfma_k(const T* __restrict__ x0, const T* __restrict__ gy0,
                                                                   float* __restrict__ part0, const WgradMfmaGeom g0,
                                                                   const T* __restrict__ x1, const T* __restrict__ gy1,
                                                                   float* __restrict__ part1, const WgradMfmaGeom g1,
                                                                   const unsigned first1) {
    const bool second = blockIdx.x >= first1;  // uniform
    const T* __restrict__ x = second ? x1 : x0;
    const T* __restrict__ gy = second ? gy1 : gy0;
    float* __restrict__ part = second ? part1 : part0;
    const WgradMfmaGeom g = second ? g1 : g0;
    const unsigned my_block = second ? blockIdx.x - first1 : blockIdx.x;
    const unsigned my_blocks = second ? gridDim.x - first1 : first1;
    using Sh = WgradMfmaShape<K>;
    constexpr int V = 8, NT = NWV * 64, CS = Sh::CS, NUB = Sh::NUB, NVG = Sh::NVG, NTILE = Sh::NTILE;
    constexpr int NPX = 6, NPG = 4;  // staging passes of the x / gy windows requested at once (more: staged directly)
    extern __shared__ uint32_t smem[];
    const int XR = g.TH + K - 1;                    // x window rows
    const int NCX = g.TW / 2 + 4 * NVG;             // x window pairs: every pair an operand reads
    uint32_t* xl = smem;                            // [XR][CS][XP]
    uint32_t* gl = smem + XR * CS * g.XP;           // [TH][CS][GP], rows one dword further apart: the 4 gy rows an
                                                    // operand read touches then fall on different banks

    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it branches uniformly
    const int bid = xcd_remap(my_block, my_blocks);
    const int sl = bid % g.slices, chunk = bid / g.slices;
    const int c0 = sl * CS;
    const int tiles_per_img = g.tiles_h * g.tiles_w;
    const int bq = lane >> 2, q = lane & 3;

    TileStager<T, CS, V, NPX, true, NT> sx;
    TileStager<T, CS, V, NPG, true, NT> sg;
    sx.init(tid, c0, g.C, XR, NCX, g.XP);
    sg.init(tid, c0, g.C, g.TH, g.TW / 2, g.GP, CS * g.GP + 1);
    auto origin = [&](int tile, int& b, int& row0, int& col0) {
        b = tile / tiles_per_img;
        const int rem = tile - b * tiles_per_img;
        const int th_i = rem / g.tiles_w;
        row0 = th_i * g.TH, col0 = (rem - th_i * g.tiles_w) * g.TW;
    };
    auto request = [&](int tile) {
        int b, row0, col0;
        origin(tile, b, row0, col0);
        sx.issue(x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, row0 - g.PH, col0 - g.PW);
        sg.issue(gy + (long long)b * g.OH * g.OW * g.C, g.OH, g.OW, g.C, row0, col0);
    };
    if (chunk < g.ntiles) request(chunk);

    f32x4 acc[NUB][NVG][2];
#pragma unroll
    for (int ub = 0; ub < NUB; ++ub)
#pragma unroll
        for (int vg = 0; vg < NVG; ++vg)
#pragma unroll
            for (int par = 0; par < 2; ++par) acc[ub][vg][par] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int RPX = CS * g.XP, RPG = CS * g.GP + 1;  // dwords per staged row
    // Work items of a tile: (group of JB column blocks, s, row range), dealt out to the wavefronts.  JB = 7 fits the
    // 14 blocks of a 56-column row in two groups; large filters keep fewer blocks in flight (registers).
    constexpr int JB = NTILE <= 16 ? 7 : 4;
    const int nblk = g.TW / 4;                       // column blocks (<= 14)
    const int ngrp = (nblk + JB - 1) / JB;
    const int nrs = NWV / (4 * ngrp) > 1 ? NWV / (4 * ngrp) : 1;  // row ranges: enough items for every wavefront
    const int nitems = 4 * ngrp * nrs;
    for (int tile = chunk; tile < g.ntiles; tile += g.nchunks) {
        int b, row0, col0;
        origin(tile, b, row0, col0);
        __syncthreads();  // the previous windows are fully consumed
        sx.commit(xl, x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, row0 - g.PH, col0 - g.PW);
        sg.commit(gl, gy + (long long)b * g.OH * g.OW * g.C, g.OH, g.OW, g.C, row0, col0);
        __syncthreads();
        for (int item = wv; item < nitems; item += NWV) {
            const int s = item & 3, grp = (item >> 2) % ngrp, rs = (item >> 2) / ngrp;
            const int jb0 = grp * JB;
            // x rows of this item: 4 rho + s for rho in [rho_lo, rho_hi)
            const int nrho = (XR - s + 3) / 4;
            const int rho_lo = rs * ((nrho + nrs - 1) / nrs);
            const int rho_hi = min(nrho, (rs + 1) * ((nrho + nrs - 1) / nrs));
            // lane addresses: x pairs start at 2 jb + n (+ 4 vg + 0..2), gy pairs at 2 jb (+0, 1)
            const uint32_t* xq = xl + bq * g.XP + 2 * jb0 + q;
            const uint32_t* gq = gl + bq * g.GP + 2 * jb0;
            uint2 ring[JB][NUB];  // G_s[rho - ub] of column block j lives in ring[j][(rho - ub) mod NUB]
#pragma unroll
            for (int j = 0; j < JB; ++j)
#pragma unroll
                for (int i = 0; i < NUB; ++i) ring[j][i] = make_uint2(0u, 0u);
            // The walk starts NUB - 1 steps early to fill the ring (no MFMAs there); the steps are unrolled NUB at
            // a time so the ring index is static.
            const int rho_start = rho_lo - (NUB - 1) > 0 ? ((rho_lo - (NUB - 1)) / NUB) * NUB : 0;
            for (int rho0 = rho_start; rho0 < rho_hi; rho0 += NUB) {
#pragma unroll
                for (int uu = 0; uu < NUB; ++uu) {
                    const int rho = rho0 + uu;
                    const int rr = 4 * rho + s;
                    // new gy operands: row rr - m of this lane (zero outside the tile)
                    const int gr = rr - q;
                    const bool gok = gr >= 0 && gr < g.TH;
                    const uint32_t* gp = gq + (gok ? gr : 0) * RPG;
#pragma unroll
                    for (int j = 0; j < JB; ++j) {
                        const bool jok = jb0 + j < nblk;  // past the tile: reread block 0 and zero the operand
                        const int jc = jok ? j : 0;
                        const uint32_t g0 = gp[2 * jc], g1 = gp[2 * jc + 1];  // always a valid address
                        ring[j][uu] = make_uint2(gok && jok ? g0 : 0u, gok && jok ? g1 : 0u);
                    }
                    if (rho >= rho_lo && rho < rho_hi) {
                        const uint32_t* xr = xq + rr * RPX;
#pragma unroll
                        for (int j = 0; j < JB; ++j) {
                            {
                                const int jc = jb0 + j < nblk ? j : 0;
                                uint2 be[NVG], bo[NVG];
#pragma unroll
                                for (int vg = 0; vg < NVG; ++vg) {
                                    const uint32_t p0 = xr[2 * jc + 4 * vg], p1 = xr[2 * jc + 4 * vg + 1],
                                                   p2 = xr[2 * jc + 4 * vg + 2];
                                    be[vg] = make_uint2(p0, p1);
                                    bo[vg] = make_uint2(__builtin_amdgcn_alignbit(p1, p0, 16),
                                                        __builtin_amdgcn_alignbit(p2, p1, 16));
                                }
#pragma unroll
                                for (int ub = 0; ub < NUB; ++ub) {
                                    // gy rows 4 (rho - ub) + s - m; outside the tile the ring holds zeros.  Skipping
                                    // those products would cost a branch per 2 NVG MFMAs, more than they do.
                                    const uint2 a = ring[j][(uu - ub + NUB) % NUB];
#pragma unroll
                                    for (int vg = 0; vg < NVG; ++vg) {
                                        acc[ub][vg][0] = mfma4(a, be[vg], acc[ub][vg][0], T());
                                        acc[ub][vg][1] = mfma4(a, bo[vg], acc[ub][vg][1], T());
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
        if (tile + g.nchunks < g.ntiles) request(tile + g.nchunks);
    }

    // ---- sum the wavefronts through LDS, red_tiles accumulator tiles per round; register m of tile (ub, vg, par):
    // filter row 4 ub + m, lane (b, n): filter column 8 vg + 2 n + par of channel b
    float* red = reinterpret_cast<float*>(smem);  // [NWV][RT][m][n][16 channels]
    float* pout = part + (long long)chunk * K * K * g.C;
    const int RT = g.red_tiles;
    const int slot = q * 16 + bq;  // lane (b, n) -> channel-fastest
    for (int t0 = 0; t0 < NTILE; t0 += RT) {
        __syncthreads();
#pragma unroll
        for (int ub = 0; ub < NUB; ++ub)
#pragma unroll
            for (int vg = 0; vg < NVG; ++vg)
#pragma unroll
                for (int par = 0; par < 2; ++par) {
                    const int ti = (ub * NVG + vg) * 2 + par;
                    if (ti >= t0 && ti < t0 + RT) {
#pragma unroll
                        for (int m = 0; m < 4; ++m)
                            red[((wv * RT + ti - t0) * 4 + m) * 64 + slot] = acc[ub][vg][par][m];
                    }
                }
        __syncthreads();
        const int nout = (NTILE - t0 < RT ? NTILE - t0 : RT) * 64;  // float4 outputs: 4 channels each
        for (int o = tid; o < nout; o += NT) {
            const int c4 = (o & 3) * 4, n = (o >> 2) & 3, m = (o >> 4) & 3, ti = t0 + (o >> 6);
            float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w2 = 0; w2 < NWV; ++w2) {
                const float4 t = *reinterpret_cast<const float4*>(red + ((w2 * RT + ti - t0) * 4 + m) * 64 + n * 16 + c4);
                s.x += t.x, s.y += t.y, s.z += t.z, s.w += t.w;
            }
            const int par = ti & 1, vg = (ti >> 1) % NVG, ub = (ti >> 1) / NVG;
            const int u = 4 * ub + m, v = 8 * vg + 2 * n + par;
            if (u < K && v < K && c0 + c4 < g.C)  // C % 8 == 0: the 4 channels are in range together
                *reinterpret_cast<float4*>(pout + (u * K + v) * g.C + c0 + c4) = s;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Host side

struct WgradMfmaPlan {
    bool ok = false;
    WgradMfmaGeom g;
    size_t lds = 0;
    int nblocks = 0;
};

template <typename T, int K, int NWV>
static WgradMfmaPlan plan_wgrad_mfma(int B, int H, int W, int C, int PH, int PW) {
    using Sh = WgradMfmaShape<K>;
    WgradMfmaPlan p;
    WgradMfmaGeom& g = p.g;
    g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    if (g.OH < 1 || g.OW < 1 || C % 8 != 0) return p;
    if ((long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL) return p;
    g.slices = cdiv(C, Sh::CS);
    // tile width: the whole row up to 56 columns, a multiple of 4
    const int ow4 = cdiv(g.OW, 4) * 4;
    g.tiles_w = cdiv(ow4, 56);
    g.TW = cdiv(cdiv(ow4, g.tiles_w), 4) * 4;
    auto pad = [](int n) {  // 4 mod 8 keeps the 16 channels x 4 lanes of an operand read on distinct banks
        while (n % 8 != 4) ++n;
        return n;
    };
    g.XP = pad(g.TW / 2 + 4 * Sh::NVG), g.GP = pad(g.TW / 2);
    if (tune_env("PDW_WG_XP") && atoi(tune_env("PDW_WG_XP")) >= g.TW / 2 + 4 * Sh::NVG) g.XP = atoi(tune_env("PDW_WG_XP"));
    if (tune_env("PDW_WG_GP") && atoi(tune_env("PDW_WG_GP")) >= g.TW / 2) g.GP = atoi(tune_env("PDW_WG_GP"));
    auto lds_of = [&](int th) { return ((size_t)(th + K - 1) * Sh::CS * g.XP + (size_t)th * (Sh::CS * g.GP + 1)) * 4; };
    // tile height: about one tile per CU, within LDS.  Where LDS forces lower tiles than that, the count of tile
    // rows is chosen for the shortest run: rounds of tiles per workgroup times (tile rows + 66), the 66 being what a
    // tile costs beside its rows (halo, staging latency, the final sum), fitted to measurements at K = 13 and 17.
    const long long per_row = (long long)B * g.slices * g.tiles_w;  // tiles per row of tiles, all slices
    int tiles_h = (int)(256 / (per_row > 0 ? per_row : 1));
    if (tune_env("PDW_WG_TILEMUL")) tiles_h *= atoi(tune_env("PDW_WG_TILEMUL"));
    if (tiles_h < 1) tiles_h = 1;
    if (tiles_h > g.OH) tiles_h = g.OH;
    int th = cdiv(g.OH, tiles_h);
    if (th < 4) th = g.OH < 4 ? g.OH : 4;
    if (lds_of(th) > 150 * 1024) {
        while (th > 1 && lds_of(th) > 150 * 1024) --th;
        if (lds_of(th) > 150 * 1024) return p;
        const int first = cdiv(g.OH, th);
        const int cap_s = 256 / g.slices > 1 ? 256 / g.slices : 1;
        long long best = -1;
        for (int cand = first; cand <= 2 * first + 2 && cand <= g.OH; ++cand) {
            const int thc = cdiv(g.OH, cand);
            if (thc < 4 || lds_of(thc) > 150 * 1024) continue;
            const long long rounds = cdiv((long long)B * cdiv(g.OH, thc) * g.tiles_w, (long long)cap_s);
            const long long cost = rounds * (thc + 66);
            if (best < 0 || cost < best) best = cost, th = thc;
        }
    }
    g.TH = th;
    g.tiles_h = cdiv(g.OH, th);
    const long long ntiles = (long long)B * g.tiles_h * g.tiles_w;
    if (ntiles > 0x7fffffffLL) return p;
    g.ntiles = (int)ntiles;
    const int cap = 256 / g.slices > 1 ? 256 / g.slices : 1;
    const long long rounds = cdiv(ntiles, (long long)cap);
    g.nchunks = (int)cdiv(ntiles, rounds);
    p.nblocks = g.nchunks * g.slices;
    size_t lds = lds_of(th);
    // final reduction: NWV wavefronts x red_tiles x 1 KB
    int rt = Sh::NTILE;
    while ((size_t)NWV * rt * 1024 > 150 * 1024) rt = (rt + 1) / 2;
    g.red_tiles = rt;
    if (lds < (size_t)NWV * rt * 1024) lds = (size_t)NWV * rt * 1024;
    p.lds = lds;
    p.ok = true;
    return p;
}

template <typename T, int K>
static size_t wgrad_mfma_workspace_t(int B, int H, int W, int C, int PH, int PW) {
    const WgradMfmaPlan p = plan_wgrad_mfma<T, K, 8>(B, H, W, C, PH, PW);
    return p.ok ? (size_t)p.g.nchunks * K * K * C * sizeof(float) : 0;
}

// -1: not covered (the caller uses the vector-ALU tiled kernel).
template <typename T, int K>
static int wgrad_mfma_launch_t(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                               int PW, hipStream_t s) {
    constexpr int NWV = 8;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(gy) & 15)) return -1;
    const WgradMfmaPlan p = plan_wgrad_mfma<T, K, NWV>(B, H, W, C, PH, PW);
    if (!p.ok) return -1;
    auto kern = dwconv_wgrad_mfma_k<T, K, NWV>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nblocks), dim3(NWV * 64), p.lds, s, (const T*)x, (const T*)gy, (float*)ws,
                       p.g, (const T*)x, (const T*)gy, (float*)ws, p.g, (unsigned)p.nblocks);
    if (int e = check_launch("dwconv_wgrad_mfma")) return e;
    return wgrad_reduce_launch<T>((const float*)ws, dw, p.g.nchunks, K * K * C, s);
}

// Two problems (same batch, channels and filter size, different extents) in one launch; -1: not covered.
template <typename T, int K>
static int wgrad_mfma_pair_launch_t(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                                    const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                                    hipStream_t s) {
    constexpr int NWV = 8;
    for (const void* ptr : {xa, gya, xb, gyb})
        if (reinterpret_cast<uintptr_t>(ptr) & 15) return -1;
    const WgradMfmaPlan pa = plan_wgrad_mfma<T, K, NWV>(B, Ha, Wa, C, PH, PW);
    const WgradMfmaPlan pb = plan_wgrad_mfma<T, K, NWV>(B, Hb, Wb, C, PH, PW);
    if (!pa.ok || !pb.ok || pa.nblocks % 8 != 0) return -1;  // a multiple of 8: problem 1 keeps its XCD mapping
    auto kern = dwconv_wgrad_mfma_k<T, K, NWV>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)(pa.nblocks + pb.nblocks)), dim3(NWV * 64), pa.lds > pb.lds ? pa.lds : pb.lds,
                       s, (const T*)xa, (const T*)gya, (float*)wsa, pa.g, (const T*)xb, (const T*)gyb, (float*)wsb, pb.g,
                       (unsigned)pa.nblocks);
    if (int e = check_launch("dwconv_wgrad_mfma pair")) return e;
    if (int e = wgrad_reduce_launch<T>((const float*)wsa, dwa, pa.g.nchunks, K * K * C, s)) return e;
    return wgrad_reduce_launch<T>((const float*)wsb, dwb, pb.g.nchunks, K * K * C, s);
}

}  // namespace pdw
