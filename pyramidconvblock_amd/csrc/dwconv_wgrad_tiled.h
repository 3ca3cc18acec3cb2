// LDS-tiled depthwise-convolution weight gradient for stride 1, dilation 1, odd square filters:
//     dw[u,v,c] = sum_{b,i,j} gy[b,i,j,c] * x[b, i+u-PH, j+v-PW, c].
//
// Pass 1 (this file).  Persistent workgroups of 4 wavefronts.  A workgroup owns a slice of 32
// channels and a chunk of the position tiles; a lane is a channel (lane % 32) of strip-group
// lane / 32, and keeps the partial sums of its taps in registers for the whole kernel:
// NU x K accumulators, where the K filter rows are split over USPLIT wavefront classes when K*K
// does not fit the register file.  Per tile the workgroup stages the x window (with halo) and
// the gy window into LDS (zeros outside the image, so ragged edges need no masks), then every
// wavefront walks its x rows: one LDS read of an x row segment serves all filter rows u (the gy
// row i = r - u is the only other operand), so LDS traffic is ~1 dword per 10 multiply-add pairs.
// 16-bit types use v_dot2_f32 over column pairs: even taps pair gy's even-aligned column pairs
// with x's even-aligned pairs, odd taps with x's odd-aligned pairs (one v_alignbit per x pair).
// At the end lanes 32..63 are folded onto 0..31, the wavefronts are summed through LDS, and the
// workgroup writes one fp32 partial [K][K][32] into the workspace.
//
// Pass 2 sums the partials in a fixed order (wgrad_reduce_parts).  No atomics anywhere, so the
// result is bit-reproducible.
#pragma once
#include <mutex>
#include <stdlib.h>

#include "common.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

struct WgradGeom {
    int H, W, C;    // x extents
    int OH, OW;     // gy extents
    int PH, PW;
    int TH, NSP;    // tile = TH rows x (2*NSP*R) columns of gy positions
    int tiles_h, tiles_w, ntiles;  // ntiles = B * tiles_h * tiles_w
    int nchunks, slices;
    int CPX, CPG;   // LDS units per staged row of x / gy
};

constexpr int kWgCS = 32;  // channels per workgroup slice (two strip groups per wavefront)

template <typename T, int K, int R, int USPLIT, int V>
__global__ __launch_bounds__(256, 2) void dwconv_wgrad_tiled_k(const T* __restrict__ x, const T* __restrict__ gy,
                                                            float* __restrict__ part, const WgradGeom g) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int CS = kWgCS;
    constexpr int NU = (K + USPLIT - 1) / USPLIT;  // filter rows per wavefront class
    constexpr int RU = R / PK;                     // gy units per strip
    constexpr int XU = (R + K - 1) / PK;           // x units per strip window
    constexpr int NWR = 4 / USPLIT;                // wavefronts sharing a class (split the rows)
    constexpr int NPX = NU * K > 100 ? 3 : (NU * K > 84 ? 5 : 6);  // staging passes of the x / gy windows held in registers
    constexpr int NPG = NU * K > 100 ? 1 : 2;      // for the next tile (fewer when the accumulators are many)
    static_assert(R % 2 == 0 && K % 2 == 1 && 4 % USPLIT == 0, "bad wgrad parameters");
    extern __shared__ uint32_t smem[];
    const int xrows = g.TH + K - 1;
    uint32_t* xl = smem;                        // [xrows][CPX][CS]
    uint32_t* gl = smem + xrows * g.CPX * CS;   // [TH][CPG][CS]

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int c = lane & (CS - 1), grp = lane / CS;
    const int us = wv % USPLIT, wr = wv / USPLIT;
    const int ubase = us * NU;
    int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int sl = bid % g.slices, chunk = bid / g.slices;
    const int c0 = sl * CS;

    float acc[NU][K];
#pragma unroll
    for (int a = 0; a < NU; ++a)
#pragma unroll
        for (int v = 0; v < K; ++v) acc[a][v] = 0.f;

    const int tiles_per_img = g.tiles_h * g.tiles_w;
    // The next tile's windows are requested while the current one is multiplied (register prefetch).
    TileStager<T, CS, V, NPX> sx;
    TileStager<T, CS, V, NPG> sg;
    sx.init(tid, c0, g.C, xrows, g.CPX);
    sg.init(tid, c0, g.C, g.TH, g.CPG);
    auto origin = [&](int tile, int& b, int& row0, int& col0) {
        b = tile / tiles_per_img;
        const int rem = tile - b * tiles_per_img;
        const int th_i = rem / g.tiles_w;
        row0 = th_i * g.TH, col0 = (rem - th_i * g.tiles_w) * (2 * g.NSP * R);
    };
    auto request = [&](int tile) {
        int b, row0, col0;
        origin(tile, b, row0, col0);
        sx.issue(x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, row0 - g.PH, col0 - g.PW);
        sg.issue(gy + (long long)b * g.OH * g.OW * g.C, g.OH, g.OW, g.C, row0, col0);
    };
    if (chunk < g.ntiles) request(chunk);
    for (int tile = chunk; tile < g.ntiles; tile += g.nchunks) {
        int b, row0, col0;
        origin(tile, b, row0, col0);
        __syncthreads();  // previous tile fully consumed
        sx.commit(xl, x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, row0 - g.PH, col0 - g.PW);
        sg.commit(gl, gy + (long long)b * g.OH * g.OW * g.C, g.OH, g.OW, g.C, row0, col0);
        __syncthreads();
        if (tile + g.nchunks < g.ntiles) request(tile + g.nchunks);
        for (int r = wr; r < xrows; r += NWR) {
            for (int sp = 0; sp < g.NSP; ++sp) {
                const int st = 2 * sp + grp;
                const uint32_t* xr = xl + (r * g.CPX + st * RU) * CS + c;
                uint32_t xe[XU];
#pragma unroll
                for (int m = 0; m < XU; ++m) xe[m] = xr[m * CS];
                uint32_t xo[XU];  // odd-aligned pairs (16-bit types only)
                if constexpr (PK == 2) {
#pragma unroll
                    for (int m = 0; m + 1 < XU; ++m) xo[m] = __builtin_amdgcn_alignbit(xe[m + 1], xe[m], 16);
                }
#pragma unroll
                for (int a = 0; a < NU; ++a) {
                    const int u = ubase + a;
                    const int i = r - u;  // gy row (tile-relative) that meets x row r under filter row u
                    if (u < K && i >= 0 && i < g.TH) {
                        const uint32_t* gr = gl + (i * g.CPG + st * RU) * CS + c;
                        uint32_t ge[RU];
#pragma unroll
                        for (int t = 0; t < RU; ++t) ge[t] = gr[t * CS];
#pragma unroll
                        for (int v = 0; v < K; ++v)
#pragma unroll
                            for (int t = 0; t < RU; ++t) {
                                if constexpr (PK == 2) {
                                    const uint32_t xv = (v & 1) ? xo[t + (v - 1) / 2] : xe[t + v / 2];
                                    acc[a][v] = dot2acc(ge[t], xv, acc[a][v], T());
                                } else {
                                    acc[a][v] = fmaf(__builtin_bit_cast(float, ge[t]),
                                                     __builtin_bit_cast(float, xe[t + v]), acc[a][v]);
                                }
                            }
                    }
                }
            }
        }
    }

    // ---- fold the two strip groups, then sum the wavefronts of each class through LDS
#pragma unroll
    for (int a = 0; a < NU; ++a)
#pragma unroll
        for (int v = 0; v < K; ++v) acc[a][v] += __shfl_xor(acc[a][v], 32);
    float* red = reinterpret_cast<float*>(smem);  // [4 waves][NU][K][CS]
    float* pout = part + (long long)chunk * K * K * g.C;
    constexpr int WSZ = NU * K * CS;  // floats per wavefront
    __syncthreads();                  // every wavefront is done with the tile buffers
    if (grp == 0) {
#pragma unroll
        for (int a = 0; a < NU; ++a)
#pragma unroll
            for (int v = 0; v < K; ++v) red[wv * WSZ + (a * K + v) * CS + c] = acc[a][v];
    }
    __syncthreads();
    // element e = ((cls * NU + a) * K + v) * CS + cc, four channels per thread and pass
    const bool vec4 = (g.C & 3) == 0;
#pragma unroll 4
    for (int e = tid * 4; e < USPLIT * WSZ; e += 1024) {
        const int cls = e / WSZ, o = e - cls * WSZ;
        const int cc = o % CS, av = o / CS;
        const int a = av / K, v = av - a * K;
        const int u = cls * NU + a;
        float4 s = *reinterpret_cast<const float4*>(red + cls * WSZ + o);
#pragma unroll
        for (int q = 1; q < NWR; ++q) {
            const float4 t = *reinterpret_cast<const float4*>(red + (q * USPLIT + cls) * WSZ + o);
            s.x += t.x, s.y += t.y, s.z += t.z, s.w += t.w;
        }
        if (u < K) {
            float* dst = pout + (u * K + v) * g.C + c0 + cc;
            if (vec4 && c0 + cc + 3 < g.C) {
                *reinterpret_cast<float4*>(dst) = s;
            } else {
                const float sv[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (c0 + cc + j < g.C) dst[j] = sv[j];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Host side

template <typename T, int K>
struct WgradCfg {
    static constexpr int PK = PackOf<T>::PK;
    static constexpr int USPLIT = (K <= 11) ? 1 : (K <= 15 ? 2 : 4);
    static constexpr int R = PK == 2 ? 14 : 8;
};

struct WgradPlan {
    bool ok = false;
    WgradGeom g;
    size_t lds = 0;
    int nblocks = 0;
};

template <typename T, int K, int R>
static WgradPlan plan_wgrad(int B, int H, int W, int C, int PH, int PW) {
    constexpr int PK = PackOf<T>::PK;
    constexpr int CS = kWgCS;
    WgradPlan p;
    WgradGeom& g = p.g;
    g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    if (g.OH < 1 || g.OW < 1) return p;
    if ((long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL) return p;
    g.slices = cdiv(C, CS);
    constexpr int USPLIT_ = WgradCfg<T, K>::USPLIT;
    const int red_bytes = 4 * ((K + USPLIT_ - 1) / USPLIT_) * K * CS * 4;  // the final cross-wavefront sum
    double best = -1;
    int best_nch = 1;
    for (int th = 1; th <= 32; ++th)
        for (int nsp = 1; nsp <= 4; ++nsp) {
            const int tw = 2 * nsp * R;
            if (th >= 2 * g.OH || (tw >= 2 * g.OW && nsp > 1)) continue;
            const int cpx = (tw + K - 1 + PK - 1) / PK, cpg = tw / PK;
            const long long lds = ((long long)(th + K - 1) * cpx + (long long)th * cpg) * CS * 4;
            if (lds > 78 * 1024) continue;
            const int t_h = cdiv(g.OH, th), t_w = cdiv(g.OW, tw);
            const long long ntiles = (long long)B * t_h * t_w;
            if (ntiles > 0x7fffffffLL) continue;
            // wave-instructions per tile: compute rounds over rows (4 waves) + staging
            const double compute = cdiv(th + K - 1, 4) * nsp * (K * K * (R / PK) * th / (double)(th + K - 1) + 60.0);
            const double stage = ((th + K - 1) * cpx + th * cpg) * (CS / 8) / 64.0 * 40.0 + 100;
            double span;
            const int nch = pick_chunks(ntiles, g.slices, 2, &span);
            // makespan in tile units times the tile cost, plus the partial-sum traffic of the chunks
            const double cost = span * (4 * compute + stage) + 0.02 * nch * K * K;
            if (best < 0 || cost < best) {
                best = cost, best_nch = nch;
                g.TH = th, g.NSP = nsp, g.tiles_h = t_h, g.tiles_w = t_w, g.CPX = cpx, g.CPG = cpg;
                p.lds = (size_t)(lds > red_bytes ? lds : red_bytes);
            }
        }
    if (best < 0) return p;
    if (tune_env("PDW_WG_TH") && tune_env("PDW_WG_NSP")) {
        g.TH = atoi(tune_env("PDW_WG_TH")), g.NSP = atoi(tune_env("PDW_WG_NSP"));
        const int tw = 2 * g.NSP * R;
        g.tiles_h = cdiv(g.OH, g.TH), g.tiles_w = cdiv(g.OW, tw);
        g.CPX = (tw + K - 1 + PK - 1) / PK, g.CPG = tw / PK;
        const long long lds = ((long long)(g.TH + K - 1) * g.CPX + (long long)g.TH * g.CPG) * CS * 4;
        p.lds = (size_t)(lds > red_bytes ? lds : red_bytes);
        best_nch = pick_chunks((long long)B * g.tiles_h * g.tiles_w, g.slices, 2, nullptr);
    }
    const long long ntiles = (long long)B * g.tiles_h * g.tiles_w;
    if (ntiles > 0x7fffffffLL) return p;
    g.ntiles = (int)ntiles;
    int nch = best_nch;
    if (tune_env("PDW_WG_NCH")) nch = atoi(tune_env("PDW_WG_NCH"));
    g.nchunks = nch < 1 ? 1 : nch;
    p.nblocks = g.nchunks * g.slices;
    p.ok = true;
    return p;
}

template <typename T, int K>
static size_t wgrad_tiled_workspace_t(int B, int H, int W, int C, int PH, int PW) {
    const WgradPlan p = plan_wgrad<T, K, WgradCfg<T, K>::R>(B, H, W, C, PH, PW);
    return p.ok ? (size_t)p.g.nchunks * K * K * C * sizeof(float) : 0;
}

template <typename T, int K>
static int wgrad_tiled_launch_t(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                                int PW, hipStream_t s) {
    constexpr int R = WgradCfg<T, K>::R;
    constexpr int USPLIT = WgradCfg<T, K>::USPLIT;
    WgradPlan p = plan_wgrad<T, K, R>(B, H, W, C, PH, PW);
    if (!p.ok) return -1;
    WgradGeom& g = p.g;
    const void* ptrs[2] = {x, gy};
    const int vec = pick_vec(C, sizeof(T), ptrs, 2);
#define PDW_GO(V)                                                                                                 \
    {                                                                                                             \
        auto kern = dwconv_wgrad_tiled_k<T, K, R, USPLIT, V>;                                                     \
        static std::once_flag attr_once;                                                                            \
        std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });                                                                                                         \
        hipLaunchKernelGGL(kern, dim3((unsigned)p.nblocks), dim3(256), p.lds, s, (const T*)x, (const T*)gy,       \
                           (float*)ws, g);                                                                        \
    }
    if constexpr (sizeof(T) == 2) {
        if (vec >= 8) PDW_GO(8) else if (vec >= 4) PDW_GO(4) else PDW_GO(1)
    } else {
        if (vec >= 4) PDW_GO(4) else PDW_GO(1)
    }
#undef PDW_GO
    if (int e = check_launch("dwconv_wgrad_tiled")) return e;
    return wgrad_reduce_launch<T>((const float*)ws, dw, g.nchunks, K * K * C, s);
}

template <int K>
static size_t wgrad_tiled_workspace_k(int B, int H, int W, int C, int PH, int PW, int dtype) {
    switch (dtype) {
        case kF32: return wgrad_tiled_workspace_t<float, K>(B, H, W, C, PH, PW);
        case kF16: return wgrad_tiled_workspace_t<f16_t, K>(B, H, W, C, PH, PW);
        default: return wgrad_tiled_workspace_t<bf16_t, K>(B, H, W, C, PH, PW);
    }
}

template <int K>
static int wgrad_tiled_launch_k(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                                int PW, int dtype, hipStream_t s) {
    switch (dtype) {
        case kF32: return wgrad_tiled_launch_t<float, K>(x, gy, dw, ws, B, H, W, C, PH, PW, s);
        case kF16: return wgrad_tiled_launch_t<f16_t, K>(x, gy, dw, ws, B, H, W, C, PH, PW, s);
        default: return wgrad_tiled_launch_t<bf16_t, K>(x, gy, dw, ws, B, H, W, C, PH, PW, s);
    }
}

}  // namespace pdw
