// fp32 depthwise convolution (stride 1, square odd filters 5 .. 17) on the fp32 matrix cores: the block-Toeplitz
// product of dwconv_tz.h restated for v_mfma_f32_16x16x4_f32 (dwconv_triton.py:52-104 forward, :154-185 input gradient
// through the rotated filter).
//
// For one channel a 4 x 4 output patch is the filter spread out as a 16 x (k+3)^2 matrix A (zero where a tap falls
// outside the filter) times the patch's (k+3)^2 window: m = the patch's 16 outputs, n = 16 patches side by side (4
// columns apart; with narrow images 8 patches of each of 2 images), k = 4 consecutive window columns of one window row
// per instruction.  A depends on the channel only and lives in registers ((k+3) * ceil((k+3)/4) of them); the window
// rows of vertically adjacent patches overlap, so the loops run over the staged rows of the tile and every B operand
// read from LDS (64 consecutive floats: no bank conflict) feeds up to four patch rows' accumulators, which are
// independent instructions.  The fp32 matrix rate is twice the unpacked vector rate and two thirds of these
// multiply-adds fall on real taps at k = 13.  A workgroup (4 wavefronts, 2 channels each) stages the tile and its halo
// channel-major for its 8 channels, multiplies, and returns the results through LDS as channels-last 16-byte stores;
// two workgroups share a compute unit, so one stages while the other multiplies.  Measured: the products run at 86 %
// of the matrix rate, but the staging costs about 50 us at [32,56,56,128] whatever the filter (8 channels are half of a
// 64-byte sector, 28 staged rows for 16 rows of results), which leaves the kernel ahead of the vector-ALU one only for
// the largest filters and for small tensors: dwconv_f32m_launch picks it there and nowhere else.
#include <stdint.h>

#include <mutex>

#include "common.h"
#include "kernels.h"

namespace pdw {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

struct F32mGeom {
    int B, H, W, C, OH, OW, PH, PW, flip;
    int nrt, nct, nsl;   // tiles of rows, of columns, channel slices (image groups are the slowest index)
};

template <int K, int NPI>
struct F32mShape {
    static constexpr int WR = K + 3;                 // window rows of a patch
    static constexpr int G = (K + 3 + 3) / 4;        // groups of 4 window columns
    static constexpr int PR = K >= 15 ? 3 : 4;       // patch rows of a tile
    static constexpr int TH = 4 * PR, TW = 4 * NPI;  // outputs of a tile (per image)
    static constexpr int NI = 16 / NPI;              // images of a tile
    static constexpr int CS = 8;                     // channels of a workgroup
    static constexpr int SR = TH + K - 1;            // staged rows
    static constexpr int SC = 4 * (NPI + G - 1);     // staged columns per image
    static constexpr int SP = SC + 1;                // row pitch (floats)
    static constexpr int PLANE = SR * SP;            // one channel of one image
    static constexpr int KK = K * K;
    static constexpr int in_floats = NI * CS * PLANE;
    static constexpr int out_floats = NI * TH * TW * CS;
    static constexpr int lds_floats = (in_floats > out_floats ? in_floats : out_floats) + CS * KK;
};

template <int K, int NPI>
__global__ __launch_bounds__(256, 2) void dwconv_f32m_k(const float* __restrict__ x, const float* __restrict__ w,
                                                        float* __restrict__ y, const F32mGeom g) {
    using Sh = F32mShape<K, NPI>;
    constexpr int WR = Sh::WR, G = Sh::G, PR = Sh::PR, TH = Sh::TH, TW = Sh::TW, NI = Sh::NI, CS = Sh::CS, SR = Sh::SR,
                  SC = Sh::SC, SP = Sh::SP, PLANE = Sh::PLANE, KK = Sh::KK;
    extern __shared__ float lds[];
    float* xl = lds;                                                        // [NI][CS][SR][SP]
    float* wl = lds + (Sh::in_floats > Sh::out_floats ? Sh::in_floats : Sh::out_floats);   // [CS][K][K]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int t = blockIdx.x;
    const int sl = t % g.nsl;
    t /= g.nsl;
    const int ctile = t % g.nct;
    t /= g.nct;
    const int rtile = t % g.nrt, ig = t / g.nrt;
    const int c0 = sl * CS, r0 = rtile * TH, cl0 = ctile * TW, b0 = ig * NI;

    // the slice's filters, rotated for the input gradient, zero for channels past C
    for (int i = tid; i < CS * KK; i += 256) {
        const int c = i % CS, tap = i / CS, ti = tap / K, tj = tap - ti * K;
        const int src = g.flip ? (K - 1 - ti) * K + (K - 1 - tj) : tap;
        wl[c * KK + tap] = c0 + c < g.C ? w[(long long)src * g.C + c0 + c] : 0.f;
    }
    // the tile and its halo, channel-major: an item is 4 channels of one pixel; rows, columns, images and channels
    // outside the tensor read as zero through the descriptor (an offset past its end)
    {
        const int nimg = g.B - b0 < NI ? g.B - b0 : NI;
        const long long img_bytes = (long long)g.H * g.W * g.C * 4;
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(x + (long long)b0 * g.H * g.W * g.C), (short)0, (int)(nimg * img_bytes), 0x00020000);
        constexpr int NQ = CS / 4, NITEM = NI * SR * SC * NQ, BATCH = 8;
        for (int base = 0; base < NITEM; base += 256 * BATCH) {
            v4u v[BATCH];
            int dst[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const int it = base + tid + u * 256;
                const int cq = it % NQ, p = it / NQ, col = p % SC, q = p / SC, row = q % SR, img = q / SR;
                const int ih = r0 - g.PH + row, iw = cl0 - g.PW + col;
                const bool ok = it < NITEM && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W && c0 + 4 * cq < g.C;
                const uint32_t off = (uint32_t)((((long long)img * g.H + ih) * g.W + iw) * g.C + c0 + 4 * cq) * 4u;
                v[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(ok ? off : 0x80000000u), 0, 0);
                dst[u] = it < NITEM ? ((img * CS + 4 * cq) * SR + row) * SP + col : -1;
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                if (dst[u] >= 0) {
                    // (each element through a scalar of its own: a bit cast applied to a vector element expression
                    // takes the vector's first element)
                    const unsigned e0 = v[u].x, e1 = v[u].y, e2 = v[u].z, e3 = v[u].w;
                    xl[dst[u]] = __uint_as_float(e0);
                    xl[dst[u] + PLANE] = __uint_as_float(e1);
                    xl[dst[u] + 2 * PLANE] = __uint_as_float(e2);
                    xl[dst[u] + 3 * PLANE] = __uint_as_float(e3);
                }
            }
        }
    }
    __syncthreads();

    // lane: n = patch (and image) of the B operand and of the results, kq = window column within a group / output row
    const int n = lane & 15, kq = lane >> 4;
    const int img = n / NPI, np = n - img * NPI;
    const int oy = n >> 2, ox = n & 3;   // as an A lane: m = n = (output row, output column) of the patch
    v4f acc[2][PR];
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int pr = 0; pr < PR; ++pr) acc[cc][pr] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
        const int ch = wave * 2 + cc;
        if (c0 + ch < g.C) {   // uniform
            // A[m][kq] of (window row r, column group gg): w[r - oy][4 gg + kq - ox], zero outside the filter
            float a[WR][G];
            const float* wc = wl + ch * KK;
#pragma unroll
            for (int r = 0; r < WR; ++r)
#pragma unroll
                for (int gg = 0; gg < G; ++gg) {
                    const int i = r - oy, j = 4 * gg + kq - ox;
                    const bool ok = i >= 0 && i < K && j >= 0 && j < K;
                    const float v = wc[ok ? i * K + j : 0];
                    a[r][gg] = ok ? v : 0.f;
                }
            // (the operands stay in registers: left alone, the compiler reads each of them from LDS again where it is
            // used, one LDS latency in front of every few instructions)
#pragma unroll
            for (int r = 0; r < WR; ++r)
#pragma unroll
                for (int gg = 0; gg < G; ++gg) asm volatile("" : "+v"(a[r][gg]));
            const float* xb = xl + (img * CS + ch) * PLANE + 4 * np + kq;
            // B operands one staged row ahead of the products that use them
            float bq[2][G];
#pragma unroll
            for (int gg = 0; gg < G; ++gg) bq[0][gg] = xb[4 * gg];
#pragma unroll
            for (int rho = 0; rho < SR; ++rho) {
                if (rho + 1 < SR) {
#pragma unroll
                    for (int gg = 0; gg < G; ++gg) bq[(rho + 1) & 1][gg] = xb[(rho + 1) * SP + 4 * gg];
                }
                __builtin_amdgcn_sched_barrier(0);   // (the reads stay in front of this row's products)
#pragma unroll
                for (int gg = 0; gg < G; ++gg) {
#pragma unroll
                    for (int pr = 0; pr < PR; ++pr) {
                        const int r = rho - 4 * pr;
                        if (r >= 0 && r < WR)
                            acc[cc][pr] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r][gg], bq[rho & 1][gg], acc[cc][pr], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    __syncthreads();   // every wavefront is done with the staged tile: the results take its place
    // results: lane (n, q = kq) holds outputs (row 4 pr + q, columns 4 np .. 4 np + 3) of its patch; tile [NI][TH][TW][CS]
    float* ol = lds;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
        const int ch = wave * 2 + cc;
#pragma unroll
        for (int pr = 0; pr < PR; ++pr)
#pragma unroll
            for (int i = 0; i < 4; ++i) ol[((img * TH + 4 * pr + kq) * TW + 4 * np + i) * CS + ch] = acc[cc][pr][i];
    }
    __syncthreads();
    {
        constexpr int NQ = CS / 4, NITEM = NI * TH * TW * NQ;
        for (int it = tid; it < NITEM; it += 256) {
            const int cq = it % NQ, p = it / NQ, col = p % TW, q = p / TW, row = q % TH, im = q / TH;
            const int b = b0 + im, oh = r0 + row, ow = cl0 + col, c = c0 + 4 * cq;
            if (b < g.B && oh < g.OH && ow < g.OW && c < g.C)
                *reinterpret_cast<float4*>(y + (((long long)b * g.OH + oh) * g.OW + ow) * g.C + c) =
                    *reinterpret_cast<const float4*>(ol + ((im * TH + row) * TW + col) * CS + 4 * cq);
        }
    }
}

template <int K, int NPI>
int f32m_go(const void* x, const void* w, void* y, int B, int H, int W, int C, int PH, int PW, bool flip, hipStream_t s) {
    using Sh = F32mShape<K, NPI>;
    F32mGeom g;
    g.B = B, g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW, g.flip = flip ? 1 : 0;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    g.nrt = cdiv(g.OH, Sh::TH), g.nct = cdiv(g.OW, Sh::TW), g.nsl = cdiv(C, Sh::CS);
    const long long nblocks = (long long)cdiv(B, Sh::NI) * g.nrt * g.nct * g.nsl;
    if (nblocks > 0x7fffffffLL || (long long)Sh::NI * H * W * C * 4 > 0x7fffffffLL) return -1;   // (32-bit byte offsets)
    auto kern = dwconv_f32m_k<K, NPI>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), (size_t)Sh::lds_floats * sizeof(float), s, (const float*)x,
                       (const float*)w, (float*)y, g);
    return check_launch("dwconv_f32m");
}

template <int K>
int f32m_k(const void* x, const void* w, void* y, int B, int H, int W, int C, int PH, int PW, bool flip, hipStream_t s) {
    const int OW = W + 2 * PW - K + 1;
    // narrow images: two per tile, 32 columns each
    if (OW <= 32 && B > 1) return f32m_go<K, 8>(x, w, y, B, H, W, C, PH, PW, flip, s);
    return f32m_go<K, 16>(x, w, y, B, H, W, C, PH, PW, flip, s);
}

}  // namespace

// -1: not covered or not worth it (the caller goes on to the vector-ALU kernel): other filter sizes, channel counts
// that are not multiples of 4, unaligned tensors, images too large for 32-bit byte offsets, shapes on which the
// vector-ALU kernel was measured as fast or faster.
int dwconv_f32m_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW, int PH, int PW,
                       bool flip, hipStream_t s) {
    if (KH != KW || C % 4 != 0 || B < 1 || H + 2 * PH - KH + 1 < 1 || W + 2 * PW - KW + 1 < 1) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 15) || (reinterpret_cast<uintptr_t>(w) & 3))
        return -1;
    if (tune_env("PDW_NO_F32M")) return -1;
    // Where it pays, by measurement against the vector-ALU kernel (1.2-1.9x): the largest filter on images wider than
    // half a tile, and filters from 11 on small tensors, where the vector-ALU kernel's 32-channel workgroups are too
    // few to fill the chip.  Elsewhere this kernel's staging (half-used 64-byte sectors: 8 channels of a pixel) and the
    // fp32 matrix rate leave it level with or behind the vector ALU (0.5-1.0x), and the caller goes on to that.
    const int OW = W + 2 * PW - KW + 1;
    const bool small = (long long)B * H * W * C <= (2 << 20);
    if (!tune_env("PDW_F32M_ALWAYS") && !(OW > 32 && (KW >= 17 || (KW >= 11 && small)))) return -1;
    switch (KW) {
        case 5: return f32m_k<5>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 7: return f32m_k<7>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 9: return f32m_k<9>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 11: return f32m_k<11>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 13: return f32m_k<13>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 15: return f32m_k<15>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case 17: return f32m_k<17>(x, w, y, B, H, W, C, PH, PW, flip, s);
        default: return -1;
    }
}

}  // namespace pdw
