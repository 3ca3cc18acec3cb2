// Depthwise convolution on the matrix cores: forward and input gradient for 16-bit types, stride 1,
// dilation 1, odd square filters (the input gradient is the same kernel run on gy with the 180-degree
// rotated filter and padding k-1-p).
//
// v_mfma_f32_4x4x4_16b_{bf16,f16} multiplies 16 independent 4x4x4 blocks per instruction.  A block is one
// channel; its product is
//     D[m][n] += sum_k A[m][k] * B[k][n]        m = output row i0+m, n = one of 4 column strips, k = 4 filter columns
// with, for the input row r = i0 + p ("phase" p = 0 .. K+2) and filter-column block vb:
//     A[m][k] = w[p - m][4 vb + k]              (zero outside the filter: the filter is stored with 3 zero rows
//                                                above and below and zero columns up to a multiple of 4)
//     B[k][n] = x[r][col(n) + t + 4 vb + k]     t = output column inside strip n
// so that one staged input row serves the 4 output rows of a row group, and K+3 phases x ceil(K/4) blocks
// cover the whole filter: 1024 multiply-adds per instruction, of which K/(K+3) * K/ceil4(K) are useful
// (66 % at K = 13), against 128 per v_dot2.  A lane is (channel b = lane / 4, q = lane % 4): q is the output
// row m in the A operand and the strip n in the B operand, and register m of the result holds output row m
// of strip q.
//
// The 4 strips of a unit are S columns wide and sit side by side (SR = 1: a unit is 4 rows x 4S columns) or
// in a 2 x 2 arrangement (SR = 2: 8 rows x 2S columns; the strips of the lower pair use input rows 4 further
// down with the same phase, so they share the A operand).  A workgroup of 4 wavefronts owns a tile of 4 units:
// CG groups of 16 channels x 4/CG unit rows.  The tile's input window is staged in LDS channel-major,
// xl[row][channel][column pair] (a dword holds two adjacent columns), which makes the B operand of an even
// output column two consecutive dwords; odd columns use the same dwords shifted by 16 bits (v_alignbit).
// Operand pairs must start at an even register, so the window is read twice, at pair offsets 0 and 1.
// Workgroups are persistent, one per CU (the window of the next tile is requested into registers while the
// current one is multiplied).
#pragma once
#include <stdlib.h>

#include "common.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma4(uint2 a, uint2 b, f32x4 c, bf16_t) {
    typedef short s4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma4(uint2 a, uint2 b, f32x4 c, f16_t) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(h4, a), __builtin_bit_cast(h4, b), c, 0, 0, 0);
}

struct MfmaGeom {
    int H, W, C;      // input extents
    int OH, OW;       // output extents
    int PH, PW;       // padding
    int tiles_h, tiles_w, ntiles, nchunks, slices;
    int CPn;          // LDS dwords per channel row (>= staged column pairs)
    int flip;         // 1: 180-degree rotated filter (input gradient)
};

template <int K, int S, int SR, int CG>
struct MfmaShape {
    static constexpr int SC = 4 / SR;            // strips side by side
    static constexpr int UH = 4 * SR, UW = S * SC;  // unit = UH x UW outputs x 16 channels
    static constexpr int RGB = 4 / CG;           // unit rows per tile
    static constexpr int TH = UH * RGB, TW = UW, CS = 16 * CG;
    static constexpr int KP = (K + 3) / 4 * 4;   // filter columns padded to the MFMA k
    static constexpr int NVB = KP / 4;
    static constexpr int NPH = K + 3;            // phases (input rows) per row group
    static constexpr int WR = K + 6;             // filter rows in LDS, 3 zero rows on either side
    static constexpr int ROWS_IN = TH + K - 1;
    static constexpr int NCOL = (TW + KP) / 2;   // staged column pairs: every pair an operand reads, the ones under
                                                 // the zero filter columns included (0 * garbage could be NaN)
};

template <typename T, int K, int S, int SR, int CG, int V>
__global__ __launch_bounds__(256, 1) void dwconv_mfma_k(const T* __restrict__ x, const T* __restrict__ w,
                                                        T* __restrict__ y, const MfmaGeom g) {
    using Sh = MfmaShape<K, S, SR, CG>;
    constexpr int SC = Sh::SC, UH = Sh::UH, TH = Sh::TH, TW = Sh::TW, CS = Sh::CS;
    constexpr int KP = Sh::KP, NVB = Sh::NVB, NPH = Sh::NPH, WR = Sh::WR, ROWS_IN = Sh::ROWS_IN, NCOL = Sh::NCOL;
    constexpr int NQ = (S / 2 + 2 * NVB + 1) / 2;  // 64-bit operand registers per copy of a lane's window
    constexpr int CV = CS / V, UPP = 256 / CV;
    constexpr int NPRE = (ROWS_IN * NCOL + UPP - 1) / UPP;  // the whole window of the next tile sits in registers
    static_assert(S % 2 == 0 && K % 2 == 1 && (SR == 1 || SR == 2) && (CG == 1 || CG == 2 || CG == 4), "bad shape");
    extern __shared__ uint32_t smem[];
    uint32_t* xl = smem;                                                // [ROWS_IN][CS][CPn]
    T* wl = reinterpret_cast<T*>(smem + ROWS_IN * CS * g.CPn);          // [CS][WR][KP]

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int sl = bid % g.slices, chunk = bid / g.slices;
    const int c0 = sl * CS;
    const int tiles_per_img = g.tiles_h * g.tiles_w;

    TileStager<T, CS, V, NPRE, true> st;
    st.init(tid, c0, g.C, ROWS_IN, NCOL, g.CPn);
    auto origin = [&](int tile, int& b, int& row0, int& col0) {
        b = tile / tiles_per_img;
        const int rem = tile - b * tiles_per_img;
        const int th_i = rem / g.tiles_w;
        row0 = th_i * TH, col0 = (rem - th_i * g.tiles_w) * TW;
    };
    auto request = [&](int tile) {
        int b, row0, col0;
        origin(tile, b, row0, col0);
        st.issue(x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, row0 - g.PH, col0 - g.PW);
    };
    if (chunk < g.ntiles) request(chunk);

    // ---- filter slice -> wl[ch][3 + u][v] (rotated for the input gradient), zero elsewhere
    {
        uint32_t* wz = reinterpret_cast<uint32_t*>(wl);
        for (int i = tid; i < CS * WR * KP / 2; i += 256) wz[i] = 0u;
        __syncthreads();
        constexpr int NW = K * K * CS, SU = 8;
        unsigned short* wls = reinterpret_cast<unsigned short*>(wl);
        for (int i0 = tid; i0 < NW; i0 += 256 * SU) {
            uint32_t val[SU];
#pragma unroll
            for (int s = 0; s < SU; ++s) {
                const int idx = min(i0 + s * 256, NW - 1);
                const int ch = idx % CS, uv = idx / CS;
                val[s] = bits16(w[(long long)uv * g.C + min(c0 + ch, g.C - 1)]);
            }
#pragma unroll
            for (int s = 0; s < SU; ++s) {
                const int idx = i0 + s * 256;
                if (idx < NW) {
                    const int ch = idx % CS, uv = idx / CS;
                    const int u = uv / K, v = uv - u * K;
                    const int uu = g.flip ? K - 1 - u : u, vv = g.flip ? K - 1 - v : v;
                    wls[(ch * WR + 3 + uu) * KP + vv] = (unsigned short)(c0 + ch < g.C ? val[s] : 0u);
                }
            }
        }
    }

    // ---- this lane's operand addresses
    const int bq = lane >> 2, q = lane & 3;
    const int cg = wv % CG, ur = wv / CG;
    const int sr = q / SC, sc = q % SC;
    const int RP = CS * g.CPn;  // dwords per staged row
    const uint32_t* xbase = xl + ((ur * UH + sr * 4) * CS + cg * 16 + bq) * g.CPn + sc * (S / 2);
    const T* wbase = wl + ((cg * 16 + bq) * WR + 3 - q) * KP;

    for (int tile = chunk; tile < g.ntiles; tile += g.nchunks) {
        int b, orow0, ocol0;
        origin(tile, b, orow0, ocol0);
        __syncthreads();  // the previous tile is fully consumed (and, first time, the filter is staged)
        st.commit(xl, x + (long long)b * g.H * g.W * g.C, g.H, g.W, g.C, orow0 - g.PH, ocol0 - g.PW);
        __syncthreads();
        if (tile + g.nchunks < g.ntiles) request(tile + g.nchunks);

        f32x4 acc[S];
#pragma unroll
        for (int t = 0; t < S; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < NPH; ++p) {
            const uint32_t* xr = xbase + p * RP;
            // window copies at pair offsets 0 and 1, and the same shifted by one column
            uint2 P0[NQ], P1[NQ], O0[NQ], O1[NQ];
#pragma unroll
            for (int i = 0; i < NQ; ++i) {
                P0[i] = make_uint2(xr[2 * i], xr[2 * i + 1]);
                P1[i] = make_uint2(xr[2 * i + 1], xr[2 * i + 2]);
            }
#pragma unroll
            for (int i = 0; i < NQ; ++i) {
                O0[i] = make_uint2(__builtin_amdgcn_alignbit(P0[i].y, P0[i].x, 16),
                                   __builtin_amdgcn_alignbit(P1[i].y, P1[i].x, 16));
                O1[i] = make_uint2(__builtin_amdgcn_alignbit(P1[i].y, P1[i].x, 16),
                                   i + 1 < NQ ? __builtin_amdgcn_alignbit(P0[i + 1].y, P0[i + 1].x, 16) : 0u);
            }
#pragma unroll
            for (int vb = 0; vb < NVB; ++vb) {
                const uint2 a = *reinterpret_cast<const uint2*>(wbase + p * KP + 4 * vb);
#pragma unroll
                for (int t = 0; t < S; ++t) {
                    const int e = t / 2, j = e + 2 * vb;  // first column pair of the operand
                    const uint2 bop = (t % 2 == 0) ? ((j % 2 == 0) ? P0[j / 2] : P1[j / 2])
                                                   : ((j % 2 == 0) ? O0[j / 2] : O1[j / 2]);
                    acc[t] = mfma4(a, bop, acc[t], T());
                }
            }
        }
        // ---- store (one rounding to T): register m of acc[t] is output row m, column t of strip q
        const int ch = c0 + cg * 16 + bq;
        const int orow_b = orow0 + ur * UH + sr * 4, ocol_b = ocol0 + sc * S;
        if (ch < g.C) {
            T* yp = y + (((long long)b * g.OH + orow_b) * g.OW + ocol_b) * g.C + ch;
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int t = 0; t < S; ++t)
                    if (orow_b + m < g.OH && ocol_b + t < g.OW) yp[(m * g.OW + t) * g.C] = from_f32<T>(acc[t][m]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Host side

template <typename T, int K, int S, int SR, int CG>
static int launch_mfma(const void* x, const void* w, void* y, int B, int H, int W, int C, int PH, int PW, bool flip,
                       hipStream_t s) {
    using Sh = MfmaShape<K, S, SR, CG>;
    MfmaGeom g;
    g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW, g.flip = flip ? 1 : 0;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    g.slices = cdiv(C, Sh::CS);
    g.tiles_h = cdiv(g.OH, Sh::TH), g.tiles_w = cdiv(g.OW, Sh::TW);
    const long long ntiles = (long long)B * g.tiles_h * g.tiles_w;
    if (ntiles > 0x7fffffffLL || (long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL)
        return -1;
    g.ntiles = (int)ntiles;
    // LDS: pitch = pairs per channel row, 4 mod 8 keeps the 16 channels x 4 strips of an operand read on
    // distinct banks; fall back to the bare width when that does not fit.
    const size_t wbytes = (size_t)Sh::CS * Sh::WR * Sh::KP * 2;
    const int need = Sh::NCOL;
    int pitch = need;
    while (pitch % 8 != 4) ++pitch;
    auto lds_of = [&](int p) { return (size_t)Sh::ROWS_IN * Sh::CS * p * 4 + wbytes; };
    if (lds_of(pitch) > 160 * 1024) pitch = need;
    if (lds_of(pitch) > 160 * 1024) return -1;
    g.CPn = pitch;
    const size_t lds = lds_of(pitch);
    // persistent workgroups, one per CU; tiles dealt out as evenly as they divide
    const int cap = 256 / g.slices > 1 ? 256 / g.slices : 1;
    const long long rounds = cdiv(ntiles, (long long)cap);
    long long nch = cdiv(ntiles, rounds);
    if (getenv("PDW_MFMA_NCH")) nch = atoi(getenv("PDW_MFMA_NCH"));
    g.nchunks = (int)(nch < 1 ? 1 : nch);
    const long long nblocks = (long long)g.nchunks * g.slices;
    auto kern = dwconv_mfma_k<T, K, S, SR, CG, 8>;
    static bool attr_done = false;
    if (!attr_done) {
        (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        attr_done = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), lds, s, (const T*)x, (const T*)w, (T*)y, g);
    return check_launch("dwconv_mfma");
}

// -1: not covered (the caller falls back to the vector-ALU tiled kernel).
template <typename T, int K>
static int launch_mfma_best(const void* x, const void* w, void* y, int B, int H, int W, int C, int PH, int PW,
                            bool flip, hipStream_t s) {
    const int OH = H + 2 * PH - K + 1, OW = W + 2 * PW - K + 1;
    if (OH < 1 || OW < 1 || C % 8 != 0) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0) return -1;
    constexpr int S = 14;
    // strips side by side (tile 8 x 56) or 2 x 2 (tile 16 x 28): whichever pads the output less
    const long long pad1 = (long long)cdiv(OH, 8) * 8 * cdiv(OW, 56) * 56;
    const long long pad2 = (long long)cdiv(OH, 16) * 16 * cdiv(OW, 28) * 28;
    if (pad1 <= pad2) return launch_mfma<T, K, S, 1, 2>(x, w, y, B, H, W, C, PH, PW, flip, s);
    const char* e = getenv("PDW_MFMA");
    if (!e || atoi(e) < 2) return -1;  // the 2 x 2 arrangement is not yet faster than the vector-ALU kernel
    return launch_mfma<T, K, S, 2, 2>(x, w, y, B, H, W, C, PH, PW, flip, s);
}

template <int K>
static int launch_mfma_dtype(const void* x, const void* w, void* y, int B, int H, int W, int C, int PH, int PW,
                             bool flip, int dtype, hipStream_t s) {
    switch (dtype) {
        case kF16: return launch_mfma_best<f16_t, K>(x, w, y, B, H, W, C, PH, PW, flip, s);
        case kBF16: return launch_mfma_best<bf16_t, K>(x, w, y, B, H, W, C, PH, PW, flip, s);
        default: return -1;
    }
}

}  // namespace pdw
