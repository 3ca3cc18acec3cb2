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
// A unit is 4 output rows x 4 strips of S columns x 16 channels, the work of one wavefront per tile; a
// workgroup of 4 wavefronts owns a tile of 16 rows x 4S columns x 16 channels.  The tile's input window is
// staged in LDS channel-major, xl[row][channel][column pair] (a dword holds two adjacent columns), which makes
// the B operand of an even output column two consecutive dwords.  The odd column next to it uses the SAME
// operand with the filter shifted by one column (w'[v+1] = w[v], which still fits the padded width because K is
// odd), so the inner loop has no vector-ALU work at all: a 4x4x4 MFMA occupies the SIMD for 8 cycles and every
// vector instruction next to it for 4 more.  Workgroups are persistent over their tiles: the filter operands are
// built in LDS once, a tile's window is requested into registers as early as possible (the first before the
// filter is staged, the next ones as soon as the operand registers are free) and written to LDS in passes,
// and the results leave through LDS as 16-byte stores.
#pragma once
#include <mutex>
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

// The two 16-bit values of a window dword as floats.
template <typename T>
__device__ __forceinline__ float pair_lo(uint32_t d) {
    return to_f32(__builtin_bit_cast(T, (unsigned short)(d & 0xffffu)));
}
template <typename T>
__device__ __forceinline__ float pair_hi(uint32_t d) {
    return to_f32(__builtin_bit_cast(T, (unsigned short)(d >> 16)));
}

// 8 values of T: a + b / 4, rounded once more (what an accumulating pool gradient does to a stored tensor).
template <typename T>
__device__ __forceinline__ uint4 add_quarter(uint4 a, uint4 b) {
    union U {
        uint4 u;
        T t[8];
    } ua, ub, uo;
    ua.u = a, ub.u = b;
#pragma unroll
    for (int i = 0; i < 8; ++i) uo.t[i] = from_f32<T>(to_f32(ua.t[i]) + 0.25f * to_f32(ub.t[i]));
    return uo.u;
}

struct MfmaGeom {
    int H, W, C;      // input extents
    int OH, OW;       // output extents
    int PH, PW;       // padding
    int tiles_h, tiles_w, ntiles, nchunks, slices;
    int CPn;          // LDS dwords per channel row (>= staged column pairs)
    int flip;         // 1: 180-degree rotated filter (input gradient)
    int AH, AW;       // extents of the half-resolution addend (OH = 2 AH, OW = 2 AW), 0 without one
    int one;          // the constant 1 (see the kernel)
};

template <int K, int S, int NWV>
struct MfmaShape {
    static constexpr int CS = 16;                   // channels per workgroup
    static constexpr int TH = 4 * NWV, TW = 4 * S;  // tile = NWV units of 4 rows, one per wavefront
    static constexpr int KP = (K + 3) / 4 * 4;      // filter columns padded to the MFMA k
    static constexpr int NVB = KP / 4;
    static constexpr int NPH = K + 3;               // phases (input rows) per row group
    static constexpr int WR = K + 6;                // filter rows in LDS, 3 zero rows on either side
    static constexpr int ROWS_IN = TH + K - 1;
    static constexpr int NCOL = (TW + KP) / 2;      // staged column pairs: every pair an operand reads, the ones under
                                                    // the zero filter columns included (0 * garbage could be NaN)
};

// MODE 0: plain.  MODE 1 (input gradient of a tensor that was also average-pooled 2x2): y += add[i/2, j/2] / 4.
// MODE 2 (forward): the 2x2 average pool of x itself is written to `pool` as a by-product, from the staged window.
template <typename T, int K, int S, int NWV, int MODE>
__global__ __launch_bounds__(NWV * 64, NWV == 4 ? 2 : 1) void dwconv_mfma_k(const T* __restrict__ x, const T* __restrict__ w,
                                                             const T* __restrict__ add, T* __restrict__ pool,
                                                             T* __restrict__ y, const MfmaGeom g) {
    constexpr bool ADD = MODE == 1;
    using Sh = MfmaShape<K, S, NWV>;
    constexpr int V = 8, NT = NWV * 64, CS = Sh::CS, TH = Sh::TH, TW = Sh::TW;
    constexpr int NVB = Sh::NVB, NPH = Sh::NPH, WR = Sh::WR, ROWS_IN = Sh::ROWS_IN, NCOL = Sh::NCOL;
    constexpr int NQ = (S / 2 + 2 * NVB + 1) / 2;  // 64-bit operand registers per copy of a lane's window
    constexpr int UPP = NT / (CS / V);
    constexpr int NPRE = (ROWS_IN * NCOL + UPP - 1) / UPP;  // passes: a whole window sits in registers
    constexpr int NE = S / 2;                               // column pairs per strip
    constexpr int WPITCH = (16 * NVB + 4) * 4;              // elements per filter row in LDS
    static_assert(S % 2 == 0 && K % 2 == 1 && (NWV == 4 || NWV == 8), "bad shape");
    extern __shared__ uint32_t smem[];
    uint32_t* xl = smem;                                                  // [ROWS_IN][CS][CPn]
    // filter operands: wl[copy][3 + u][vb][channel] as 4 columns (8 bytes) each, copy 1 shifted by one column; a
    // row pitch of 16 NVB + 4 operands puts consecutive filter rows an odd multiple of 32 bytes apart modulo 256,
    // measured the best of the paddings 0..24 (the 4 rows an MFMA's lanes read then fall on different banks)
    T* wl = reinterpret_cast<T*>(smem + ROWS_IN * CS * g.CPn);

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int sl = bid % g.slices, chunk = bid / g.slices;
    const int c0 = sl * CS;
    const int tiles_per_img = g.tiles_h * g.tiles_w;

    TileStager<T, CS, V, NPRE, true, NT> st;
    st.init(tid, c0, g.C, ROWS_IN, NCOL, g.CPn);
    auto origin = [&](int tile, int& b, int& row0, int& col0) {
        b = tile / tiles_per_img;
        const int rem = tile - b * tiles_per_img;
        const int th_i = rem / g.tiles_w;
        row0 = th_i * TH, col0 = (rem - th_i * g.tiles_w) * TW;
    };
    // ---- filter slice, 8 channels of a tap per load (requested first: it is in LDS by the time the window arrives)
    constexpr int NW = K * K * (CS / 8), IT = (NW + NT - 1) / NT;
    uint4 val[IT];
#pragma unroll
    for (int s = 0; s < IT; ++s) {  // all loads of a thread in flight together
        const int idx = min(tid + s * NT, NW - 1);
        const int oct = idx & 1, uv = idx >> 1;
        val[s] = *reinterpret_cast<const uint4*>(w + uv * g.C + min(c0 + 8 * oct, g.C - 8));  // C % 8 == 0
    }
    int nb = 0, nrow0 = 0, ncol0 = 0;  // tile whose window is in flight
    if (chunk < g.ntiles) {
        origin(chunk, nb, nrow0, ncol0);
        st.issue(x + (long long)nb * g.H * g.W * g.C, g.H, g.W, g.C, nrow0 - g.PH, ncol0 - g.PW);
    }

    // ---- filter operands in LDS (rotated for the input gradient), zero elsewhere: cleared here, filled behind a
    // barrier that does not wait for the loads in flight, while the window is still on its way
    {
        uint4* wz = reinterpret_cast<uint4*>(wl);  // both copies: 2 * WR * WPITCH elements, a multiple of 8
        for (int i = tid; i < WR * WPITCH / 4; i += NT) wz[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    auto fill_filter = [&]() {
        unsigned short* wls = reinterpret_cast<unsigned short*>(wl);
#pragma unroll
        for (int s = 0; s < IT; ++s) {
            const int idx = tid + s * NT;
            if (idx < NW) {
                const int oct = idx & 1, uv = idx >> 1;
                const int u = uv / K, v = uv - u * K;
                const int uu = g.flip ? K - 1 - u : u, vv = g.flip ? K - 1 - v : v;
                const bool chok = c0 + 8 * oct < g.C;
                const uint32_t d[4] = {val[s].x, val[s].y, val[s].z, val[s].w};
                unsigned short* w0 = wls + (3 + uu) * WPITCH + ((vv >> 2) * 16 + 8 * oct) * 4 + (vv & 3);
                unsigned short* w1 = wls + (WR + 3 + uu) * WPITCH + (((vv + 1) >> 2) * 16 + 8 * oct) * 4 + ((vv + 1) & 3);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const unsigned short val16 = (unsigned short)(chok ? (d[e >> 1] >> (16 * (e & 1))) & 0xffffu : 0u);
                    w0[4 * e] = val16;
                    w1[4 * e] = val16;
                }
            }
        }
    };
    // LDS accesses of this wavefront are complete, then the workgroup barrier: unlike __syncthreads this leaves
    // global loads in flight
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // ---- this lane's operand addresses: wavefront = unit row, lane = (channel bq, q)
    const int bq = lane >> 2, q = lane & 3;
    const int RP = CS * g.CPn;  // dwords per staged row
    const uint32_t* xbase = xl + (wv * 4 * CS + bq) * g.CPn + q * (S / 2);
    const T* wbase = wl + (3 - q) * WPITCH + bq * 4;   // + WR * WPITCH: the shifted copy
    const int one = g.one;  // 1, opaque to the compiler: the second window copy is a load of its own, not a register shuffle

    for (int tile = chunk; tile < g.ntiles; tile += g.nchunks) {
        int b, orow0, ocol0;
        origin(tile, b, orow0, ocol0);
        lds_barrier();  // the previous window is fully consumed; first tile: the filter area is cleared
        if (tile == chunk) fill_filter();  // waits for the filter's loads only
        st.commit_begin();
#pragma unroll
        for (int it = 0; it < NPRE; ++it) st.commit_next(xl, it, g.H, g.W, orow0 - g.PH, ocol0 - g.PW);
        __syncthreads();
        if constexpr (MODE == 2) {
            // 2x2 means of the tile's own input pixels (H = OH, W = OW, both even, PW even: a window dword is one of
            // the pool's column pairs), 8 channels per item, summed in the order of the stand-alone pool kernel
            constexpr int PWh = TW / 2, NITEM = (TH / 2) * PWh * 2;
            const int AH = g.H >> 1, AW = g.W >> 1;
            T* pb = pool + ((long long)b * AH * AW) * g.C + c0;
            for (int it = tid; it < NITEM; it += NT) {
                const int oct = it & 1, px = it >> 1;
                const int pi = px / PWh, pj = px - pi * PWh;
                const int gi = (orow0 >> 1) + pi, gj = (ocol0 >> 1) + pj;
                if (gi < AH && gj < AW && c0 + 8 * oct < g.C) {
                    const uint32_t* wp = xl + ((g.PH + 2 * pi) * CS + 8 * oct) * g.CPn + (g.PW >> 1) + pj;
                    union {
                        uint4 u;
                        T t[8];
                    } o;
#pragma unroll
                    for (int ch = 0; ch < 8; ++ch) {
                        const uint32_t d0 = wp[ch * g.CPn], d1 = wp[CS * g.CPn + ch * g.CPn];
                        const float s = ((pair_lo<T>(d0) + pair_hi<T>(d0)) + pair_lo<T>(d1)) + pair_hi<T>(d1);
                        o.t[ch] = from_f32<T>(s * 0.25f);
                    }
                    *reinterpret_cast<uint4*>(pb + ((long long)gi * AW + gj) * g.C + 8 * oct) = o.u;
                }
            }
        }
        const int orow_b = orow0 + wv * 4;
        const bool has_next = tile + g.nchunks < g.ntiles;
        const bool active = orow_b < g.OH;  // this wavefront's unit has outputs (uniform per wavefront)
        f32x4 acc[S];
#pragma unroll
        for (int t = 0; t < S; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (active) {
            // Operands of a phase: the lane's window at pair offsets 0 and 1 (operand pairs must start at an even
            // register) and the 2 NVB filter operands.  They are requested one phase ahead, all at the top of the
            // phase, so the LDS latency lies under the 4 S NVB MFMAs of the current phase.
            constexpr bool REUSE = NWV == 4;
            struct Ops {
                uint2 P0[NQ], P1[NQ], ae[NVB], ao[NVB];
            };
            auto fetch = [&](Ops& o, const uint32_t* xr, const T* wr) {
                const uint32_t* xr1 = xr + one;
#pragma unroll
                for (int i = 0; i < NQ; ++i) {
                    if (2 * i < NE + 2 * NVB - 1) o.P0[i] = make_uint2(xr[2 * i], xr[2 * i + 1]);
                    if constexpr (!REUSE)
                        if (2 * i + 1 < NE + 2 * NVB - 1) o.P1[i] = make_uint2(xr1[2 * i], xr1[2 * i + 1]);
                }
                if constexpr (REUSE) {
                    // one wavefront per SIMD: the loop is bound by LDS traffic and the vector ALU is idle, so the
                    // copy at pair offset 1 is put together from the registers of the first (2 moves per operand)
#pragma unroll
                    for (int i = 0; i < NQ; ++i)
                        if (2 * i + 1 < NE + 2 * NVB - 1) o.P1[i] = make_uint2(o.P0[i].y, o.P0[i + 1 < NQ ? i + 1 : i].x);
                }
#pragma unroll
                for (int vb = 0; vb < NVB; ++vb) {
                    o.ae[vb] = *reinterpret_cast<const uint2*>(wr + vb * 64);
                    o.ao[vb] = *reinterpret_cast<const uint2*>(wr + WR * WPITCH + vb * 64);
                }
            };
            auto multiply = [&](const Ops& o) {
#pragma unroll
                for (int vb = 0; vb < NVB; ++vb)
#pragma unroll
                    for (int e = 0; e < NE; ++e) {
                        const int j = e + 2 * vb;  // first column pair of the operand
                        const uint2 bop = (j % 2 == 0) ? o.P0[j / 2] : o.P1[j / 2];
                        acc[2 * e] = mfma4(o.ae[vb], bop, acc[2 * e], T());
                        acc[2 * e + 1] = mfma4(o.ao[vb], bop, acc[2 * e + 1], T());
                    }
            };
            const uint32_t* xr = xbase;
            const T* wr = wbase;
            // two operand sets when the registers allow it (2 wavefronts per SIMD: 256 registers each)
            constexpr bool kAhead = 2 * (4 * NQ + 4 * NVB) + 4 * S <= 176;
            if constexpr (kAhead) {
                Ops oa, ob;
                fetch(oa, xr, wr);
                static_assert(NPH % 2 == 0, "phases are processed in pairs");
                // LDS reads of the next phase interleaved with the MFMAs of this one, one read per MPR MFMAs: issued
                // in a block they would leave the matrix pipe idle, a wavefront issues in order
                constexpr int NLD = NE + 2 * NVB + NVB, MPR = (2 * NE * NVB) / NLD > 1 ? (2 * NE * NVB) / NLD : 1;
                auto interleave = [&]() {
#pragma unroll
                    for (int i = 0; i < NLD; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
                    }
                };
#pragma unroll 1
                for (int p = 0; p < NPH; p += 2) {
                    xr += RP, wr += WPITCH;
                    fetch(ob, xr, wr);
                    multiply(oa);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    xr += RP, wr += WPITCH;
                    fetch(oa, xr, wr);  // after the last phase: one row past the window and the filter, unused
                    multiply(ob);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll 1
                for (int p = 0; p < NPH; ++p) {
                    Ops oa;
                    fetch(oa, xr, wr);
                    multiply(oa);
                    xr += RP, wr += WPITCH;
                }
            }
        }
        // ---- results -> LDS as yl[row][column][16 channels] (one rounding to T), then out in 16-byte pieces:
        // the 2-byte values a lane owns are 4 rows x S scattered pixels, far too many store instructions.
        constexpr int NIT = (TH * TW * 2 + NT - 1) / NT;  // 16-byte pieces (8 channels of a pixel) per thread
        __syncthreads();  // every wavefront is done reading the window
        T* yl = reinterpret_cast<T*>(smem);
        if (active) {
            T* yq = yl + ((wv * 4) * TW + q * S) * CS + bq;  // register m of acc[t]: row m, column t of strip q
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int t = 0; t < S; ++t) yq[(m * TW + t) * CS] = from_f32<T>(acc[t][m]);
        }
        // The addend (gradient of a 2x2 average pool taken of the same tensor: a quarter of the pooled gradient at
        // every pixel of its window) is requested once the accumulators are free.
        uint4 av[NIT];
        if constexpr (ADD) {
            __builtin_amdgcn_sched_barrier(0);
            const T* ab = add + ((long long)b * g.AH * g.AW) * g.C + c0;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int idx = tid + it * NT;
                const int half = idx & 1, pix = idx >> 1;
                const int r = pix / TW, cc = pix - r * TW;
                const int ar = min((orow0 + r) >> 1, g.AH - 1), ac = min((ocol0 + cc) >> 1, g.AW - 1);
                const int ach = min(8 * half, g.C - c0 - 8);  // C % 8 == 0: always a whole piece inside the tensor
                av[it] = *reinterpret_cast<const uint4*>(ab + ((long long)ar * g.AW + ac) * g.C + ach);
            }
        }
        __syncthreads();
        {
            T* yb = y + ((long long)b * g.OH * g.OW) * g.C + c0;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int idx = tid + it * NT;
                const int half = idx & 1, pix = idx >> 1;
                const int r = pix / TW, cc = pix - r * TW;
                if (pix < TH * TW && orow0 + r < g.OH && ocol0 + cc < g.OW && c0 + 8 * half < g.C) {
                    uint4 o = *reinterpret_cast<const uint4*>(yl + pix * CS + 8 * half);
                    if constexpr (ADD) o = add_quarter<T>(o, av[it]);
                    *reinterpret_cast<uint4*>(yb + ((long long)(orow0 + r) * g.OW + ocol0 + cc) * g.C + 8 * half) = o;
                }
            }
        }
        if (has_next) {  // the next window is requested only now: its registers were the operand registers above
            origin(tile + g.nchunks, nb, nrow0, ncol0);
            st.issue(x + (long long)nb * g.H * g.W * g.C, g.H, g.W, g.C, nrow0 - g.PH, ncol0 - g.PW);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Host side

template <typename T, int K, int S, int NWV>
static int launch_mfma(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C,
                       int PH, int PW, bool flip, hipStream_t s) {
    using Sh = MfmaShape<K, S, NWV>;
    MfmaGeom g;
    g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW, g.flip = flip ? 1 : 0, g.one = 1;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    g.AH = add ? g.OH / 2 : 0, g.AW = add ? g.OW / 2 : 0;
    g.slices = cdiv(C, Sh::CS);
    g.tiles_h = cdiv(g.OH, Sh::TH), g.tiles_w = cdiv(g.OW, Sh::TW);
    const long long ntiles = (long long)B * g.tiles_h * g.tiles_w;
    if (ntiles > 0x7fffffffLL || (long long)H * W * C > 0x7fffffffLL || (long long)g.OH * g.OW * C > 0x7fffffffLL)
        return -1;
    g.ntiles = (int)ntiles;
    // LDS: pitch = pairs per channel row.  A lane's operand reads start at pitch * channel + S/2 * strip: measured
    // on the part, a pitch of 4 mod 8 is free of bank conflicts for strips of 14 columns, an odd one for strips of 8.
    const size_t wbytes = (size_t)(2 * Sh::WR + 1) * (16 * Sh::NVB + 4) * 8;  // + the row the last prefetch reads
    auto lds_of = [&](int p) { return (size_t)Sh::ROWS_IN * Sh::CS * p * 4 + wbytes; };
    int pitch = Sh::NCOL;
    while (S == 14 ? pitch % 8 != 4 : pitch % 2 != 1) ++pitch;
    if (lds_of(pitch) > 160 * 1024) pitch = Sh::NCOL;
    if (tune_env("PDW_MFMA_PITCH") && atoi(tune_env("PDW_MFMA_PITCH")) >= Sh::NCOL) pitch = atoi(tune_env("PDW_MFMA_PITCH"));
    if (lds_of(pitch) > 160 * 1024) return -1;
    g.CPn = pitch;
    size_t lds = lds_of(pitch);
    if (tune_env("PDW_MFMA_LDSMIN") && lds < (size_t)atoi(tune_env("PDW_MFMA_LDSMIN"))) lds = atoi(tune_env("PDW_MFMA_LDSMIN"));
    // persistent workgroups: as many as are resident at once, tiles dealt out as evenly as they divide
    const int resident = (int)((160 * 1024) / (lds + 1024)) >= 2 && NWV == 4 ? 2 : 1;
    const int cap = (256 * resident) / g.slices > 1 ? (256 * resident) / g.slices : 1;
    const long long rounds = cdiv(ntiles, (long long)cap);
    long long nch = cdiv(ntiles, rounds);
    if (tune_env("PDW_MFMA_NCH")) nch = atoi(tune_env("PDW_MFMA_NCH"));
    g.nchunks = (int)(nch < 1 ? 1 : nch);
    const long long nblocks = (long long)g.nchunks * g.slices;
    const int mode = add ? 1 : (pool ? 2 : 0);
    auto kern = mode == 1 ? dwconv_mfma_k<T, K, S, NWV, 1> : (mode == 2 ? dwconv_mfma_k<T, K, S, NWV, 2> : dwconv_mfma_k<T, K, S, NWV, 0>);
    static std::once_flag attr_once[3];
    std::call_once(attr_once[mode], [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(NWV * 64), lds, s, (const T*)x, (const T*)w, (const T*)add,
                       (T*)pool, (T*)y, g);
    return check_launch("dwconv_mfma");
}

// -1: not covered (the caller falls back to the vector-ALU tiled kernel).
template <typename T, int K>
static int launch_mfma_best(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W,
                            int C, int PH, int PW, bool flip, hipStream_t s) {
    const int OH = H + 2 * PH - K + 1, OW = W + 2 * PW - K + 1;
    if (OH < 1 || OW < 1 || C % 8 != 0) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(w) & 15) != 0)
        return -1;
    if (add && ((OH | OW) & 1 || (reinterpret_cast<uintptr_t>(add) & 15) != 0)) return -1;
    if (pool && (add || flip || OH != H || OW != W || ((H | W | PW) & 1) || (reinterpret_cast<uintptr_t>(pool) & 15) != 0))
        return -1;
    // strips of 14 columns (tile 56 wide) or 8 (tile 32 wide): whichever pads the output width less
    const bool s14 = (long long)cdiv(OW, 56) * 56 <= (long long)cdiv(OW, 32) * 32;
    const int tw = s14 ? 56 : 32;
    // 8 wavefronts per workgroup (tile 32 rows) when that still yields a workgroup for most CUs
    const long long t8 = (long long)B * cdiv(OH, 32) * cdiv(OW, tw) * cdiv(C, 16);
    bool w8 = t8 >= 192;
    if (tune_env("PDW_MFMA_NWV")) w8 = atoi(tune_env("PDW_MFMA_NWV")) == 8;
    if (s14) {
        if (w8) return launch_mfma<T, K, 14, 8>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
        return launch_mfma<T, K, 14, 4>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
    }
    if (w8) return launch_mfma<T, K, 8, 8>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
    return launch_mfma<T, K, 8, 4>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
}

template <int K>
static int launch_mfma_dtype(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W,
                             int C, int PH, int PW, bool flip, int dtype, hipStream_t s) {
    switch (dtype) {
        case kF16: return launch_mfma_best<f16_t, K>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
        case kBF16: return launch_mfma_best<bf16_t, K>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, s);
        default: return -1;
    }
}

}  // namespace pdw
