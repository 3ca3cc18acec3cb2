// Thin dense layers of the block (inner dimensions <= 128, millions of rows) on the matrix
// cores.  These products are HBM-bound: the row matrix is streamed once with 16-byte vector loads
// straight into MFMA operand registers, the small weight matrix is staged to LDS once per
// workgroup, and the bias / per-image broadcast add is fused into the store.
//
//   rows:  Y[n,o] = sum_k X[n,k] * W(o,k) + bias[o] + rowbias[n / P][o]
//          computed as D = Wtile (32 features x 16 k) * Xtile^T (16 k x 32 rows) with
//          v_mfma_f32_32x32x16_{bf16,f16}; a lane then owns one row and 4 consecutive features per
//          accumulator group; the tile is transposed through a per-wave LDS buffer so the global
//          stores are whole 128-byte lines.
//   wgrad: dW[m,o] = sum_n A[n,m] * B[n,o]   (reduction over the rows)
//          64-row stages of A and B are copied to LDS with coalesced loads (requested one stage
//          ahead); the MFMA k dimension is the row index, so fragments are read from LDS column-wise.
//          Every wavefront accumulates all (m,o) tiles in registers, the wavefronts of a workgroup
//          are summed through LDS and the per-workgroup fp32 partials are reduced in a fixed order by
//          wgrad_reduce_parts (no atomics).
#include <math.h>
#include <stdlib.h>

#include "bilinear.h"
#include "common.h"
#include "kernels.h"
#include "reduce_parts.h"
#include "tile_common.h"

namespace pdw {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

struct alignas(16) Frag {
    uint32_t v[4];  // 8 16-bit values
};

__device__ __forceinline__ f32x16 mfma32(const Frag& a, const Frag& b, f32x16 c, bf16_t) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
}
__device__ __forceinline__ f32x16 mfma32(const Frag& a, const Frag& b, f32x16 c, f16_t) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
}


constexpr int kKT = 8;  // k tiles of 16  (inner dimension <= 128)
constexpr int kNT = 4;  // feature tiles of 32 (<= 128 features)

__device__ __forceinline__ uint32_t ld16(const bf16_t* p) { return (uint32_t) * reinterpret_cast<const unsigned short*>(p); }
__device__ __forceinline__ uint32_t ld16(const f16_t* p) { return (uint32_t) * reinterpret_cast<const unsigned short*>(p); }

// The 16-bit pattern `h` (in the low half of a register) as a float.
template <typename T>
__device__ __forceinline__ float half_to_f32(uint32_t h) {
    if constexpr (sizeof(T) == 2 && __is_same(T, bf16_t)) {
        return __builtin_bit_cast(float, h << 16);
    } else {
        return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
    }
}

// 8 values p[0], p[stride], ..., p[7*stride] packed as a fragment (zeros where !ok; p must be readable
// either way, so the 8 reads are issued back to back without a branch).
template <typename T>
__device__ __forceinline__ Frag gather8(const T* p, long long stride, bool ok) {
    uint32_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = ld16(p + j * stride);
    Frag f;
#pragma unroll
    for (int j = 0; j < 4; ++j) f.v[j] = ok ? (e[2 * j] | (e[2 * j + 1] << 16)) : 0u;
    return f;
}

// Offsets out[i] = (c / per_row) * pitch + (c % per_row) * unit for c = first + i * step, i < L (-1 once
// c / per_row >= max_rows), with one integer division instead of 2 L: a runtime division costs ~40 instructions.
template <int L>
__device__ __forceinline__ void strided_offsets(int first, int step, int per_row, int pitch, int unit, int max_rows,
                                                int (&out)[L]) {
    int r, c;
    if ((per_row & (per_row - 1)) == 0) {  // uniform; the usual widths: a shift instead of ~40 dependent instructions
        r = first >> (31 - __builtin_clz(per_row)), c = first & (per_row - 1);
    } else {
        r = first / per_row, c = first - r * per_row;
    }
    const int qr = step / per_row, qc = step - qr * per_row;  // uniform: scalar ALU
#pragma unroll
    for (int i = 0; i < L; ++i) {
        out[i] = r < max_rows ? r * pitch + c * unit : -1;
        r += qr, c += qc;
        if (c >= per_row) c -= per_row, ++r;
    }
}

// W[k][o] (K x NO, o fastest) -> wl[o][k] (pitch ldw) in 4 x 4 sub-blocks: a thread loads 4 consecutive o of 4
// consecutive k (four 8-byte loads), transposes them with 8 byte-permutes and writes 4 consecutive k of each o
// as one 8-byte LDS store; consecutive threads take consecutive k groups, so the stores fall on consecutive banks.
// Split in two so that the caller can put other global loads between the request and the LDS writes.
template <typename T, int IT>
struct WTransposer {
    uint2 row[IT][4];
    int dst[IT];
    __device__ __forceinline__ void load(const T* __restrict__ W, int K, int NO, int ldw, int tid) {
        const int kq = K / 4, nitem = kq * (NO / 4);
        int src[IT];
        strided_offsets<IT>(tid, 256, kq, 4, 4 * NO, NO / 4, src);       // W offset   4 kq * NO + 4 oq
        strided_offsets<IT>(tid, 256, kq, 4 * ldw, 4, NO / 4, dst);      // wl offset  4 oq * ldw + 4 kq
        (void)nitem;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                row[it][r] = *reinterpret_cast<const uint2*>(W + (src[it] >= 0 ? src[it] : 0) + r * NO);
    }
    __device__ __forceinline__ void store(T* wl, int ldw) const {
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            if (dst[it] >= 0) {
                T* q = wl + dst[it];
                const uint2* r = row[it];
                // o = 0: low halves of .x, o = 1: high halves of .x, o = 2 / 3: the same of .y
                *reinterpret_cast<uint2*>(q) = make_uint2(__builtin_amdgcn_perm(r[1].x, r[0].x, 0x05040100u),
                                                          __builtin_amdgcn_perm(r[3].x, r[2].x, 0x05040100u));
                *reinterpret_cast<uint2*>(q + ldw) = make_uint2(__builtin_amdgcn_perm(r[1].x, r[0].x, 0x07060302u),
                                                                __builtin_amdgcn_perm(r[3].x, r[2].x, 0x07060302u));
                *reinterpret_cast<uint2*>(q + 2 * ldw) = make_uint2(__builtin_amdgcn_perm(r[1].y, r[0].y, 0x05040100u),
                                                                    __builtin_amdgcn_perm(r[3].y, r[2].y, 0x05040100u));
                *reinterpret_cast<uint2*>(q + 3 * ldw) = make_uint2(__builtin_amdgcn_perm(r[1].y, r[0].y, 0x07060302u),
                                                                    __builtin_amdgcn_perm(r[3].y, r[2].y, 0x07060302u));
            }
        }
    }
};

// Weights live in LDS as wl[NO][K + 8] (the pad keeps 16-byte fragment reads of 32 consecutive rows off
// the same banks); every MFMA reads its weight fragment from there.  Row tiles (32 rows x K) are loaded
// fully coalesced - a wavefront reads its 32*K*2 contiguous bytes as 16-byte chunks, lane after lane -
// and re-shaped into MFMA fragments through a per-wave LDS buffer: row-strided fragment loads straight
// from global memory run ~2.5x slower on this part.  The same buffer transposes the result tile so the
// global stores are whole 128-byte lines as well.
//
// COLSUM: the kernel also writes colsum[tile][k] = sum over the tile's 32 rows of X[., k] (fp32), for callers that
// need per-image sums of X over the positions and would otherwise read X a second time.  Chunk i*64+lane of a tile
// is 8 columns of one row, and with 64 % (K/8) == 0 a lane keeps the same 8 columns for every chunk: 8 running
// sums per lane, combined over the 512/K lanes that share them through the tile buffer once the fragments are out.
//
// SK, SNO: the inner dimension and the feature count as compile-time constants (0: taken from the arguments).
// With both fixed (and then K % 16 == 0, NO % 32 == 0) a full tile is whole passes of 64 chunks in and out and
// whole MFMA steps, and its code has no per-lane predicates and no loop bounds to test: those were a third of the
// generic kernel's vector-ALU work.
//
// POOL (static widths; rows are the pixels of [B, Himg, Wimg] images, Himg % 4 == 0, Wimg % 8 == 0, no rowbias): a
// tile is a block of 4 image rows x 8 columns instead of 32 consecutive pixels (a load or store instruction still
// covers 1 KB of consecutive bytes of an image row: 4 pixels of 128 values in, 8 pixels of 64 out; with other widths
// an instruction's 64 chunks run over the end of the tile's image row into its next one), so that it holds 2 x 4 whole windows of
// the 2x2 average pool of Y, which the kernel writes to `pool` [B, Himg/2, Wimg/2, NO] from the result tile in LDS:
// (((y00 + y01) + y10) + y11) / 4 in fp32 of the rounded results, as the pooling kernel computes it.
//
// MID (rows = the pixels of [B, Himg, Wimg] images in the 4 x 8 tiles of POOL; written here for K = 64, NO = 128): the rows are not
// loaded but made, from the convolution outputs of a two-scale block (conv_block.py:18-21, 41-44): row (b, i, j) =
// [ gate(cf[b, i, j]) | bilinear resize to Himg x Wimg of gate(ch[b]) at (i, j) ], cf [B, Himg, Wimg, 64] the full
// scale, ch [B, Himg/2, Wimg/2, 64] the half scale, gate(v) = v[:32] * v[32:] * gs rounded to T.  A tile's resized
// half needs the 4 x 6 patch of the half scale around it: the patch is gated once into the tile buffer's spare columns
// and the tile's 32 pixels take their four taps from there (gated per output pixel it would be 4 gates per value
// instead of 0.75).  The rows are also written to mid->cat ([B, Himg, Wimg, 64], when not null): the arithmetic, and
// therefore every bit, is that of the gate kernels followed by this layer on their output.
// MID = 2: both scales arrive gated (cf [B, Himg, Wimg, 32] at a pixel stride of ldf values, ch [B, Himg/2, Wimg/2, 32]):
// the inference forward, whose convolutions gate in their stores; nothing but y is written.
struct MidRows {
    const void *cf, *ch;
    void* cat;
    int ldf;
    float gs;
};

// `x` rounded to T, as its 16-bit pattern in the low half of a register.
template <typename T>
__device__ __forceinline__ uint32_t f32_to_half(float x) {
    return (uint32_t)__builtin_bit_cast(unsigned short, from_f32<T>(x));
}

// 8 gate values a * b * s, each rounded to T (the arithmetic of the stand-alone gate kernels).
template <typename T>
__device__ __forceinline__ Frag gate8(const Frag& a, const Frag& b, float s) {
    Frag o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = gate_f32(half_to_f32<T>(a.v[j] & 0xffffu), half_to_f32<T>(b.v[j] & 0xffffu), s);
        const float hi = gate_f32(half_to_f32<T>(a.v[j] >> 16), half_to_f32<T>(b.v[j] >> 16), s);
        o.v[j] = f32_to_half<T>(lo) | (f32_to_half<T>(hi) << 16);
    }
    return o;
}

// 8 bilinear values of four taps (row y0: g00, g01; row y1: g10, g11), rounded to T (the arithmetic of the
// stand-alone resize kernels).
template <typename T>
__device__ __forceinline__ Frag bilinear8(const Frag& g00, const Frag& g01, const Frag& g10, const Frag& g11, float ly,
                                          float lx) {
    Frag o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = bl_mix(half_to_f32<T>(g00.v[j] & 0xffffu), half_to_f32<T>(g01.v[j] & 0xffffu),
                                half_to_f32<T>(g10.v[j] & 0xffffu), half_to_f32<T>(g11.v[j] & 0xffffu), ly, lx);
        const float hi = bl_mix(half_to_f32<T>(g00.v[j] >> 16), half_to_f32<T>(g01.v[j] >> 16),
                                half_to_f32<T>(g10.v[j] >> 16), half_to_f32<T>(g11.v[j] >> 16), ly, lx);
        o.v[j] = f32_to_half<T>(lo) | (f32_to_half<T>(hi) << 16);
    }
    return o;
}

template <typename T, bool KMAJOR, bool COLSUM, int SK = 0, int SNO = 0, bool POOL = false, int MID = 0>
__device__ __forceinline__ void dense_rows_body(const T* __restrict__ X, const T* __restrict__ W,
                                                const T* __restrict__ bias, const float* __restrict__ rowbias,
                                                T* __restrict__ Y, float* __restrict__ colsum, long long N, int Kd,
                                                int NOd, int P, int nktd, int nntd, int bid, int nblocks,
                                                uint32_t* dsm, T* __restrict__ pool = nullptr, int Himg = 0,
                                                int Wimg = 0, const MidRows* mid = nullptr) {
    constexpr bool STATIC = SK > 0 && SNO > 0;
    static_assert(!POOL || (STATIC && !KMAJOR), "pooled output: layers with their extents as constants");
    static_assert(MID == 0 || (((STATIC && SK <= 64) || (SK == 0 && SNO == 0)) && !KMAJOR && !COLSUM && !POOL),
                  "made rows: a layer with its extents as constants (inner width up to 64), or any covered widths");
    // POOL: first pixel of a tile and first pixel of its part of the pooled tensor (two 32-bit divisions per tile,
    // taken once, when the tile is requested, and kept for its way out)
    int px_next = 0, pp_next = 0, px_cur = 0, pp_cur = 0;
    [[maybe_unused]] int rb_next = 0, cb_next = 0, rb_cur = 0, cb_cur = 0;   // MID: the tile's block row and column
    auto tile_pixel = [&](long long t) {
        const unsigned tw = (unsigned)Wimg >> 3, tpi = ((unsigned)Himg >> 2) * tw;
        const unsigned ti = (unsigned)t, b = ti / tpi, r = ti - b * tpi, rb = r / tw, cb = r - rb * tw;
        px_next = (int)((b * (unsigned)Himg + 4 * rb) * (unsigned)Wimg + 8 * cb);
        pp_next = (int)((b * ((unsigned)Himg >> 1) + 2 * rb) * ((unsigned)Wimg >> 1) + 4 * cb);
        rb_next = (int)rb, cb_next = (int)cb;
        return (int)b;
    };
    static_assert(!STATIC || (SK % 16 == 0 && SNO % 16 == 0 && SK <= 128 && SNO <= 128), "static dense shape");
    const int K = STATIC ? SK : Kd, NO = STATIC ? SNO : NOd;
    const int nkt = STATIC ? SK / 16 : nktd, nnt = STATIC ? (SNO + 31) / 32 : nntd;
    T* wl = reinterpret_cast<T*>(dsm);
    // The weights are multiplied as NOP x KP (whole feature tiles, 4 or 8 steps of the inner dimension) with zeros
    // in the padding, so that the multiplication below is straight-line code without predicates.
    const int KP = nkt > 4 ? 128 : 64, NOP = nnt * 32;
    const int ldw = KP + 8;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int ldt = (K > NO ? K : NO) + 8;             // pitch of the per-wave tile buffer (elements)
    T* tl = wl + NOP * ldw + wave * 32 * ldt;
    // bias[o] + rowbias[image][o] for the (at most two) images of the wavefront's current tile: [2][NOP] floats
    float* bl = reinterpret_cast<float*>(wl + NOP * ldw + 4 * 32 * ldt) + wave * 2 * NOP;
    const bool hasb = bias != nullptr || rowbias != nullptr;
    const int bcol = 4 * l32;                           // this lane's 4 columns of that table (row `half`)
    const int nimg = rowbias ? (int)((N + P - 1) / P) : 1;
    // this lane's four bias values: an unconditional 8-byte load (of the weights when there is no bias), converted
    // where the table is written, so that nothing waits for it before the weights and the first tile are requested
    const ChanVec<T, 4> braw = *reinterpret_cast<const ChanVec<T, 4>*>(bias && bcol < NO ? bias + bcol : W);
    if (K != KP || NO != NOP) {  // uniform
        for (int i = tid; i < NOP * ldw / 8; i += 256) reinterpret_cast<uint4*>(wl)[i] = make_uint4(0u, 0u, 0u, 0u);
        __syncthreads();
    }
    const long long ntiles = (N + 31) / 32;
    const long long gw = (long long)bid * 4 + wave, nw = (long long)nblocks * 4;
    const int cpk = K / 8;                              // 16-byte chunks per input row
    const int nin = 32 * cpk;                           // chunks per input tile (<= 512)
    constexpr int LP = 8;                               // chunk loads per lane (K <= 128)
    Frag raw[LP];
    float4 brow = make_float4(0.f, 0.f, 0.f, 0.f);
    // MID: with G = K / 2 gated values per scale and ncc = G / 8 chunks of 8, a lane makes the chunks (pixel idx / ncc,
    // values 8 (idx % ncc) ..) of both halves of the rows for idx = lane, lane + 64 (idx < 32 ncc: K <= 64), and gates
    // the chunks (patch pixel idx / ncc < 24, same values) of the half-scale patch.  Lane constants, the same for every
    // tile: the item's pixel and chunk (clamped for the loads, which then read valid addresses) and whether it exists.
    const int MG = K >> 1;
    [[maybe_unused]] int mpix[2] = {0, 0}, mcc[2] = {0, 0};
    [[maybe_unused]] bool mok[2] = {false, false};
    if constexpr (MID != 0) {
        const int ncc = MG >> 3;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int idx = p * 64 + lane;
            if constexpr (STATIC && SK == 64) {
                mpix[p] = idx >> 2, mcc[p] = idx & 3, mok[p] = true;
            } else {
                const int pix = idx / ncc;
                mok[p] = pix < 32;
                mpix[p] = min(pix, 31), mcc[p] = idx - pix * ncc;
            }
        }
    }
    // POOL / MID with widths whose passes of 64 chunks are not whole pixels: where in global memory, relative to the
    // tile's first pixel, this lane's chunk i*64 + lane = (pixel, 8 values) of a tile of 4 x 8 pixels lies (lane
    // constants; input rows of K values, output rows of NO)
    [[maybe_unused]] int gin[LP], gout[2 * kNT];
    if constexpr (STATIC && (POOL || MID != 0)) {
#pragma unroll
        for (int i = 0; i < LP; ++i) {
            const int cidx = i * 64 + lane, pix = cidx / (SK / 8), cc = cidx - pix * (SK / 8);
            gin[i] = ((pix >> 3) * Wimg + (pix & 7)) * SK + 8 * cc;
        }
#pragma unroll
        for (int i = 0; i < 2 * kNT; ++i) {
            const int cidx = i * 64 + lane, pix = cidx / (SNO / 8), cc = cidx - pix * (SNO / 8);
            gout[i] = ((pix >> 3) * Wimg + (pix & 7)) * SNO + 8 * cc;
        }
    }
    [[maybe_unused]] Frag fa[2], fb[2], ha[2], hb[2];
    [[maybe_unused]] auto mid_load = [&](long long t) {
        const int b = tile_pixel(t);
        const int hh = Himg >> 1, hw = Wimg >> 1;
        const int ldf = MID == 1 ? K : mid->ldf, ldh = MID == 1 ? K : MG;
        const T* cf = static_cast<const T*>(mid->cf) + (long long)px_next * ldf;
        const T* chb = static_cast<const T*>(mid->ch) + (long long)b * hh * hw * ldh;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int pix = mpix[p], cc = mcc[p];
            const T* f = cf + (long long)((pix >> 3) * Wimg + (pix & 7)) * ldf + 8 * cc;
            fa[p] = *reinterpret_cast<const Frag*>(f);
            if constexpr (MID == 1) fb[p] = *reinterpret_cast<const Frag*>(f + MG);
            // (patch entries past the image are never used as taps: clamped, they are readable)
            const int q = min(pix, 23), qr = q / 6, qc = q - 6 * qr;
            const int hy = min(max(2 * rb_next - 1 + qr, 0), hh - 1), hx = min(max(4 * cb_next - 1 + qc, 0), hw - 1);
            const T* hp = chb + (long long)(hy * hw + hx) * ldh + 8 * cc;
            ha[p] = *reinterpret_cast<const Frag*>(hp);
            if constexpr (MID == 1) hb[p] = *reinterpret_cast<const Frag*>(hp + MG);
        }
    };
    auto load_tile = [&](long long t) {                 // coalesced: chunk i*64+lane of the tile's byte range
        const T* base = X + t * 32 * K;
        const long long rows_left = N - t * 32;         // rows of this tile that exist
        if constexpr (MID != 0) {
            mid_load(t);
        } else if constexpr (POOL) {
            tile_pixel(t);
            base = X + (long long)px_next * K;
            if constexpr (SK == 128) {
#pragma unroll
                for (int i = 0; i < LP; ++i)   // chunks i*64 .. of the tile: its pixels 4 i .. 4 i + 3 = image row i / 2, 4 columns
                    raw[i] = *reinterpret_cast<const Frag*>(base + (long long)((i >> 1) * Wimg + 4 * (i & 1)) * K + lane * 8);
            } else {
#pragma unroll
                for (int i = 0; i < LP; ++i) {   // chunk i*64 + lane = (pixel, 8 values) of the tile; whole passes (K % 16 == 0)
                    // (built from its four words: copied as a whole, an array that nothing reads word by word stays
                    // in scratch memory)
                    if (i * 64 < 32 * (SK / 8)) {
                        const uint4 u = *reinterpret_cast<const uint4*>(base + gin[i]);
                        raw[i] = Frag{{u.x, u.y, u.z, u.w}};
                    } else {
                        raw[i] = Frag{{0u, 0u, 0u, 0u}};
                    }
                }
            }
        } else if (STATIC && rows_left >= 32) {
#pragma unroll
            for (int i = 0; i < LP; ++i) {
                if (i * 64 < nin)
                    raw[i] = *reinterpret_cast<const Frag*>(base + (long long)(i * 64 + lane) * 8);
                else
                    raw[i] = Frag{{0u, 0u, 0u, 0u}};
            }
        } else {
            const int valid = rows_left >= 32 ? nin : (int)rows_left * cpk;
#pragma unroll
            for (int i = 0; i < LP; ++i) {
                const int cidx = i * 64 + lane;
                raw[i] = cidx < valid ? *reinterpret_cast<const Frag*>(base + (long long)cidx * 8)
                                      : Frag{{0u, 0u, 0u, 0u}};
            }
        }
        if (rowbias) {  // the tile's per-image rows ride behind its data: a tile of 32 rows meets two images at most
            const int img = min((int)(t * 32 / P) + half, nimg - 1);
            if (bcol < NO) brow = *reinterpret_cast<const float4*>(rowbias + (long long)img * NO + bcol);
        }
    };
    // The weights are requested first and written to LDS after the first tile's loads have been issued: loads
    // return in order, so the other way round the weights would wait for the whole tile.
    constexpr int ITW = kKT * kNT * 64 / 256;   // 16-byte copies (W[o][k]) or 4 x 4 sub-blocks (W[k][o]) per thread
    if constexpr (!KMAJOR) {
        const int kv = K / 8;
        Frag wv[ITW];
        int src[ITW], wdst[ITW];
        strided_offsets<ITW>(tid, 256, kv, K, 8, NO, src);
        strided_offsets<ITW>(tid, 256, kv, ldw, 8, NO, wdst);
#pragma unroll
        for (int it = 0; it < ITW; ++it) wv[it] = *reinterpret_cast<const Frag*>(W + (src[it] >= 0 ? src[it] : 0));
        if (gw < ntiles) load_tile(gw);
        // The stores are predicated, and a load whose only use is predicated is sunk into the branch: one load
        // latency per item.  Naming the registers here keeps the eight loads above, in flight together.
#pragma unroll
        for (int it = 0; it < ITW; ++it)
            asm volatile("" : "+v"(wv[it].v[0]), "+v"(wv[it].v[1]), "+v"(wv[it].v[2]), "+v"(wv[it].v[3]));
#pragma unroll
        for (int it = 0; it < ITW; ++it)
            if (wdst[it] >= 0) *reinterpret_cast<Frag*>(wl + wdst[it]) = wv[it];
    } else {
        // (K/4)(NO/4) sub-blocks over 256 threads: 2 per thread for 64 x 128, 4 at most (uniform switch, so that
        // a small matrix does not pay for the largest one's address arithmetic and predicated passes)
        const int nsub = (K / 4) * (NO / 4);
        if (nsub <= 512) {
            WTransposer<T, 2> wt;
            wt.load(W, K, NO, ldw, tid);
            if (gw < ntiles) load_tile(gw);
            wt.store(wl, ldw);
        } else {
            WTransposer<T, 4> wt;
            wt.load(W, K, NO, ldw, tid);
            if (gw < ntiles) load_tile(gw);
            wt.store(wl, ldw);
        }
    }
    const int cpr = NO / 8;  // 16-byte chunks per output row (NO % 8 == 0 on this path)
    constexpr int LO = 2 * kNT;  // 16-byte chunks per lane of a 32 x NO tile (NO <= 32 * kNT)
    int oin[LP], oout[LO];   // LDS offsets of this lane's input / output chunks (the same for every tile)
    strided_offsets<LP>(lane, 64, cpk, ldt, 8, 32, oin);
    strided_offsets<LO>(lane, 64, cpr, ldt, 8, 32, oout);
    __syncthreads();
    for (long long tile = gw; tile < ntiles; tile += nw) {
        [[maybe_unused]] const bool first = tile == gw;
        px_cur = px_next, pp_cur = pp_next;   // (POOL, MID) set when this tile was requested
        if constexpr (MID != 0) {
            rb_cur = rb_next, cb_cur = cb_next;
            const int hh = Himg >> 1, hw = Wimg >> 1;
            T* cat = MID == 1 ? static_cast<T*>(mid->cat) : nullptr;
            // the gated patch of the half scale: [24 pixels][G] in columns K.. of the tile buffer's rows
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int q = mpix[p], cc = mcc[p];
                Frag hg;
                if constexpr (MID == 1) hg = gate8<T>(ha[p], hb[p], mid->gs);
                else hg = Frag{{ha[p].v[0], ha[p].v[1], ha[p].v[2], ha[p].v[3]}};
                if (mok[p] && q < 24) *reinterpret_cast<Frag*>(tl + q * ldt + K + 8 * cc) = hg;
            }
            // the full scale's half of the rows
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int pix = mpix[p], cc = mcc[p];
                Frag full;
                if constexpr (MID == 1) full = gate8<T>(fa[p], fb[p], mid->gs);
                else full = Frag{{fa[p].v[0], fa[p].v[1], fa[p].v[2], fa[p].v[3]}};
                if (mok[p]) {
                    *reinterpret_cast<Frag*>(tl + pix * ldt + 8 * cc) = full;
                    if (cat)
                        *reinterpret_cast<Frag*>(cat + ((long long)px_cur + (pix >> 3) * Wimg + (pix & 7)) * K + 8 * cc) = full;
                }
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the patch is in LDS (written by other lanes of this wavefront)
            // the resized half: four taps of the patch per pixel, bl_src's rows, columns and weights
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int pix = mpix[p], cc = mcc[p];
                int y0, y1, x0, x1;
                float ly, lx;
                bl_src(4 * rb_cur + (pix >> 3), 0.5f, hh, y0, y1, ly);
                bl_src(8 * cb_cur + (pix & 7), 0.5f, hw, x0, x1, lx);
                const int oy = 2 * rb_cur - 1, ox = 4 * cb_cur - 1;   // source row / column of patch entry (0, 0)
                const T* pt = tl + K + 8 * cc;
                const Frag g00 = *reinterpret_cast<const Frag*>(pt + ((y0 - oy) * 6 + (x0 - ox)) * ldt);
                const Frag g01 = *reinterpret_cast<const Frag*>(pt + ((y0 - oy) * 6 + (x1 - ox)) * ldt);
                const Frag g10 = *reinterpret_cast<const Frag*>(pt + ((y1 - oy) * 6 + (x0 - ox)) * ldt);
                const Frag g11 = *reinterpret_cast<const Frag*>(pt + ((y1 - oy) * 6 + (x1 - ox)) * ldt);
                const Frag up = bilinear8<T>(g00, g01, g10, g11, ly, lx);
                if (mok[p]) {
                    *reinterpret_cast<Frag*>(tl + pix * ldt + MG + 8 * cc) = up;
                    if (cat)
                        *reinterpret_cast<Frag*>(cat + ((long long)px_cur + (pix >> 3) * Wimg + (pix & 7)) * K + MG + 8 * cc) = up;
                }
            }
        } else {
        // raw chunks -> LDS [row][k] -> MFMA fragments (row l32, k = kt*16 + 8*half ..)
#pragma unroll
        for (int i = 0; i < LP; ++i)
            if (STATIC ? i * 64 < nin : oin[i] >= 0) *reinterpret_cast<Frag*>(tl + oin[i]) = raw[i];
        }
        if (hasb && bcol < NOP) {
            const bool hb = bias != nullptr && bcol < NO;
            *reinterpret_cast<float4*>(bl + half * NOP + bcol) =
                make_float4((hb ? to_f32(braw.v[0]) : 0.f) + brow.x, (hb ? to_f32(braw.v[1]) : 0.f) + brow.y,
                            (hb ? to_f32(braw.v[2]) : 0.f) + brow.z, (hb ? to_f32(braw.v[3]) : 0.f) + brow.w);
        }
        float cs[8];
        const bool cs_lanes = K == 128 || K == 64;   // a lane keeps its 8 columns over all chunks (64 % (K/8) == 0)
        if (COLSUM && cs_lanes) {
#pragma unroll
            for (int j = 0; j < 8; ++j) cs[j] = 0.f;
#pragma unroll
            for (int i = 0; i < LP; ++i)   // chunks past the tile or the tensor are zero
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    cs[2 * j] += half_to_f32<T>(raw[i].v[j] & 0xffffu);
                    cs[2 * j + 1] += half_to_f32<T>(raw[i].v[j] >> 16);
                }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS writes have landed
        Frag xf[kKT];
#pragma unroll
        for (int kt = 0; kt < kKT; ++kt) {
            if (kt < nkt && (STATIC || kt * 16 + 8 * half < K))
                xf[kt] = *reinterpret_cast<const Frag*>(tl + l32 * ldt + kt * 16 + 8 * half);
            else
                xf[kt] = Frag{{0u, 0u, 0u, 0u}};
        }
        if (COLSUM && !cs_lanes) {
            // other widths: lane sums one dword column (two features) of the tile in LDS over its 32 rows (rows past
            // the tensor were written as zeros)
            float s0 = 0.f, s1 = 0.f;
            if (2 * lane < K) {
#pragma unroll 8
                for (int r = 0; r < 32; ++r) {
                    const uint32_t v = *reinterpret_cast<const uint32_t*>(tl + r * ldt + 2 * lane);
                    s0 += half_to_f32<T>(v & 0xffffu), s1 += half_to_f32<T>(v >> 16);
                }
                *reinterpret_cast<float2*>(colsum + tile * K + 2 * lane) = make_float2(s0, s1);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // fragments are in registers: the buffer may be overwritten
        if constexpr (MID != 0) {
            // unconditionally (the last tile asks for itself again, from the caches): behind a branch the loaded
            // registers are copied into the loop's own at the end of the branch, which waits for the data there
            load_tile(tile + nw < ntiles ? tile + nw : tile);
        } else {
            if (tile + nw < ntiles) load_tile(tile + nw);  // next tile in flight during the MFMAs and the store
        }
        if (COLSUM && cs_lanes) {
            float* tf = reinterpret_cast<float*>(tl);  // [512 / K lane groups][K]
            *reinterpret_cast<float4*>(tf + lane * 8) = make_float4(cs[0], cs[1], cs[2], cs[3]);
            *reinterpret_cast<float4*>(tf + lane * 8 + 4) = make_float4(cs[4], cs[5], cs[6], cs[7]);
            __builtin_amdgcn_s_waitcnt(0xc07f);
            float* dst = colsum + tile * K;
            if (K == 128) {
                float2 t = *reinterpret_cast<const float2*>(tf + 2 * lane);
#pragma unroll
                for (int gidx = 1; gidx < 4; ++gidx) {
                    const float2 u = *reinterpret_cast<const float2*>(tf + gidx * 128 + 2 * lane);
                    t.x += u.x, t.y += u.y;
                }
                *reinterpret_cast<float2*>(dst + 2 * lane) = t;
            } else {  // K == 64
                float t = tf[lane];
#pragma unroll
                for (int gidx = 1; gidx < 8; ++gidx) t += tf[gidx * 64 + lane];
                dst[lane] = t;
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // read before the result tile is written to the same buffer
        }
        // this lane's row of the bias table: the image of tile row l32 relative to the tile's first image
        const float* blr = bl + 4 * half;
        if (rowbias) {
            const long long m = tile * 32 + l32;
            const int img = min((int)((m < N ? m : N - 1) / P), nimg - 1);
            blr += (img - (int)(tile * 32 / P)) * NOP;
        }
        // One 32-feature tile: its weight fragments and bias values (all LDS reads issued before the first MFMA), the
        // product, and the way out (bias added, rounded, into the tile buffer).
        auto load_w = [&](int nt, Frag (&wf)[kKT], float4 (&r4)[4]) {
            const T* wr = wl + (nt * 32 + l32) * ldw + 8 * half;
            if constexpr (STATIC) {
#pragma unroll
                for (int kt = 0; kt < SK / 16; ++kt) wf[kt] = *reinterpret_cast<const Frag*>(wr + kt * 16);
            } else {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) wf[kt] = *reinterpret_cast<const Frag*>(wr + kt * 16);
                if (nkt > 4) {
#pragma unroll
                    for (int kt = 4; kt < 8; ++kt) wf[kt] = *reinterpret_cast<const Frag*>(wr + kt * 16);
                }
            }
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                r4[g4] = hasb ? *reinterpret_cast<const float4*>(blr + nt * 32 + g4 * 8) : make_float4(0.f, 0.f, 0.f, 0.f);
        };
        auto product = [&](const Frag (&wf)[kKT]) {
            f32x16 acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.f;
            if constexpr (STATIC) {
#pragma unroll
                for (int kt = 0; kt < SK / 16; ++kt) acc = mfma32(wf[kt], xf[kt], acc, T());
            } else {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) acc = mfma32(wf[kt], xf[kt], acc, T());
                if (nkt > 4) {
#pragma unroll
                    for (int kt = 4; kt < 8; ++kt) acc = mfma32(wf[kt], xf[kt], acc, T());
                }
            }
            return acc;
        };
        auto way_out = [&](int nt, const f32x16& acc, const float4 (&r4)[4]) {
            // lane owns row l32 of the tile and features n0..n0+3 of each accumulator group
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int n0 = nt * 32 + g4 * 8 + half * 4;
                // (static widths are multiples of 16: both halves of a group of 8 features exist or neither does)
                if (STATIC ? nt * 32 + g4 * 8 < NO : n0 < NO) {
                    float o[4];
                    o[0] = acc[g4 * 4] + r4[g4].x, o[1] = acc[g4 * 4 + 1] + r4[g4].y;
                    o[2] = acc[g4 * 4 + 2] + r4[g4].z, o[3] = acc[g4 * 4 + 3] + r4[g4].w;
                    store_f32<T, 4>(tl + l32 * ldt + n0, o);
                }
            }
        };
        if constexpr (STATIC) {
            // Software pipeline over the feature tiles (unrolled): tile nt + 1's LDS reads are issued before tile nt's
            // MFMAs, and tile nt's way out follows the issue of tile nt + 1's MFMAs, so neither the read latency nor
            // the MFMA latency of a tile sits between two tiles.
            constexpr int NNT = (SNO + 31) / 32;
            Frag wf[2][kKT];
            float4 r4[3][4];   // (three tiles' bias values are alive at once: nt - 1 on its way out, nt, nt + 1 read ahead)
            f32x16 acc[2];
            load_w(0, wf[0], r4[0]);
#pragma unroll
            for (int nt = 0; nt < NNT; ++nt) {
                if (nt + 1 < NNT) load_w(nt + 1, wf[(nt + 1) % 2], r4[(nt + 1) % 3]);
                acc[nt % 2] = product(wf[nt % 2]);
                if (nt > 0) way_out(nt - 1, acc[(nt - 1) % 2], r4[(nt - 1) % 3]);
            }
            way_out(NNT - 1, acc[(NNT - 1) % 2], r4[(NNT - 1) % 3]);
        } else {
            for (int nt = 0; nt < nnt; ++nt) {
                Frag wf[kKT];
                float4 r4[4];
                load_w(nt, wf, r4);
                const f32x16 acc = product(wf);
                way_out(nt, acc, r4);
            }
        }
        // coalesced copy-out of the 32 x NO tile (same wavefront wrote it: no workgroup barrier needed)
        __builtin_amdgcn_s_waitcnt(0xc07f);
        {
            const long long rows_left = N - tile * 32;
            T* yb = Y + tile * 32 * NO;
            if constexpr (POOL) {
                yb = Y + (long long)px_cur * NO;
                Frag of[LO];
#pragma unroll
                for (int i = 0; i < LO; ++i)
                    if (i * 64 < 32 * cpr) of[i] = *reinterpret_cast<const Frag*>(tl + oout[i]);
                // the lane's window of the pool (2 x 4 per tile) and 8 of its features
                constexpr int CPR = SNO / 8;
                int wr = lane >> 5, wc = (lane >> 3) & 3, ch = (lane & 7) * 8;
                if constexpr (CPR != 8) {
                    const int win = min(lane / CPR, 7);
                    wr = win >> 2, wc = win & 3, ch = (lane - (lane / CPR) * CPR) * 8;
                }
                const bool wok = CPR == 8 || lane < 8 * CPR;
                const T* p00 = tl + (16 * wr + 2 * wc) * ldt + ch;
                const Frag q00 = *reinterpret_cast<const Frag*>(p00), q01 = *reinterpret_cast<const Frag*>(p00 + ldt);
                const Frag q10 = *reinterpret_cast<const Frag*>(p00 + 8 * ldt), q11 = *reinterpret_cast<const Frag*>(p00 + 9 * ldt);
                if constexpr (SNO == 64) {
#pragma unroll
                    for (int i = 0; i < LO; ++i)   // chunks i*64 .. = image row i of the tile, 8 pixels
                        if (i * 64 < 32 * cpr) *reinterpret_cast<Frag*>(yb + (long long)i * Wimg * NO + lane * 8) = of[i];
                } else {
#pragma unroll
                    for (int i = 0; i < LO; ++i)   // whole passes (NO % 16 == 0)
                        if (i * 64 < 32 * CPR) *reinterpret_cast<Frag*>(yb + gout[i]) = of[i];
                }
                Frag o;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float lo = (((half_to_f32<T>(q00.v[j] & 0xffffu) + half_to_f32<T>(q01.v[j] & 0xffffu)) +
                                       half_to_f32<T>(q10.v[j] & 0xffffu)) + half_to_f32<T>(q11.v[j] & 0xffffu)) * 0.25f;
                    const float hi = (((half_to_f32<T>(q00.v[j] >> 16) + half_to_f32<T>(q01.v[j] >> 16)) +
                                       half_to_f32<T>(q10.v[j] >> 16)) + half_to_f32<T>(q11.v[j] >> 16)) * 0.25f;
                    ChanVec<T, 2> pv;
                    pv.v[0] = from_f32<T>(lo), pv.v[1] = from_f32<T>(hi);
                    o.v[j] = *reinterpret_cast<const uint32_t*>(&pv);
                }
                T* pb = pool + ((long long)pp_cur + wr * (Wimg >> 1) + wc) * NO + ch;
                if (wok) *reinterpret_cast<Frag*>(pb) = o;
            } else if constexpr (MID != 0) {
                yb = Y + (long long)px_cur * NO;
                Frag of[LO];
#pragma unroll
                for (int i = 0; i < LO; ++i) of[i] = *reinterpret_cast<const Frag*>(tl + (oout[i] >= 0 ? oout[i] : 0));
                if constexpr (STATIC && SNO == 128) {
#pragma unroll
                    for (int i = 0; i < LO; ++i)   // chunks i*64 .. = pixels 4 i .. 4 i + 3 of the tile: image row i / 2, 4 columns
                        *reinterpret_cast<Frag*>(yb + (long long)((i >> 1) * Wimg + 4 * (i & 1)) * NO + lane * 8) = of[i];
                } else if constexpr (STATIC) {
#pragma unroll
                    for (int i = 0; i < LO; ++i)   // whole passes (NO % 16 == 0)
                        if (i * 64 < 32 * (SNO / 8)) *reinterpret_cast<Frag*>(yb + gout[i]) = of[i];
                } else {
#pragma unroll
                    for (int i = 0; i < LO; ++i)
                        asm volatile("" : "+v"(of[i].v[0]), "+v"(of[i].v[1]), "+v"(of[i].v[2]), "+v"(of[i].v[3]));
#pragma unroll
                    for (int i = 0; i < LO; ++i) {   // chunk i*64 + lane = (pixel, 8 features) of the tile
                        const int cidx = i * 64 + lane, pix = cidx / cpr, cc = cidx - pix * cpr;
                        if (pix < 32)
                            *reinterpret_cast<Frag*>(yb + (long long)((pix >> 3) * Wimg + (pix & 7)) * NO + 8 * cc) = of[i];
                    }
                }
            } else if (STATIC && rows_left >= 32) {  // (an array of its own: one array written on both paths ends up in scratch)
                Frag of[LO];
#pragma unroll
                for (int i = 0; i < LO; ++i)
                    if (i * 64 < 32 * cpr) of[i] = *reinterpret_cast<const Frag*>(tl + oout[i]);
#pragma unroll
                for (int i = 0; i < LO; ++i)
                    if (i * 64 < 32 * cpr) *reinterpret_cast<Frag*>(yb + (long long)(i * 64 + lane) * 8) = of[i];
            } else {
                const int valid = (rows_left >= 32 ? 32 : (int)rows_left) * cpr;
                Frag ov[LO];
#pragma unroll
                for (int i = 0; i < LO; ++i) ov[i] = *reinterpret_cast<const Frag*>(tl + (oout[i] >= 0 ? oout[i] : 0));
                // (naming the registers keeps the reads together: a read whose only use is a conditional store is
                // otherwise moved to that store, one LDS latency per chunk)
#pragma unroll
                for (int i = 0; i < LO; ++i)
                    asm volatile("" : "+v"(ov[i].v[0]), "+v"(ov[i].v[1]), "+v"(ov[i].v[2]), "+v"(ov[i].v[3]));
#pragma unroll
                for (int i = 0; i < LO; ++i) {
                    const int cidx = i * 64 + lane;
                    if (cidx < valid) *reinterpret_cast<Frag*>(yb + (long long)cidx * 8) = ov[i];
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // copy-out reads done before the next tile overwrites the buffer
    }
}

template <typename T, bool KMAJOR, bool COLSUM, int SK, int SNO>
__global__ __launch_bounds__(256, 2) void dense_rows_k(const T* __restrict__ X, const T* __restrict__ W,
                                                    const T* __restrict__ bias, const float* __restrict__ rowbias,
                                                    T* __restrict__ Y, float* __restrict__ colsum, long long N, int K,
                                                    int NO, int P, int nkt, int nnt) {
    extern __shared__ uint32_t dsm[];
    dense_rows_body<T, KMAJOR, COLSUM, SK, SNO>(X, W, bias, rowbias, Y, colsum, N, K, NO, P, nkt, nnt, blockIdx.x,
                                                gridDim.x, dsm);
}

// The 128 -> 64 layer over the pixels of [B, Himg, Wimg] images with the tile sums of X and the 2x2 average pool of Y
// (dense_rows_body, POOL).
template <typename T, int SK, int SNO>
__global__ __launch_bounds__(256, 2) void dense_rows_pool_k(const T* __restrict__ X, const T* __restrict__ W,
                                                         const T* __restrict__ bias, T* __restrict__ Y,
                                                         float* __restrict__ colsum, T* __restrict__ pool, long long N,
                                                         int Himg, int Wimg) {
    extern __shared__ uint32_t dsm[];
    dense_rows_body<T, false, true, SK, SNO, true>(X, W, bias, nullptr, Y, colsum, N, SK, SNO, 1, SK / 16,
                                                   (SNO + 31) / 32, blockIdx.x, gridDim.x, dsm, pool, Himg, Wimg);
}

// The 64 -> 128 layer on rows made from the two scales of a pyramid block (dense_rows_body, MID).
template <typename T, int MID, int SK, int SNO>
__global__ __launch_bounds__(256, 2) void dense_mid_rows_k(const T* __restrict__ W, const T* __restrict__ bias,
                                                        const float* __restrict__ rowbias, T* __restrict__ Y,
                                                        long long N, int Himg, int Wimg, int K, int NO,
                                                        const MidRows mid) {
    extern __shared__ uint32_t dsm[];
    // (workgroup ids go to the 8 XCDs round-robin: each XCD gets a contiguous range of tiles, so that the half-scale
    // patches of neighbouring tiles, which overlap, meet in one L2)
    dense_rows_body<T, false, false, SK, SNO, false, MID>(nullptr, W, bias, rowbias, Y, nullptr, N, K, NO, Himg * Wimg,
                                                           (K + 15) / 16, (NO + 31) / 32, xcd_remap(blockIdx.x, gridDim.x),
                                                           gridDim.x, dsm, nullptr, Himg, Wimg, &mid);
}

// The same with the deferred partial-sum reductions of a backward pass in the first gridDim.x - nblocks
// workgroups: they are a few microseconds of latency that need no launch of their own when a dense layer runs
// after the last of the kernels that produce the partials.
template <typename T, bool KMAJOR, int SK, int SNO>
__global__ __launch_bounds__(256, 2) void dense_rows_rider_k(const T* __restrict__ X, const T* __restrict__ W,
                                                          const T* __restrict__ bias,
                                                          const float* __restrict__ rowbias, T* __restrict__ Y,
                                                          long long N, int K, int NO, int P, int nkt, int nnt,
                                                          int nblocks, const ReduceJobs jobs) {
    extern __shared__ uint32_t dsm[];
    const int nride = (int)gridDim.x - nblocks;
    if ((int)blockIdx.x < nride) {
        reduce_jobs_block(jobs, blockIdx.x, reinterpret_cast<float*>(dsm));
    } else {
        dense_rows_body<T, KMAJOR, false, SK, SNO>(X, W, bias, rowbias, Y, nullptr, N, K, NO, P, nkt, nnt,
                                                   blockIdx.x - nride, nblocks, dsm);
    }
}

// dW partials.  A workgroup of 4 wavefronts walks 64-row stages b, b + gridDim.x, ...: the stage's rows
// of A and B are copied to LDS with coalesced 16-byte loads (requested one stage ahead and held in
// registers while the current stage is multiplied), then wavefront w multiplies rows 16w..16w+15, reading
// the k-major MFMA fragments (8 consecutive rows of one feature) from LDS with 16-bit reads.
constexpr int kWgRows = 64;

// EXACT: M = 32 MT and NO = 32 NT, as compile-time facts: the staging map is shifts and masks, every pass is a
// whole one and no fragment needs a clamp or a zero (the generic form spends a quarter of its time on those).
// SM, SN > 0 (without EXACT): other extents as compile-time facts (multiples of 8): the staging map divides by
// constants, a whole stage is read as one contiguous range, and only the last, partial tiles clamp their fragments.
template <typename T, int MT, int NT, bool EXACT, int SM = 0, int SN = 0>
__device__ __forceinline__ void dense_wgrad_body(const T* __restrict__ A, const T* __restrict__ Bm,
                                                 float* __restrict__ part, long long N, int Md, int NOd, int nblocks,
                                                 uint32_t* dsm) {
    constexpr bool SDIM = !EXACT && SM > 0 && SN > 0;
    static_assert(!SDIM || (SM % 8 == 0 && SN % 8 == 0 && SM <= 32 * MT && SN <= 32 * NT && SM > 32 * (MT - 1) &&
                            SN > 32 * (NT - 1)), "static extents of the weight gradient");
    const int M = EXACT ? 32 * MT : SDIM ? SM : Md, NO = EXACT ? 32 * NT : SDIM ? SN : NOd;
    const int lda = M + 8, ldb = NO + 8;  // LDS row pitches (elements)
    const int buf_elems = kWgRows * (lda + ldb);
    T* lds = reinterpret_cast<T*>(dsm);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    f32x16 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

    // staging map: 16-byte vectors; A has M/8 vectors per row, B has NO/8
    const int va = M / 8, vb = NO / 8;
    const int nva = kWgRows * va, nvb = kWgRows * vb;
    constexpr int PA = (kWgRows * 16 * MT / 8 * 2 + 255) / 256;  // passes over A vectors (upper bound)
    constexpr int PB = (kWgRows * 16 * NT / 8 * 2 + 255) / 256;
    Frag pa[PA], pb[PB];
    const long long nstages = (N + kWgRows - 1) / kWgRows;
    // workgroup b takes stages b, b + gridDim.x, ...: at any moment the chip reads one contiguous window
    const long long st0 = blockIdx.x, sstep = nblocks;
    const long long st1 = nstages;

    auto fetch = [&](long long st) {
        const long long r0 = st * kWgRows;
        if (EXACT && r0 + kWgRows <= N) {  // a whole stage of an exact shape: contiguous, nothing to test
            const T* ab = A + r0 * M + tid * 8;
            const T* bb = Bm + r0 * NO + tid * 8;
#pragma unroll
            for (int p = 0; p < PA; ++p) pa[p] = *reinterpret_cast<const Frag*>(ab + p * 2048);
#pragma unroll
            for (int p = 0; p < PB; ++p) pb[p] = *reinterpret_cast<const Frag*>(bb + p * 2048);
            return;
        }
        if (SDIM && r0 + kWgRows <= N) {   // a whole stage: contiguous; the last pass may be a partial one
            const T* ab = A + r0 * M + tid * 8;
            const T* bb = Bm + r0 * NO + tid * 8;
#pragma unroll
            for (int p = 0; p < PA; ++p)
                pa[p] = tid + p * 256 < nva ? *reinterpret_cast<const Frag*>(ab + p * 2048) : Frag{{0u, 0u, 0u, 0u}};
#pragma unroll
            for (int p = 0; p < PB; ++p)
                pb[p] = tid + p * 256 < nvb ? *reinterpret_cast<const Frag*>(bb + p * 2048) : Frag{{0u, 0u, 0u, 0u}};
            return;
        }
#pragma unroll
        for (int p = 0; p < PA; ++p) {
            const int idx = tid + p * 256;
            const long long r = r0 + idx / va;
            pa[p] = (idx < nva && r < N) ? *reinterpret_cast<const Frag*>(A + r * M + (idx % va) * 8)
                                         : Frag{{0u, 0u, 0u, 0u}};
        }
#pragma unroll
        for (int p = 0; p < PB; ++p) {
            const int idx = tid + p * 256;
            const long long r = r0 + idx / vb;
            pb[p] = (idx < nvb && r < N) ? *reinterpret_cast<const Frag*>(Bm + r * NO + (idx % vb) * 8)
                                         : Frag{{0u, 0u, 0u, 0u}};
        }
    };
    auto commit = [&](int buf) {
        T* la = lds + buf * buf_elems;
        T* lb = la + kWgRows * lda;
#pragma unroll
        for (int p = 0; p < PA; ++p) {
            const int idx = tid + p * 256;
            if (EXACT || idx < nva) *reinterpret_cast<Frag*>(la + (idx / va) * lda + (idx % va) * 8) = pa[p];
        }
#pragma unroll
        for (int p = 0; p < PB; ++p) {
            const int idx = tid + p * 256;
            if (EXACT || idx < nvb) *reinterpret_cast<Frag*>(lb + (idx / vb) * ldb + (idx % vb) * 8) = pb[p];
        }
    };

    if (st0 < st1) {
        fetch(st0);
        commit(0);
    }
    __syncthreads();
    int buf = 0;
    for (long long st = st0; st < st1; st += sstep, buf ^= 1) {
        if (st + sstep < st1) fetch(st + sstep);  // in flight while this stage is multiplied
        const T* la = lds + buf * buf_elems + (wave * 16 + 8 * half) * lda;
        const T* lb = lds + buf * buf_elems + kWgRows * lda + (wave * 16 + 8 * half) * ldb;
        Frag af[MT], bf[NT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const bool whole = EXACT || (SDIM && (t + 1) * 32 <= SM);   // (t is a constant once unrolled)
            const int m = whole ? t * 32 + l32 : min(t * 32 + l32, M - 1);
            const bool ok = whole || t * 32 + l32 < M;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = ld16(la + (2 * j) * lda + m), hi = ld16(la + (2 * j + 1) * lda + m);
                af[t].v[j] = ok ? (lo | (hi << 16)) : 0u;
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const bool whole = EXACT || (SDIM && (t + 1) * 32 <= SN);
            const int n = whole ? t * 32 + l32 : min(t * 32 + l32, NO - 1);
            const bool ok = whole || t * 32 + l32 < NO;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = ld16(lb + (2 * j) * ldb + n), hi = ld16(lb + (2 * j + 1) * ldb + n);
                bf[t].v[j] = ok ? (lo | (hi << 16)) : 0u;
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = mfma32(af[mt], bf[nt], acc[mt][nt], T());
        if (st + sstep < st1) commit(buf ^ 1);
        __syncthreads();
    }
    // sum the 4 waves through LDS, tile by tile; D lane map: column n = l32, row m = 8*(i/4) + 4*half + i%4
    float* red = reinterpret_cast<float*>(dsm);  // [4][16][64]
    float* pout = part + (long long)blockIdx.x * M * NO;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 16; ++i) red[(wave * 16 + i) * 64 + lane] = acc[mt][nt][i];
            __syncthreads();
            {   // thread -> 4 consecutive lanes' values = 4 consecutive n of one dW row
                const int idx = threadIdx.x * 4;
                const int i = idx >> 6, l = idx & 63;
                const float4 a = *reinterpret_cast<const float4*>(red + idx), b = *reinterpret_cast<const float4*>(red + 1024 + idx);
                const float4 c = *reinterpret_cast<const float4*>(red + 2048 + idx), d = *reinterpret_cast<const float4*>(red + 3072 + idx);
                const int m = mt * 32 + 8 * (i / 4) + 4 * (l >> 5) + (i % 4), n = nt * 32 + (l & 31);
                if (EXACT || (m < M && n < NO))  // NO % 8 == 0: the four values are in range together
                    *reinterpret_cast<float4*>(pout + (long long)m * NO + n) =
                        make_float4((a.x + b.x) + (c.x + d.x), (a.y + b.y) + (c.y + d.y), (a.z + b.z) + (c.z + d.z),
                                    (a.w + b.w) + (c.w + d.w));
            }
        }
}

template <typename T, int MT, int NT, bool EXACT>
__global__ __launch_bounds__(256, 2) void dense_wgrad_k(const T* __restrict__ A, const T* __restrict__ Bm,
                                                        float* __restrict__ part, long long N, int M, int NO) {
    extern __shared__ uint32_t dsm[];
    dense_wgrad_body<T, MT, NT, EXACT>(A, Bm, part, N, M, NO, gridDim.x, dsm);
}

// The same with earlier summations in the workgroups behind the first `nblocks` (one workgroup of the product per
// compute unit leaves room for a second one beside it from the start).
template <typename T, int MT, int NT, bool EXACT>
__global__ __launch_bounds__(256, 2) void dense_wgrad_rider_k(const T* __restrict__ A, const T* __restrict__ Bm,
                                                              float* __restrict__ part, long long N, int M, int NO,
                                                              int nblocks, const ReduceJobs jobs) {
    extern __shared__ uint32_t dsm[];
    if ((int)blockIdx.x >= nblocks) {
        reduce_jobs_block(jobs, blockIdx.x - nblocks, reinterpret_cast<float*>(dsm));
        return;
    }
    dense_wgrad_body<T, MT, NT, EXACT>(A, Bm, part, N, M, NO, nblocks, dsm);
}

// Input gradient and weight gradient of one dense layer (y = x W^T, W[O][I]) in one launch, for the layer shapes of
// pyramid blocks of 128, 96 and 64 features, (O, I) = (128, 64), (64, 128), (96, 48), (48, 96), (64, 32), (32, 64): dx[N][I] = gy W (dense_rows_body, W as W[k][o]) and the
// partials of dW[O][I] = gy^T x (dense_wgrad_body).  Both read gy and neither fills the chip alone (the weight gradient is one
// workgroup per compute unit, the row product waits on memory in lockstep): the weight gradient's workgroups come
// first in the grid, one per compute unit, and the row product's persistent workgroups take the second slot.
template <typename T, bool COLSUM, int O, int I>
__global__ __launch_bounds__(256, 2) void dense_bwd_pair_k(const T* __restrict__ gy, const T* __restrict__ W,
                                                           const T* __restrict__ xin, T* __restrict__ dx,
                                                           float* __restrict__ colsum, float* __restrict__ part,
                                                           const float* __restrict__ rowbias, int P, long long N,
                                                           int nwg, int nrows) {
    extern __shared__ uint32_t dsm[];
    constexpr bool EX = O % 32 == 0 && I % 32 == 0;   // else: the extents as constants, partial last tiles
    if ((int)blockIdx.x < nwg)
        dense_wgrad_body<T, (O + 31) / 32, (I + 31) / 32, EX, EX ? 0 : O, EX ? 0 : I>(gy, xin, part, N, O, I, nwg, dsm);
    else
        dense_rows_body<T, true, COLSUM, O, I>(gy, W, nullptr, rowbias, dx, colsum, N, O, I, P, O / 16, (I + 31) / 32,
                                               blockIdx.x - nwg, nrows, dsm);
}

// The same for any widths the two bodies cover (multiples of 8 up to 128 with at most 8 accumulator tiles): extents
// from the arguments, MT = ceil(O / 32), NT = ceil(I / 32).
template <typename T, int MT, int NT, bool COLSUM>
__global__ __launch_bounds__(256, 2) void dense_bwd_pair_gen_k(const T* __restrict__ gy, const T* __restrict__ W,
                                                               const T* __restrict__ xin, T* __restrict__ dx,
                                                               float* __restrict__ colsum, float* __restrict__ part,
                                                               const float* __restrict__ rowbias, int P, long long N,
                                                               int O, int I, int nwg, int nrows) {
    extern __shared__ uint32_t dsm[];
    if ((int)blockIdx.x < nwg)
        dense_wgrad_body<T, MT, NT, false>(gy, xin, part, N, O, I, nwg, dsm);
    else
        dense_rows_body<T, true, COLSUM>(gy, W, nullptr, rowbias, dx, colsum, N, O, I, P, (O + 15) / 16, (I + 31) / 32,
                                         blockIdx.x - nwg, nrows, dsm);
}

static bool dense_dims_ok(int K, int NO, int dtype) {
    return dtype != kF32 && K >= 8 && K <= 16 * kKT && K % 8 == 0 && NO >= 8 && NO <= 32 * kNT && NO % 8 == 0;
}

// (the tiled kernels of this file, or the one-tile-per-wavefront kernels of dense_any.hip: fp32, other widths)
int dense_rows_supported(int K, int NO, int dtype) { return (dense_dims_ok(K, NO, dtype) || dense_any_dims_ok(K, NO)) ? 1 : 0; }

int dense_colsum_rows() { return 32; }

int dense_colsum_supported(int K, int NO, int dtype) { return dense_dims_ok(K, NO, dtype) ? 1 : 0; }

int dense_rows_launch(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                      long long N, int K, int NO, int P, int dtype, hipStream_t s, float* colsum,
                      const ReduceJobs* rider) {
    if (!dense_dims_ok(K, NO, dtype)) {
        // fp32 and the widths the tiled kernels do not take: no tile sums there, and summations that were to ride
        // in this launch get one of their own
        if (colsum || !dense_any_dims_ok(K, NO)) return -1;
        if (rider)
            if (int e = reduce_jobs_launch(*rider, s)) return e;
        return dense_any_rows_launch(x, w, w_kmajor, bias, rowbias, y, N, K, NO, P, dtype, s);
    }
    if (rider && colsum) return -1;
    if (colsum && (!dense_colsum_supported(K, NO, dtype) || (reinterpret_cast<uintptr_t>(colsum) & 15))) return -1;
    if (N == 0) return 0;
    if (N > 0x7fffffffLL) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 15) ||
        (reinterpret_cast<uintptr_t>(rowbias) & 15) || (reinterpret_cast<uintptr_t>(bias) & 7) ||
        (reinterpret_cast<uintptr_t>(w) & 15))
        return -1;
    if (rowbias && P < 32) {
        // The kernel's bias table holds two images per 32-row tile; smaller images get their rows in a second pass.
        if (int e = dense_rows_launch(x, w, w_kmajor, bias, nullptr, y, N, K, NO, P, dtype, s, colsum, rider)) return e;
        const long long full = N / P, rest = N - full * P;
        if (full > 0)
            if (int e = add_rowbias_launch(y, rowbias, (int)full, P, NO, dtype, s)) return e;
        if (rest > 0)
            return add_rowbias_launch(static_cast<char*>(y) + (size_t)full * P * NO * 2, rowbias + full * NO, 1, (int)rest,
                                      NO, dtype, s);
        return 0;
    }
    const int nkt = cdiv(K, 16), nnt = cdiv(NO, 32);
    const long long ntiles = (N + 31) / 32;
    long long blocks = (ntiles + 3) / 4;  // one row tile per wavefront until the cap
    const int cap = tune_env("PDW_DENSE_BLOCKS") ? atoi(tune_env("PDW_DENSE_BLOCKS")) : 512;
    if (blocks > cap) blocks = cap;  // persistent workgroups: the weights are staged to LDS once each
    if (blocks < 1) blocks = 1;
    const size_t lds = ((size_t)nnt * 32 * ((nkt > 4 ? 128 : 64) + 8) + 4 * 32 * ((K > NO ? K : NO) + 8)) * 2 +
                       ((bias || rowbias) ? (size_t)4 * 2 * nnt * 32 * sizeof(float) : 0);
    const int shape = tune_env("PDW_DENSE_GENERIC") ? 0 : (K == 128 && NO == 64) ? 1 : (K == 64 && NO == 128) ? 2 : 0;
    if (rider) {
        // The summations come first in the grid and take resident slots of their own from the start (the slots
        // are two per compute unit; waiting for finished row workgroups would put their latency behind the
        // product's): as long as they are few, the product gives up that many of its persistent workgroups.
        const int nride = rider->first_block[rider->njobs];
        if (blocks + nride > cap && nride <= cap / 4) blocks = cap - nride;
        const unsigned total = (unsigned)blocks + (unsigned)nride;
        // shapes of the block's layers as compile-time constants (shape = 0: from the arguments)
#define PDW_RIDE(T, KM, SK, SNO)                                                                                    \
    hipLaunchKernelGGL((dense_rows_rider_k<T, KM, SK, SNO>), dim3(total), dim3(256), lds, s, (const T*)x,            \
                       (const T*)w, (const T*)bias, rowbias, (T*)y, N, K, NO, P > 0 ? P : 1, nkt, nnt, (int)blocks,   \
                       *rider)
#define PDW_RIDE_S(T, KM)                 \
    if (shape == 1)                       \
        PDW_RIDE(T, KM, 128, 64);         \
    else if (shape == 2)                  \
        PDW_RIDE(T, KM, 64, 128);         \
    else                                  \
        PDW_RIDE(T, KM, 0, 0)
        if (dtype == kF16) {
            if (w_kmajor) { PDW_RIDE_S(f16_t, true); } else { PDW_RIDE_S(f16_t, false); }
        } else {
            if (w_kmajor) { PDW_RIDE_S(bf16_t, true); } else { PDW_RIDE_S(bf16_t, false); }
        }
#undef PDW_RIDE_S
#undef PDW_RIDE
        return check_launch("dense_rows_rider");
    }
#define PDW_GO(T, KM, CSUM, SK, SNO)                                                                             \
    hipLaunchKernelGGL((dense_rows_k<T, KM, CSUM, SK, SNO>), dim3((unsigned)blocks), dim3(256), lds, s, (const T*)x, \
                       (const T*)w, (const T*)bias, rowbias, (T*)y, colsum, N, K, NO, P > 0 ? P : 1, nkt, nnt)
#define PDW_GO_S(T, KM, CSUM)             \
    if (shape == 1)                       \
        PDW_GO(T, KM, CSUM, 128, 64);     \
    else if (shape == 2)                  \
        PDW_GO(T, KM, CSUM, 64, 128);     \
    else                                  \
        PDW_GO(T, KM, CSUM, 0, 0)
#define PDW_GO2(T, KM)                    \
    if (colsum) {                         \
        PDW_GO_S(T, KM, true);            \
    } else {                              \
        PDW_GO_S(T, KM, false);           \
    }
    // conv_up of a 96- or 64-feature pyramid block (with the tile sums): its extents as constants, too
    if (K == 96 && NO == 48 && colsum && !w_kmajor && !tune_env("PDW_DENSE_GENERIC")) {
        if (dtype == kF16) PDW_GO(f16_t, false, true, 96, 48); else PDW_GO(bf16_t, false, true, 96, 48);
    } else if (K == 64 && NO == 32 && colsum && !w_kmajor && !tune_env("PDW_DENSE_GENERIC")) {
        if (dtype == kF16) PDW_GO(f16_t, false, true, 64, 32); else PDW_GO(bf16_t, false, true, 64, 32);
    } else
    if (dtype == kF16) {
        if (w_kmajor) { PDW_GO2(f16_t, true) } else { PDW_GO2(f16_t, false) }
    } else {
        if (w_kmajor) { PDW_GO2(bf16_t, true) } else { PDW_GO2(bf16_t, false) }
    }
#undef PDW_GO2
#undef PDW_GO_S
#undef PDW_GO
    return check_launch("dense_rows");
}

// y = x W^T (+ bias) for the pixels of [B, H, W] images with (K, NO) = (128, 64), (96, 48) or (64, 32) features in / out
// (conv_up of a pyramid block of 128, 96 or 64 features), the sums of x over
// each 32-pixel tile (tiles of 4 rows x 8 columns here: still H * W / 32 per image, image after image) and the 2x2
// average pool of y.  -1: not covered (other widths, extents that are not multiples of 4 x 8, fp32).
int dense_rows_pool_launch(const void* x, const void* w, const void* bias, void* y, float* colsum, void* pool, int B,
                           int H, int W, int K, int NO, int dtype, hipStream_t s) {
    const bool s128 = K == 128 && NO == 64, s96 = K == 96 && NO == 48, s64 = K == 64 && NO == 32;
    if (dtype == kF32 || !(s128 || s96 || s64) || H % 4 != 0 || W % 8 != 0 || B < 1 || H < 4 || W < 8) return -1;
    if (tune_env("PDW_DENSE_GENERIC") || tune_env("PDW_NO_DENSE_POOL")) return -1;
    const long long N = (long long)B * H * W;
    if (N > 0x7fffffffLL) return -1;
    for (const void* p : {x, w, (const void*)y, (const void*)colsum, (const void*)pool})
        if (!p || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    if (reinterpret_cast<uintptr_t>(bias) & 7) return -1;
    const long long ntiles = N / 32;
    long long blocks = (ntiles + 3) / 4;
    const int cap = tune_env("PDW_DENSE_BLOCKS") ? atoi(tune_env("PDW_DENSE_BLOCKS")) : 512;
    if (blocks > cap) blocks = cap;
    // (weights as whole feature tiles x 64 or 128 padded inner values, four tile buffers of 32 rows x (K + 8), the
    // bias table)
    const int nnt = cdiv(NO, 32);
    const size_t lds = ((size_t)nnt * 32 * ((K > 64 ? 128 : 64) + 8) + 4 * 32 * (K + 8)) * 2 +
                       (bias ? (size_t)4 * 2 * nnt * 32 * sizeof(float) : 0);
#define PDW_POOL(T, SK, SNO)                                                                                         \
    hipLaunchKernelGGL((dense_rows_pool_k<T, SK, SNO>), dim3((unsigned)blocks), dim3(256), lds, s, (const T*)x,       \
                       (const T*)w, (const T*)bias, (T*)y, colsum, (T*)pool, N, H, W)
    if (dtype == kF16) {
        if (s128) PDW_POOL(f16_t, 128, 64); else if (s96) PDW_POOL(f16_t, 96, 48); else PDW_POOL(f16_t, 64, 32);
    } else {
        if (s128) PDW_POOL(bf16_t, 128, 64); else if (s96) PDW_POOL(bf16_t, 96, 48); else PDW_POOL(bf16_t, 64, 32);
    }
#undef PDW_POOL
    return check_launch("dense_rows_pool");
}

// y[N][128] = rows w^T + bias + rowbias[image] for the rows made from a pyramid block's two convolution outputs
// (dense_rows_body, MID): cf [B,H,W,64], ch [B,H/2,W/2,64]; cat (optional) receives the rows.  ldf > 0: both scales
// arrive gated, cf [B,H,W,32] at a pixel stride of ldf values, ch [B,H/2,W/2,32], no cat.  -1: not covered (other
// widths, extents that are not multiples of 4 x 8, fp32).
// Whether dense_mid_rows_launch covers the widths and extents (aligned tensors assumed).
int dense_mid_rows_supported(int H, int W, int I, int D, int dtype) {
    if (dtype == kF32 || I < 16 || I > 64 || I % 16 != 0 || !dense_dims_ok(I, D, dtype) || I + I / 2 > (I > D ? I : D) + 8)
        return 0;
    return (H % 4 == 0 && W % 8 == 0 && H >= 4 && W >= 8 && !tune_env("PDW_NO_DENSE_MID")) ? 1 : 0;
}

int dense_mid_rows_launch(const void* cf, const void* ch, void* cat, const void* w, const void* bias,
                          const float* rowbias, void* y, int B, int H, int W, int I, int D, int dtype, hipStream_t s,
                          int ldf) {
    // widths: the inner one a multiple of 16 up to 64 (two items per lane make a tile's rows), the outer one whatever the
    // row kernel covers, wide enough that the half scale's patch fits beside a tile's rows in the tile buffer
    if (!dense_mid_rows_supported(H, W, I, D, dtype) || B < 1) return -1;
    if (ldf != 0 && (ldf < I / 2 || ldf % 8 != 0 || cat)) return -1;
    const long long N = (long long)B * H * W;
    if (N > 0x7fffffffLL / 128) return -1;
    const bool exact = I == 64 && D == 128 && !tune_env("PDW_DENSE_GENERIC");
    const bool exact96 = I == 48 && D == 96 && !tune_env("PDW_DENSE_GENERIC");
    const bool exact64 = I == 32 && D == 64 && !tune_env("PDW_DENSE_GENERIC");
    const int nnt = cdiv(D, 32);
    for (const void* p : {cf, ch, w, (const void*)y})
        if (!p || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    if ((reinterpret_cast<uintptr_t>(cat) & 15) || (reinterpret_cast<uintptr_t>(rowbias) & 15) ||
        (reinterpret_cast<uintptr_t>(bias) & 7))
        return -1;
    const long long ntiles = N / 32;
    long long blocks = (ntiles + 3) / 4;
    const int cap = tune_env("PDW_DENSE_BLOCKS") ? atoi(tune_env("PDW_DENSE_BLOCKS")) : 512;
    if (blocks > cap) blocks = cap;
    const size_t lds = ((size_t)nnt * 32 * (64 + 8) + 4 * 32 * ((I > D ? I : D) + 8)) * 2 +
                       ((bias || rowbias) ? (size_t)4 * 2 * nnt * 32 * sizeof(float) : 0);
    const MidRows mid{cf, ch, cat, ldf, sqrtf((float)(I / 2))};
#define PDW_MID(T, M, SK, SNO)                                                                                   \
    hipLaunchKernelGGL((dense_mid_rows_k<T, M, SK, SNO>), dim3((unsigned)blocks), dim3(256), lds, s, (const T*)w, \
                       (const T*)bias, rowbias, (T*)y, N, H, W, I, D, mid)
#define PDW_MID_S(T, M)            \
    if (exact)                     \
        PDW_MID(T, M, 64, 128);    \
    else if (exact96)              \
        PDW_MID(T, M, 48, 96);     \
    else if (exact64)              \
        PDW_MID(T, M, 32, 64);     \
    else                           \
        PDW_MID(T, M, 0, 0)
    if (dtype == kF16) {
        if (ldf) { PDW_MID_S(f16_t, 2); } else { PDW_MID_S(f16_t, 1); }
    } else {
        if (ldf) { PDW_MID_S(bf16_t, 2); } else { PDW_MID_S(bf16_t, 1); }
    }
#undef PDW_MID_S
#undef PDW_MID
    return check_launch("dense_mid_rows");
}

static void dense_wgrad_plan(long long N, int* blocks, int* stages_per_block) {
    const long long nstages = (N + kWgRows - 1) / kWgRows;
    long long nb = tune_env("PDW_DWG_BLOCKS") ? atoi(tune_env("PDW_DWG_BLOCKS")) : 256;
    if (nb > nstages) nb = nstages;
    if (nb < 1) nb = 1;
    const long long spb = (nstages + nb - 1) / nb;
    *stages_per_block = (int)(spb < 1 ? 1 : spb);
    *blocks = (int)((nstages + *stages_per_block - 1) / *stages_per_block);
    if (*blocks < 1) *blocks = 1;
}

// the staged kernel of this file
static bool dense_wgrad_tiled_ok(int M, int NO, int dtype) {
    const int mt = cdiv(M, 32), nt = cdiv(NO, 32);
    return dtype != kF32 && M >= 8 && NO >= 8 && M % 8 == 0 && NO % 8 == 0 && mt <= 4 && nt <= 4 && mt * nt <= 8;
}

int dense_wgrad_supported(int M, int NO, int dtype) {
    return (dense_wgrad_tiled_ok(M, NO, dtype) || dense_any_wgrad_dims_ok(M, NO)) ? 1 : 0;
}

size_t dense_wgrad_workspace(long long N, int M, int NO) {
    int blocks, spb;
    dense_wgrad_plan(N, &blocks, &spb);
    return (size_t)blocks * M * NO * sizeof(float);
}

template <typename T, int MT, int NT, bool EXACT>
static int dense_wgrad_go(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, hipStream_t s) {
    int blocks, spb;
    dense_wgrad_plan(N, &blocks, &spb);
    size_t lds = (size_t)2 * kWgRows * (M + 8 + NO + 8) * 2;
    if (lds < 4 * 16 * 64 * sizeof(float)) lds = 4 * 16 * 64 * sizeof(float);
    // While reductions are being deferred, the ones recorded so far run in this launch; its own joins the list.
    ReduceJobs jobs;
    if (reduce_defer_take(&jobs) > 0) {
        hipLaunchKernelGGL((dense_wgrad_rider_k<T, MT, NT, EXACT>), dim3(blocks + jobs.first_block[jobs.njobs]),
                           dim3(256), lds, s, (const T*)a, (const T*)b, (float*)ws, N, M, NO, blocks, jobs);
    } else {
        hipLaunchKernelGGL((dense_wgrad_k<T, MT, NT, EXACT>), dim3(blocks), dim3(256), lds, s, (const T*)a,
                           (const T*)b, (float*)ws, N, M, NO);
    }
    if (int e = check_launch("dense_wgrad")) return e;
    return wgrad_reduce_launch<T>((const float*)ws, dw, blocks, M * NO, s);
}

template <typename T>
static int dense_wgrad_t(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, hipStream_t s) {
    const int mt = cdiv(M, 32), nt = cdiv(NO, 32);
    // the block's two layer shapes (64 x 128 and 128 x 64) have variants with the extents as constants
    if (M == 64 && NO == 128 && !tune_env("PDW_DENSE_GENERIC")) return dense_wgrad_go<T, 2, 4, true>(a, b, dw, ws, N, M, NO, s);
    if (M == 128 && NO == 64 && !tune_env("PDW_DENSE_GENERIC")) return dense_wgrad_go<T, 4, 2, true>(a, b, dw, ws, N, M, NO, s);
#define PDW_CASE(MT, NT) \
    if (mt == MT && nt == NT) return dense_wgrad_go<T, MT, NT, false>(a, b, dw, ws, N, M, NO, s);
    PDW_CASE(1, 1) PDW_CASE(1, 2) PDW_CASE(2, 1) PDW_CASE(2, 2) PDW_CASE(1, 3) PDW_CASE(3, 1) PDW_CASE(2, 3)
    PDW_CASE(3, 2) PDW_CASE(1, 4) PDW_CASE(4, 1) PDW_CASE(2, 4) PDW_CASE(4, 2)
#undef PDW_CASE
    return -1;
}

int dense_wgrad_launch(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, int dtype,
                       hipStream_t s) {
    if (!dense_wgrad_tiled_ok(M, NO, dtype)) {   // fp32, other widths: at most as many partials as the workspace holds
        int blocks, spb;
        dense_wgrad_plan(N, &blocks, &spb);
        return dense_any_wgrad_launch(a, b, dw, ws, N, M, NO, dtype, blocks, s);
    }
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15)) return -1;
    if (dtype == kF16) return dense_wgrad_t<f16_t>(a, b, dw, ws, N, M, NO, s);
    return dense_wgrad_t<bf16_t>(a, b, dw, ws, N, M, NO, s);
}

static bool pair_exact(int O, int I) {
    return (O == 128 && I == 64) || (O == 64 && I == 128) || (O == 64 && I == 32) || (O == 32 && I == 64) ||
           (O == 96 && I == 48) || (O == 48 && I == 96);
}

int dense_bwd_pair_supported(int O, int I, int dtype) {
    if (dtype == kF32) return 0;
    if (pair_exact(O, I)) return 1;
    // any widths both bodies cover: the row product with K = O, NO = I and the weight gradient with M = O, NO = I
    return (dense_dims_ok(O, I, dtype) && dense_wgrad_tiled_ok(O, I, dtype)) ? 1 : 0;
}

// with the 32-row tile sums of gy (the `colsum` argument of the launch)
int dense_bwd_pair_colsum_supported(int O, int I, int dtype) {
    return (dense_bwd_pair_supported(O, I, dtype) && (!pair_exact(O, I) || O >= 64) && dense_colsum_supported(O, I, dtype))
               ? 1
               : 0;
}

// -1: shape not covered.  ws: dense_wgrad_workspace(N, O, I) bytes.
int dense_bwd_pair_launch(const void* gy, const void* w, const void* xin, void* dx, float* colsum, void* dw, void* ws,
                          const float* rowbias, int P, long long N, int O, int I, int dtype, hipStream_t s) {
    if (!dense_bwd_pair_supported(O, I, dtype)) return -1;
    if (rowbias && (P < 32 || (reinterpret_cast<uintptr_t>(rowbias) & 15))) return -1;  // two images per tile at most
    if (N <= 0 || N > 0x7fffffffLL) return -1;
    const void* ptrs[5] = {gy, w, xin, dx, colsum};
    for (const void* p : ptrs)
        if (reinterpret_cast<uintptr_t>(p) & 15) return -1;
    int nwg, spb;
    dense_wgrad_plan(N, &nwg, &spb);
    const long long ntiles = (N + 31) / 32;
    long long nrows = (ntiles + 3) / 4;
    const int cap = tune_env("PDW_PAIR_ROWS") ? atoi(tune_env("PDW_PAIR_ROWS")) : 256;  // the second slot of every CU
    if (nrows > cap) nrows = cap;
    if (colsum && !dense_bwd_pair_colsum_supported(O, I, dtype)) return -1;
    // rows product: K = O, NO = I (inner dimension padded to 64 or 128 in LDS); weight gradient: M = O, NO = I
    const int nnt = cdiv(I, 32);
    const size_t lds_rows = ((size_t)nnt * 32 * ((O > 64 ? 128 : 64) + 8) + 4 * 32 * ((O > I ? O : I) + 8)) * 2 +
                            (rowbias ? (size_t)4 * 2 * nnt * 32 * sizeof(float) : 0);
    const size_t lds_wg = (size_t)2 * kWgRows * (O + 8 + I + 8) * 2;
    const size_t lds = lds_rows > lds_wg ? lds_rows : lds_wg;
    const dim3 grid((unsigned)(nwg + nrows));
#define PDW_PAIR(T, CS, OO, II)                                                                                      \
    hipLaunchKernelGGL((dense_bwd_pair_k<T, CS, OO, II>), grid, dim3(256), lds, s, (const T*)gy, (const T*)w,        \
                       (const T*)xin, (T*)dx, colsum, (float*)ws, rowbias, P > 0 ? P : 1, N, nwg, (int)nrows)
#define PDW_PAIR_T(T)                                           \
    if (O == 128) {                                             \
        if (colsum) PDW_PAIR(T, true, 128, 64); else PDW_PAIR(T, false, 128, 64); \
    } else if (O == 96) {                                       \
        if (colsum) PDW_PAIR(T, true, 96, 48); else PDW_PAIR(T, false, 96, 48); \
    } else if (O == 48) {                                       \
        PDW_PAIR(T, false, 48, 96);                             \
    } else if (O == 64 && I == 128) {                           \
        if (colsum) PDW_PAIR(T, true, 64, 128); else PDW_PAIR(T, false, 64, 128); \
    } else if (O == 64) {                                       \
        if (colsum) PDW_PAIR(T, true, 64, 32); else PDW_PAIR(T, false, 64, 32); \
    } else {                                                    \
        PDW_PAIR(T, false, 32, 64);                             \
    }
#define PDW_PAIR_GEN(T, MT_, NT_)                                                                                   \
    if (mt == MT_ && nt == NT_) {                                                                                    \
        if (colsum)                                                                                                  \
            hipLaunchKernelGGL((dense_bwd_pair_gen_k<T, MT_, NT_, true>), grid, dim3(256), lds, s, (const T*)gy,     \
                               (const T*)w, (const T*)xin, (T*)dx, colsum, (float*)ws, rowbias, P > 0 ? P : 1, N, O, \
                               I, nwg, (int)nrows);                                                                  \
        else                                                                                                         \
            hipLaunchKernelGGL((dense_bwd_pair_gen_k<T, MT_, NT_, false>), grid, dim3(256), lds, s, (const T*)gy,    \
                               (const T*)w, (const T*)xin, (T*)dx, colsum, (float*)ws, rowbias, P > 0 ? P : 1, N, O, \
                               I, nwg, (int)nrows);                                                                  \
    }
#define PDW_PAIR_GEN_T(T)                                                                                           \
    PDW_PAIR_GEN(T, 1, 1) PDW_PAIR_GEN(T, 1, 2) PDW_PAIR_GEN(T, 2, 1) PDW_PAIR_GEN(T, 2, 2) PDW_PAIR_GEN(T, 1, 3)     \
    PDW_PAIR_GEN(T, 3, 1) PDW_PAIR_GEN(T, 2, 3) PDW_PAIR_GEN(T, 3, 2) PDW_PAIR_GEN(T, 1, 4) PDW_PAIR_GEN(T, 4, 1)     \
    PDW_PAIR_GEN(T, 2, 4) PDW_PAIR_GEN(T, 4, 2)
    if (pair_exact(O, I)) {
        if (dtype == kF16) { PDW_PAIR_T(f16_t) } else { PDW_PAIR_T(bf16_t) }
    } else {
        const int mt = cdiv(O, 32), nt = cdiv(I, 32);
        if (dtype == kF16) { PDW_PAIR_GEN_T(f16_t) } else { PDW_PAIR_GEN_T(bf16_t) }
    }
#undef PDW_PAIR_GEN_T
#undef PDW_PAIR_GEN
#undef PDW_PAIR_T
#undef PDW_PAIR
    if (int e = check_launch("dense_bwd_pair")) return e;
    if (dtype == kF16) return wgrad_reduce_launch<f16_t>((const float*)ws, dw, nwg, O * I, s);
    return wgrad_reduce_launch<bf16_t>((const float*)ws, dw, nwg, O * I, s);
}

}  // namespace pdw

