// Dense layers for the shapes that the tiled matrix-core kernels of dense.hip do not take: fp32, and 16-bit layers
// whose widths are multiples of 4 only or wider than 128 (nn.Linear of conv_block.py:37, 44 on any dim and in fp32).
//
//   rows:  Y[n,o] = sum_k X[n,k] * W(o,k) + bias[o] + rowbias[n / P][o]
//   wgrad: dW[m,o] = sum_n A[n,m] * B[n,o]
//
// One wavefront makes one 32 x 32 tile of the result with v_mfma_f32_32x32x2_f32 (fp32) or
// v_mfma_f32_32x32x16_{bf16,f16}: every operand value is used once per instruction, there is no loop over feature
// tiles and no per-wave tile buffer, so the code has no width limit beyond what its one LDS slab holds and no
// alignment need beyond 4 values.  The row operand X is read straight from global memory (a lane: one row, 16 bytes
// of consecutive k per step, eight steps requested ahead); the 32 x K slab of W that a workgroup's four wavefronts
// share is staged to LDS once, transposed on the way in when W is stored [K][NO].  The same rows are read again by
// the wavefronts of the other feature tiles: from the caches, which is what these small or ragged layers fit in.
// fp32 runs at the fp32 matrix rate (a sixteenth of the 16-bit one), which at the widths of a pyramid block is as
// long as the memory traffic takes.
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "common.h"
#include "kernels.h"
#include "reduce_parts.h"

namespace pdw {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kAnyMaxK = 256;   // inner width the LDS slab is sized for (33 KB in fp32)

// Per element type: the k values one step covers (a lane holds half of them, 16 bytes, consecutive) and the product.
template <typename T>
struct AnyStep;
template <>
struct AnyStep<float> {
    static constexpr int KS = 8;
    static __device__ __forceinline__ v16f mul(const uint4& a, const uint4& b, v16f c) {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.x), __builtin_bit_cast(float, b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.y), __builtin_bit_cast(float, b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.z), __builtin_bit_cast(float, b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.w), __builtin_bit_cast(float, b.w), c, 0, 0, 0);
        return c;
    }
};
template <>
struct AnyStep<bf16_t> {
    static constexpr int KS = 16;
    static __device__ __forceinline__ v16f mul(const uint4& a, const uint4& b, v16f c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    }
};
template <>
struct AnyStep<f16_t> {
    static constexpr int KS = 16;
    static __device__ __forceinline__ v16f mul(const uint4& a, const uint4& b, v16f c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
    }
};

typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// Loads go through buffer descriptors: an offset past the descriptor's end reads as zero and moves no data, so rows
// past the tensor and values past a row's end need no branch (a vector-memory instruction behind a branch makes the
// compiler wait for every load in flight).  kPast added to any offset of a descriptor of less than 2^31 bytes stays
// past its end.
constexpr uint32_t kPast = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t any_rsrc(const void* p, long long bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// Y = X W^T (+ bias + rowbias).  A workgroup's four wavefronts are CT feature tiles x 4 / CT row tiles (CT = 1, 2, 4):
// the wavefronts that need the same rows run side by side.  Grid: x = groups of 128 / CT rows, y = groups of CT feature
// tiles.  KMAJOR: W is stored [K][NO] (the input gradient of a layer whose weights are [NO_layer = K][K_layer = NO]).
//
// A wavefront walks its 32 rows in chunks of 256 bytes per row (64 fp32 or 128 16-bit values: 8 steps): the chunk is
// read with coalesced loads (a lane takes 16 or 8 consecutive bytes, lane after lane along the row: whole 64-byte
// sectors; row-strided operand loads straight from global memory ask the L1 for four times the sectors), held in
// registers while the previous chunk is multiplied, and reshaped into MFMA operands through the wavefront's own LDS
// tile.  Values past K read as zero; the weight slab is zero there as well.
template <typename T, bool KMAJOR, int CT>
__global__ __launch_bounds__(256) void dense_any_rows_k(const T* __restrict__ X, const T* __restrict__ W,
                                                        const T* __restrict__ bias, const float* __restrict__ rowbias,
                                                        T* __restrict__ Y, int N, int K, int NO, int P, int nimg) {
    constexpr int KS = AnyStep<T>::KS, KL = KS / 2, PAD = 16 / (int)sizeof(T), ES = (int)sizeof(T);
    constexpr int CE = 256 / ES;                           // values of a row per chunk
    constexpr int VE = 4;                                  // a lane's load: 4 values
    constexpr int NV = CE / VE, PASSES = 32 * NV / 64;     // loads per row and chunk; per lane and chunk
    constexpr int TP = CE + PAD;                           // pitch of the wavefront's tile
    constexpr int ITW = 8;                                 // groups of 4 weights per thread and pass
    constexpr int NC = 32 * CT;                            // features of the slab
    extern __shared__ uint32_t dsm[];
    T* wl = reinterpret_cast<T*>(dsm);                    // [NC features][KP]
    const int KR = (K + CE - 1) / CE * CE, KP = KR + PAD;  // k padded to whole chunks, pitch off the banks
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (scalar: the tile loop and its descriptors are uniform)
    T* tl = wl + NC * KP + wave * 32 * TP;                 // [32 rows][TP]
    const int c0 = blockIdx.y * NC;
    const int ct = wave % CT, rt = wave / CT;
    // row tiles of 32: this wavefront takes tiles first, first + stride, ...; a tile's descriptor ends with its rows (or
    // with the tensor), one past the last tile holds nothing
    const long long ntiles = ((long long)N + 31) / 32;
    const long long first = (long long)blockIdx.x * (4 / CT) + rt, stride = (long long)gridDim.x * (4 / CT);
    auto tile_rsrc = [&](long long t) {
        const long long r0 = t * 32;
        const int nrows = t < ntiles ? (int)(N - r0 < 32 ? N - r0 : 32) : 0;
        return any_rsrc(X + (t < ntiles ? r0 : 0) * K, (long long)nrows * K * ES);
    };
    typedef typename std::conditional<ES == 4, v4u, v2u>::type Vec;
    Vec st[PASSES];
    uint32_t goff[PASSES];   // byte offset of this lane's load in chunk 0; its first value's k
    int gk[PASSES], ldst[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int v = p * 64 + lane, row = v / NV, cv = v - row * NV;
        goff[p] = (uint32_t)((row * K + cv * VE) * ES), gk[p] = cv * VE, ldst[p] = row * TP + cv * VE;
    }
    auto request = [&](const __amdgpu_buffer_rsrc_t& r, int c) {   // chunk c of a tile
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const uint32_t off = gk[p] + c * CE < K ? goff[p] + (uint32_t)(c * CE * ES) : kPast;
            if constexpr (ES == 4) st[p] = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
            else st[p] = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
        }
    };
    request(tile_rsrc(first), 0);
    const int col = c0 + 32 * ct + l32;
    const bool cok = col < NO;
    const float bv0 = bias && cok ? to_f32(bias[col]) : 0.f;
    // the slab, zero where W has nothing (features past NO, k past K): groups of 4 consecutive k of one feature
    // (W[NO][K]) or of 4 consecutive features of one k (W[K][NO]: NO % 4 == 0, a group exists whole or not at all)
    const __amdgpu_buffer_rsrc_t wrsrc = any_rsrc(W, (long long)K * NO * ES);
    {
        const int kq = KR / 4, ngroups = KMAJOR ? (NC / 4) * KR : NC * kq;
        for (int base = 0; base < ngroups; base += 256 * ITW) {
            ChanVec<T, 4> wv[ITW];
            int wdst[ITW];
#pragma unroll
            for (int it = 0; it < ITW; ++it) {
                const int i = base + tid + it * 256;
                uint32_t off;
                bool ok;
                if constexpr (!KMAJOR) {
                    const int c = i / kq, q = i - c * kq;
                    ok = c0 + c < NO && 4 * q < K;
                    off = (uint32_t)(((c0 + c) * K + 4 * q) * ES);
                    wdst[it] = i < ngroups ? c * KP + 4 * q : -1;
                } else {
                    const int k = i / (NC / 4), q = i - k * (NC / 4);
                    ok = k < K && c0 + 4 * q < NO;
                    off = (uint32_t)((k * NO + c0 + 4 * q) * ES);
                    wdst[it] = i < ngroups ? 4 * q * KP + k : -1;
                }
                if constexpr (ES == 4) {
                    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)(ok ? off : kPast), 0, 0);
                    wv[it] = __builtin_bit_cast(ChanVec<T, 4>, v);
                } else {
                    const v2u v = __builtin_amdgcn_raw_buffer_load_b64(wrsrc, (int)(ok ? off : kPast), 0, 0);
                    wv[it] = __builtin_bit_cast(ChanVec<T, 4>, v);
                }
            }
#pragma unroll
            for (int it = 0; it < ITW; ++it) {
                if (wdst[it] >= 0) {
                    if constexpr (!KMAJOR) {
                        *reinterpret_cast<ChanVec<T, 4>*>(wl + wdst[it]) = wv[it];
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t) wl[wdst[it] + t * KP] = wv[it].v[t];
                    }
                }
            }
        }
    }
    __syncthreads();
    const T* wr = wl + (32 * ct + l32) * KP + KL * h;
    const T* ar = tl + l32 * TP + KL * h;
    const int nsteps = (K + KS - 1) / KS, nchunks = KR / CE;
    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    long long tile = first;
    int c = 0;
    while (tile < ntiles) {
        // the chunk goes to the tile buffer (the wavefront's own LDS operations stay in order: no barrier), the next
        // one - of this tile or of the wavefront's next - is requested, and the chunk's 8 steps run on operands read
        // back from the buffer
#pragma unroll
        for (int p = 0; p < PASSES; ++p) *reinterpret_cast<Vec*>(tl + ldst[p]) = st[p];
        const bool last = c + 1 == nchunks;
        const long long tnext = last ? tile + stride : tile;
        const int cnext = last ? 0 : c + 1;
        request(tile_rsrc(tnext), cnext);
#pragma unroll
        for (int sidx = 0; sidx < CE / KS; ++sidx) {
            if (c * (CE / KS) + sidx < nsteps) {   // uniform
                const uint4 av = *reinterpret_cast<const uint4*>(ar + sidx * KS);
                const uint4 bv = *reinterpret_cast<const uint4*>(wr + (c * (CE / KS) + sidx) * KS);
                acc = AnyStep<T>::mul(av, bv, acc);
            }
        }
        if (last) {
            // lane: feature col, rows r0 + 8 (i / 4) + 4 h + i % 4; bias and the per-image rows of the (at most two:
            // P >= 32) images of the tile
            const long long r0 = tile * 32;
            if (cok) {
                float add = bv0, add1 = bv0;
                long long edge = (long long)N;   // first row of the tile's second image
                if (rowbias) {
                    const int img = (int)(r0 / P);
                    edge = (long long)(img + 1) * P;
                    add += rowbias[(long long)img * NO + col];
                    add1 += rowbias[(long long)(img + 1 < nimg ? img + 1 : img) * NO + col];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const long long r = r0 + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (r < N) Y[r * NO + col] = from_f32<T>(acc[i] + (r < edge ? add : add1));
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        }
        tile = tnext, c = cnext;
    }
}

// Partials of dW[M][NO] = A^T B over row chunks: grid x = chunk, y = groups of 4 tiles (a wavefront: one 32 x 32
// tile of dW for the chunk's rows).  The MFMA k is the row index: a lane holds one feature of 4 (fp32) or 8 (16-bit)
// rows, so consecutive lanes read consecutive features of a row.
template <typename T>
__global__ __launch_bounds__(256) void dense_any_wgrad_k(const T* __restrict__ A, const T* __restrict__ Bm,
                                                         float* __restrict__ part, int N, int M, int NO, int rows_per_chunk,
                                                         int nt) {
    constexpr int KS = AnyStep<T>::KS, KL = KS / 2, ES = (int)sizeof(T);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int mt_total = (M + 31) / 32;
    const int tile = blockIdx.y * 4 + wave;
    if (tile >= mt_total * nt) return;
    const int tm = tile / nt, tn = tile - tm * nt;
    const long long rb = (long long)blockIdx.x * rows_per_chunk;
    const int nrows = (int)(rb + rows_per_chunk < N ? rows_per_chunk : N - rb);
    const int m = tm * 32 + l32, n = tn * 32 + l32;
    // descriptors over the chunk's rows: rows past the chunk read as zero; so does a feature past the width
    const __amdgpu_buffer_rsrc_t arsrc = any_rsrc(A + rb * M, (long long)nrows * M * ES);
    const __amdgpu_buffer_rsrc_t brsrc = any_rsrc(Bm + rb * NO, (long long)nrows * NO * ES);
    const uint32_t aoff = m < M ? (uint32_t)((KL * h * M + m) * ES) : kPast;
    const uint32_t boff = n < NO ? (uint32_t)((KL * h * NO + n) * ES) : kPast;
    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    // one step: rows r .. r + KS - 1 of the chunk, this lane's are r + KL h .. + KL - 1
    auto fetch = [&](int r, uint4& a, uint4& b) {
        if constexpr (ES == 4) {
            uint32_t av[4], bv[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                av[t] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(arsrc, (int)(aoff + (uint32_t)((r + t) * M * ES)), 0, 0));
                bv[t] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(brsrc, (int)(boff + (uint32_t)((r + t) * NO * ES)), 0, 0));
            }
            a = make_uint4(av[0], av[1], av[2], av[3]);
            b = make_uint4(bv[0], bv[1], bv[2], bv[3]);
        } else {
            uint32_t av[8], bv[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                av[t] = (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(arsrc, (int)(aoff + (uint32_t)((r + t) * M * ES)), 0, 0);
                bv[t] = (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(brsrc, (int)(boff + (uint32_t)((r + t) * NO * ES)), 0, 0);
            }
            a = make_uint4(av[0] | (av[1] << 16), av[2] | (av[3] << 16), av[4] | (av[5] << 16), av[6] | (av[7] << 16));
            b = make_uint4(bv[0] | (bv[1] << 16), bv[2] | (bv[3] << 16), bv[4] | (bv[5] << 16), bv[6] | (bv[7] << 16));
        }
    };
    constexpr int D = 4;
    uint4 a[D], b[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        fetch(d * KS, a[d], b[d]);
        __builtin_amdgcn_sched_barrier(0);   // (requested in the order in which the loop re-requests them)
    }
    for (int r = 0; r < nrows; r += D * KS) {   // (steps past the chunk multiply zeros)
#pragma unroll
        for (int d = 0; d < D; ++d) {
            acc = AnyStep<T>::mul(a[d], b[d], acc);
            fetch(r + (d + D) * KS, a[d], b[d]);
            // (keeps the steps in order: moved together, the loads of all steps end up behind all products, and the
            // next round then waits for every one of them instead of the oldest)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // lane: column n of dW, rows tm * 32 + 8 (i / 4) + 4 h + i % 4
    float* po = part + (long long)blockIdx.x * M * NO;
    if (n < NO) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int mm = tm * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
            if (mm < M) po[(long long)mm * NO + n] = acc[i];
        }
    }
}

size_t any_slab_bytes(int K, int esize) {   // 32 features of the weight slab: k padded to whole 256-byte chunks
    const int ce = 256 / esize;
    return (size_t)32 * ((K + ce - 1) / ce * ce + 16 / esize) * esize;
}
constexpr size_t kAnyTileBytes = 4 * 32 * (256 + 16);   // the four wavefronts' row tiles

template <typename T, bool KM, int CT>
int any_rows_go(const void* x, const void* w, const void* bias, const float* rowbias, void* y, long long N, int K, int NO,
                int P, int nimg, hipStream_t s) {
    auto kern = dense_any_rows_k<T, KM, CT>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    // persistent workgroups (the weight slab is staged once each): at most 512 per group of feature tiles
    const int rows_per_wg = 32 * (4 / CT), nct = (NO + 31) / 32;
    long long gx = (N + rows_per_wg - 1) / rows_per_wg;
    if (gx > 512) gx = 512;
    const dim3 grid((unsigned)gx, (unsigned)((nct + CT - 1) / CT));
    hipLaunchKernelGGL(kern, grid, dim3(256), CT * any_slab_bytes(K, (int)sizeof(T)) + kAnyTileBytes, s, (const T*)x, (const T*)w,
                       (const T*)bias, rowbias, (T*)y, (int)N, K, NO, P > 0 ? P : 1, nimg);
    return check_launch("dense_any_rows");
}

}  // namespace

bool dense_any_dims_ok(int K, int NO) { return K >= 4 && NO >= 4 && K % 4 == 0 && NO % 4 == 0 && K <= kAnyMaxK; }

// -1: not covered (widths, alignment, more than 2^31 - 1 rows).
int dense_any_rows_launch(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                          long long N, int K, int NO, int P, int dtype, hipStream_t s) {
    if (!dense_any_dims_ok(K, NO)) return -1;
    if (N == 0) return 0;
    const int es = dtype == kF32 ? 4 : 2;
    if (N > 0x7fffffffLL) return -1;   // (descriptors are per 32-row tile: no limit on the bytes of x)
    const uintptr_t amask = es == 4 ? 15 : 7;   // groups of 4 values
    if ((reinterpret_cast<uintptr_t>(x) & amask) || (reinterpret_cast<uintptr_t>(w) & amask)) return -1;
    if (rowbias && P < 32) {
        // a 32-row tile takes its per-image rows from two images at most; smaller images get theirs in a second pass
        if (int e = dense_any_rows_launch(x, w, w_kmajor, bias, nullptr, y, N, K, NO, P, dtype, s)) return e;
        const long long full = N / P, rest = N - full * P;
        if (full > 0)
            if (int e = add_rowbias_launch(y, rowbias, (int)full, P, NO, dtype, s)) return e;
        if (rest > 0)
            return add_rowbias_launch(static_cast<char*>(y) + (size_t)full * P * NO * es, rowbias + full * NO, 1, (int)rest,
                                      NO, dtype, s);
        return 0;
    }
    const int nimg = rowbias ? (int)((N + P - 1) / P) : 1;
    // feature tiles per workgroup: all of them up to 4 (the wavefronts that read the same rows side by side), as long as
    // their slabs fit in 96 KB of LDS; a small problem (fewer row tiles than the persistent grid has wavefronts) is
    // better off with more, smaller workgroups that stage one slab each
    const int nct = (NO + 31) / 32;
    const long long ntiles = (N + 31) / 32;
    int ct = ntiles < 2048 ? 1 : nct >= 3 ? 4 : nct;
    while (ct > 1 && ct * any_slab_bytes(K, es) > 96 * 1024) ct /= 2;
#define PDW_ANY_CT(T, KM)                                                                               \
    (ct == 4   ? any_rows_go<T, KM, 4>(x, w, bias, rowbias, y, N, K, NO, P, nimg, s)                    \
     : ct == 2 ? any_rows_go<T, KM, 2>(x, w, bias, rowbias, y, N, K, NO, P, nimg, s)                    \
               : any_rows_go<T, KM, 1>(x, w, bias, rowbias, y, N, K, NO, P, nimg, s))
    if (dtype == kF32) return w_kmajor ? PDW_ANY_CT(float, true) : PDW_ANY_CT(float, false);
    if (dtype == kF16) return w_kmajor ? PDW_ANY_CT(f16_t, true) : PDW_ANY_CT(f16_t, false);
    return w_kmajor ? PDW_ANY_CT(bf16_t, true) : PDW_ANY_CT(bf16_t, false);
#undef PDW_ANY_CT
}

bool dense_any_wgrad_dims_ok(int M, int NO) { return M >= 4 && NO >= 4 && M % 4 == 0 && NO % 4 == 0; }

// Row chunks of the weight gradient: enough wavefronts for the chip, at most `max_chunks` partials.
static int any_wgrad_chunks(long long N, int M, int NO, int max_chunks) {
    const int tiles = ((M + 31) / 32) * ((NO + 31) / 32);
    long long c = (2048 + tiles - 1) / tiles;
    const long long by_rows = (N + 63) / 64;   // 64 rows per chunk at least
    if (c > by_rows) c = by_rows;
    if (c > max_chunks) c = max_chunks;
    return (int)(c < 1 ? 1 : c);
}

// ws: max_chunks * M * NO floats (max_chunks as the caller sized it: dense_wgrad_workspace).
int dense_any_wgrad_launch(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, int dtype,
                           int max_chunks, hipStream_t s) {
    if (!dense_any_wgrad_dims_ok(M, NO) || N > 0x7fffffffLL || max_chunks < 1) return -1;
    if (N == 0) {   // an empty sum: the summation of no partials writes the zeros (a kernel, so that it can be captured)
        if (dtype == kF32) return wgrad_reduce_launch<float>((const float*)ws, dw, 0, M * NO, s);
        if (dtype == kF16) return wgrad_reduce_launch<f16_t>((const float*)ws, dw, 0, M * NO, s);
        return wgrad_reduce_launch<bf16_t>((const float*)ws, dw, 0, M * NO, s);
    }
    const int chunks0 = any_wgrad_chunks(N, M, NO, max_chunks);
    const int ks = dtype == kF32 ? 8 : 16;
    long long rpc = (N + chunks0 - 1) / chunks0;
    rpc = (rpc + ks - 1) / ks * ks;
    const int chunks = (int)((N + rpc - 1) / rpc);
    if (rpc * (M > NO ? M : NO) * (dtype == kF32 ? 4 : 2) > 0x7fffffffLL) return -1;   // (32-bit byte offsets into a chunk)
    const int nt = (NO + 31) / 32, tiles = ((M + 31) / 32) * nt;
    const dim3 grid((unsigned)chunks, (unsigned)((tiles + 3) / 4));
#define PDW_ANYW(T) \
    hipLaunchKernelGGL((dense_any_wgrad_k<T>), grid, dim3(256), 0, s, (const T*)a, (const T*)b, (float*)ws, (int)N, M, NO, (int)rpc, nt)
    if (dtype == kF32) PDW_ANYW(float);
    else if (dtype == kF16) PDW_ANYW(f16_t);
    else PDW_ANYW(bf16_t);
#undef PDW_ANYW
    if (int e = check_launch("dense_any_wgrad")) return e;
    if (dtype == kF32) return wgrad_reduce_launch<float>((const float*)ws, dw, chunks, M * NO, s);
    if (dtype == kF16) return wgrad_reduce_launch<f16_t>((const float*)ws, dw, chunks, M * NO, s);
    return wgrad_reduce_launch<bf16_t>((const float*)ws, dw, chunks, M * NO, s);
}

}  // namespace pdw
