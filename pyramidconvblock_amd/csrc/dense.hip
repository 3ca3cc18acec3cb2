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
#include <stdlib.h>

#include "common.h"
#include "kernels.h"

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

// 8 values p[0], p[stride], ..., p[7*stride] (zeros where !ok) packed as a fragment.
template <typename T>
__device__ __forceinline__ Frag gather8(const T* p, long long stride, bool ok) {
    Frag f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t lo = ok ? ld16(p + (2 * j) * stride) : 0u;
        const uint32_t hi = ok ? ld16(p + (2 * j + 1) * stride) : 0u;
        f.v[j] = lo | (hi << 16);
    }
    return f;
}

// Weights live in LDS as wl[NO][K + 8] (the pad keeps 16-byte fragment reads of 32 consecutive rows off
// the same banks); every MFMA reads its weight fragment from there.  Row tiles (32 rows x K) are loaded
// fully coalesced - a wavefront reads its 32*K*2 contiguous bytes as 16-byte chunks, lane after lane -
// and re-shaped into MFMA fragments through a per-wave LDS buffer: row-strided fragment loads straight
// from global memory run ~2.5x slower on this part.  The same buffer transposes the result tile so the
// global stores are whole 128-byte lines as well.
template <typename T>
__global__ __launch_bounds__(256) void dense_rows_k(const T* __restrict__ X, const T* __restrict__ W, int w_kmajor,
                                                    const T* __restrict__ bias, const float* __restrict__ rowbias,
                                                    T* __restrict__ Y, long long N, int K, int NO, int P, int nkt,
                                                    int nnt) {
    extern __shared__ uint32_t dsm[];
    T* wl = reinterpret_cast<T*>(dsm);
    const int ldw = K + 8;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int ldt = (K > NO ? K : NO) + 8;             // pitch of the per-wave tile buffer (elements)
    T* tl = wl + NO * ldw + wave * 32 * ldt;
    const long long ntiles = (N + 31) / 32;
    const long long gw = (long long)blockIdx.x * 4 + wave, nw = (long long)gridDim.x * 4;
    const int cpk = K / 8;                              // 16-byte chunks per input row
    const int nin = 32 * cpk;                           // chunks per input tile (<= 512)
    constexpr int LP = 8;                               // chunk loads per lane (K <= 128)
    Frag raw[LP];
    auto load_tile = [&](long long t) {                 // coalesced: chunk i*64+lane of the tile's byte range
        const T* base = X + t * 32 * K;
        const long long rows_left = N - t * 32;         // rows of this tile that exist
        const int valid = rows_left >= 32 ? nin : (int)rows_left * cpk;
#pragma unroll
        for (int i = 0; i < LP; ++i) {
            const int cidx = i * 64 + lane;
            raw[i] = cidx < valid ? *reinterpret_cast<const Frag*>(base + (long long)cidx * 8) : Frag{{0u, 0u, 0u, 0u}};
        }
    };
    if (gw < ntiles) load_tile(gw);                     // requested before the weights are staged
    if (!w_kmajor) {  // W[o][k]: 16-byte copies
        const int kv = K / 8;
        for (int idx = tid; idx < NO * kv; idx += 256) {
            const int n = idx / kv, k8 = (idx % kv) * 8;
            *reinterpret_cast<Frag*>(wl + n * ldw + k8) = *reinterpret_cast<const Frag*>(W + (long long)n * K + k8);
        }
    } else {  // W[k][o]: read along o, write transposed
        const int nv = NO / 4;
        for (int idx = tid; idx < K * nv; idx += 256) {
            const int k = idx / nv, n4 = (idx % nv) * 4;
            const ChanVec<T, 4> v = *reinterpret_cast<const ChanVec<T, 4>*>(W + (long long)k * NO + n4);
#pragma unroll
            for (int i = 0; i < 4; ++i) wl[(n4 + i) * ldw + k] = v.v[i];
        }
    }
    __syncthreads();
    const int cpr = NO / 8;  // 16-byte chunks per output row (NO % 8 == 0 on this path)
    for (long long tile = gw; tile < ntiles; tile += nw) {
        // raw chunks -> LDS [row][k] -> MFMA fragments (row l32, k = kt*16 + 8*half ..)
#pragma unroll
        for (int i = 0; i < LP; ++i) {
            const int cidx = i * 64 + lane;
            if (cidx < nin) *reinterpret_cast<Frag*>(tl + (cidx / cpk) * ldt + (cidx % cpk) * 8) = raw[i];
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS writes have landed
        Frag xf[kKT];
#pragma unroll
        for (int kt = 0; kt < kKT; ++kt) {
            if (kt < nkt && kt * 16 + 8 * half < K)
                xf[kt] = *reinterpret_cast<const Frag*>(tl + l32 * ldt + kt * 16 + 8 * half);
            else
                xf[kt] = Frag{{0u, 0u, 0u, 0u}};
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // fragments are in registers: the buffer may be overwritten
        if (tile + nw < ntiles) load_tile(tile + nw);  // next tile in flight during the MFMAs and the store
        const long long m = tile * 32 + l32;
        const float* rb = rowbias ? rowbias + (long long)((int)(m < N ? m : N - 1) / P) * NO : nullptr;
        for (int nt = 0; nt < nnt; ++nt) {
            f32x16 acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.f;
            const int n = nt * 32 + l32;
            const T* wr = wl + (n < NO ? n : 0) * ldw + 8 * half;
#pragma unroll
            for (int kt = 0; kt < kKT; ++kt)
                if (kt < nkt) {
                    Frag wf = Frag{{0u, 0u, 0u, 0u}};
                    if (n < NO && kt * 16 + 8 * half < K) wf = *reinterpret_cast<const Frag*>(wr + kt * 16);
                    acc = mfma32(wf, xf[kt], acc, T());
                }
            // lane owns row l32 of the tile and features n0..n0+3 of each accumulator group
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int n0 = nt * 32 + g4 * 8 + half * 4;
                if (n0 < NO) {
                    float o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[i] = acc[g4 * 4 + i];
                    if (bias) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) o[i] += to_f32(bias[n0 + i]);
                    }
                    if (rb) {
                        const float4 r4 = *reinterpret_cast<const float4*>(rb + n0);
                        o[0] += r4.x, o[1] += r4.y, o[2] += r4.z, o[3] += r4.w;
                    }
                    store_f32<T, 4>(tl + l32 * ldt + n0, o);
                }
            }
        }
        // coalesced copy-out of the 32 x NO tile (same wavefront wrote it: no workgroup barrier needed)
        __builtin_amdgcn_s_waitcnt(0xc07f);
        const int nchunk = 32 * cpr;
        for (int cidx = lane; cidx < nchunk; cidx += 64) {
            const int r = cidx / cpr, cc = (cidx % cpr) * 8;
            const long long row = tile * 32 + r;
            if (row < N) *reinterpret_cast<Frag*>(Y + row * NO + cc) = *reinterpret_cast<const Frag*>(tl + r * ldt + cc);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // copy-out reads done before the next tile overwrites the buffer
    }
}

// dW partials.  A workgroup of 4 wavefronts walks its contiguous range of 64-row stages: the stage's rows
// of A and B are copied to LDS with coalesced 16-byte loads (requested one stage ahead and held in
// registers while the current stage is multiplied), then wavefront w multiplies rows 16w..16w+15, reading
// the k-major MFMA fragments (8 consecutive rows of one feature) from LDS with 16-bit reads.
constexpr int kWgRows = 64;

template <typename T, int MT, int NT>
__global__ __launch_bounds__(256, 2) void dense_wgrad_k(const T* __restrict__ A, const T* __restrict__ Bm,
                                                        float* __restrict__ part, long long N, int M, int NO,
                                                        int stages_per_block) {
    extern __shared__ uint32_t dsm[];
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
    const long long st0 = (long long)blockIdx.x * stages_per_block;
    long long st1 = st0 + stages_per_block;
    if (st1 > nstages) st1 = nstages;

    auto fetch = [&](long long st) {
        const long long r0 = st * kWgRows;
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
            if (idx < nva) *reinterpret_cast<Frag*>(la + (idx / va) * lda + (idx % va) * 8) = pa[p];
        }
#pragma unroll
        for (int p = 0; p < PB; ++p) {
            const int idx = tid + p * 256;
            if (idx < nvb) *reinterpret_cast<Frag*>(lb + (idx / vb) * ldb + (idx % vb) * 8) = pb[p];
        }
    };

    if (st0 < st1) {
        fetch(st0);
        commit(0);
    }
    __syncthreads();
    for (long long st = st0; st < st1; ++st) {
        const int buf = (int)((st - st0) & 1);
        if (st + 1 < st1) fetch(st + 1);  // in flight while this stage is multiplied
        const T* la = lds + buf * buf_elems + (wave * 16 + 8 * half) * lda;
        const T* lb = lds + buf * buf_elems + kWgRows * lda + (wave * 16 + 8 * half) * ldb;
        Frag af[MT], bf[NT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = min(t * 32 + l32, M - 1);
            const bool ok = t * 32 + l32 < M;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = ld16(la + (2 * j) * lda + m), hi = ld16(la + (2 * j + 1) * lda + m);
                af[t].v[j] = ok ? (lo | (hi << 16)) : 0u;
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int n = min(t * 32 + l32, NO - 1);
            const bool ok = t * 32 + l32 < NO;
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
        if (st + 1 < st1) commit(buf ^ 1);
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
            for (int idx = threadIdx.x; idx < 16 * 64; idx += 256) {
                const int i = idx >> 6, l = idx & 63;
                const float sum = (red[idx] + red[1024 + idx]) + (red[2048 + idx] + red[3072 + idx]);
                const int m = mt * 32 + 8 * (i / 4) + 4 * (l >> 5) + (i % 4), n = nt * 32 + (l & 31);
                if (m < M && n < NO) pout[(long long)m * NO + n] = sum;
            }
        }
}

static bool dense_dims_ok(int K, int NO, int dtype) {
    return dtype != kF32 && K >= 8 && K <= 16 * kKT && K % 8 == 0 && NO >= 8 && NO <= 32 * kNT && NO % 8 == 0;
}

int dense_rows_supported(int K, int NO, int dtype) { return dense_dims_ok(K, NO, dtype) ? 1 : 0; }

int dense_rows_launch(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                      long long N, int K, int NO, int P, int dtype, hipStream_t s) {
    if (!dense_dims_ok(K, NO, dtype)) return -1;
    if (N == 0) return 0;
    if (N > 0x7fffffffLL) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 15) ||
        (reinterpret_cast<uintptr_t>(rowbias) & 15))
        return -1;
    const int nkt = cdiv(K, 16), nnt = cdiv(NO, 32);
    const long long ntiles = (N + 31) / 32;
    long long blocks = (ntiles + 7) / 8;  // about two row tiles per wavefront
    const int cap = getenv("PDW_DENSE_BLOCKS") ? atoi(getenv("PDW_DENSE_BLOCKS")) : 512;
    if (blocks > cap) blocks = cap;  // persistent workgroups: the weights are staged to LDS once each
    if (blocks < 1) blocks = 1;
    const size_t lds = ((size_t)NO * (K + 8) + 4 * 32 * ((K > NO ? K : NO) + 8)) * 2;
    if (dtype == kF16)
        hipLaunchKernelGGL((dense_rows_k<f16_t>), dim3((unsigned)blocks), dim3(256), lds, s, (const f16_t*)x,
                           (const f16_t*)w, w_kmajor, (const f16_t*)bias, rowbias, (f16_t*)y, N, K, NO, P > 0 ? P : 1,
                           nkt, nnt);
    else
        hipLaunchKernelGGL((dense_rows_k<bf16_t>), dim3((unsigned)blocks), dim3(256), lds, s, (const bf16_t*)x,
                           (const bf16_t*)w, w_kmajor, (const bf16_t*)bias, rowbias, (bf16_t*)y, N, K, NO,
                           P > 0 ? P : 1, nkt, nnt);
    return check_launch("dense_rows");
}

static void dense_wgrad_plan(long long N, int* blocks, int* stages_per_block) {
    const long long nstages = (N + kWgRows - 1) / kWgRows;
    long long nb = getenv("PDW_DWG_BLOCKS") ? atoi(getenv("PDW_DWG_BLOCKS")) : 256;
    if (nb > nstages) nb = nstages;
    if (nb < 1) nb = 1;
    const long long spb = (nstages + nb - 1) / nb;
    *stages_per_block = (int)(spb < 1 ? 1 : spb);
    *blocks = (int)((nstages + *stages_per_block - 1) / *stages_per_block);
    if (*blocks < 1) *blocks = 1;
}

int dense_wgrad_supported(int M, int NO, int dtype) {
    const int mt = cdiv(M, 32), nt = cdiv(NO, 32);
    return (dtype != kF32 && M >= 8 && NO >= 8 && M % 8 == 0 && NO % 8 == 0 && mt <= 4 && nt <= 4 && mt * nt <= 8) ? 1
                                                                                                                  : 0;
}

size_t dense_wgrad_workspace(long long N, int M, int NO) {
    int blocks, spb;
    dense_wgrad_plan(N, &blocks, &spb);
    return (size_t)blocks * M * NO * sizeof(float);
}

template <typename T, int MT, int NT>
static int dense_wgrad_go(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, hipStream_t s) {
    int blocks, spb;
    dense_wgrad_plan(N, &blocks, &spb);
    size_t lds = (size_t)2 * kWgRows * (M + 8 + NO + 8) * 2;
    if (lds < 4 * 16 * 64 * sizeof(float)) lds = 4 * 16 * 64 * sizeof(float);
    hipLaunchKernelGGL((dense_wgrad_k<T, MT, NT>), dim3(blocks), dim3(256), lds, s, (const T*)a, (const T*)b,
                       (float*)ws, N, M, NO, spb);
    if (int e = check_launch("dense_wgrad")) return e;
    return wgrad_reduce_launch<T>((const float*)ws, dw, blocks, M * NO, s);
}

template <typename T>
static int dense_wgrad_t(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, hipStream_t s) {
    const int mt = cdiv(M, 32), nt = cdiv(NO, 32);
#define PDW_CASE(MT, NT) \
    if (mt == MT && nt == NT) return dense_wgrad_go<T, MT, NT>(a, b, dw, ws, N, M, NO, s);
    PDW_CASE(1, 1) PDW_CASE(1, 2) PDW_CASE(2, 1) PDW_CASE(2, 2) PDW_CASE(1, 3) PDW_CASE(3, 1) PDW_CASE(2, 3)
    PDW_CASE(3, 2) PDW_CASE(1, 4) PDW_CASE(4, 1) PDW_CASE(2, 4) PDW_CASE(4, 2)
#undef PDW_CASE
    return -1;
}

int dense_wgrad_launch(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, int dtype,
                       hipStream_t s) {
    if (!dense_wgrad_supported(M, NO, dtype)) return -1;
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15)) return -1;
    if (dtype == kF16) return dense_wgrad_t<f16_t>(a, b, dw, ws, N, M, NO, s);
    return dense_wgrad_t<bf16_t>(a, b, dw, ws, N, M, NO, s);
}

}  // namespace pdw
