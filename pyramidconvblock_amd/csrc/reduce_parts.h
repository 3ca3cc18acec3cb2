// Fixed-order summation of fp32 partial results (the last step of every weight gradient), as a device function
// that other kernels can run in spare workgroups, and the table of several such summations for one launch.
#pragma once
#include "common.h"

namespace pdw {

// Pass 2 of wgrad (shared with the tiled kernels): dw[e] = sum over parts in a fixed order.
// Block = EL output lanes x QL part lanes (EL * QL = 256); an output lane owns V consecutive outputs (V = 4:
// 16-byte loads), part lane q adds parts q, q + QL, ... with up to sixteen loads in flight, and the QL lanes are
// combined through LDS, so the reads of one part are contiguous and many parts are in flight.  The pass is pure
// latency.  QL = 8 keeps the workgroups few (they ride in other kernels' grids, where resident slots are scarce);
// QL = 32 takes 256 parts in one round of loads, for the stand-alone launch.  V = 4 needs n % 4 == 0 and 16-byte
// aligned partials (reduce_vec_ok).  The order of the additions, and so the result, depends on QL.
constexpr int kReduceVec = 4;
constexpr int kReduceLds = 8 * 32 * kReduceVec;  // floats of LDS a workgroup needs

template <typename T, int V, int QL>
__device__ __forceinline__ void reduce_parts_block(const float* __restrict__ part, T* __restrict__ dw, int nparts, int n,
                                                   int blk, float* red) {
    constexpr int EL = 256 / QL, ROW = EL * V;  // red[QL][ROW]
    const int el = threadIdx.x % EL, q = threadIdx.x / EL;
    const int e = (blk * EL + el) * V;
    float s0[V], s1[V];
#pragma unroll
    for (int i = 0; i < V; ++i) s0[i] = 0.f, s1[i] = 0.f;
    auto ld = [&](int p, float (&v)[V]) {
        if constexpr (V == 4) {
            const float4 t = *reinterpret_cast<const float4*>(part + (long long)p * n + e);
            v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
        } else {
            v[0] = part[(long long)p * n + e];
        }
    };
    if (e < n) {
        int p = q;
        for (; p + 15 * QL < nparts; p += 16 * QL) {  // sixteen loads in flight per lane
            float v[16][V];
#pragma unroll
            for (int u = 0; u < 16; ++u) ld(p + QL * u, v[u]);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                s0[i] += ((v[0][i] + v[2][i]) + (v[4][i] + v[6][i])) + ((v[8][i] + v[10][i]) + (v[12][i] + v[14][i]));
                s1[i] += ((v[1][i] + v[3][i]) + (v[5][i] + v[7][i])) + ((v[9][i] + v[11][i]) + (v[13][i] + v[15][i]));
            }
        }
        for (; p + 7 * QL < nparts; p += 8 * QL) {
            float v[8][V];
#pragma unroll
            for (int u = 0; u < 8; ++u) ld(p + QL * u, v[u]);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                s0[i] += (v[0][i] + v[2][i]) + (v[4][i] + v[6][i]);
                s1[i] += (v[1][i] + v[3][i]) + (v[5][i] + v[7][i]);
            }
        }
        for (; p + QL < nparts; p += 2 * QL) {
            float a[V], b[V];
            ld(p, a), ld(p + QL, b);
#pragma unroll
            for (int i = 0; i < V; ++i) s0[i] += a[i], s1[i] += b[i];
        }
        if (p < nparts) {
            float a[V];
            ld(p, a);
#pragma unroll
            for (int i = 0; i < V; ++i) s0[i] += a[i];
        }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) red[q * ROW + el * V + i] = s0[i] + s1[i];
    __syncthreads();
    if constexpr (QL == 32) {  // 32 rows -> 8, by the threads of the first 8 part lanes
        if (q < 8) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const int c = el * V + i;
                red[q * ROW + c] = (red[q * ROW + c] + red[(q + 8) * ROW + c]) +
                                   (red[(q + 16) * ROW + c] + red[(q + 24) * ROW + c]);
            }
        }
        __syncthreads();
    }
    if (q == 0 && e < n) {
        float o[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const int c = el * V + i;
            o[i] = ((red[c] + red[ROW + c]) + (red[2 * ROW + c] + red[3 * ROW + c])) +
                   ((red[4 * ROW + c] + red[5 * ROW + c]) + (red[6 * ROW + c] + red[7 * ROW + c]));
        }
        store_f32<T, V>(dw + e, o);
    }
}

// Whether the 4-wide form applies to a summation.
inline bool reduce_vec_ok(const float* part, const void* dw, int n, int esize) {
    return n % kReduceVec == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(dw) & (size_t)(kReduceVec * esize - 1)) == 0;
}

// Outputs one workgroup covers, for `vec` outputs per lane and `ql` part lanes.
inline int reduce_block_outputs(int vec, int ql) { return 256 / ql * vec; }

template <typename T>
__device__ __forceinline__ void reduce_parts_any(const float* part, T* dw, int nparts, int n, int blk, int vec, int ql,
                                                 float* red) {
    if (vec == kReduceVec) {
        if (ql == 32) reduce_parts_block<T, kReduceVec, 32>(part, dw, nparts, n, blk, red);
        else reduce_parts_block<T, kReduceVec, 8>(part, dw, nparts, n, blk, red);
    } else {
        if (ql == 32) reduce_parts_block<T, 1, 32>(part, dw, nparts, n, blk, red);
        else reduce_parts_block<T, 1, 8>(part, dw, nparts, n, blk, red);
    }
}

// out[o * D + d] = sum over b < B of g[b * D + o] * m[b * D + d]: the weight gradient of a small dense layer
// applied to one row per image (g: fp32 output gradients, m: its inputs), 1024 outputs per workgroup of 256
// threads, D % 4 == 0.  The same kind of deferred work as the sums of partials: nothing needs it before the
// backward pass is over.
constexpr int kOuterBlock = 1024;

template <typename T>
__device__ __forceinline__ void outer_sum_block(const float* __restrict__ g, const T* __restrict__ m,
                                                T* __restrict__ out, int B, int D, int blk, int tid) {
    const int e = (blk * 256 + tid) * 4;
    if (e >= D * D) return;
    const int o = e / D, d = e - o * D;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    int b = 0;
    for (; b + 8 <= B; b += 8) {  // sixteen loads in flight
        float gv[8], mv[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            gv[u] = g[(long long)(b + u) * D + o];
            load_f32<T, 4>(m + (long long)(b + u) * D + d, mv[u]);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = fmaf(gv[u], mv[u][i], acc[i]);
    }
    for (; b < B; ++b) {
        float mv[4];
        const float gv = g[(long long)b * D + o];
        load_f32<T, 4>(m + (long long)b * D + d, mv);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(gv, mv[i], acc[i]);
    }
    store_f32<T, 4>(out + e, acc);
}

// Several such reductions in one launch: the weight gradients of a backward pass are each a few microseconds of
// latency, and nothing reads them before the pass is over.
constexpr int kMaxReduceJobs = 8;
struct ReduceJobs {
    const float* part[kMaxReduceJobs];
    void* out[kMaxReduceJobs];
    const void* aux[kMaxReduceJobs];  // outer products: the second factor (element type of `out`)
    int nparts[kMaxReduceJobs], n[kMaxReduceJobs], dtype[kMaxReduceJobs];
    int vec[kMaxReduceJobs];  // outputs per lane: kReduceVec or 1; 0 = outer product (n = D * D, nparts = B)
    int ql[kMaxReduceJobs];   // part lanes: 8 or 32
    int dim[kMaxReduceJobs];  // outer products: D
    int first_block[kMaxReduceJobs + 1];
    int njobs;
};

// Workgroup `wg` (of 256 threads) of the table's grid; red: kReduceLds floats of LDS.
__device__ __forceinline__ void reduce_jobs_block(const ReduceJobs& jobs, int wg, float* red) {
    int j = 0;
    while (j + 1 < jobs.njobs && wg >= jobs.first_block[j + 1]) ++j;  // uniform: scalar ALU
    const int blk = wg - jobs.first_block[j];
    const float* part = jobs.part[j];
    const int nparts = jobs.nparts[j], n = jobs.n[j], vec = jobs.vec[j], ql = jobs.ql[j];
    if (vec == 0) {  // outer product; fp32 outputs are not produced this way
        if (jobs.dtype[j] == kF16)
            outer_sum_block<f16_t>(part, (const f16_t*)jobs.aux[j], (f16_t*)jobs.out[j], nparts, jobs.dim[j], blk, threadIdx.x);
        else
            outer_sum_block<bf16_t>(part, (const bf16_t*)jobs.aux[j], (bf16_t*)jobs.out[j], nparts, jobs.dim[j], blk, threadIdx.x);
        return;
    }
    switch (jobs.dtype[j]) {
        case kF32: reduce_parts_any<float>(part, (float*)jobs.out[j], nparts, n, blk, vec, ql, red); break;
        case kF16: reduce_parts_any<f16_t>(part, (f16_t*)jobs.out[j], nparts, n, blk, vec, ql, red); break;
        default: reduce_parts_any<bf16_t>(part, (bf16_t*)jobs.out[j], nparts, n, blk, vec, ql, red); break;
    }
}

}  // namespace pdw
