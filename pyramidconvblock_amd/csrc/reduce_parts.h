// Fixed-order summation of fp32 partial results (the last step of every weight gradient), as a device function
// that other kernels can run in spare workgroups, and the table of several such summations for one launch.
#pragma once
#include "common.h"

namespace pdw {

// Pass 2 of wgrad (shared with the tiled kernels): dw[e] = sum over parts in a fixed order.
// Block = 32 outputs x 8 part lanes; lane q adds parts q, q+8, ... and the 8 lanes are combined
// through LDS, so the reads of one part are contiguous and many parts are in flight.
template <typename T>
__device__ __forceinline__ void reduce_parts_block(const float* __restrict__ part, T* __restrict__ dw, int nparts, int n,
                                                   int blk, float (*red)[32]) {
    const int el = threadIdx.x & 31, q = threadIdx.x >> 5;
    const int e = blk * 32 + el;
    float s0 = 0.f, s1 = 0.f;
    if (e < n) {
        int p = q;
        for (; p + 56 < nparts; p += 64) {  // eight loads in flight per lane: the pass is pure latency
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(long long)(p + 8 * u) * n + e];
            s0 += (v[0] + v[2]) + (v[4] + v[6]);
            s1 += (v[1] + v[3]) + (v[5] + v[7]);
        }
        for (; p + 8 < nparts; p += 16) {
            s0 += part[(long long)p * n + e];
            s1 += part[(long long)(p + 8) * n + e];
        }
        if (p < nparts) s0 += part[(long long)p * n + e];
    }
    red[q][el] = s0 + s1;
    __syncthreads();
    if (q == 0 && e < n) {
        const float s = ((red[0][el] + red[1][el]) + (red[2][el] + red[3][el])) +
                        ((red[4][el] + red[5][el]) + (red[6][el] + red[7][el]));
        dw[e] = from_f32<T>(s);
    }
}

// Several such reductions in one launch: the weight gradients of a backward pass are each a few microseconds of
// latency, and nothing reads them before the pass is over.
constexpr int kMaxReduceJobs = 8;
struct ReduceJobs {
    const float* part[kMaxReduceJobs];
    void* out[kMaxReduceJobs];
    int nparts[kMaxReduceJobs], n[kMaxReduceJobs], dtype[kMaxReduceJobs];
    int first_block[kMaxReduceJobs + 1];
    int njobs;
};

// Workgroup `wg` (of 256 threads) of the table's grid; red: 8 x 32 floats of LDS.
__device__ __forceinline__ void reduce_jobs_block(const ReduceJobs& jobs, int wg, float (*red)[32]) {
    int j = 0;
    while (j + 1 < jobs.njobs && wg >= jobs.first_block[j + 1]) ++j;  // uniform: scalar ALU
    const int blk = wg - jobs.first_block[j];
    switch (jobs.dtype[j]) {
        case kF32: reduce_parts_block<float>(jobs.part[j], (float*)jobs.out[j], jobs.nparts[j], jobs.n[j], blk, red); break;
        case kF16: reduce_parts_block<f16_t>(jobs.part[j], (f16_t*)jobs.out[j], jobs.nparts[j], jobs.n[j], blk, red); break;
        default: reduce_parts_block<bf16_t>(jobs.part[j], (bf16_t*)jobs.out[j], jobs.nparts[j], jobs.n[j], blk, red); break;
    }
}

}  // namespace pdw
