// The forward of a block's global-mean branch (conv_block.py:46-49: mean over the positions -> conv_pool -> one row per
// image that is added to every output row) as a workgroup body, so that it can ride in the grid of whichever large
// launch runs at that point of the dataflow.
#pragma once
#include "common.h"

namespace pdw {

struct PoolFwdJob {
    const float* part;
    int nchunks, B, D;
    float inv_p;
    const void *wp, *bp, *bo;
    void* m;
    float* rowbias;
};

// sm[c] = sum over q < nchunks of pp[q * D + c] for c < D, by the whole workgroup of 256: thread = (4-column vector
// tid % 32, chunk lane tid / 32), up to 8 loads of a thread in flight, the 8 chunk lanes combined through
// red[8][D].  D % 4 == 0, D <= 128.  Ends with a barrier; the order of the additions is fixed.  In a larger workgroup
// the threads from 256 on only join the barriers.
__device__ __forceinline__ void colsum_coop(const float* __restrict__ pp, int nchunks, int D, float* sm, float* red) {
    const int tid = threadIdx.x, cv = tid & 31, ql = tid >> 5;
    float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0;
    if (tid < 256 && cv * 4 < D) {
        const float* p = pp + cv * 4;
        int q = ql;
        for (; q + 56 < nchunks; q += 64) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4*>(p + (long long)(q + 8 * u) * D);
#pragma unroll
            for (int u = 0; u < 8; u += 2) {
                a0.x += v[u].x, a0.y += v[u].y, a0.z += v[u].z, a0.w += v[u].w;
                a1.x += v[u + 1].x, a1.y += v[u + 1].y, a1.z += v[u + 1].z, a1.w += v[u + 1].w;
            }
        }
        for (; q < nchunks; q += 8) {
            const float4 v = *reinterpret_cast<const float4*>(p + (long long)q * D);
            a0.x += v.x, a0.y += v.y, a0.z += v.z, a0.w += v.w;
        }
        *reinterpret_cast<float4*>(red + ql * D + cv * 4) =
            make_float4(a0.x + a1.x, a0.y + a1.y, a0.z + a1.z, a0.w + a1.w);
    }
    __syncthreads();
    if (tid < D) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) t += red[k * D + tid];
        sm[tid] = t;
    }
    __syncthreads();
}

template <typename T>
__device__ __forceinline__ void pool_branch_fwd_v8_body(const float* __restrict__ part, int nchunks, int D,
                                                        float inv_p, const T* __restrict__ wp,
                                                        const T* __restrict__ bp, const T* __restrict__ bo,
                                                        T* __restrict__ m, float* __restrict__ rowbias, int b,
                                                        float* sm) {  // sm: [D] means, [8][D] partial column sums
    const int tid = threadIdx.x;   // (a workgroup of 256, or a larger one whose other threads only join the barriers)
    // weight rows of this thread: outputs o = tid/8 + 32*pass, channel vectors sub + 8*i  (requested first)
    const int sub = tid & 7, ol = tid >> 3;
    ChanVec<T, 8> wv[4][2];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int o = ol + 32 * pass, v = sub + 8 * i;
            const bool ok = tid < 256 && o < D && v * 8 < D;
            wv[pass][i] = *reinterpret_cast<const ChanVec<T, 8>*>(wp + (ok ? (long long)o * D + v * 8 : 0));
        }
    // the biases of this thread's outputs, requested here as well: read where they are added, after the last
    // barrier, they would be eight dependent trips to memory at the end of the workgroup
    // (unconditional loads from a readable address, converted where they are used: no branch, no early wait)
    const T* bpp = bp ? bp : wp;
    const T* bop = bo ? bo : wp;
    T braw[4][2];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int oc = min(ol + 32 * pass, D - 1);
        braw[pass][0] = bpp[oc], braw[pass][1] = bop[oc];
    }
    colsum_coop(part + (long long)b * nchunks * D, nchunks, D, sm, sm + D);
    if (tid < D) {
        const T mv = from_f32<T>(sm[tid] * inv_p);
        m[(long long)b * D + tid] = mv;
        sm[tid] = to_f32(mv);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int o = ol + 32 * pass;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int v = sub + 8 * i;
            if (o < D && v * 8 < D) {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc = fmaf(sm[v * 8 + j], to_f32(wv[pass][i].v[j]), acc);
            }
        }
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
        acc += __shfl_xor(acc, 4);
        acc += (bp ? to_f32(braw[pass][0]) : 0.f) + (bo ? to_f32(braw[pass][1]) : 0.f);
        if (sub == 0 && o < D && tid < 256) rowbias[(long long)b * D + o] = acc;
    }
}

// Whether the 8-channel-vector bodies of the mean branch cover the case (host side).
inline bool pool_branch_v8_ok(const void* wp, const void* m_or_null, const float* parts, int B, int D, int dtype) {
    return dtype != kF32 && D % 8 == 0 && D <= 128 && (reinterpret_cast<uintptr_t>(wp) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(m_or_null) & 15) == 0 && (reinterpret_cast<uintptr_t>(parts) & 15) == 0 &&
           (size_t)(B + 16 * D) * sizeof(float) <= 64 * 1024;
}

}  // namespace pdw
