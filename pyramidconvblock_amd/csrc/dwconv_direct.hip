// General-parameter depthwise convolution kernels (any stride / padding / dilation /
// kernel extent).  They read straight from global memory, so they are the slow but
// fully general member of the family; the LDS-tiled kernels take over for stride 1,
// dilation 1.  One thread owns VEC consecutive channels of one pixel, so a wavefront's
// loads of one tap are one contiguous run of channels-last memory.
#include "common.h"
#include "kernels.h"
#include "reduce_parts.h"

namespace pdw {

struct ConvGeom {
    int B, H, W, C, OH, OW, KH, KW, SH, SW, PH, PW, DH, DW;
};

template <typename T, int VEC>
__global__ __launch_bounds__(256) void dwconv_fwd_direct(const T* __restrict__ x, const T* __restrict__ w,
                                                         T* __restrict__ y, ConvGeom g, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = g.C / VEC;
    const int c = (int)(idx % CV) * VEC;
    long long t = idx / CV;
    const int j = (int)(t % g.OW);
    t /= g.OW;
    const int i = (int)(t % g.OH);
    const int b = (int)(t / g.OH);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    const T* xb = x + (long long)b * g.H * g.W * g.C;
    for (int kh = 0; kh < g.KH; ++kh) {
        const int ih = i * g.SH - g.PH + kh * g.DH;
        if (ih < 0 || ih >= g.H) continue;
        for (int kw = 0; kw < g.KW; ++kw) {
            const int iw = j * g.SW - g.PW + kw * g.DW;
            if (iw < 0 || iw >= g.W) continue;
            float xv[VEC], wv[VEC];
            load_f32<T, VEC>(xb + ((long long)ih * g.W + iw) * g.C + c, xv);
            load_f32<T, VEC>(w + ((long long)kh * g.KW + kw) * g.C + c, wv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = fmaf(xv[v], wv[v], acc[v]);
        }
    }
    store_f32<T, VEC>(y + (((long long)b * g.OH + i) * g.OW + j) * g.C + c, acc);
}

// dx[b,ih,iw,c] = sum over taps with (ih + PH - kh*DH) divisible by SH of gy[b,(..)/SH,..,c] * w[kh,kw,c]
template <typename T, int VEC>
__global__ __launch_bounds__(256) void dwconv_dgrad_direct(const T* __restrict__ gy, const T* __restrict__ w,
                                                           T* __restrict__ dx, ConvGeom g, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = g.C / VEC;
    const int c = (int)(idx % CV) * VEC;
    long long t = idx / CV;
    const int iw = (int)(t % g.W);
    t /= g.W;
    const int ih = (int)(t % g.H);
    const int b = (int)(t / g.H);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    const T* gb = gy + (long long)b * g.OH * g.OW * g.C;
    for (int kh = 0; kh < g.KH; ++kh) {
        const int ni = ih + g.PH - kh * g.DH;
        if (ni < 0 || ni % g.SH) continue;
        const int i = ni / g.SH;
        if (i >= g.OH) continue;
        for (int kw = 0; kw < g.KW; ++kw) {
            const int nj = iw + g.PW - kw * g.DW;
            if (nj < 0 || nj % g.SW) continue;
            const int j = nj / g.SW;
            if (j >= g.OW) continue;
            float gv[VEC], wv[VEC];
            load_f32<T, VEC>(gb + ((long long)i * g.OW + j) * g.C + c, gv);
            load_f32<T, VEC>(w + ((long long)kh * g.KW + kw) * g.C + c, wv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = fmaf(gv[v], wv[v], acc[v]);
        }
    }
    store_f32<T, VEC>(dx + (((long long)b * g.H + ih) * g.W + iw) * g.C + c, acc);
}

// Pass 1 of wgrad: block (tap, channel slice of 64, chunk) sums gy*x over its chunk of the
// B*OH*OW output positions; 4 position lanes per channel are combined through LDS and the
// block writes part[chunk][tap][c] (fp32).
template <typename T>
__global__ __launch_bounds__(256) void dwconv_wgrad_direct(const T* __restrict__ x, const T* __restrict__ gy,
                                                           float* __restrict__ part, ConvGeom g, int chunk_len) {
    __shared__ float red[4][64];
    const int tap = blockIdx.x;
    const int kh = tap / g.KW, kw = tap % g.KW;
    const int lane_c = threadIdx.x & 63, lane_p = threadIdx.x >> 6;
    const int c = blockIdx.y * 64 + lane_c;
    const long long npos = (long long)g.B * g.OH * g.OW;
    const long long p0 = (long long)blockIdx.z * chunk_len;
    long long p1 = p0 + chunk_len;
    if (p1 > npos) p1 = npos;
    float acc = 0.f;
    if (c < g.C) {
        for (long long p = p0 + lane_p; p < p1; p += 4) {
            const int j = (int)(p % g.OW);
            const long long t = p / g.OW;
            const int i = (int)(t % g.OH);
            const int b = (int)(t / g.OH);
            const int ih = i * g.SH - g.PH + kh * g.DH;
            const int iw = j * g.SW - g.PW + kw * g.DW;
            if (ih < 0 || ih >= g.H || iw < 0 || iw >= g.W) continue;
            const float gv = to_f32(gy[p * g.C + c]);
            const float xv = to_f32(x[(((long long)b * g.H + ih) * g.W + iw) * g.C + c]);
            acc = fmaf(gv, xv, acc);
        }
    }
    red[lane_p][lane_c] = acc;
    __syncthreads();
    if (lane_p == 0 && c < g.C) {
        const float s = (red[0][lane_c] + red[1][lane_c]) + (red[2][lane_c] + red[3][lane_c]);
        part[((long long)blockIdx.z * gridDim.x + tap) * g.C + c] = s;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void wgrad_reduce_parts(const float* __restrict__ part, T* __restrict__ dw,
                                                          int nparts, int n, int vec, int ql) {
    __shared__ float red[kReduceLds];
    reduce_parts_any<T>(part, dw, nparts, n, blockIdx.x, vec, ql, red);
}

__global__ __launch_bounds__(256) void wgrad_reduce_many(const ReduceJobs jobs) {
    __shared__ float red[kReduceLds];
    reduce_jobs_block(jobs, blockIdx.x, red);
}

// Deferred mode (per host thread): between reduce_defer_begin and reduce_defer_flush the reductions are only
// recorded; the flush runs them all in one launch.
static thread_local bool t_defer = false;
static thread_local ReduceJobs t_jobs;

// Part lanes of a stand-alone summation: 32 when 8 would need more than one round of loads.
static int standalone_part_lanes(int nparts) { return nparts > 128 ? 32 : 8; }

// A launch of its own has the whole chip's slots: the jobs that were laid out for riding (few workgroups, 8 part
// lanes) are laid out again with as many part lanes as make their loads a single round.
int reduce_jobs_launch(const ReduceJobs& recorded, hipStream_t s) {
    if (recorded.njobs == 0) return 0;
    ReduceJobs jobs = recorded;
    for (int j = 0; j < jobs.njobs; ++j) {
        int nb = recorded.first_block[j + 1] - recorded.first_block[j];
        if (recorded.vec[j] != 0) {
            jobs.ql[j] = standalone_part_lanes(jobs.nparts[j]);
            nb = cdiv(jobs.n[j], reduce_block_outputs(jobs.vec[j], jobs.ql[j]));
        }
        jobs.first_block[j + 1] = jobs.first_block[j] + nb;
    }
    hipLaunchKernelGGL(wgrad_reduce_many, dim3(jobs.first_block[jobs.njobs]), dim3(256), 0, s, jobs);
    return check_launch("wgrad_reduce_many");
}

int reduce_defer_begin() {
    if (t_defer) return set_error("pdw_reduce_defer_begin: already deferring on this thread"), 1;
    t_defer = true;
    t_jobs.njobs = 0;
    t_jobs.first_block[0] = 0;
    return 0;
}

int reduce_defer_flush(hipStream_t s) {
    if (!t_defer) return set_error("pdw_reduce_defer_flush: pdw_reduce_defer_begin was not called"), 1;
    t_defer = false;
    if (t_jobs.njobs == 0) return 0;
    const int r = reduce_jobs_launch(t_jobs, s);
    t_jobs.njobs = 0;
    return r;
}

bool reduce_deferring() { return t_defer; }

int reduce_defer_room() { return t_defer ? kMaxReduceJobs - t_jobs.njobs : 0; }

// Records out[o * D + d] = sum_b g[b * D + o] * m[b * D + d] (see outer_sum_block); only while deferring.
int reduce_defer_outer(const float* g, const void* m, void* out, int B, int D, int dtype) {
    if (reduce_defer_room() < 1 || dtype == kF32 || D % 4 != 0) return -1;
    const int j = t_jobs.njobs++;
    t_jobs.part[j] = g, t_jobs.aux[j] = m, t_jobs.out[j] = out, t_jobs.nparts[j] = B, t_jobs.n[j] = D * D;
    t_jobs.dtype[j] = dtype, t_jobs.vec[j] = 0, t_jobs.ql[j] = 8, t_jobs.dim[j] = D;
    t_jobs.first_block[j + 1] = t_jobs.first_block[j] + cdiv((long long)D * D, kOuterBlock);
    return 0;
}

// Hands the recorded jobs to a caller that runs them inside another kernel's grid; the later flush then finds
// nothing left to do.  Returns the number of jobs.
int reduce_defer_take(ReduceJobs* out) {
    if (!t_defer || t_jobs.njobs == 0) return 0;
    *out = t_jobs;
    const int n = t_jobs.njobs;
    t_jobs.njobs = 0;
    t_jobs.first_block[0] = 0;
    return n;
}

template <typename T>
static constexpr int dtype_of() {
    return sizeof(T) == 4 ? kF32 : (__is_same(T, f16_t) ? kF16 : kBF16);
}

static ConvGeom make_geom(int B, int H, int W, int C, int KH, int KW, int SH, int SW, int PH, int PW, int DH,
                          int DW) {
    ConvGeom g{B, H, W, C, conv_out_size(H, KH, SH, PH, DH), conv_out_size(W, KW, SW, PW, DW), KH, KW, SH, SW, PH, PW, DH, DW};
    return g;
}

template <typename T>
static int fwd_direct_t(const void* x, const void* w, void* y, const ConvGeom& g, hipStream_t s, bool dgrad) {
    const void* ptrs[3] = {x, w, y};
    const int vec = pick_vec(g.C, sizeof(T), ptrs, 3);
    const long long npix = dgrad ? (long long)g.B * g.H * g.W : (long long)g.B * g.OH * g.OW;
    const long long total = npix * (g.C / vec);
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)((total + 255) / 256);
#define PDW_LAUNCH(V)                                                                                              \
    if (dgrad)                                                                                                     \
        hipLaunchKernelGGL((dwconv_dgrad_direct<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (const T*)w,  \
                           (T*)y, g, total);                                                                       \
    else                                                                                                           \
        hipLaunchKernelGGL((dwconv_fwd_direct<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (const T*)w,    \
                           (T*)y, g, total);
    switch (vec) {
        case 8: if constexpr (sizeof(T) == 2) { PDW_LAUNCH(8) } break;
        case 4: PDW_LAUNCH(4) break;
        case 2: PDW_LAUNCH(2) break;
        default: PDW_LAUNCH(1) break;
    }
#undef PDW_LAUNCH
    return check_launch(dgrad ? "dwconv_dgrad_direct" : "dwconv_fwd_direct");
}

int dwconv_fwd_direct_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW,
                             int SH, int SW, int PH, int PW, int DH, int DW, int dtype, hipStream_t s) {
    const ConvGeom g = make_geom(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW);
    switch (dtype) {
        case kF32: return fwd_direct_t<float>(x, w, y, g, s, false);
        case kF16: return fwd_direct_t<f16_t>(x, w, y, g, s, false);
        default: return fwd_direct_t<bf16_t>(x, w, y, g, s, false);
    }
}

int dwconv_dgrad_direct_launch(const void* gy, const void* w, void* dx, int B, int H, int W, int C, int KH, int KW,
                               int SH, int SW, int PH, int PW, int DH, int DW, int dtype, hipStream_t s) {
    const ConvGeom g = make_geom(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW);
    switch (dtype) {
        case kF32: return fwd_direct_t<float>(gy, w, dx, g, s, true);
        case kF16: return fwd_direct_t<f16_t>(gy, w, dx, g, s, true);
        default: return fwd_direct_t<bf16_t>(gy, w, dx, g, s, true);
    }
}

static void wgrad_direct_plan(const ConvGeom& g, int* nchunks, int* chunk_len) {
    const long long npos = (long long)g.B * g.OH * g.OW;
    long long n = (npos + 1023) / 1024;  // >= 1024 positions per chunk
    if (n > 64) n = 64;
    if (n < 1) n = 1;
    *nchunks = (int)n;
    *chunk_len = (int)((npos + n - 1) / n);
}

size_t dwconv_wgrad_direct_workspace(int B, int H, int W, int C, int KH, int KW, int SH, int SW, int PH, int PW,
                                     int DH, int DW) {
    const ConvGeom g = make_geom(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW);
    int nchunks, chunk_len;
    wgrad_direct_plan(g, &nchunks, &chunk_len);
    return (size_t)nchunks * KH * KW * C * sizeof(float);
}

template <typename T>
int wgrad_reduce_launch(const float* part, void* dw, int nparts, int n, hipStream_t s) {
    const int vec = reduce_vec_ok(part, dw, n, (int)sizeof(T)) ? kReduceVec : 1;
    if (t_defer && t_jobs.njobs < kMaxReduceJobs) {
        const int j = t_jobs.njobs++;
        t_jobs.part[j] = part, t_jobs.out[j] = dw, t_jobs.nparts[j] = nparts, t_jobs.n[j] = n;
        t_jobs.dtype[j] = dtype_of<T>();
        t_jobs.vec[j] = vec, t_jobs.ql[j] = 8;
        t_jobs.first_block[j + 1] = t_jobs.first_block[j] + cdiv(n, reduce_block_outputs(vec, 8));
        return 0;
    }
    const int ql = standalone_part_lanes(nparts);
    hipLaunchKernelGGL((wgrad_reduce_parts<T>), dim3(cdiv(n, reduce_block_outputs(vec, ql))), dim3(256), 0, s, part,
                       (T*)dw, nparts, n, vec, ql);
    return check_launch("wgrad_reduce_parts");
}
template int wgrad_reduce_launch<float>(const float*, void*, int, int, hipStream_t);
template int wgrad_reduce_launch<f16_t>(const float*, void*, int, int, hipStream_t);
template int wgrad_reduce_launch<bf16_t>(const float*, void*, int, int, hipStream_t);

template <typename T>
static int wgrad_direct_t(const void* x, const void* gy, void* dw, float* part, const ConvGeom& g, hipStream_t s) {
    int nchunks, chunk_len;
    wgrad_direct_plan(g, &nchunks, &chunk_len);
    const dim3 grid(g.KH * g.KW, cdiv(g.C, 64), nchunks);
    hipLaunchKernelGGL((dwconv_wgrad_direct<T>), grid, dim3(256), 0, s, (const T*)x, (const T*)gy, part, g,
                       chunk_len);
    if (int e = check_launch("dwconv_wgrad_direct")) return e;
    return wgrad_reduce_launch<T>(part, dw, nchunks, g.KH * g.KW * g.C, s);
}

int dwconv_wgrad_direct_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C,
                               int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW, int dtype,
                               hipStream_t s) {
    const ConvGeom g = make_geom(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW);
    switch (dtype) {
        case kF32: return wgrad_direct_t<float>(x, gy, dw, (float*)ws, g, s);
        case kF16: return wgrad_direct_t<f16_t>(x, gy, dw, (float*)ws, g, s);
        default: return wgrad_direct_t<bf16_t>(x, gy, dw, (float*)ws, g, s);
    }
}

}  // namespace pdw
