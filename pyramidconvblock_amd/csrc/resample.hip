// HBM-bound helpers around the depthwise conv: adaptive average pooling, bilinear
// resize (align_corners=False) and the multiplicative gate, forward and backward.
// Channels-last; one thread owns VEC consecutive channels of one pixel (up to 16 bytes),
// so every wavefront access is a contiguous run.  Both backward kernels are gathers:
// each input element sums the few outputs that touch it, in a fixed order, so there are
// no atomics and results are bit-reproducible.
#include "common.h"
#include "kernels.h"
#include "bilinear.h"
#include "pool_branch.h"

namespace pdw {

// idx = ((q * n2 + r2) * n1 + r1) * n0 + r0 taken apart.  A thread's flat item index almost always fits 31 bits, and
// three 32-bit divisions cost a fifth of three 64-bit ones: in these kernels the index arithmetic, not the memory
// system, was what a wavefront spent most of its instructions on.
__device__ __forceinline__ void split_idx(long long idx, int n0, int n1, int n2, int& r0, int& r1, int& r2, long long& q) {
    if ((unsigned long long)idx < 0x80000000ull) {
        const unsigned u = (unsigned)idx, t0 = u / (unsigned)n0, t1 = t0 / (unsigned)n1, t2 = t1 / (unsigned)n2;
        r0 = (int)(u - t0 * (unsigned)n0), r1 = (int)(t0 - t1 * (unsigned)n1), r2 = (int)(t1 - t2 * (unsigned)n2);
        q = (long long)t2;
    } else {
        long long t = idx / n0;
        r0 = (int)(idx - t * n0);
        const long long t1 = t / n1;
        r1 = (int)(t - t1 * n1);
        q = t1 / n2;
        r2 = (int)(t1 - q * n2);
    }
}
// idx = q * n0 + r0
__device__ __forceinline__ void split_idx(long long idx, int n0, int& r0, long long& q) {
    if ((unsigned long long)idx < 0x80000000ull) {
        const unsigned u = (unsigned)idx, t0 = u / (unsigned)n0;
        r0 = (int)(u - t0 * (unsigned)n0), q = (long long)t0;
    } else {
        q = idx / n0, r0 = (int)(idx - q * n0);
    }
}

// ---------------------------------------------------------------- adaptive average pool
// Host side guarantees in * out < 2^31 (checked in the launchers), so 32-bit arithmetic is exact.
__device__ __forceinline__ int bin_start(int i, int in, int out) { return (int)((unsigned)(i * in) / (unsigned)out); }
__device__ __forceinline__ int bin_end(int i, int in, int out) {
    return (int)((unsigned)((i + 1) * in + out - 1) / (unsigned)out);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void avgpool_fwd_k(const T* __restrict__ x, T* __restrict__ y, int H, int W, int C,
                                                     int h, int w, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = C / VEC;
    int cq, j, i;
    long long b;
    split_idx(idx, CV, w, h, cq, j, i, b);
    const int c = cq * VEC;
    if (H == 2 * h && W == 2 * w) {   // (uniform) exact halves: the four loads of the 2 x 2 bin in flight together
        const T* p = x + ((b * H + 2 * i) * W + 2 * j) * C + c;
        float x00[VEC], x01[VEC], x10[VEC], x11[VEC], o[VEC];
        load_f32<T, VEC>(p, x00), load_f32<T, VEC>(p + C, x01);
        load_f32<T, VEC>(p + (long long)W * C, x10), load_f32<T, VEC>(p + (long long)W * C + C, x11);
#pragma unroll
        for (int v = 0; v < VEC; ++v) o[v] = (((x00[v] + x01[v]) + x10[v]) + x11[v]) * 0.25f;   // the loop's order
        store_f32<T, VEC>(y + ((b * h + i) * w + j) * C + c, o);
        return;
    }
    const int hs = bin_start(i, H, h), he = bin_end(i, H, h);
    const int ws = bin_start(j, W, w), we = bin_end(j, W, w);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    for (int ih = hs; ih < he; ++ih)
        for (int iw = ws; iw < we; ++iw) {
            float xv[VEC];
            load_f32<T, VEC>(x + ((b * H + ih) * W + iw) * C + c, xv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] += xv[v];
        }
    const float inv = 1.f / (float)((he - hs) * (we - ws));
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] *= inv;
    store_f32<T, VEC>(y + ((b * h + i) * w + j) * C + c, acc);
}

// Input row ih lies in bins i with floor(ih*h/H) <= i <= ceil((ih+1)*h/H) - 1.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void avgpool_bwd_k(const T* __restrict__ gy, T* __restrict__ gx, int H, int W,
                                                     int C, int h, int w, int accumulate, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = C / VEC;
    int cq, iw, ih;
    long long b;
    split_idx(idx, CV, W, H, cq, iw, ih, b);
    const int c = cq * VEC;
    const int i0 = (int)((unsigned)(ih * h) / (unsigned)H), i1 = (int)((unsigned)((ih + 1) * h + H - 1) / (unsigned)H) - 1;
    const int j0 = (int)((unsigned)(iw * w) / (unsigned)W), j1 = (int)((unsigned)((iw + 1) * w + W - 1) / (unsigned)W) - 1;
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    for (int i = i0; i <= i1; ++i) {
        const int kh = bin_end(i, H, h) - bin_start(i, H, h);
        for (int j = j0; j <= j1; ++j) {
            const int kw = bin_end(j, W, w) - bin_start(j, W, w);
            const float inv = 1.f / (float)(kh * kw);
            float gv[VEC];
            load_f32<T, VEC>(gy + ((b * h + i) * w + j) * C + c, gv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = fmaf(gv[v], inv, acc[v]);
        }
    }
    T* dst = gx + ((b * H + ih) * W + iw) * C + c;
    if (accumulate) {  // gx += pooled gradient (fp32 add, one rounding)
        float old[VEC];
        load_f32<T, VEC>(dst, old);
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += old[v];
    }
    store_f32<T, VEC>(dst, acc);
}

// Exact halves (H = 2h, W = 2w): a thread takes one pooled pixel's gradient and writes the four input pixels of its
// bin (one load, four stores; the values are those of the general kernel: gy * 0.25, plus the old value when
// accumulating).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void avgpool_bwd_x2_k(const T* __restrict__ gy, T* __restrict__ gx, int h, int w, int C,
                                                        int accumulate, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = C / VEC, W = 2 * w;
    int cq, j, i;
    long long b;
    split_idx(idx, CV, w, h, cq, j, i, b);
    const int c = cq * VEC;
    float gv[VEC];
    load_f32<T, VEC>(gy + ((b * h + i) * w + j) * C + c, gv);
    T* dst = gx + ((b * 2 * h + 2 * i) * W + 2 * j) * C + c;
    const long long off[4] = {0, C, (long long)W * C, (long long)W * C + C};
    float old[4][VEC];
    if (accumulate) {
#pragma unroll
        for (int k = 0; k < 4; ++k) load_f32<T, VEC>(dst + off[k], old[k]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float o[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) o[v] = fmaf(gv[v], 0.25f, 0.f) + (accumulate ? old[k][v] : 0.f);
        store_f32<T, VEC>(dst + off[k], o);
    }
}

// ---------------------------------------------------------------- bilinear, align_corners=False (bilinear.h)
template <typename T, int VEC>
__device__ __forceinline__ void bilinear_fwd_item(const T* __restrict__ x, T* __restrict__ y, int h, int w, int C,
                                                  int H, int W, int ldy, float sy, float sx, long long idx) {
    const int CV = C / VEC;
    int cq, j, i;
    long long b;
    split_idx(idx, CV, W, H, cq, j, i, b);
    const int c = cq * VEC;
    int y0, y1, x0, x1;
    float ly, lx;
    bl_src(i, sy, h, y0, y1, ly);
    bl_src(j, sx, w, x0, x1, lx);
    const T* xb = x + b * h * w * C + c;
    float a[VEC], bb[VEC], cc[VEC], d[VEC], o[VEC];
    load_f32<T, VEC>(xb + ((long long)y0 * w + x0) * C, a);
    load_f32<T, VEC>(xb + ((long long)y0 * w + x1) * C, bb);
    load_f32<T, VEC>(xb + ((long long)y1 * w + x0) * C, cc);
    load_f32<T, VEC>(xb + ((long long)y1 * w + x1) * C, d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = bl_mix(a[v], bb[v], cc[v], d[v], ly, lx);
    store_f32<T, VEC>(y + ((b * H + i) * W + j) * ldy + c, o);
}

// Exactly doubled extents, a 2 x 2 block of outputs per thread: their 16 taps fall on a 3 x 3 neighbourhood of the
// source (rows m-1 .. m+1, columns n-1 .. n+1, clamped to the image), so 9 loads serve 4 outputs instead of 16.  Same
// weights (bl_src), same values: at the image border bl_src moves the tap pair one row inwards, but the clamped
// neighbourhood then holds that row twice, so the static entries (di, di+1) give the same sums.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinear_fwd_x2_k(const T* __restrict__ x, T* __restrict__ y, int h, int w, int C,
                                                         int ldy, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int H = 2 * h, W = 2 * w, CV = C / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, CV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    const T* xb = x + b * h * w * C + c;
    ChanVec<T, VEC> p[3][3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int rr = min(max(m - 1 + r, 0), h - 1);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int cc = min(max(n - 1 + k, 0), w - 1);
            p[r][k] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + ((long long)rr * w + cc) * C);
        }
    }
#pragma unroll
    for (int di = 0; di < 2; ++di) {
        int y0, y1;
        float ly;
        bl_src(2 * m + di, 0.5f, h, y0, y1, ly);
#pragma unroll
        for (int dj = 0; dj < 2; ++dj) {
            int x0, x1;
            float lx;
            bl_src(2 * n + dj, 0.5f, w, x0, x1, lx);
            float o[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                o[v] = bl_mix(to_f32(p[di][dj].v[v]), to_f32(p[di][dj + 1].v[v]), to_f32(p[di + 1][dj].v[v]),
                              to_f32(p[di + 1][dj + 1].v[v]), ly, lx);
            store_f32<T, VEC>(y + ((b * H + 2 * m + di) * W + 2 * n + dj) * ldy + c, o);
        }
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinear_fwd_k(const T* __restrict__ x, T* __restrict__ y, int h, int w,
                                                      int C, int H, int W, int ldy, float sy, float sx,
                                                      long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) bilinear_fwd_item<T, VEC>(x, y, h, w, C, H, W, ldy, sy, sx, idx);
}

// Weight with which destination index `dst` reads source index m along one axis.
__device__ __forceinline__ float bl_weight(int dst, float scale, int in, int m) {
    int i0, i1;
    float lam;
    bl_src(dst, scale, in, i0, i1, lam);
    return (i0 == m ? 1.f - lam : 0.f) + (i1 == m ? lam : 0.f);
}

// Destination indices whose taps can include source m: src in [m-1, m+1), padded by 2 for fp rounding.
__device__ __forceinline__ void bl_dst_range(int m, float scale, int out, int& lo, int& hi) {
    const float inv = 1.f / scale;
    lo = (int)floorf(((float)m - 0.5f) * inv - 0.5f) - 2;
    hi = (int)ceilf(((float)m + 1.5f) * inv - 0.5f) + 2;
    if (lo < 0 || m == 0) lo = 0;
    if (hi > out - 1) hi = out - 1;
}

// Exactly doubled extents (H = 2h, W = 2w, the block's half-resolution gate): source m is read by the 4
// destinations 2m-1 .. 2m+2 and no others, so the taps are fixed and all 16 loads go out together.  The weights
// come from the same bl_weight as the general kernel (bit-identical results, borders included).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinear_bwd_x2_k(const T* __restrict__ gy, T* __restrict__ gx, int h, int w,
                                                         int C, int ldg, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int H = 2 * h, W = 2 * w;
    const int CV = C / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, CV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    float wy[4], wx[4];
    int iy[4], ix[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int di = 2 * m - 1 + k, dj = 2 * n - 1 + k;
        const bool oky = di >= 0 && di < H, okx = dj >= 0 && dj < W;
        iy[k] = oky ? di : 0, ix[k] = okx ? dj : 0;
        wy[k] = oky ? bl_weight(iy[k], 0.5f, h, m) : 0.f;
        wx[k] = okx ? bl_weight(ix[k], 0.5f, w, n) : 0.f;
    }
    const T* gb = gy + b * H * W * ldg + c;
    ChanVec<T, VEC> gv[4][4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            gv[p][q] = *reinterpret_cast<const ChanVec<T, VEC>*>(gb + ((long long)iy[p] * W + ix[q]) * ldg);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    // same order of accumulation as the general kernel: destinations ascending, rows outer
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float ww = wy[p] * wx[q];
            if (ww != 0.f) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = fmaf(ww, to_f32(gv[p][q].v[v]), acc[v]);
            }
        }
    store_f32<T, VEC>(gx + ((b * h + m) * w + n) * C + c, acc);
}

// acc = the gradient of source (m, n) of one image: the sum over the destinations that read it of their weight times
// gy (gb: the image's gy at the lane's channels, pixel stride ldg), for any ratio of extents.
template <typename T, int VEC>
__device__ __forceinline__ void bilinear_bwd_gather(const T* __restrict__ gb, int h, int w, int H, int W, int ldg, float sy,
                                                    float sx, int m, int n, float (&acc)[VEC]) {
    int ilo, ihi, jlo, jhi;
    bl_dst_range(m, sy, H, ilo, ihi);
    bl_dst_range(n, sx, W, jlo, jhi);
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    // The candidate ranges are generous (up to 11 wide when the output is about twice the input); the destinations
    // that really weigh in are a contiguous run of about 2 * out/in.  Up to NS of them per axis are handled
    // without branches: weights beyond the run are zero and addresses clamped, so the NS loads of a row are issued
    // together (a load behind a per-lane `continue` is a trip to memory of its own).
    constexpr int NC = 12, NS = 5;
    int i0 = ihi + 1, i1 = ilo - 1, j0 = jhi + 1, j1 = jlo - 1;
    if (ihi - ilo < NC && jhi - jlo < NC) {
#pragma unroll
        for (int q = NC - 1; q >= 0; --q) {
            if (ilo + q <= ihi && bl_weight(ilo + q, sy, h, m) != 0.f) i0 = ilo + q;
            if (jlo + q <= jhi && bl_weight(jlo + q, sx, w, n) != 0.f) j0 = jlo + q;
        }
#pragma unroll
        for (int q = 0; q < NC; ++q) {
            if (ilo + q <= ihi && bl_weight(ilo + q, sy, h, m) != 0.f) i1 = ilo + q;
            if (jlo + q <= jhi && bl_weight(jlo + q, sx, w, n) != 0.f) j1 = jlo + q;
        }
    }
    if (i1 - i0 < NS && j1 - j0 < NS && i1 >= i0 && j1 >= j0) {
        float wy[NS], wx[NS];
        int jo[NS];
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            wy[q] = i0 + q <= i1 ? bl_weight(i0 + q, sy, h, m) : 0.f;
            wx[q] = j0 + q <= j1 ? bl_weight(j0 + q, sx, w, n) : 0.f;
            jo[q] = min(j0 + q, j1) * ldg;
        }
#pragma unroll
        for (int p = 0; p < NS; ++p) {
            const T* gr = gb + (long long)min(i0 + p, i1) * W * ldg;
            ChanVec<T, VEC> gv[NS];
#pragma unroll
            for (int q = 0; q < NS; ++q) gv[q] = *reinterpret_cast<const ChanVec<T, VEC>*>(gr + jo[q]);
#pragma unroll
            for (int q = 0; q < NS; ++q) {
                const float ww = wy[p] * wx[q];
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = fmaf(ww, to_f32(gv[q].v[v]), acc[v]);
            }
        }
    } else {
        for (int i = ilo; i <= ihi; ++i) {
            const float wy = bl_weight(i, sy, h, m);
            if (wy == 0.f) continue;
            for (int j = jlo; j <= jhi; ++j) {
                const float wx = bl_weight(j, sx, w, n);
                if (wx == 0.f) continue;
                float gv[VEC];
                load_f32<T, VEC>(gb + ((long long)i * W + j) * ldg, gv);
                const float ww = wy * wx;
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = fmaf(ww, gv[v], acc[v]);
            }
        }
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinear_bwd_k(const T* __restrict__ gy, T* __restrict__ gx, int h, int w,
                                                      int C, int H, int W, int ldg, float sy, float sx,
                                                      long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = C / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, CV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    float acc[VEC];
    bilinear_bwd_gather<T, VEC>(gy + b * H * W * ldg + c, h, w, H, W, ldg, sy, sx, m, n, acc);
    store_f32<T, VEC>(gx + ((b * h + m) * w + n) * C + c, acc);
}

// ---------------------------------------------------------------- gate
template <typename T, int VEC>
__device__ __forceinline__ void gate_fwd_item(const T* __restrict__ x, T* __restrict__ y, int I, int ldy, float s,
                                              long long idx) {
    const int G = I / 2, GV = G / VEC;
    int cq;
    long long m;
    split_idx(idx, GV, cq, m);
    const int c = cq * VEC;
    float a[VEC], b[VEC], o[VEC];
    load_f32<T, VEC>(x + m * I + c, a);
    load_f32<T, VEC>(x + m * I + G + c, b);
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = gate_f32(a[v], b[v], s);
    store_f32<T, VEC>(y + m * ldy + c, o);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_fwd_k(const T* __restrict__ x, T* __restrict__ y, int I, int ldy, float s,
                                                  long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) gate_fwd_item<T, VEC>(x, y, I, ldy, s, idx);
}

template <typename T, int VEC>
__device__ __forceinline__ void gate_bwd_item(const T* __restrict__ x, const T* __restrict__ gy, T* __restrict__ gx,
                                              int I, int ldg, float s, long long idx) {
    const int G = I / 2, GV = G / VEC;
    int cq;
    long long m;
    split_idx(idx, GV, cq, m);
    const int c = cq * VEC;
    float a[VEC], b[VEC], g[VEC], ga[VEC], gb[VEC];
    load_f32<T, VEC>(x + m * I + c, a);
    load_f32<T, VEC>(x + m * I + G + c, b);
    load_f32<T, VEC>(gy + m * ldg + c, g);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        ga[v] = gate_f32(g[v], b[v], s);
        gb[v] = gate_f32(g[v], a[v], s);
    }
    store_f32<T, VEC>(gx + m * I + c, ga);
    store_f32<T, VEC>(gx + m * I + G + c, gb);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_bwd_k(const T* __restrict__ x, const T* __restrict__ gy,
                                                  T* __restrict__ gx, int I, int ldg, float s, long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) gate_bwd_item<T, VEC>(x, gy, gx, I, ldg, s, idx);
}


// U items per thread, every load of a thread requested before the first use (a streaming kernel lives on the number
// of loads in flight); items past the end read the last item's data and store nothing.
constexpr int kGateItems = 8;  // full-resolution items per thread of the paired kernels
constexpr int kGateAhead = 2;  // items whose loads are in flight when an item is stored

template <typename T, int VEC, int U>
__device__ __forceinline__ void gate_fwd_items(const T* __restrict__ x, T* __restrict__ y, int I, int ldy, float s,
                                               long long first, long long step, long long total) {
    // A rolling pipeline: the loads of item u + kGateAhead are issued before item u is stored, so that a
    // thread's reads and writes alternate.  With every thread of the grid resident at once, "load everything,
    // then store everything" puts the whole kernel's reads before the whole kernel's writes.
    const int G = I / 2, GV = G / VEC;
    // item -> (pixel, channel vector): a shift and a mask for the usual power-of-two channel counts; the general
    // 64-bit division costs more vector-ALU time per item than the gate itself
    const int sh = (GV & (GV - 1)) == 0 ? 31 - __builtin_clz(GV) : -1;
    ChanVec<T, VEC> a[U], b[U];
    long long m[U];
    int c[U];
    auto load = [&](int u) {
        const long long idx = min(first + u * step, total - 1);
        if (sh >= 0)
            c[u] = ((int)idx & (GV - 1)) * VEC, m[u] = idx >> sh;
        else {
            split_idx(idx, GV, c[u], m[u]);
            c[u] *= VEC;
        }
        a[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(x + m[u] * I + c[u]);
        b[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(x + m[u] * I + G + c[u]);
    };
#pragma unroll
    for (int u = 0; u < kGateAhead && u < U; ++u) load(u);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (u + kGateAhead < U) load(u + kGateAhead);
        float o[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) o[v] = gate_f32(to_f32(a[u].v[v]), to_f32(b[u].v[v]), s);
        if (first + u * step < total) store_f32<T, VEC>(y + m[u] * ldy + c[u], o);
    }
}

template <typename T, int VEC, int U>
__device__ __forceinline__ void gate_bwd_items(const T* __restrict__ x, const T* __restrict__ gy, T* __restrict__ gx,
                                               int I, int ldg, float s, long long first, long long step,
                                               long long total) {
    const int G = I / 2, GV = G / VEC;
    const int sh = (GV & (GV - 1)) == 0 ? 31 - __builtin_clz(GV) : -1;  // as in gate_fwd_items
    ChanVec<T, VEC> a[U], b[U], g[U];
    long long m[U];
    int c[U];
    auto load = [&](int u) {
        const long long idx = min(first + u * step, total - 1);
        if (sh >= 0)
            c[u] = ((int)idx & (GV - 1)) * VEC, m[u] = idx >> sh;
        else {
            split_idx(idx, GV, c[u], m[u]);
            c[u] *= VEC;
        }
        a[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(x + m[u] * I + c[u]);
        b[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(x + m[u] * I + G + c[u]);
        g[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(gy + m[u] * ldg + c[u]);
    };
#pragma unroll
    for (int u = 0; u < kGateAhead && u < U; ++u) load(u);
#pragma unroll
    for (int u = 0; u < U; ++u) {  // loads run kGateAhead items ahead of the stores, as in gate_fwd_items
        if (u + kGateAhead < U) load(u + kGateAhead);
        float ga[VEC], gb[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            const float gv = to_f32(g[u].v[v]);
            ga[v] = gate_f32(gv, to_f32(b[u].v[v]), s);
            gb[v] = gate_f32(gv, to_f32(a[u].v[v]), s);
        }
        if (first + u * step < total) {
            store_f32<T, VEC>(gx + m[u] * I + c[u], ga);
            store_f32<T, VEC>(gx + m[u] * I + G + c[u], gb);
        }
    }
}

// ---------------------------------------------------------------- gate fused with the resampling next to it
// Gate then bilinear resize in one pass: y[b,i,j,c] = interp of gate(x)[b,:,:,c], x[B,h,w,I] -> y[B,H,W,G] (G = I/2).
// The gate value of each of the 4 source pixels is rounded to T first, exactly what the two separate kernels
// produce, so the gated tensor never exists in memory.
template <typename T, int VEC>
__device__ __forceinline__ void gate_bilinear_fwd_item(const T* __restrict__ x, T* __restrict__ y, int h, int w, int I,
                                                       int H, int W, int ldy, float sy, float sx, float s,
                                                       long long idx) {
    const int G = I / 2, GV = G / VEC;
    int cq, j, i;
    long long b;
    split_idx(idx, GV, W, H, cq, j, i, b);
    const int c = cq * VEC;
    int y0, y1, x0, x1;
    float ly, lx;
    bl_src(i, sy, h, y0, y1, ly);
    bl_src(j, sx, w, x0, x1, lx);
    const T* xb = x + b * h * w * I + c;
    const long long o00 = ((long long)y0 * w + x0) * I, o01 = ((long long)y0 * w + x1) * I;
    const long long o10 = ((long long)y1 * w + x0) * I, o11 = ((long long)y1 * w + x1) * I;
    ChanVec<T, VEC> pa[4], pb[4];  // all eight loads in flight
    pa[0] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o00), pb[0] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o00 + G);
    pa[1] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o01), pb[1] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o01 + G);
    pa[2] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o10), pb[2] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o10 + G);
    pa[3] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o11), pb[3] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + o11 + G);
    float o[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        float gv[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) gv[k] = to_f32(from_f32<T>(gate_f32(to_f32(pa[k].v[v]), to_f32(pb[k].v[v]), s)));
        o[v] = bl_mix(gv[0], gv[1], gv[2], gv[3], ly, lx);
    }
    store_f32<T, VEC>(y + ((b * H + i) * W + j) * ldy + c, o);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_bilinear_fwd_k(const T* __restrict__ x, T* __restrict__ y, int h, int w,
                                                           int I, int H, int W, int ldy, float sy, float sx, float s,
                                                           long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) gate_bilinear_fwd_item<T, VEC>(x, y, h, w, I, H, W, ldy, sy, sx, s, idx);
}

// The same for exactly doubled extents, a 2 x 2 block of outputs per thread: their 16 taps fall on a 3 x 3
// neighbourhood of the source (rows m-1 .. m+1, columns n-1 .. n+1, clamped to the image), so 18 loads and 9 gate
// values serve 4 outputs instead of 32 and 16.  Same weights (bl_src), same rounding.
template <typename T, int VEC>
__device__ __forceinline__ void gate_bilinear_fwd_x2_item(const T* __restrict__ x, T* __restrict__ y, int h, int w,
                                                          int I, int ldy, float s, long long idx) {
    const int H = 2 * h, W = 2 * w;
    const int G = I / 2, GV = G / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, GV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    const T* xb = x + b * h * w * I + c;
    ChanVec<T, VEC> pa[3][3], pb[3][3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int rr = min(max(m - 1 + r, 0), h - 1);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int cc = min(max(n - 1 + k, 0), w - 1);
            const T* p = xb + ((long long)rr * w + cc) * I;
            pa[r][k] = *reinterpret_cast<const ChanVec<T, VEC>*>(p);
            pb[r][k] = *reinterpret_cast<const ChanVec<T, VEC>*>(p + G);
        }
    }
    float gv[3][3][VEC];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                gv[r][k][v] = to_f32(from_f32<T>(gate_f32(to_f32(pa[r][k].v[v]), to_f32(pb[r][k].v[v]), s)));
#pragma unroll
    for (int di = 0; di < 2; ++di) {
        // Output row 2m + di takes source rows m-1+di and m+di; at the image border bl_src moves the pair one
        // row inwards, but the clamped neighbourhood then holds the same row twice, so the static entries
        // (di, di+1) with bl_src's weights give the same sums.
        int y0, y1;
        float ly;
        bl_src(2 * m + di, 0.5f, h, y0, y1, ly);
#pragma unroll
        for (int dj = 0; dj < 2; ++dj) {
            int x0, x1;
            float lx;
            bl_src(2 * n + dj, 0.5f, w, x0, x1, lx);
            float o[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                o[v] = bl_mix(gv[di][dj][v], gv[di][dj + 1][v], gv[di + 1][dj][v], gv[di + 1][dj + 1][v], ly, lx);
            store_f32<T, VEC>(y + ((b * H + 2 * m + di) * W + 2 * n + dj) * ldy + c, o);
        }
    }
}

// Both branches of a two-scale block in one launch: workgroups below nblk_full gate the full-resolution tensor into
// channels [0, G) of y, the others gate and resize the pooled one into channels [G, 2G).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_pair_fwd_k(const T* __restrict__ xf, const T* __restrict__ xh,
                                                       T* __restrict__ y, int h, int w, int I, int H, int W, int ldy,
                                                       float sy, float sx, float s, unsigned nblk_full,
                                                       long long total_full, long long total_half) {
    if (blockIdx.x < nblk_full) {
        const long long first = (long long)blockIdx.x * (kGateItems * 256) + threadIdx.x;
        if (first < total_full) gate_fwd_items<T, VEC, kGateItems>(xf, y, I, ldy, s, first, 256, total_full);
    } else {
        const long long idx = (long long)(blockIdx.x - nblk_full) * blockDim.x + threadIdx.x;
        if (idx < total_half) {
            if (H == 2 * h && W == 2 * w)  // total_half then counts 2 x 2 output blocks
                gate_bilinear_fwd_x2_item<T, VEC>(xh, y + I / 2, h, w, I, ldy, s, idx);
            else
                gate_bilinear_fwd_item<T, VEC>(xh, y + I / 2, h, w, I, H, W, ldy, sy, sx, s, idx);
        }
    }
}

// Backward of the pair for exactly doubled extents: the bilinear gather of bilinear_bwd_x2_k (rounded to T),
// then the gate's gradient, written as gx[B,h,w,I].
template <typename T, int VEC>
__device__ __forceinline__ void bilinear_gate_bwd_x2_item(const T* __restrict__ gy, const T* __restrict__ x,
                                                          T* __restrict__ gx, int h, int w, int I, int ldg, float s,
                                                          long long idx) {
    const int H = 2 * h, W = 2 * w;
    const int G = I / 2, GV = G / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, GV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    float wy[4], wx[4];
    int iy[4], ix[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int di = 2 * m - 1 + k, dj = 2 * n - 1 + k;
        const bool oky = di >= 0 && di < H, okx = dj >= 0 && dj < W;
        iy[k] = oky ? di : 0, ix[k] = okx ? dj : 0;
        wy[k] = oky ? bl_weight(iy[k], 0.5f, h, m) : 0.f;
        wx[k] = okx ? bl_weight(ix[k], 0.5f, w, n) : 0.f;
    }
    const T* gb = gy + b * H * W * ldg + c;
    const T* xp = x + ((b * h + m) * w + n) * I + c;
    const ChanVec<T, VEC> xa = *reinterpret_cast<const ChanVec<T, VEC>*>(xp);
    const ChanVec<T, VEC> xb = *reinterpret_cast<const ChanVec<T, VEC>*>(xp + G);
    ChanVec<T, VEC> gv[4][4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            gv[p][q] = *reinterpret_cast<const ChanVec<T, VEC>*>(gb + ((long long)iy[p] * W + ix[q]) * ldg);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float ww = wy[p] * wx[q];
            if (ww != 0.f) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = fmaf(ww, to_f32(gv[p][q].v[v]), acc[v]);
            }
        }
    float ga[VEC], gbv[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const float g = to_f32(from_f32<T>(acc[v]));  // the resampled gradient as the separate kernel stores it
        ga[v] = gate_f32(g, to_f32(xb.v[v]), s);
        gbv[v] = gate_f32(g, to_f32(xa.v[v]), s);
    }
    T* op = gx + ((b * h + m) * w + n) * I + c;
    store_f32<T, VEC>(op, ga);
    store_f32<T, VEC>(op + G, gbv);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinear_gate_bwd_x2_k(const T* __restrict__ gy, const T* __restrict__ x,
                                                              T* __restrict__ gx, int h, int w, int I, int ldg, float s,
                                                              long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) bilinear_gate_bwd_x2_item<T, VEC>(gy, x, gx, h, w, I, ldg, s, idx);
}

// Gradient of gate_pair_fwd_k for exactly doubled extents, the two branches again in one launch.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_pair_bwd_k(const T* __restrict__ gy, const T* __restrict__ xf,
                                                       const T* __restrict__ xh, T* __restrict__ gxf,
                                                       T* __restrict__ gxh, int h, int w, int I, int ldg, float s,
                                                       unsigned nblk_full, long long total_full,
                                                       long long total_half) {
    if (blockIdx.x < nblk_full) {
        const long long first = (long long)blockIdx.x * (kGateItems * 256) + threadIdx.x;
        if (first < total_full) gate_bwd_items<T, VEC, kGateItems>(xf, gy, gxf, I, ldg, s, first, 256, total_full);
    } else {
        const long long idx = (long long)(blockIdx.x - nblk_full) * blockDim.x + threadIdx.x;
        if (idx < total_half) bilinear_gate_bwd_x2_item<T, VEC>(gy + I / 2, xh, gxh, h, w, I, ldg, s, idx);
    }
}

// The same for any ratio of extents: the half-resolution items gather their gradient with bilinear_bwd_gather
// (rounded to T, as the separate kernel stores it) and apply the gate's gradient.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_pair_bwd_gen_k(const T* __restrict__ gy, const T* __restrict__ xf,
                                                           const T* __restrict__ xh, T* __restrict__ gxf,
                                                           T* __restrict__ gxh, int h, int w, int H, int W, int I, int ldg,
                                                           float s, float sy, float sx, unsigned nblk_full,
                                                           long long total_full, long long total_half) {
    if (blockIdx.x < nblk_full) {
        const long long first = (long long)blockIdx.x * (kGateItems * 256) + threadIdx.x;
        if (first < total_full) gate_bwd_items<T, VEC, kGateItems>(xf, gy, gxf, I, ldg, s, first, 256, total_full);
        return;
    }
    const long long idx = (long long)(blockIdx.x - nblk_full) * blockDim.x + threadIdx.x;
    if (idx >= total_half) return;
    const int G = I / 2, GV = G / VEC;
    int cq, n, m;
    long long b;
    split_idx(idx, GV, w, h, cq, n, m, b);
    const int c = cq * VEC;
    const T* xp = xh + ((b * h + m) * w + n) * I + c;
    const ChanVec<T, VEC> xa = *reinterpret_cast<const ChanVec<T, VEC>*>(xp);
    const ChanVec<T, VEC> xb = *reinterpret_cast<const ChanVec<T, VEC>*>(xp + G);
    float acc[VEC];
    bilinear_bwd_gather<T, VEC>(gy + b * H * W * ldg + G + c, h, w, H, W, ldg, sy, sx, m, n, acc);
    float ga[VEC], gbv[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const float g = to_f32(from_f32<T>(acc[v]));
        ga[v] = gate_f32(g, to_f32(xb.v[v]), s);
        gbv[v] = gate_f32(g, to_f32(xa.v[v]), s);
    }
    T* op = gxh + ((b * h + m) * w + n) * I + c;
    store_f32<T, VEC>(op, ga);
    store_f32<T, VEC>(op + G, gbv);
}

// ---------------------------------------------------------------- per-image column sums and broadcast add
// Pass 1 of the spatial sum: block (chunk, b) adds its share of the P positions of image b for all C
// channels; threads are (channel vector, position lane); position lanes are combined through LDS.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void spatial_sum_part_k(const T* __restrict__ x, float* __restrict__ part, int P, int C,
                                                          int chunk_len) {
    extern __shared__ float red[];  // [PL][CV*VEC]
    const int CV = C / VEC;
    const int PL = 256 / CV;  // position lanes (host guarantees CV <= 256)
    const int cv = threadIdx.x % CV, pl = threadIdx.x / CV;
    const int b = blockIdx.y, ch = blockIdx.x;
    const int p0 = ch * chunk_len, p1 = min(p0 + chunk_len, P);
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    if (pl < PL) {
        const T* xb = x + ((long long)b * P) * C + cv * VEC;
        int p = p0 + pl;
        for (; p + 3 * PL < p1; p += 4 * PL) {  // four loads in flight per thread
            ChanVec<T, VEC> xv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) xv[u] = *reinterpret_cast<const ChanVec<T, VEC>*>(xb + (long long)(p + u * PL) * C);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] += to_f32(xv[u].v[v]);
        }
        for (; p < p1; p += PL) {
            float xv[VEC];
            load_f32<T, VEC>(xb + (long long)p * C, xv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] += xv[v];
        }
#pragma unroll
        for (int v = 0; v < VEC; ++v) red[pl * C + cv * VEC + v] = acc[v];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < C; c += 256) {
        float s = 0.f;
        for (int q = 0; q < PL; ++q) s += red[q * C + c];
        part[((long long)b * gridDim.x + ch) * C + c] = s;
    }
}

__global__ __launch_bounds__(256) void spatial_sum_final_k(const float* __restrict__ part, float* __restrict__ out,
                                                           int nchunks, int C, int total) {
    __shared__ float red[8][32];
    const int el = threadIdx.x & 31, ql = threadIdx.x >> 5;
    const int idx = blockIdx.x * 32 + el;
    float s = 0.f;
    if (idx < total) {
        const int c = idx % C, b = idx / C;
        for (int q = ql; q < nchunks; q += 8) s += part[((long long)b * nchunks + q) * C + c];
    }
    red[ql][el] = s;
    __syncthreads();
    if (ql == 0 && idx < total)
        out[idx] = ((red[0][el] + red[1][el]) + (red[2][el] + red[3][el])) +
                   ((red[4][el] + red[5][el]) + (red[6][el] + red[7][el]));
}

// ---------------------------------------------------------------- pooled branch (global mean -> dense layer)
// Forward, one workgroup per image: m[b,:] = (sum of the chunk partials) / P rounded to T, then
// rowbias[b,o] = sum_c m[b,c] * Wp[o,c] + bp[o] + bo[o]  (fp32).  The dot products are spread over
// Sum of one column of the chunk partials of an image, 8 loads in flight (fixed order: bit-reproducible).
__device__ __forceinline__ float chunk_column_sum(const float* __restrict__ pp, int nchunks, int D) {
    float s[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] = 0.f;
    int q = 0;
    for (; q + 32 <= nchunks; q += 32) {   // 32 loads in flight, added in the order of the 8-wide loop below
        float v[32];
#pragma unroll
        for (int j = 0; j < 32; ++j) v[j] = pp[(long long)(q + j) * D];
#pragma unroll
        for (int j = 0; j < 32; ++j) s[j & 7] += v[j];
    }
    for (; q + 8 <= nchunks; q += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = pp[(long long)(q + j) * D];
#pragma unroll
        for (int j = 0; j < 8; ++j) s[j] += v[j];
    }
    {   // the last, partial group: requested together, added to s[0] one after the other
        float v[7];
#pragma unroll
        for (int j = 0; j < 7; ++j) v[j] = q + j < nchunks ? pp[(long long)(q + j) * D] : 0.f;
#pragma unroll
        for (int j = 0; j < 7; ++j)
            if (q + j < nchunks) s[0] += v[j];
    }
    return ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
}

// 8 lanes per output feature (strided over c, combined with wavefront shuffles).  gridDim.y slices of 32 output
// features each (every slice forms the image's mean again: the partials are a few KB in L2).
template <typename T>
__global__ __launch_bounds__(256) void pool_branch_fwd_k(const float* __restrict__ part, int nchunks, int D, float inv_p,
                                                         const T* __restrict__ wp, const T* __restrict__ bp,
                                                         const T* __restrict__ bo, T* __restrict__ m,
                                                         float* __restrict__ rowbias) {
    extern __shared__ float sm[];  // [D]
    const int b = blockIdx.x;
    for (int c = threadIdx.x; c < D; c += 256) {
        const T mv = from_f32<T>(chunk_column_sum(part + (long long)b * nchunks * D + c, nchunks, D) * inv_p);
        if (blockIdx.y == 0) m[(long long)b * D + c] = mv;
        sm[c] = to_f32(mv);
    }
    __syncthreads();
    const int sub = threadIdx.x & 7;
    for (int o = blockIdx.y * 32 + (threadIdx.x >> 3); o < D; o += 32 * gridDim.y) {
        const T* wr = wp + (long long)o * D;
        float acc = 0.f;
#pragma unroll 8
        for (int c = sub; c < D; c += 8) acc = fmaf(sm[c], to_f32(wr[c]), acc);
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
        acc += __shfl_xor(acc, 4);
        if (sub == 0) {
            if (bp) acc += to_f32(bp[o]);
            if (bo) acc += to_f32(bo[o]);
            rowbias[(long long)b * D + o] = acc;
        }
    }
}

// Backward part A, one workgroup per image: gs[b,:] = sum of the chunk partials of gy's column sums and
// dmean[b,c] = inv_p * sum_o gs[b,o] * Wp[o,c]   (the gradient that flows back through the mean).
template <typename T>
__global__ __launch_bounds__(256) void pool_branch_bwd_a_k(const float* __restrict__ part, int nchunks, int D,
                                                           float inv_p, const T* __restrict__ wp,
                                                           float* __restrict__ gs, float* __restrict__ dmean) {
    extern __shared__ float sm[];  // [D] column sums, then [OL][D] partial products
    const int b = blockIdx.x;
    for (int c = threadIdx.x; c < D; c += 256) {
        const float s = chunk_column_sum(part + (long long)b * nchunks * D + c, nchunks, D);
        if (blockIdx.y == 0) gs[(long long)b * D + c] = s;
        sm[c] = s;
    }
    __syncthreads();
    if (gridDim.y > 1) {
        // wide layers (D > 128): gridDim.y slices of 32 columns of dmean (every slice forms the column sums again: a
        // few KB from L2), 8 row lanes per column with 32 loads in flight each, combined through LDS
        const int cl = threadIdx.x & 31, ol = threadIdx.x >> 5, c = blockIdx.y * 32 + cl;
        float* pr = sm + D;   // [8][32]
        float a4[4] = {0.f, 0.f, 0.f, 0.f};
        if (c < D) {
            for (int o = ol; o < D; o += 256) {   // 32 loads in flight: one round for D <= 256
                float wv[32], sv[32];
#pragma unroll
                for (int j = 0; j < 32; ++j) {
                    const int oo = o + 8 * j;
                    const bool ok = oo < D;
                    wv[j] = ok ? to_f32(wp[(long long)oo * D + c]) : 0.f;
                    sv[j] = ok ? sm[oo] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < 32; ++j) a4[j & 3] = fmaf(sv[j], wv[j], a4[j & 3]);
            }
        }
        pr[ol * 32 + cl] = (a4[0] + a4[1]) + (a4[2] + a4[3]);
        __syncthreads();
        if (ol == 0 && c < D) {
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < 8; ++q) t += pr[q * 32 + cl];
            dmean[(long long)b * D + c] = t * inv_p;
        }
        return;
    }
    // thread (ol, c): rows o = ol, ol+OL, ...  of Wp, coalesced over c; OL row lanes combined through LDS
    const int OL = D <= 128 ? 256 / (D < 32 ? 32 : D) : 1;   // row lanes when D <= 128
    float* prod = sm + D;
    if (OL > 1) {
        const int cw = 256 / OL;
        const int c = threadIdx.x % cw, ol = threadIdx.x / cw;
        float acc = 0.f;
        if (c < D) {
#pragma unroll 4
            for (int o = ol; o < D; o += OL) acc = fmaf(sm[o], to_f32(wp[(long long)o * D + c]), acc);
            prod[ol * D + c] = acc;
        }
        __syncthreads();
        if (ol == 0 && c < D) {
            float t = 0.f;
            for (int q = 0; q < OL; ++q) t += prod[q * D + c];
            dmean[(long long)b * D + c] = t * inv_p;
        }
    } else {
        for (int c = threadIdx.x; c < D; c += 256) {
            float a4[4] = {0.f, 0.f, 0.f, 0.f};   // four independent chains, 16 loads in flight
            int o = 0;
            for (; o + 16 <= D; o += 16) {
                float wv[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) wv[j] = to_f32(wp[(long long)(o + j) * D + c]);
#pragma unroll
                for (int j = 0; j < 16; ++j) a4[j & 3] = fmaf(sm[o + j], wv[j], a4[j & 3]);
            }
            for (; o < D; ++o) a4[0] = fmaf(sm[o], to_f32(wp[(long long)o * D + c]), a4[0]);
            dmean[(long long)b * D + c] = ((a4[0] + a4[1]) + (a4[2] + a4[3])) * inv_p;
        }
    }
}

// Backward part B, one workgroup per output feature o: gbias[o] = sum_b gs[b,o] and
// gwp[o,c] = sum_b gs[b,o] * m[b,c].
template <typename T>
__global__ __launch_bounds__(256) void pool_branch_bwd_b_k(const float* __restrict__ gs, const T* __restrict__ m, int B,
                                                           int D, T* __restrict__ gbias, T* __restrict__ gbias2,
                                                           T* __restrict__ gwp) {
    extern __shared__ float gcol[];  // [B] = gs[:, o]
    const int o = blockIdx.x;
    for (int b = threadIdx.x; b < B; b += 256) gcol[b] = gs[(long long)b * D + o];
    __syncthreads();
    for (int c = threadIdx.x; c < D; c += 256) {
        float a0 = 0.f, a1 = 0.f;
        int b = 0;
        for (; b + 2 <= B; b += 2) {
            a0 = fmaf(gcol[b], to_f32(m[(long long)b * D + c]), a0);
            a1 = fmaf(gcol[b + 1], to_f32(m[(long long)(b + 1) * D + c]), a1);
        }
        if (b < B) a0 = fmaf(gcol[b], to_f32(m[(long long)b * D + c]), a0);
        gwp[(long long)o * D + c] = from_f32<T>(a0 + a1);
    }
    if (threadIdx.x == 0) {
        float s = 0.f;
        for (int b = 0; b < B; ++b) s += gcol[b];
        gbias[o] = from_f32<T>(s);
        if (gbias2) gbias2[o] = from_f32<T>(s);
    }
}

// ---- the same three kernels for 16-bit types with D % 8 == 0 and D <= 128 (the block's widths): 16-byte weight
// loads, every global load of a thread issued before the first use (these kernels are pure latency), partial
// products combined through LDS.
template <typename T>
__device__ __forceinline__ float colsum_parts(const float* __restrict__ pp, int nchunks, int D) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int q = 0;
#pragma unroll 4
    for (; q + 4 <= nchunks; q += 4) {
        s0 += pp[(long long)q * D], s1 += pp[(long long)(q + 1) * D];
        s2 += pp[(long long)(q + 2) * D], s3 += pp[(long long)(q + 3) * D];
    }
    for (; q < nchunks; ++q) s0 += pp[(long long)q * D];
    return (s0 + s1) + (s2 + s3);
}

template <typename T>
__global__ __launch_bounds__(256) void pool_branch_fwd_v8_k(const float* __restrict__ part, int nchunks, int D,
                                                            float inv_p, const T* __restrict__ wp,
                                                            const T* __restrict__ bp, const T* __restrict__ bo,
                                                            T* __restrict__ m, float* __restrict__ rowbias) {
    extern __shared__ float sm[];
    pool_branch_fwd_v8_body<T>(part, nchunks, D, inv_p, wp, bp, bo, m, rowbias, blockIdx.x, sm);
}

template <typename T>
__device__ __forceinline__ void pool_branch_bwd_a_v8_body(const float* __restrict__ part, int nchunks, int D,
                                                          float inv_p, const T* __restrict__ wp,
                                                          float* __restrict__ gs, float* __restrict__ dmean, int b,
                                                          float* sm) {  // sm: [D] column sums, then [16][D] products
    const int tid = threadIdx.x;
    const int cv = tid & 15, ol = tid >> 4;  // channel vector, row lane: rows o = ol + 16*it
    ChanVec<T, 8> wv[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int o = ol + 16 * it;
        const bool ok = o < D && cv * 8 < D;
        wv[it] = *reinterpret_cast<const ChanVec<T, 8>*>(wp + (ok ? (long long)o * D + cv * 8 : 0));
    }
    colsum_coop(part + (long long)b * nchunks * D, nchunks, D, sm, sm + D);
    if (tid < D) gs[(long long)b * D + tid] = sm[tid];
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int o = ol + 16 * it;
        if (o < D && cv * 8 < D) {
            const float gsv = sm[o];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf(gsv, to_f32(wv[it].v[j]), acc[j]);
        }
    }
    float* prod = sm + D;
    if (cv * 8 < D) {
#pragma unroll
        for (int j = 0; j < 8; ++j) prod[ol * D + cv * 8 + j] = acc[j];
    }
    __syncthreads();
    if (tid < D) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) t += prod[q * D + tid];
        dmean[(long long)b * D + tid] = t * inv_p;
    }
}

// sm: [B] = column sums gs[:, o] (filled by the caller, barrier included), then [16][D] partial products
template <typename T>
__device__ __forceinline__ void pool_branch_bwd_b_v8_body(const T* __restrict__ m, int B, int D, T* __restrict__ gbias,
                                                          T* __restrict__ gbias2, T* __restrict__ gwp, int o,
                                                          float* sm) {
    const int tid = threadIdx.x;
    const int cv = tid & 15, bl = tid >> 4;  // channel vector, batch lane: images b = bl + 16*it
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    if (cv * 8 < D) {
        int b = bl;
        for (; b + 16 < B; b += 32) {  // two loads in flight
            const ChanVec<T, 8> m0 = *reinterpret_cast<const ChanVec<T, 8>*>(m + (long long)b * D + cv * 8);
            const ChanVec<T, 8> m1 = *reinterpret_cast<const ChanVec<T, 8>*>(m + (long long)(b + 16) * D + cv * 8);
            const float g0 = sm[b], g1 = sm[b + 16];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf(g1, to_f32(m1.v[j]), fmaf(g0, to_f32(m0.v[j]), acc[j]));
        }
        for (; b < B; b += 16) {
            const ChanVec<T, 8> m0 = *reinterpret_cast<const ChanVec<T, 8>*>(m + (long long)b * D + cv * 8);
            const float g0 = sm[b];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf(g0, to_f32(m0.v[j]), acc[j]);
        }
    }
    float* prod = sm + B;
    if (cv * 8 < D) {
#pragma unroll
        for (int j = 0; j < 8; ++j) prod[bl * D + cv * 8 + j] = acc[j];
    }
    __syncthreads();
    if (tid < D) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) t += prod[q * D + tid];
        gwp[(long long)o * D + tid] = from_f32<T>(t);
    }
    if (tid == 0) {
        float sv = 0.f;
        for (int b = 0; b < B; ++b) sv += sm[b];
        gbias[o] = from_f32<T>(sv);
        if (gbias2) gbias2[o] = from_f32<T>(sv);
    }
}

// Both parts in one launch: workgroups [0, B) are part A for image b, workgroups [B, B + D) part B for feature o.
// Part B sums its column of the per-chunk sums itself (8 lanes per image), so it does not wait for part A.
template <typename T>
__device__ __forceinline__ void pool_branch_bwd_v8_block(const float* __restrict__ part, int nchunks, int B, int D,
                                                         float inv_p, const T* __restrict__ wp,
                                                         const T* __restrict__ m, float* __restrict__ gs,
                                                         float* __restrict__ dmean, T* __restrict__ gbias,
                                                         T* __restrict__ gbias2, T* __restrict__ gwp, int bid,
                                                         float* sm) {
    if (bid < B) {
        pool_branch_bwd_a_v8_body<T>(part, nchunks, D, inv_p, wp, gs, dmean, bid, sm);
        return;
    }
    const int o = bid - B, tid = threadIdx.x, l8 = tid & 7;
    for (int b = tid >> 3; b < B; b += 32) {
        const float* pp = part + (long long)b * nchunks * D + o;
        float sv = 0.f;
        for (int q = l8; q < nchunks; q += 8) sv += pp[(long long)q * D];
        sv += __shfl_xor(sv, 1);
        sv += __shfl_xor(sv, 2);
        sv += __shfl_xor(sv, 4);
        if (l8 == 0) sm[b] = sv;
    }
    __syncthreads();
    pool_branch_bwd_b_v8_body<T>(m, B, D, gbias, gbias2, gwp, o, sm);
}

template <typename T>
__global__ __launch_bounds__(256) void pool_branch_bwd_v8_k(const float* __restrict__ part, int nchunks, int B, int D,
                                                            float inv_p, const T* __restrict__ wp,
                                                            const T* __restrict__ m, float* __restrict__ gs,
                                                            float* __restrict__ dmean, T* __restrict__ gbias,
                                                            T* __restrict__ gbias2, T* __restrict__ gwp) {
    extern __shared__ float sm[];
    pool_branch_bwd_v8_block<T>(part, nchunks, B, D, inv_p, wp, m, gs, dmean, gbias, gbias2, gwp, blockIdx.x, sm);
}

// ---- the middle of a two-scale block in one launch each way: the (tiny, latency-bound) mean branch rides on the
// gate kernels.  Its workgroups come first in the grid, the gate workgroups after them.
struct PoolBwdJob {
    const float* part;
    int nchunks, B, D;
    float inv_p;
    const void *wp, *m;
    float *gs, *dmean;
    void *gbias, *gbias2, *gwp;
};

template <typename T>
__global__ __launch_bounds__(256) void block_mid_fwd_k(const T* __restrict__ xf, const T* __restrict__ xh,
                                                       T* __restrict__ y, int h, int w, int I, int H, int W, int ldy,
                                                       float sy, float sx, float s, unsigned nblk_full,
                                                       long long total_full, long long total_half,
                                                       const PoolFwdJob job) {
    extern __shared__ float sm[];
    constexpr int VEC = 8;
    unsigned bid = blockIdx.x;
    if (bid < (unsigned)job.B) {
        pool_branch_fwd_v8_body<T>(job.part, job.nchunks, job.D, job.inv_p, (const T*)job.wp, (const T*)job.bp,
                                   (const T*)job.bo, (T*)job.m, job.rowbias, bid, sm);
        return;
    }
    bid -= job.B;
    if (bid < nblk_full) {
        const long long first = (long long)bid * (kGateItems * 256) + threadIdx.x;
        if (first < total_full) gate_fwd_items<T, VEC, kGateItems>(xf, y, I, ldy, s, first, 256, total_full);
    } else {
        const long long idx = (long long)(bid - nblk_full) * blockDim.x + threadIdx.x;
        if (idx < total_half) {
            if (H == 2 * h && W == 2 * w)
                gate_bilinear_fwd_x2_item<T, VEC>(xh, y + I / 2, h, w, I, ldy, s, idx);
            else
                gate_bilinear_fwd_item<T, VEC>(xh, y + I / 2, h, w, I, H, W, ldy, sy, sx, s, idx);
        }
    }
}

// Inference: the gated half-resolution scale upsampled into its slice of the concatenation, with the mean branch
// riding in front as above.
template <typename T>
__global__ __launch_bounds__(256) void bilinear_pool_fwd_k(const T* __restrict__ x, T* __restrict__ y, int h, int w, int C,
                                                           int H, int W, int ldy, float sy, float sx, long long total,
                                                           const PoolFwdJob job) {
    extern __shared__ float sm[];
    unsigned bid = blockIdx.x;
    if (bid < (unsigned)job.B) {
        pool_branch_fwd_v8_body<T>(job.part, job.nchunks, job.D, job.inv_p, (const T*)job.wp, (const T*)job.bp,
                                   (const T*)job.bo, (T*)job.m, job.rowbias, bid, sm);
        return;
    }
    const long long idx = (long long)(bid - job.B) * blockDim.x + threadIdx.x;
    if (idx < total) bilinear_fwd_item<T, 8>(x, y, h, w, C, H, W, ldy, sy, sx, idx);
}

template <typename T>
__global__ __launch_bounds__(256) void block_mid_bwd_k(const T* __restrict__ gy, const T* __restrict__ xf,
                                                       const T* __restrict__ xh, T* __restrict__ gxf,
                                                       T* __restrict__ gxh, int h, int w, int I, int ldg, float s,
                                                       unsigned nblk_full, long long total_full,
                                                       long long total_half, const PoolBwdJob job, unsigned npool) {
    // npool = B + D, or B when the per-feature part (the gradients of the pooled layer's weight and bias) is
    // left to deferred work
    extern __shared__ float sm[];
    constexpr int VEC = 8;
    unsigned bid = blockIdx.x;
    if (bid < npool) {
        pool_branch_bwd_v8_block<T>(job.part, job.nchunks, job.B, job.D, job.inv_p, (const T*)job.wp, (const T*)job.m,
                                    job.gs, job.dmean, (T*)job.gbias, (T*)job.gbias2, (T*)job.gwp, (int)bid, sm);
    } else {
        bid -= npool;
        // the half-resolution workgroups (16 gathered taps per item, the slowest to finish) come first in the grid
        const unsigned nblk_half = gridDim.x - npool - nblk_full;
        if (bid >= nblk_half) {
            const long long first = (long long)(bid - nblk_half) * (kGateItems * 256) + threadIdx.x;
            if (first < total_full) gate_bwd_items<T, VEC, kGateItems>(xf, gy, gxf, I, ldg, s, first, 256, total_full);
        } else {
            __builtin_amdgcn_s_setprio(2);
            const long long idx = (long long)bid * blockDim.x + threadIdx.x;
            if (idx < total_half) bilinear_gate_bwd_x2_item<T, VEC>(gy + I / 2, xh, gxh, h, w, I, ldg, s, idx);
        }
    }
}

// y[b,p,c] += v[b,c]  (v in fp32, one rounding)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void add_rowbias_k(T* __restrict__ y, const float* __restrict__ v, int P, int C,
                                                     long long total) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int CV = C / VEC;
    int cq;
    long long bp;
    split_idx(idx, CV, cq, bp);
    const int c = cq * VEC;
    const int b = (int)(bp / P);
    float a[VEC];
    load_f32<T, VEC>(y + bp * C + c, a);
#pragma unroll
    for (int i = 0; i < VEC; ++i) a[i] += v[(long long)b * C + c + i];
    store_f32<T, VEC>(y + bp * C + c, a);
}

// ---------------------------------------------------------------- launch plumbing
// Instantiates KERNEL<T, VEC> for the element type and the widest legal channel vector.
#define PDW_VEC_SWITCH(T, vec, CALL)                       \
    switch (vec) {                                         \
        case 8: if constexpr (sizeof(T) == 2) { CALL(T, 8) } break; \
        case 4: CALL(T, 4) break;                          \
        case 2: CALL(T, 2) break;                          \
        default: CALL(T, 1) break;                         \
    }
#define PDW_TYPE_SWITCH(dtype, vec, CALL)                  \
    switch (dtype) {                                       \
        case kF32: PDW_VEC_SWITCH(float, vec, CALL) break; \
        case kF16: PDW_VEC_SWITCH(f16_t, vec, CALL) break; \
        default: PDW_VEC_SWITCH(bf16_t, vec, CALL) break;  \
    }

static inline size_t esize(int dtype) { return dtype == kF32 ? 4 : 2; }
static inline int gcd_int(int a, int b) {
    while (b) {
        const int t = a % b;
        a = b, b = t;
    }
    return a;
}

static bool grid_for(long long total, unsigned* blocks) {
    const long long nb = (total + 255) / 256;
    if (nb > 0x7fffffffLL) {
        set_error("problem too large for one launch (%lld threads)", total);
        return false;
    }
    *blocks = (unsigned)nb;
    return true;
}

int avgpool_fwd_launch(const void* x, void* y, int B, int H, int W, int C, int h, int w, int dtype, hipStream_t s) {
    const void* ptrs[2] = {x, y};
    const int vec = pick_vec(C, esize(dtype), ptrs, 2);
    const long long total = (long long)B * h * w * (C / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
#define CALL(T, V) hipLaunchKernelGGL((avgpool_fwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (T*)y, H, W, C, h, w, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("avgpool_fwd");
}

int avgpool_bwd_launch(const void* gy, void* gx, int B, int H, int W, int C, int h, int w, int accumulate, int dtype,
                       hipStream_t s) {
    const void* ptrs[2] = {gy, gx};
    const int vec = pick_vec(C, esize(dtype), ptrs, 2);
    unsigned blocks;
    if (H == 2 * h && W == 2 * w) {
        const long long items = (long long)B * h * w * (C / vec);
        if (items == 0) return 0;
        if (!grid_for(items, &blocks)) return 1;
#define CALL(T, V) hipLaunchKernelGGL((avgpool_bwd_x2_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)gy, (T*)gx, h, w, C, accumulate, items);
        PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
        return check_launch("avgpool_bwd");
    }
    const long long total = (long long)B * H * W * (C / vec);
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
#define CALL(T, V) hipLaunchKernelGGL((avgpool_bwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)gy, (T*)gx, H, W, C, h, w, accumulate, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("avgpool_bwd");
}

int bilinear_fwd_launch(const void* x, void* y, int B, int h, int w, int C, int H, int W, int ldy, int dtype,
                        hipStream_t s) {
    const void* ptrs[2] = {x, y};
    const int vec = pick_vec(gcd_int(C, ldy), esize(dtype), ptrs, 2);
    unsigned blocks;
    if (H == 2 * h && W == 2 * w) {
        const long long items = (long long)B * h * w * (C / vec);
        if (items == 0) return 0;
        if (!grid_for(items, &blocks)) return 1;
#define CALL(T, V) hipLaunchKernelGGL((bilinear_fwd_x2_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (T*)y, h, w, C, ldy, items);
        PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
        return check_launch("bilinear_fwd");
    }
    const long long total = (long long)B * H * W * (C / vec);
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W;
#define CALL(T, V) hipLaunchKernelGGL((bilinear_fwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (T*)y, h, w, C, H, W, ldy, sy, sx, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("bilinear_fwd");
}

int bilinear_bwd_launch(const void* gy, void* gx, int B, int h, int w, int C, int H, int W, int ldg, int dtype,
                        hipStream_t s) {
    const void* ptrs[2] = {gy, gx};
    const int vec = pick_vec(gcd_int(C, ldg), esize(dtype), ptrs, 2);
    const long long total = (long long)B * h * w * (C / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W;
    if (H == 2 * h && W == 2 * w && h >= 2 && w >= 2) {
#define CALL(T, V) hipLaunchKernelGGL((bilinear_bwd_x2_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)gy, (T*)gx, h, w, C, ldg, total);
        PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
        return check_launch("bilinear_bwd");
    }
#define CALL(T, V) hipLaunchKernelGGL((bilinear_bwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)gy, (T*)gx, h, w, C, H, W, ldg, sy, sx, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("bilinear_bwd");
}

int gate_bilinear_fwd_launch(const void* x, void* y, int B, int h, int w, int I, int H, int W, int ldy, int dtype,
                             hipStream_t s) {
    const void* ptrs[2] = {x, y};
    const int vec = pick_vec(gcd_int(I / 2, ldy), esize(dtype), ptrs, 2);
    const long long total = (long long)B * H * W * (I / 2 / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W, sc = sqrtf((float)(I / 2));
#define CALL(T, V) hipLaunchKernelGGL((gate_bilinear_fwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (T*)y, h, w, I, H, W, ldy, sy, sx, sc, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("gate_bilinear_fwd");
}

// -1: extents are not exactly doubled (the caller runs the two separate kernels).
int bilinear_gate_bwd_launch(const void* gy, const void* x, void* gx, int B, int h, int w, int I, int H, int W, int ldg,
                             int dtype, hipStream_t s) {
    if (H != 2 * h || W != 2 * w || h < 2 || w < 2) return -1;
    const void* ptrs[3] = {gy, x, gx};
    const int vec = pick_vec(gcd_int(I / 2, ldg), esize(dtype), ptrs, 3);
    const long long total = (long long)B * h * w * (I / 2 / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sc = sqrtf((float)(I / 2));
#define CALL(T, V) hipLaunchKernelGGL((bilinear_gate_bwd_x2_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)gy, (const T*)x, (T*)gx, h, w, I, ldg, sc, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("bilinear_gate_bwd");
}

int gate_pair_fwd_launch(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                         int dtype, hipStream_t s) {
    const void* ptrs[3] = {xf, xh, y};
    const int vec = pick_vec(gcd_int(I / 2, ldy), esize(dtype), ptrs, 3);
    const long long tf = (long long)B * H * W * (I / 2 / vec);
    const long long th = (H == 2 * h && W == 2 * w) ? (long long)B * h * w * (I / 2 / vec) : tf;
    unsigned bf, bh;
    if (tf == 0) return 0;
    if (!grid_for((tf + kGateItems - 1) / kGateItems, &bf) || !grid_for(th, &bh) ||
        (unsigned long long)bf + bh > 0x7fffffffULL)
        return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W, sc = sqrtf((float)(I / 2));
#define CALL(T, V) hipLaunchKernelGGL((gate_pair_fwd_k<T, V>), dim3(bf + bh), dim3(256), 0, s, (const T*)xf, (const T*)xh, (T*)y, h, w, I, H, W, ldy, sy, sx, sc, bf, tf, th);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("gate_pair_fwd");
}

// -1: extents are not exactly doubled (the caller runs the separate kernels).
int gate_pair_bwd_launch(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                         int w, int I, int ldg, int dtype, hipStream_t s) {
    const void* ptrs[5] = {gy, xf, xh, gxf, gxh};
    const int vec = pick_vec(gcd_int(I / 2, ldg), esize(dtype), ptrs, 5);
    const long long tf = (long long)B * H * W * (I / 2 / vec), th = (long long)B * h * w * (I / 2 / vec);
    unsigned bf, bh;
    if (tf == 0 || th == 0) return tf == 0 && th == 0 ? 0 : -1;
    if (!grid_for((tf + kGateItems - 1) / kGateItems, &bf) || !grid_for(th, &bh) ||
        (unsigned long long)bf + bh > 0x7fffffffULL)
        return 1;
    const float sc = sqrtf((float)(I / 2));
    if (H != 2 * h || W != 2 * w || h < 2 || w < 2) {   // any ratio of extents
        const float sy = (float)h / (float)H, sx = (float)w / (float)W;
#define CALL(T, V) hipLaunchKernelGGL((gate_pair_bwd_gen_k<T, V>), dim3(bf + bh), dim3(256), 0, s, (const T*)gy, (const T*)xf, (const T*)xh, (T*)gxf, (T*)gxh, h, w, H, W, I, ldg, sc, sy, sx, bf, tf, th);
        PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
        return check_launch("gate_pair_bwd");
    }
#define CALL(T, V) hipLaunchKernelGGL((gate_pair_bwd_k<T, V>), dim3(bf + bh), dim3(256), 0, s, (const T*)gy, (const T*)xf, (const T*)xh, (T*)gxf, (T*)gxh, h, w, I, ldg, sc, bf, tf, th);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("gate_pair_bwd");
}

// The gate pair and the mean branch (from per-chunk sums `parts`) of a two-scale block in one launch; -1 when the
// combination is not covered (the caller launches the two separately).

int block_mid_fwd_launch(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                         const float* parts, int nparts, const void* wp, const void* bp, const void* bo, void* m,
                         float* rowbias, int P, int D, int dtype, hipStream_t s) {
    const void* ptrs[3] = {xf, xh, y};
    if (pick_vec(gcd_int(I / 2, ldy), esize(dtype), ptrs, 3) != 8 || !pool_branch_v8_ok(wp, nullptr, parts, B, D, dtype))
        return -1;
    const long long tf = (long long)B * H * W * (I / 2 / 8);
    const long long th = (H == 2 * h && W == 2 * w) ? (long long)B * h * w * (I / 2 / 8) : tf;
    unsigned bf, bh;
    if (tf == 0) return -1;
    if (!grid_for((tf + kGateItems - 1) / kGateItems, &bf) || !grid_for(th, &bh) ||
        (unsigned long long)bf + bh + B > 0x7fffffffULL)
        return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W, sc = sqrtf((float)(I / 2));
    const PoolFwdJob job{parts, nparts, B, D, 1.f / (float)P, wp, bp, bo, m, rowbias};
    const size_t lds = (size_t)9 * D * sizeof(float);
    if (dtype == kF16)
        hipLaunchKernelGGL((block_mid_fwd_k<f16_t>), dim3(bf + bh + B), dim3(256), lds, s, (const f16_t*)xf,
                           (const f16_t*)xh, (f16_t*)y, h, w, I, H, W, ldy, sy, sx, sc, bf, tf, th, job);
    else
        hipLaunchKernelGGL((block_mid_fwd_k<bf16_t>), dim3(bf + bh + B), dim3(256), lds, s, (const bf16_t*)xf,
                           (const bf16_t*)xh, (bf16_t*)y, h, w, I, H, W, ldy, sy, sx, sc, bf, tf, th, job);
    return check_launch("block_mid_fwd");
}

// Bilinear upsample (x[B,h,w,C] -> y[..., :C] with pixel stride ldy) and the mean branch in one launch; -1 when the
// combination is not covered.
int bilinear_pool_fwd_launch(const void* x, void* y, int B, int h, int w, int C, int H, int W, int ldy, const float* parts,
                             int nparts, const void* wp, const void* bp, const void* bo, void* m, float* rowbias, int P,
                             int D, int dtype, hipStream_t s) {
    const void* ptrs[2] = {x, y};
    if (pick_vec(gcd_int(C, ldy), esize(dtype), ptrs, 2) != 8 || !pool_branch_v8_ok(wp, nullptr, parts, B, D, dtype)) return -1;
    const long long total = (long long)B * H * W * (C / 8);
    unsigned blocks;
    if (total == 0) return -1;
    if (!grid_for(total, &blocks) || (unsigned long long)blocks + B > 0x7fffffffULL) return 1;
    const float sy = (float)h / (float)H, sx = (float)w / (float)W;
    const PoolFwdJob job{parts, nparts, B, D, 1.f / (float)P, wp, bp, bo, m, rowbias};
    const size_t lds = (size_t)9 * D * sizeof(float);
    if (dtype == kF16)
        hipLaunchKernelGGL((bilinear_pool_fwd_k<f16_t>), dim3(blocks + B), dim3(256), lds, s, (const f16_t*)x, (f16_t*)y, h,
                           w, C, H, W, ldy, sy, sx, total, job);
    else
        hipLaunchKernelGGL((bilinear_pool_fwd_k<bf16_t>), dim3(blocks + B), dim3(256), lds, s, (const bf16_t*)x,
                           (bf16_t*)y, h, w, C, H, W, ldy, sy, sx, total, job);
    return check_launch("bilinear_pool_fwd");
}

int block_mid_bwd_launch(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                         int w, int I, int ldg, const float* parts, int nparts, const void* m, const void* wp,
                         void* gbias, void* gbias2, void* gwp, float* dmean, float* ws, int P, int D, int dtype,
                         hipStream_t s) {
    if (H != 2 * h || W != 2 * w || h < 2 || w < 2) return -1;
    const void* ptrs[5] = {gy, xf, xh, gxf, gxh};
    if (pick_vec(gcd_int(I / 2, ldg), esize(dtype), ptrs, 5) != 8 || !pool_branch_v8_ok(wp, m, parts, B, D, dtype)) return -1;
    const long long tf = (long long)B * H * W * (I / 2 / 8), th = (long long)B * h * w * (I / 2 / 8);
    unsigned bf, bh;
    if (tf == 0) return -1;
    if (!grid_for((tf + kGateItems - 1) / kGateItems, &bf) || !grid_for(th, &bh) ||
        (unsigned long long)bf + bh + B + D > 0x7fffffffULL)
        return 1;
    const float sc = sqrtf((float)(I / 2));
    float* gs = ws + spatial_sum_workspace(B, P, D) / sizeof(float);
    const PoolBwdJob job{parts, nparts, B, D, 1.f / (float)P, wp, m, gs, dmean, gbias, gbias2, gwp};
    const size_t la = (size_t)17 * D * sizeof(float), lb = (size_t)(B + 16 * D) * sizeof(float);
    const size_t lds = la > lb ? la : lb;
    // While reductions are deferred (and the table has room) the weight and bias gradients of the pooled layer
    // join them: they are sums over the images of what the per-image workgroups leave in `gs`, nothing reads
    // them before the backward pass is over, and their D workgroups are the slowest of this launch.
    const bool later = reduce_defer_room() >= (gbias2 ? 3 : 2) && D % 4 == 0;
    const unsigned npool = later ? B : B + D;
    if (dtype == kF16)
        hipLaunchKernelGGL((block_mid_bwd_k<f16_t>), dim3(bf + bh + npool), dim3(256), lds, s, (const f16_t*)gy,
                           (const f16_t*)xf, (const f16_t*)xh, (f16_t*)gxf, (f16_t*)gxh, h, w, I, ldg, sc, bf, tf, th,
                           job, npool);
    else
        hipLaunchKernelGGL((block_mid_bwd_k<bf16_t>), dim3(bf + bh + npool), dim3(256), lds, s, (const bf16_t*)gy,
                           (const bf16_t*)xf, (const bf16_t*)xh, (bf16_t*)gxf, (bf16_t*)gxh, h, w, I, ldg, sc, bf, tf,
                           th, job, npool);
    if (int e = check_launch("block_mid_bwd")) return e;
    if (later) {
        if (reduce_defer_outer(gs, m, gwp, B, D, dtype) != 0) return set_error("block_mid_bwd: deferred job refused"), 1;
        int e = dtype == kF16 ? wgrad_reduce_launch<f16_t>(gs, gbias, B, D, s) : wgrad_reduce_launch<bf16_t>(gs, gbias, B, D, s);
        if (!e && gbias2)
            e = dtype == kF16 ? wgrad_reduce_launch<f16_t>(gs, gbias2, B, D, s) : wgrad_reduce_launch<bf16_t>(gs, gbias2, B, D, s);
        return e;
    }
    return 0;
}

int gate_fwd_launch(const void* x, void* y, long long M, int I, int ldy, int dtype, hipStream_t s) {
    const void* ptrs[2] = {x, y};
    const int vec = pick_vec(gcd_int(I / 2, ldy), esize(dtype), ptrs, 2);
    const long long total = M * (I / 2 / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sc = sqrtf((float)(I / 2));
#define CALL(T, V) hipLaunchKernelGGL((gate_fwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (T*)y, I, ldy, sc, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("gate_fwd");
}

int gate_bwd_launch(const void* x, const void* gy, void* gx, long long M, int I, int ldg, int dtype, hipStream_t s) {
    const void* ptrs[3] = {x, gy, gx};
    const int vec = pick_vec(gcd_int(I / 2, ldg), esize(dtype), ptrs, 3);
    const long long total = M * (I / 2 / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
    const float sc = sqrtf((float)(I / 2));
#define CALL(T, V) hipLaunchKernelGGL((gate_bwd_k<T, V>), dim3(blocks), dim3(256), 0, s, (const T*)x, (const T*)gy, (T*)gx, I, ldg, sc, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("gate_bwd");
}

static void spatial_sum_plan(int B, int P, int* nchunks, int* chunk_len) {
    int n = cdiv(512, B > 0 ? B : 1);  // about two workgroups per CU over the batch
    if (n > cdiv(P, 64)) n = cdiv(P, 64);
    if (n < 1) n = 1;
    *chunk_len = cdiv(P, n);
    *nchunks = cdiv(P, *chunk_len);
}

size_t spatial_sum_workspace(int B, int P, int C) {
    int n, len;
    spatial_sum_plan(B, P, &n, &len);
    return (size_t)B * n * C * sizeof(float);
}

// Pass 1 only: ws[b][chunk][c]; returns the number of chunks through *nchunks.
static int spatial_sum_parts(const void* x, float* ws, int B, int P, int C, int dtype, hipStream_t s, int* nchunks) {
    int n, len;
    spatial_sum_plan(B, P, &n, &len);
    *nchunks = n;
    const void* ptrs[1] = {x};
    int vec = pick_vec(C, esize(dtype), ptrs, 1);
    if (C / vec > 256) return set_error("spatial sum: more than %d channels not supported", 256 * vec), 1;
    const int pl = 256 / (C / vec);
    const size_t lds = (size_t)pl * C * sizeof(float);
    if (lds > 64 * 1024) return set_error("spatial sum: channel count %d too large", C), 1;
#define CALL(T, V) hipLaunchKernelGGL((spatial_sum_part_k<T, V>), dim3(n, B), dim3(256), lds, s, (const T*)x, ws, P, C, len);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("spatial_sum_part");
}

int spatial_sum_launch(const void* x, float* out, float* ws, int B, int P, int C, int dtype, hipStream_t s) {
    int n, len;
    spatial_sum_plan(B, P, &n, &len);
    const void* ptrs[1] = {x};
    int vec = pick_vec(C, esize(dtype), ptrs, 1);
    if (C / vec > 256) return set_error("pdw_spatial_sum: more than %d channels not supported", 256 * vec), 1;
    const int pl = 256 / (C / vec);
    const size_t lds = (size_t)pl * C * sizeof(float);
    if (lds > 64 * 1024) return set_error("pdw_spatial_sum: channel count %d too large", C), 1;
#define CALL(T, V) hipLaunchKernelGGL((spatial_sum_part_k<T, V>), dim3(n, B), dim3(256), lds, s, (const T*)x, ws, P, C, len);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    if (int e = check_launch("spatial_sum_part")) return e;
    const int total = B * C;
    hipLaunchKernelGGL(spatial_sum_final_k, dim3(cdiv(total, 32)), dim3(256), 0, s, ws, out, n, C, total);
    return check_launch("spatial_sum_final");
}

int add_rowbias_launch(void* y, const float* v, int B, int P, int C, int dtype, hipStream_t s) {
    const void* ptrs[1] = {y};
    const int vec = pick_vec(C, esize(dtype), ptrs, 1);
    const long long total = (long long)B * P * (C / vec);
    unsigned blocks;
    if (total == 0) return 0;
    if (!grid_for(total, &blocks)) return 1;
#define CALL(T, V) hipLaunchKernelGGL((add_rowbias_k<T, V>), dim3(blocks), dim3(256), 0, s, (T*)y, v, P, C, total);
    PDW_TYPE_SWITCH(dtype, vec, CALL)
#undef CALL
    return check_launch("add_rowbias");
}

size_t pool_branch_workspace(int B, int P, int D) { return spatial_sum_workspace(B, P, D) + (size_t)B * D * sizeof(float); }

int pool_branch_fwd_launch(const void* x, const void* wp, const void* bp, const void* bo, void* m, float* rowbias,
                           float* ws, int B, int P, int D, int dtype, hipStream_t s, const float* parts, int nparts) {
    int n = nparts;
    if (!parts) {
        if (int e = spatial_sum_parts(x, ws, B, P, D, dtype, s, &n)) return e;
        parts = ws;
    }
    ws = const_cast<float*>(parts);
    const float inv_p = 1.f / (float)P;
    const size_t lds = (size_t)D * sizeof(float);
    const bool v8 = dtype != kF32 && D % 8 == 0 && D <= 128 && (reinterpret_cast<uintptr_t>(wp) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(parts) & 15) == 0;
    if (v8) {
        const size_t l8 = (size_t)9 * D * sizeof(float);
        if (dtype == kF16)
            hipLaunchKernelGGL((pool_branch_fwd_v8_k<f16_t>), dim3(B), dim3(256), l8, s, ws, n, D, inv_p,
                               (const f16_t*)wp, (const f16_t*)bp, (const f16_t*)bo, (f16_t*)m, rowbias);
        else
            hipLaunchKernelGGL((pool_branch_fwd_v8_k<bf16_t>), dim3(B), dim3(256), l8, s, ws, n, D, inv_p,
                               (const bf16_t*)wp, (const bf16_t*)bp, (const bf16_t*)bo, (bf16_t*)m, rowbias);
        return check_launch("pool_branch_fwd");
    }
    switch (dtype) {
        case kF32:
            hipLaunchKernelGGL((pool_branch_fwd_k<float>), dim3(B, (D + 31) / 32), dim3(256), lds, s, ws, n, D, inv_p, (const float*)wp,
                               (const float*)bp, (const float*)bo, (float*)m, rowbias);
            break;
        case kF16:
            hipLaunchKernelGGL((pool_branch_fwd_k<f16_t>), dim3(B, (D + 31) / 32), dim3(256), lds, s, ws, n, D, inv_p, (const f16_t*)wp,
                               (const f16_t*)bp, (const f16_t*)bo, (f16_t*)m, rowbias);
            break;
        default:
            hipLaunchKernelGGL((pool_branch_fwd_k<bf16_t>), dim3(B, (D + 31) / 32), dim3(256), lds, s, ws, n, D, inv_p,
                               (const bf16_t*)wp, (const bf16_t*)bp, (const bf16_t*)bo, (bf16_t*)m, rowbias);
    }
    return check_launch("pool_branch_fwd");
}

int pool_branch_bwd_launch(const void* gy, const void* m, const void* wp, void* gbias, void* gbias2, void* gwp,
                           float* dmean, float* ws, int B, int P, int D, int dtype, hipStream_t s, const float* parts,
                           int nparts) {
    int n = nparts;
    float* gs = ws + spatial_sum_workspace(B, P, D) / sizeof(float);  // the workspace always has both regions
    if (!parts) {
        if (int e = spatial_sum_parts(gy, ws, B, P, D, dtype, s, &n)) return e;
        parts = ws;
    }
    ws = const_cast<float*>(parts);
    const float inv_p = 1.f / (float)P;
    const size_t lds = (size_t)D * 9 * sizeof(float);
    const size_t ldsb = (size_t)B * sizeof(float);
    if (lds > 64 * 1024 || ldsb > 64 * 1024) return set_error("pool branch: extents too large"), 1;
    const bool v8 = dtype != kF32 && D % 8 == 0 && D <= 128 && (reinterpret_cast<uintptr_t>(wp) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(m) & 15) == 0 && (size_t)(B + 16 * D) * sizeof(float) <= 64 * 1024 &&
                    (reinterpret_cast<uintptr_t>(parts) & 15) == 0;
    if (v8) {
        const size_t la = (size_t)17 * D * sizeof(float), lb = (size_t)(B + 16 * D) * sizeof(float);
        const size_t l = la > lb ? la : lb;
        if (dtype == kF16)
            hipLaunchKernelGGL((pool_branch_bwd_v8_k<f16_t>), dim3(B + D), dim3(256), l, s, ws, n, B, D, inv_p,
                               (const f16_t*)wp, (const f16_t*)m, gs, dmean, (f16_t*)gbias, (f16_t*)gbias2, (f16_t*)gwp);
        else
            hipLaunchKernelGGL((pool_branch_bwd_v8_k<bf16_t>), dim3(B + D), dim3(256), l, s, ws, n, B, D, inv_p,
                               (const bf16_t*)wp, (const bf16_t*)m, gs, dmean, (bf16_t*)gbias, (bf16_t*)gbias2,
                               (bf16_t*)gwp);
        return check_launch("pool_branch_bwd");
    }
#define PDW_PB(T)                                                                                                  \
    hipLaunchKernelGGL((pool_branch_bwd_a_k<T>), dim3(B, D > 128 ? (D + 31) / 32 : 1), dim3(256), lds, s, ws, n, D,    \
                       inv_p, (const T*)wp, gs, dmean);                                                            \
    if (int e = check_launch("pool_branch_bwd_a")) return e;                                                       \
    hipLaunchKernelGGL((pool_branch_bwd_b_k<T>), dim3(D), dim3(256), ldsb, s, gs, (const T*)m, B, D, (T*)gbias,    \
                       (T*)gbias2, (T*)gwp);
    switch (dtype) {
        case kF32: PDW_PB(float) break;
        case kF16: PDW_PB(f16_t) break;
        default: PDW_PB(bf16_t) break;
    }
#undef PDW_PB
    return check_launch("pool_branch_bwd_b");
}

}  // namespace pdw

