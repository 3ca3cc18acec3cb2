/*
 * CPU oracle for the pyramid depthwise-conv hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, the smoke check and
 * the cpu_baseline leg of the bench may load it.  The shipped library must not
 * call into it and has no CPU fallback.
 *
 * Everything is computed in IEEE double on NHWC (channels-last) arrays so that a
 * float/half device result can be compared against an effectively exact value.
 * Each routine restates the arithmetic of the reference operator it names
 * (paths relative to the reference tree):
 *
 *   pdwo_dwconv_fwd     pyramid_dwconv/dwconv_triton.py:52-104  (cross-correlation,
 *                       zero outside the image, arbitrary stride/pad/dilation),
 *                       output size per dwconv_triton.py:311-312
 *   pdwo_dwconv_dgrad   exact adjoint of pdwo_dwconv_fwd in x.  For stride 1 and
 *                       2*pad == dil*(k-1) it equals the reference's flipped-tap
 *                       correlation, dwconv_triton.py:154-185
 *   pdwo_dwconv_dgrad_flipped  the reference formula itself, dwconv_triton.py:154-185
 *   pdwo_dwconv_wgrad   exact adjoint of pdwo_dwconv_fwd in w; equals
 *                       dwconv_triton.py:266-296 under the same condition
 *   pdwo_avgpool_fwd/bwd  F.adaptive_avg_pool2d as called at conv_block.py:16;
 *                       integer bins start=floor(i*H/h), end=ceil((i+1)*H/h)
 *                       (the NHWC twin is avgpool_triton.py:42-47,84-89 and
 *                       avgpool_triton.py:166-203 for the gradient)
 *   pdwo_bilinear_fwd/bwd F.interpolate(mode='bilinear', align_corners=False) as
 *                       called at conv_block.py:21 (NHWC twin: up_triton.py:41-125);
 *                       the reference has no backward, the adjoint is used
 *   pdwo_gate_fwd/bwd   conv_block.py:18-19   y = x1 * (x2 / scale)
 *
 * Parity status: the reference ships no golden vectors for any of these, so each
 * routine is pinned in tests/ against torch's CPU library operators in float64,
 * closed forms (delta kernel, all-ones window areas, exact 2x2 means, exact 2x
 * bilinear weights), adjoint identities and finite differences.
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

#define IDX4(b, i, j, c, H, W, C) ((((size_t)(b) * (H) + (i)) * (W) + (j)) * (C) + (c))

static int out_size(int in, int k, int s, int p, int d) {
    /* dwconv_triton.py:311-312 */
    int num = in + 2 * p - d * (k - 1) - 1;
    if (num < 0) return 0;
    return num / s + 1;
}

int pdwo_out_size(int in, int k, int s, int p, int d) { return out_size(in, k, s, p, d); }

void pdwo_dwconv_fwd(const double *x, const double *w, double *y, int B, int H, int W, int C,
                     int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW) {
    const int OH = out_size(H, KH, SH, PH, DH), OW = out_size(W, KW, SW, PW, DW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < OH; ++i)
            for (int j = 0; j < OW; ++j) {
                double *yo = y + IDX4(b, i, j, 0, OH, OW, C);
                for (int c = 0; c < C; ++c) yo[c] = 0.0;
                for (int kh = 0; kh < KH; ++kh) {
                    const int ih = i * SH - PH + kh * DH;
                    if (ih < 0 || ih >= H) continue;
                    for (int kw = 0; kw < KW; ++kw) {
                        const int iw = j * SW - PW + kw * DW;
                        if (iw < 0 || iw >= W) continue;
                        const double *xi = x + IDX4(b, ih, iw, 0, H, W, C);
                        const double *wk = w + ((size_t)kh * KW + kw) * C;
                        for (int c = 0; c < C; ++c) yo[c] += xi[c] * wk[c];
                    }
                }
            }
}

/* dx[b,ih,iw,c] = sum over (kh,kw,i,j) with i*SH-PH+kh*DH == ih (same for w) of gy[b,i,j,c]*w[kh,kw,c] */
void pdwo_dwconv_dgrad(const double *gy, const double *w, double *dx, int B, int H, int W, int C,
                       int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW) {
    const int OH = out_size(H, KH, SH, PH, DH), OW = out_size(W, KW, SW, PW, DW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int ih = 0; ih < H; ++ih)
            for (int iw = 0; iw < W; ++iw) {
                double *dxo = dx + IDX4(b, ih, iw, 0, H, W, C);
                for (int c = 0; c < C; ++c) dxo[c] = 0.0;
                for (int kh = 0; kh < KH; ++kh) {
                    const int ni = ih + PH - kh * DH;
                    if (ni < 0 || ni % SH) continue;
                    const int i = ni / SH;
                    if (i >= OH) continue;
                    for (int kw = 0; kw < KW; ++kw) {
                        const int nj = iw + PW - kw * DW;
                        if (nj < 0 || nj % SW) continue;
                        const int j = nj / SW;
                        if (j >= OW) continue;
                        const double *g = gy + IDX4(b, i, j, 0, OH, OW, C);
                        const double *wk = w + ((size_t)kh * KW + kw) * C;
                        for (int c = 0; c < C; ++c) dxo[c] += g[c] * wk[c];
                    }
                }
            }
}

/* The reference's own dgrad: correlate gy with the 180-degree rotated filter, using the
 * forward padding (dwconv_triton.py:154-185; gy and dx have the same H x W there). */
void pdwo_dwconv_dgrad_flipped(const double *gy, const double *w, double *dx, int B, int H, int W,
                               int C, int KH, int KW, int PH, int PW) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < H; ++i)
            for (int j = 0; j < W; ++j) {
                double *dxo = dx + IDX4(b, i, j, 0, H, W, C);
                for (int c = 0; c < C; ++c) dxo[c] = 0.0;
                for (int kh = 0; kh < KH; ++kh) {
                    const int ih = i - PH + kh;
                    if (ih < 0 || ih >= H) continue;
                    for (int kw = 0; kw < KW; ++kw) {
                        const int iw = j - PW + kw;
                        if (iw < 0 || iw >= W) continue;
                        const double *g = gy + IDX4(b, ih, iw, 0, H, W, C);
                        const double *wk = w + ((size_t)(KH - 1 - kh) * KW + (KW - 1 - kw)) * C;
                        for (int c = 0; c < C; ++c) dxo[c] += g[c] * wk[c];
                    }
                }
            }
}

/* dw[kh,kw,c] = sum_{b,i,j} gy[b,i,j,c] * x[b, i*SH-PH+kh*DH, j*SW-PW+kw*DW, c] */
void pdwo_dwconv_wgrad(const double *x, const double *gy, double *dw, int B, int H, int W, int C,
                       int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW) {
    const int OH = out_size(H, KH, SH, PH, DH), OW = out_size(W, KW, SW, PW, DW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw) {
            double *d = dw + ((size_t)kh * KW + kw) * C;
            for (int c = 0; c < C; ++c) d[c] = 0.0;
            for (int b = 0; b < B; ++b)
                for (int i = 0; i < OH; ++i) {
                    const int ih = i * SH - PH + kh * DH;
                    if (ih < 0 || ih >= H) continue;
                    for (int j = 0; j < OW; ++j) {
                        const int iw = j * SW - PW + kw * DW;
                        if (iw < 0 || iw >= W) continue;
                        const double *g = gy + IDX4(b, i, j, 0, OH, OW, C);
                        const double *xi = x + IDX4(b, ih, iw, 0, H, W, C);
                        for (int c = 0; c < C; ++c) d[c] += g[c] * xi[c];
                    }
                }
        }
}

static inline int bin_start(int i, int in, int out) { return (int)(((long long)i * in) / out); }
static inline int bin_end(int i, int in, int out) {
    return (int)((((long long)(i + 1)) * in + out - 1) / out);
}

void pdwo_avgpool_fwd(const double *x, double *y, int B, int H, int W, int C, int h, int w) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < h; ++i) {
            const int hs = bin_start(i, H, h), he = bin_end(i, H, h);
            for (int j = 0; j < w; ++j) {
                const int ws = bin_start(j, W, w), we = bin_end(j, W, w);
                double *yo = y + IDX4(b, i, j, 0, h, w, C);
                for (int c = 0; c < C; ++c) yo[c] = 0.0;
                for (int ih = hs; ih < he; ++ih)
                    for (int iw = ws; iw < we; ++iw) {
                        const double *xi = x + IDX4(b, ih, iw, 0, H, W, C);
                        for (int c = 0; c < C; ++c) yo[c] += xi[c];
                    }
                const double area = (double)(he - hs) * (double)(we - ws);
                for (int c = 0; c < C; ++c) yo[c] /= area;
            }
        }
}

void pdwo_avgpool_bwd(const double *gy, double *gx, int B, int H, int W, int C, int h, int w) {
    memset(gx, 0, sizeof(double) * (size_t)B * H * W * C);
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < h; ++i) {
            const int hs = bin_start(i, H, h), he = bin_end(i, H, h);
            for (int j = 0; j < w; ++j) {
                const int ws = bin_start(j, W, w), we = bin_end(j, W, w);
                const double area = (double)(he - hs) * (double)(we - ws);
                const double *g = gy + IDX4(b, i, j, 0, h, w, C);
                for (int ih = hs; ih < he; ++ih)
                    for (int iw = ws; iw < we; ++iw) {
                        double *o = gx + IDX4(b, ih, iw, 0, H, W, C);
                        for (int c = 0; c < C; ++c) o[c] += g[c] / area;
                    }
            }
        }
}

/* Source coordinate of destination index `dst`, align_corners=False, no explicit scale
 * factor: src = max((dst+0.5)*in/out - 0.5, 0); i0=floor(src); i1=min(i0+1,in-1). */
static inline void bilinear_src(int dst, int in, int out, int *i0, int *i1, double *lam) {
    double src = ((double)dst + 0.5) * ((double)in / (double)out) - 0.5;
    if (src < 0.0) src = 0.0;
    int lo = (int)floor(src);
    if (lo > in - 1) lo = in - 1;
    *i0 = lo;
    *i1 = lo + 1 < in ? lo + 1 : in - 1;
    *lam = src - (double)lo;
}

/* x [B,h,w,C] -> y [B,H,W,C] */
void pdwo_bilinear_fwd(const double *x, double *y, int B, int h, int w, int C, int H, int W) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < H; ++i) {
            int y0, y1;
            double ly;
            bilinear_src(i, h, H, &y0, &y1, &ly);
            for (int j = 0; j < W; ++j) {
                int x0, x1;
                double lx;
                bilinear_src(j, w, W, &x0, &x1, &lx);
                const double *p00 = x + IDX4(b, y0, x0, 0, h, w, C);
                const double *p01 = x + IDX4(b, y0, x1, 0, h, w, C);
                const double *p10 = x + IDX4(b, y1, x0, 0, h, w, C);
                const double *p11 = x + IDX4(b, y1, x1, 0, h, w, C);
                double *o = y + IDX4(b, i, j, 0, H, W, C);
                for (int c = 0; c < C; ++c)
                    o[c] = (1.0 - ly) * ((1.0 - lx) * p00[c] + lx * p01[c]) +
                           ly * ((1.0 - lx) * p10[c] + lx * p11[c]);
            }
        }
}

/* gy [B,H,W,C] -> gx [B,h,w,C] (transpose of pdwo_bilinear_fwd) */
void pdwo_bilinear_bwd(const double *gy, double *gx, int B, int h, int w, int C, int H, int W) {
    memset(gx, 0, sizeof(double) * (size_t)B * h * w * C);
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < H; ++i) {
            int y0, y1;
            double ly;
            bilinear_src(i, h, H, &y0, &y1, &ly);
            for (int j = 0; j < W; ++j) {
                int x0, x1;
                double lx;
                bilinear_src(j, w, W, &x0, &x1, &lx);
                const double *g = gy + IDX4(b, i, j, 0, H, W, C);
                double *p00 = gx + IDX4(b, y0, x0, 0, h, w, C);
                double *p01 = gx + IDX4(b, y0, x1, 0, h, w, C);
                double *p10 = gx + IDX4(b, y1, x0, 0, h, w, C);
                double *p11 = gx + IDX4(b, y1, x1, 0, h, w, C);
                for (int c = 0; c < C; ++c) {
                    p00[c] += (1.0 - ly) * (1.0 - lx) * g[c];
                    p01[c] += (1.0 - ly) * lx * g[c];
                    p10[c] += ly * (1.0 - lx) * g[c];
                    p11[c] += ly * lx * g[c];
                }
            }
        }
}

/* x [M, I] -> y [M, I/2];  y = x[:, :G] * (x[:, G:] / scale), scale = (I/2)^-0.5 (conv_block.py:10,18-19) */
void pdwo_gate_fwd(const double *x, double *y, long long M, int I) {
    const int G = I / 2;
    const double scale = pow((double)I / 2.0, -0.5);
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < M; ++m)
        for (int c = 0; c < G; ++c) y[m * G + c] = x[m * I + c] * (x[m * I + G + c] / scale);
}

void pdwo_gate_bwd(const double *x, const double *gy, double *gx, long long M, int I) {
    const int G = I / 2;
    const double scale = pow((double)I / 2.0, -0.5);
#pragma omp parallel for schedule(static)
    for (long long m = 0; m < M; ++m)
        for (int c = 0; c < G; ++c) {
            const double g = gy[m * G + c];
            gx[m * I + c] = g * (x[m * I + G + c] / scale);
            gx[m * I + G + c] = g * x[m * I + c] / scale;
        }
}
