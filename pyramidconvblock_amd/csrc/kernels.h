// Internal launcher interface between the C ABI (api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace pdw {

inline int conv_out_size(int in, int k, int s, int p, int d) {
    const int num = in + 2 * p - d * (k - 1) - 1;
    return num < 0 ? 0 : num / s + 1;
}

// dwconv_direct.hip: any stride / padding / dilation
int dwconv_fwd_direct_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW,
                             int SH, int SW, int PH, int PW, int DH, int DW, int dtype, hipStream_t s);
int dwconv_dgrad_direct_launch(const void* gy, const void* w, void* dx, int B, int H, int W, int C, int KH, int KW,
                               int SH, int SW, int PH, int PW, int DH, int DW, int dtype, hipStream_t s);
size_t dwconv_wgrad_direct_workspace(int B, int H, int W, int C, int KH, int KW, int SH, int SW, int PH, int PW,
                                     int DH, int DW);
int dwconv_wgrad_direct_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C,
                               int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW, int dtype,
                               hipStream_t s);
template <typename T>
int wgrad_reduce_launch(const float* part, void* dw, int nparts, int n, hipStream_t s);
struct ReduceJobs;
int reduce_defer_take(ReduceJobs* out);  // moves the recorded jobs out (0 = none); the flush then has nothing to do
int reduce_jobs_launch(const ReduceJobs& jobs, hipStream_t s);
int reduce_defer_begin();
bool reduce_deferring();  // between reduce_defer_begin and the flush on this thread
int reduce_defer_room();  // jobs that can still be recorded (0 when not deferring)
int reduce_defer_outer(const float* g, const void* m, void* out, int B, int D, int dtype);  // -1: not recorded
int reduce_defer_flush(hipStream_t s);

// dwconv_tiled.hip: LDS-tiled forward / input gradient for stride 1, dilation 1, odd KW <= 17.
// Returns -1 if the case is not covered (the caller then uses the direct kernel).
// `add` (optional, [B, OH/2, OW/2, C]): y += a quarter of add at [i/2, j/2].  `pool` (optional, [B, H/2, W/2, C]):
// receives the 2x2 average pool of x.  -1 if the case with either is not covered.
int dwconv_tiled_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW, int PH,
                        int PW, bool flip, int dtype, hipStream_t s, const void* add = nullptr, void* pool = nullptr);

// Fused gate of the matrix-core forward kernel (dwconv_tz.h): the output is C/2 channels wide, written with a pixel
// stride of ldy channels from channel ych on; gs is the gate factor sqrt(C/2).
struct TzGate {
    int ldy, ych;
    float gs;
};
// Forward convolution with the gate of conv_block.py:18-19 applied in the store, and optionally the 2x2 average pool
// of x written to `pool`.  -1: not covered (16-bit types, C % 16 == 0, stride 1, odd square filters that leave room
// for 16 channels per workgroup).
int dwconv_gate_launch(const void* x, const void* w, void* y, void* pool, int B, int H, int W, int C, int K, int PH,
                       int PW, int ldy, int ych, int dtype, hipStream_t s);

// dwconv_wgrad_tiled.hip: LDS-tiled weight gradient for stride 1, dilation 1, odd square filters <= 17.
size_t dwconv_wgrad_tiled_workspace(int B, int H, int W, int C, int KH, int KW, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int KH,
                              int KW, int PH, int PW, int dtype, hipStream_t s);
int dwconv_wgrad_pair_launch(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                             const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int K, int PH, int PW,
                             int dtype, hipStream_t s);

// resample.hip: adaptive average pool, bilinear resize, gate
int avgpool_fwd_launch(const void* x, void* y, int B, int H, int W, int C, int h, int w, int dtype, hipStream_t s);
int avgpool_bwd_launch(const void* gy, void* gx, int B, int H, int W, int C, int h, int w, int accumulate, int dtype,
                       hipStream_t s);
int bilinear_fwd_launch(const void* x, void* y, int B, int h, int w, int C, int H, int W, int ldy, int dtype,
                        hipStream_t s);
int bilinear_bwd_launch(const void* gy, void* gx, int B, int h, int w, int C, int H, int W, int ldg, int dtype,
                        hipStream_t s);
int gate_fwd_launch(const void* x, void* y, long long M, int I, int ldy, int dtype, hipStream_t s);
int gate_pair_fwd_launch(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                         int dtype, hipStream_t s);
int gate_pair_bwd_launch(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                         int w, int I, int ldg, int dtype, hipStream_t s);
int bilinear_pool_fwd_launch(const void* x, void* y, int B, int h, int w, int C, int H, int W, int ldy, const float* parts,
                             int nparts, const void* wp, const void* bp, const void* bo, void* m, float* rowbias, int P,
                             int D, int dtype, hipStream_t s);
int block_mid_fwd_launch(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                         const float* parts, int nparts, const void* wp, const void* bp, const void* bo, void* m,
                         float* rowbias, int P, int D, int dtype, hipStream_t s);
int block_mid_bwd_launch(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                         int w, int I, int ldg, const float* parts, int nparts, const void* m, const void* wp,
                         void* gbias, void* gbias2, void* gwp, float* dmean, float* ws, int P, int D, int dtype,
                         hipStream_t s);
int gate_bilinear_fwd_launch(const void* x, void* y, int B, int h, int w, int I, int H, int W, int ldy, int dtype,
                             hipStream_t s);
int bilinear_gate_bwd_launch(const void* gy, const void* x, void* gx, int B, int h, int w, int I, int H, int W, int ldg,
                             int dtype, hipStream_t s);
int gate_bwd_launch(const void* x, const void* gy, void* gx, long long M, int I, int ldg, int dtype, hipStream_t s);
size_t spatial_sum_workspace(int B, int P, int C);
int spatial_sum_launch(const void* x, float* out, float* ws, int B, int P, int C, int dtype, hipStream_t s);
int add_rowbias_launch(void* y, const float* v, int B, int P, int C, int dtype, hipStream_t s);
size_t pool_branch_workspace(int B, int P, int D);
// parts (optional): per-chunk column sums [B][nparts][D] already computed by the caller (x / gy is then not read)
int pool_branch_fwd_launch(const void* x, const void* wp, const void* bp, const void* bo, void* m, float* rowbias,
                           float* ws, int B, int P, int D, int dtype, hipStream_t s, const float* parts = nullptr,
                           int nparts = 0);
int pool_branch_bwd_launch(const void* gy, const void* m, const void* wp, void* gbias, void* gbias2, void* gwp,
                           float* dmean, float* ws, int B, int P, int D, int dtype, hipStream_t s,
                           const float* parts = nullptr, int nparts = 0);

// dense.hip: thin dense layers on the matrix cores (16-bit types, inner dims <= 128); -1 = not covered
int dense_rows_supported(int K, int NO, int dtype);
// colsum (optional, fp32 [ceil(N/R)][K], K = 64 or 128, R = dense_colsum_rows()): sums of x over groups of R rows
int dense_rows_launch(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                      long long N, int K, int NO, int P, int dtype, hipStream_t s, float* colsum = nullptr,
                      const struct ReduceJobs* rider = nullptr);
// the 128 -> 64 layer over the pixels of [B, H, W] images with the tile sums of x (tiles of 4 rows x 8 columns) and the
// 2x2 average pool of y; -1 = not covered
int dense_rows_pool_launch(const void* x, const void* w, const void* bias, void* y, float* colsum, void* pool, int B,
                           int H, int W, int K, int NO, int dtype, hipStream_t s);
// the 64 -> 128 layer on rows made from the two convolution outputs of a pyramid block (gates and resize where the
// tile is staged); cat (optional) receives the rows; ldf > 0: the scales arrive gated, I / 2 wide, the full one at a pixel
// stride of ldf values; -1 = not covered
int dense_mid_rows_supported(int H, int W, int I, int D, int dtype);
int dense_mid_rows_launch(const void* cf, const void* ch, void* cat, const void* w, const void* bias,
                          const float* rowbias, void* y, int B, int H, int W, int I, int D, int dtype, hipStream_t s,
                          int ldf = 0);
int dense_colsum_supported(int K, int NO, int dtype);
int dense_colsum_rows();
int dense_wgrad_supported(int M, int NO, int dtype);
size_t dense_wgrad_workspace(long long N, int M, int NO);
int dense_wgrad_launch(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, int dtype,
                       hipStream_t s);
// input gradient (optionally with the column sums of gy) and weight gradient of a layer W[O][I] in one launch
// dwconv_f32m.hip: fp32 forward / input gradient on the fp32 matrix cores; -1 = not covered
int dwconv_f32m_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW, int PH, int PW,
                       bool flip, hipStream_t s);
// dense_any.hip: one 32 x 32 tile per wavefront, any dtype, widths that are multiples of 4 (inner width <= 256)
bool dense_any_dims_ok(int K, int NO);
int dense_any_rows_launch(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                          long long N, int K, int NO, int P, int dtype, hipStream_t s);
bool dense_any_wgrad_dims_ok(int M, int NO);
int dense_any_wgrad_launch(const void* a, const void* b, void* dw, void* ws, long long N, int M, int NO, int dtype,
                           int max_chunks, hipStream_t s);
int dense_bwd_pair_supported(int O, int I, int dtype);
int dense_bwd_pair_colsum_supported(int O, int I, int dtype);
int dense_bwd_pair_launch(const void* gy, const void* w, const void* xin, void* dx, float* colsum, void* dw, void* ws,
                          const float* rowbias, int P, long long N, int O, int I, int dtype, hipStream_t s);

// dwconv_bwd3.hip: input gradient (+ pooled branch's) of the full scale and the weight gradients of both scales of a
// two-scale block in one launch; -1 = not covered
int dwconv_bwd3_launch(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0,
                       const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int K, int dtype,
                       hipStream_t s, int* plan_out = nullptr);

// dwconv_fwd2.hip: the forward convolutions of both scales of a two-scale block (the second at half the extents, its
// own input) in one launch; -1 = not covered
bool dwconv_fwd2_covers(int B, int H, int W, int C, int K, int dtype);
// (ldy0 > 0: each convolution with the gate applied in its store, written at pixel strides ldy0 / ldy1 from channels
// ych0 / ych1)
int dwconv_fwd2_launch(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H,
                       int W, int C, int K, int dtype, hipStream_t s, int ldy0 = 0, int ych0 = 0, int ldy1 = 0,
                       int ych1 = 0, const struct PoolFwdJob* mean = nullptr);

}  // namespace pdw
