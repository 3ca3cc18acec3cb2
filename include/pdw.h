/*
 * pdw.h - C ABI of libpdw.so: hand-written gfx950 (MI355X) kernels for the pyramid
 * depthwise-convolution block.
 *
 * The reference (IrisRainbowNeko/PyramidConvBlock) has no FFI: its device code is reached
 * through Triton's `kernel[grid](...)` launches inside Python autograd Functions.  Each
 * entry point below replaces one such launch site (cited per function, paths relative to
 * the reference tree) and is what a binding for that site would call.
 *
 * Conventions
 *   - All tensors are dense channels-last: x[B][H][W][C] with C fastest; depthwise
 *     weights are w[KH][KW][C]  (dwconv_triton.py:413-416).
 *   - Every pointer is a DEVICE pointer borrowed for the duration of the call; nothing is
 *     allocated, freed or synchronised inside the library.  Work is enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the null stream) of the current device.
 *   - `dtype` is one of PDW_F32 / PDW_F16 / PDW_BF16 and applies to every tensor of the
 *     call.  Arithmetic is fp32 (bf16/fp16 products are exact in fp32), one rounding on store.
 *   - Return value: 0 on success; non-zero on invalid arguments or a failed launch, with a
 *     message available from pdw_last_error() (thread-local).
 *   - Callable from several host threads at once.  The library keeps four pieces of state: the per-thread
 *     error text, the per-thread list of summations recorded between pdw_reduce_defer_begin() and
 *     pdw_reduce_defer_flush(), a once-per-process set-up of each large kernel's LDS limit (guarded by
 *     std::call_once), and a bounded cache of launch plans per shape for the launches that hold several problems (behind a
 *     mutex, emptied when it reaches 256 shapes; a plan is a function of the shape alone, so the cache changes no
 *     result).  The no-allocation entry point
 *     has a device buffer of its own, described there.  The library reads no environment variables: every launch plan
 *     is a function of the arguments.
 *   - Non-finite inputs: the matrix-core convolution kernels multiply a window of input pixels somewhat larger
 *     than the filter by zero-padded filter operands, so an Inf or NaN input pixel can turn outputs up to
 *     PDW_NONFINITE_REACH pixels beyond the filter's own footprint into NaN (0 * Inf).  Outputs further away, and
 *     all outputs for finite inputs, are unaffected.  The reference masks its loads (dwconv_triton.py:55-86), so
 *     there the value reaches the footprint only.
 */
#ifndef PDW_H_
#define PDW_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { PDW_F32 = 0, PDW_F16 = 1, PDW_BF16 = 2 };

/* See "Non-finite inputs" above: extra pixels, in every direction, by which a non-finite input value can reach
 * beyond the K x K footprint of the filter. */
#define PDW_NONFINITE_REACH 16

/* ABI version of the library (bumped when a signature changes). */
int pdw_version(void);
/* Text of the last error raised on the calling thread ("" if none). */
const char *pdw_last_error(void);

/* Output extent of a convolution axis: (in + 2p - d(k-1) - 1)/s + 1, 0 if empty.
 * dwconv_triton.py:311-312. */
int pdw_conv_out_size(int in, int k, int stride, int pad, int dil);

/* Depthwise cross-correlation  y[b,i,j,c] = sum_{kh,kw} x[b, i*sh-ph+kh*dh, j*sw-pw+kw*dw, c] * w[kh,kw,c],
 * zero outside the image.  x[B,H,W,C] -> y[B,OH,OW,C].
 * Replaces the launch of _depthwise_conv_kernel_optimized, dwconv_triton.py:325-333 (kernel :20-104). */
int pdw_dwconv_fwd(const void *x, const void *w, void *y, int B, int H, int W, int C, int KH, int KW,
                   int SH, int SW, int PH, int PW, int DH, int DW, int dtype, void *stream);

/* pdw_dwconv_fwd plus the adaptive average pool of the same input to (h, wp): y = conv(x), xp[B,h,wp,C] = pool(x).
 * ConvBlock feeds one tensor to the full-resolution conv and, pooled, to the next scale (conv_block.py:14-16, 41);
 * when the pool halves both extents exactly (and the conv keeps them: stride 1, 2*pad = k-1, pad even, 16-bit
 * types, C % 8 == 0) the conv kernel writes the pooled tensor from its staged input window, otherwise
 * pdw_dwconv_fwd and pdw_avgpool_fwd run one after the other. */
int pdw_dwconv_fwd_pool(const void *x, const void *w, void *y, void *xp, int B, int H, int W, int C, int KH, int KW,
                        int SH, int SW, int PH, int PW, int DH, int DW, int h, int wp, int dtype, void *stream);

/* Inference form of SimpleGate's convolution and gate (conv_block.py:17-19) for stride 1 and a square filter:
 *   y[b,i,j, ych + c] = conv(x)[b,i,j,c] * conv(x)[b,i,j,C/2 + c] * sqrt(C/2),   c < C/2,
 * written with a pixel stride of ldy channels (0: C/2), e.g. straight into its slice of the concatenation of
 * conv_block.py:43, so that the convolution output itself never reaches HBM.  The product is formed from the rounded
 * convolution outputs in fp32 and rounded once, as pdw_gate_fwd does.  xp (may be NULL): the 2x2 average pool of x,
 * [B,H/2,W/2,C] (needs even H, W, pad and 2*pad = K-1).  Returns 3 when the fused kernel does not cover the case
 * (it needs a 16-bit dtype, C % 16 == 0, odd K <= 17, ldy and ych multiples of 8, and K <= 13 when xp is asked for): the
 * caller then runs pdw_dwconv_fwd
 * (or pdw_dwconv_fwd_pool) and pdw_gate_fwd.  No counterpart in the reference, which keeps the convolution output for
 * its backward. */
int pdw_dwconv_fwd_gate(const void *x, const void *w, void *y, void *xp, int B, int H, int W, int C, int K, int pad,
                        int ldy, int ych, int dtype, void *stream);

/* Input gradient (exact adjoint of pdw_dwconv_fwd in x): gy[B,OH,OW,C] -> dx[B,H,W,C]; H,W are
 * the forward INPUT extents.  Fully overwrites dx (no pre-zeroing needed).
 * Replaces the launch of _depthwise_conv_backward_input_kernel, dwconv_triton.py:358-366
 * (kernel :119-203), which is only correct for stride 1 and 2*pad == dil*(k-1); this entry
 * point is correct for every stride/pad/dilation. */
int pdw_dwconv_dgrad(const void *gy, const void *w, void *dx, int B, int H, int W, int C, int KH, int KW,
                     int SH, int SW, int PH, int PW, int DH, int DW, int dtype, void *stream);

/* pdw_dwconv_dgrad plus the gradient of an adaptive average pool taken of the same tensor:
 * dx[B,H,W,C] = dgrad(gy) + avgpool_bwd(gp[B,h,wp,C] -> (H,W)).  This is the sum autograd forms for the
 * tensor that feeds both the full-resolution gate and, through conv_block.py:14, a pooled one
 * (conv_block.py:41).  One kernel when the pool halves both extents exactly (stride 1, dilation 1, 16-bit
 * types, C % 8 == 0), otherwise pdw_dwconv_dgrad followed by an accumulating pdw_avgpool_bwd; either way dx is
 * rounded to the storage type after each of the two terms. */
int pdw_dwconv_dgrad_addpool(const void *gy, const void *w, const void *gp, void *dx, int B, int H, int W, int C,
                             int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW, int h, int wp,
                             int dtype, void *stream);

/* The weight-gradient entry points (pdw_dwconv_wgrad, pdw_dense_wgrad) end with a small kernel that sums their
 * fp32 partial results.  Between pdw_reduce_defer_begin() and pdw_reduce_defer_flush(stream), on the calling host
 * thread, that last step is only recorded (up to 8 of them, further ones run at once as usual), and the flush
 * runs all recorded ones in a single launch on `stream`: the outputs are not valid, and the workspaces must not
 * be reused or freed, until then.  Two entry points take recorded work along in spare workgroups of their own
 * launch, after which the list is empty again: pdw_dense_wgrad (what was recorded before it; its own summation is
 * recorded afterwards) and pdw_dense_fwd_flush below.  pdw_block_mid_bwd records the gradients of the pooled
 * layer's weight and bias (gw_pool, gbias, gbias2) in the same way instead of computing them in its own launch.
 * No counterpart in the reference (its backward launches every kernel separately, dwconv_triton.py:358-385);
 * the ConvBlock backward (conv_block.py:36-49 under autograd) uses it for its weight gradients. */
/* out[i] = sum over p < nparts of parts[p * n + i], added in fp32 in a fixed order and rounded once to `dtype`: the
 * last step of every weight gradient here, on its own for callers that make the partial products themselves (the
 * operator's weight gradient of conv_up / conv_out for widths the dense kernels do not cover is a batched library
 * product over row slabs; autograd of conv_block.py:37, 44).  Subject to the deferral below like the others. */
int pdw_sum_parts(const float *parts, void *out, int nparts, long long n, int dtype, void *stream);
int pdw_reduce_defer_begin(void);
int pdw_reduce_defer_flush(void *stream);
/* pdw_dense_fwd that also runs the reductions recorded so far (see above) in spare workgroups of its own launch;
 * the later pdw_reduce_defer_flush then launches nothing.  For a dense layer that runs after the last kernel that
 * produced the partial results: the input gradient of conv_up at the end of the block's backward. */
int pdw_dense_fwd_flush(const void *x, const void *w, int w_kmajor, const void *bias, const float *rowbias, void *y,
                        long long N, int K, int NO, int P, int dtype, void *stream);

/* Bytes of device scratch pdw_dwconv_wgrad needs for these extents (fp32 partial sums). */
size_t pdw_dwconv_wgrad_workspace_bytes(int B, int H, int W, int C, int KH, int KW, int SH, int SW,
                                        int PH, int PW, int DH, int DW, int dtype);

/* Weight gradient dw[kh,kw,c] = sum_{b,i,j} gy[b,i,j,c] * x[b, i*sh-ph+kh*dh, j*sw-pw+kw*dw, c].
 * Two deterministic passes (per-block fp32 partials in `workspace`, then a fixed-order sum);
 * no atomics, so results are bit-reproducible.  Fully overwrites dw.
 * Replaces the launch of _depthwise_conv_weight_grad_kernel, dwconv_triton.py:377-385
 * (kernel :219-296). */
int pdw_dwconv_wgrad(const void *x, const void *gy, void *dw, void *workspace, size_t workspace_bytes,
                     int B, int H, int W, int C, int KH, int KW, int SH, int SW, int PH, int PW, int DH,
                     int DW, int dtype, void *stream);

/* pdw_dwconv_wgrad for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments and bitwise the same result, but the fp32 partial sums
 * go to a buffer of pdw_static_scratch_bytes() (32 MiB) that is part of the library's device image instead of a
 * caller-supplied workspace.  The call allocates and frees nothing.  Extents whose
 * pdw_dwconv_wgrad_workspace_bytes exceeds that size are rejected with an error (use pdw_dwconv_wgrad).  Every
 * call on a device shares that device's one buffer, so calls that overlap on one device (two streams, two host
 * threads) race; the kernels overwrite what they read of it, nothing has to be cleared between calls.  Not
 * available between pdw_reduce_defer_begin and the flush.  The buffer's address on the current device is looked
 * up on the first call there (hipGetSymbolAddress); pdw_static_scratch_init() does that ahead of time, e.g.
 * before a graph capture begins.  No counterpart in the reference. */
size_t pdw_static_scratch_bytes(void);
int pdw_static_scratch_init(void);
int pdw_dwconv_wgrad_static(const void *x, const void *gy, void *dw, int B, int H, int W, int C, int KH, int KW,
                            int SH, int SW, int PH, int PW, int DH, int DW, int dtype, void *stream);

/* Two pdw_dwconv_wgrad calls of one pyramid block as one call: the same batch, channel count and odd square
 * filter (stride 1, padding K/2, dilation 1) on two tensors of different extents, each with its own workspace
 * (sized by pdw_dwconv_wgrad_workspace_bytes).  For 16-bit types the two problems share one launch, the second
 * one's workgroups starting as compute units finish with the first; otherwise this is the two calls in turn.
 * Results are bitwise those of the separate calls.  Replaces the two launches of
 * _depthwise_conv_weight_grad_kernel (dwconv_triton.py:377-385) that the backward of conv_block.py:41 makes
 * for the block's two scales. */
int pdw_dwconv_wgrad_pair(const void *x0, const void *gy0, void *dw0, void *workspace0, size_t workspace0_bytes,
                          int H0, int W0, const void *x1, const void *gy1, void *dw1, void *workspace1,
                          size_t workspace1_bytes, int H1, int W1, int B, int C, int K, int dtype, void *stream);
/* The three convolution launches at the end of a two-scale block's backward pass that do not depend on one another, as
 * one launch (backward of conv_block.py:14-16, 41 under autograd): dx = the full scale's input gradient from gy0 and w0
 * plus a quarter of gp per 2x2 block (what pdw_dwconv_dgrad_addpool computes; gp [B,H/2,W/2,C] is the pooled scale's
 * input gradient), dw0 = the full scale's weight gradient from x0 and gy0, dw1 = the half scale's from x1 and gy1
 * [B,H/2,W/2,C].  Square odd filter, stride 1, padding K/2, even H and W; workspaces as for the two pdw_dwconv_wgrad
 * calls.  Status 3 (nothing launched) when the fused kernel does not cover the case (fp32, C % 16, images narrower than
 * 33 columns...): the caller then makes the three calls.  dx is bitwise that of the separate call; the weight gradients
 * are the same sums taken over other bands of the images (the launch chooses its own band heights: as few bands as fill
 * the chip together with the other two problems), so they can differ from pdw_dwconv_wgrad's in the last bit, and are
 * the same from call to call.  Between pdw_reduce_defer_begin/flush the two summations are recorded like any other. */
int pdw_dwconv_bwd3(const void *gy0, const void *w0, const void *gp, void *dx, const void *x0, void *dw0,
                    void *workspace0, size_t workspace0_bytes, const void *x1, const void *gy1, void *dw1,
                    void *workspace1, size_t workspace1_bytes, int B, int H, int W, int C, int K, int dtype,
                    void *stream);
/* Host only: the cut pdw_dwconv_bwd3 would choose for these extents (launch planning of the same call sites; no
 * reference counterpart, the Triton grid is fixed at dwconv_triton.py:318-333).  bands[0..2] receive the number of row
 * bands per image of the input gradient, the full scale's and the half scale's weight gradient (each >= 1).  Returns 0,
 * 3 when pdw_dwconv_bwd3 does not cover the case, 1 on invalid arguments.  Touches no device. */
int pdw_dwconv_bwd3_plan(int B, int H, int W, int C, int K, int dtype, int *bands);

/* The forward convolutions of both scales of a two-scale block as one launch (conv_block.py:14-16 at scales 1 and
 * 1/2): y0 = conv(x0, w0) on [B,H,W,C] and y1 = conv(x1, w1) on [B,H/2,W/2,C], x1 being an input (the caller's 2x2
 * average pool of x0, pdw_avgpool_fwd).  Square odd filter, stride 1, padding K/2, even H and W.  Status 3 (nothing
 * launched) when the fused kernel does not cover the case (fp32, C % 8, images narrower than 33 columns;
 * pdw_dwconv_fwd2_supported says so beforehand, so that a caller can have the full scale's convolution write the pool
 * instead: pdw_dwconv_fwd_pool): the caller then makes two pdw_dwconv_fwd calls.  Results are bitwise those of the
 * separate calls. */
int pdw_dwconv_fwd2_supported(int B, int H, int W, int C, int K, int dtype); /* 1: pdw_dwconv_fwd2 takes the case */
int pdw_dwconv_fwd2(const void *x0, const void *w0, void *y0, const void *x1, const void *w1, void *y1, int B, int H,
                    int W, int C, int K, int dtype, void *stream);
/* pdw_dwconv_fwd2 with the block's mean branch in B more workgroups of the same launch (conv_block.py:46-49:
 * m[b] = mean of x over the positions, rounded; rowbias[b] = m[b] w_pool^T + b_pool + b_out in fp32, the row that
 * pdw_dense_fwd adds to every output row of image b), from the sums of x over groups of positions that conv_up's
 * kernel left in parts [B][nparts][D] (pdw_dense_fwd_colsum): what pdw_pool_branch_fwd_parts computes, bitwise.  The
 * branch is three dependent trips to memory and a few kilobytes; in a launch of its own, or in one that saturates the
 * memory system, it costs microseconds, here it runs beside the convolutions.  Status 3 (nothing launched) where
 * pdw_dwconv_fwd2 does not take the case or the branch is not covered (D % 8, D > 128).  ldy0 = ldy1 = 0: the
 * convolution outputs y0, y1 as pdw_dwconv_fwd2 writes them; both > 0: the gated outputs of pdw_dwconv_fwd2_gate at these
 * pixel strides and channel offsets (inference). */
int pdw_dwconv_fwd2_mean(const void *x0, const void *w0, void *y0, int ldy0, int ych0, const void *x1, const void *w1,
                         void *y1, int ldy1, int ych1, int B, int H, int W, int C, int K, const float *parts,
                         int nparts, const void *w_pool, const void *b_pool, const void *b_out, void *m,
                         float *rowbias, int P, int D, int dtype, void *stream);

/* pdw_dwconv_fwd2 with the gate of pdw_dwconv_fwd_gate applied in the store of each scale (inference: neither
 * convolution output reaches HBM): y0[b,i,j, ych0 + c] and y1[b,i,j, ych1 + c], c < C/2, at pixel strides of ldy0 / ldy1
 * channels (0: C/2).  Covered where pdw_dwconv_fwd2 is and C % 16 == 0, strides and offsets multiples of 8;
 * status 3 otherwise (the caller then makes two pdw_dwconv_fwd_gate calls).  Results bitwise those calls'. */
int pdw_dwconv_fwd2_gate(const void *x0, const void *w0, void *y0, int ldy0, int ych0, const void *x1, const void *w1,
                         void *y1, int ldy1, int ych1, int B, int H, int W, int C, int K, int dtype, void *stream);

/* Adaptive average pooling x[B,H,W,C] -> y[B,h,w,C]; bin i covers [floor(i*H/h), ceil((i+1)*H/h)).
 * Replaces F.adaptive_avg_pool2d at conv_block.py:16 and the launch at avgpool_triton.py:225-229
 * (kernel :14-107; integer bin arithmetic here instead of the fp16 one at :42-47). */
int pdw_avgpool_fwd(const void *x, void *y, int B, int H, int W, int C, int h, int w, int dtype, void *stream);

/* Its gradient gy[B,h,w,C] -> gx[B,H,W,C], gather form (no atomics).  With accumulate != 0 the result
 * is added to gx (fp32 add, one rounding), otherwise gx is fully overwritten.
 * Replaces avgpool_triton.py:253-257 (kernel :118-203). */
int pdw_avgpool_bwd(const void *gy, void *gx, int B, int H, int W, int C, int h, int w, int accumulate, int dtype,
                    void *stream);

/* Bilinear resize, align_corners=False, no explicit scale factor: x[B,h,w,C] -> y[B,H,W,C].  Output pixels are
 * ldy elements apart (0 = dense, ldy = C), so the result can be written into a channel slice of a wider tensor
 * (the torch.cat of conv_block.py:43).
 * Replaces F.interpolate at conv_block.py:21 and the launch at up_triton.py:157-161 (kernel :14-125). */
int pdw_bilinear_fwd(const void *x, void *y, int B, int h, int w, int C, int H, int W, int ldy, int dtype,
                     void *stream);

/* Its gradient gy[B,H,W,C] (pixels ldgy elements apart, 0 = dense) -> gx[B,h,w,C], transpose of the above in
 * gather form.  The reference has no backward for up_triton.py; inside ConvBlock autograd supplies
 * upsample_bilinear2d_backward. */
int pdw_bilinear_bwd(const void *gy, void *gx, int B, int h, int w, int C, int H, int W, int ldgy, int dtype,
                     void *stream);

/* Gate  y[m,c] = x[m,c] * x[m,G+c] * sqrt(G),  G = I/2,  x[M,I] -> y[M,G] with rows ldy elements apart
 * (0 = dense)   (conv_block.py:10,18-19). */
int pdw_gate_fwd(const void *x, void *y, long long M, int I, int ldy, int dtype, void *stream);
/* gx[m,c] = gy*x[m,G+c]*sqrt(G);  gx[m,G+c] = gy*x[m,c]*sqrt(G); gy rows ldgy elements apart (0 = dense). */
int pdw_gate_bwd(const void *x, const void *gy, void *gx, long long M, int I, int ldgy, int dtype, void *stream);

/* Gate followed by the bilinear resize, in one pass: x[B,h,w,I] -> y[B,H,W,I/2], pixels of y ldy elements apart
 * (0 = dense).  Each gate value is rounded to the storage type before it is interpolated, as when pdw_gate_fwd
 * and pdw_bilinear_fwd run one after the other; the gated tensor itself is never written.
 * Replaces conv_block.py:18-21 for a branch with scale_factor != 1. */
int pdw_gate_bilinear_fwd(const void *x, void *y, int B, int h, int w, int I, int H, int W, int ldy, int dtype,
                          void *stream);
/* Gradient of the pair for exactly doubled extents (H = 2h, W = 2w, h,w >= 2; anything else is an error and the
 * caller runs pdw_bilinear_bwd then pdw_gate_bwd): gy[B,H,W,I/2] (pixels ldgy apart) and the gate's input
 * x[B,h,w,I] -> gx[B,h,w,I].  What autograd derives for conv_block.py:18-21. */
int pdw_bilinear_gate_bwd(const void *gy, const void *x, void *gx, int B, int h, int w, int I, int H, int W,
                          int ldgy, int dtype, void *stream);

/* The two gates of a block with scales (1, s) in one launch: y[..., 0:G] = gate(xf[B,H,W,I]) and
 * y[..., G:2G] = bilinear(gate(xh[B,h,w,I])) -> (H,W), G = I/2, pixels of y ldy elements apart (0 = 2G): the
 * torch.cat of conv_block.py:43 written directly (conv_block.py:18-21 for both entries of self.gates). */
int pdw_gate_pair_fwd(const void *xf, const void *xh, void *y, int B, int H, int W, int h, int w, int I, int ldy,
                      int dtype, void *stream);
/* Its gradient, one launch for any extents (exactly doubled ones take a kernel with fixed taps): gy[B,H,W,2G] (pixels
 * ldgy apart) -> gxf[B,H,W,I], gxh[B,h,w,I]; the same bits as pdw_gate_bwd on the first half and pdw_bilinear_bwd +
 * pdw_gate_bwd on the second. */
int pdw_gate_pair_bwd(const void *gy, const void *xf, const void *xh, void *gxf, void *gxh, int B, int H, int W,
                      int h, int w, int I, int ldgy, int dtype, void *stream);

/* Per-image sum over positions: x[B,P,C] -> out[B,C] (fp32), two deterministic passes through `workspace`.
 * Replaces x.mean(dim=(1,2)) at conv_block.py:46 (divide by P on the host side) and, in the backward, the
 * reduction of the broadcast add at conv_block.py:49. */
size_t pdw_spatial_sum_workspace_bytes(int B, int P, int C);
int pdw_spatial_sum(const void *x, float *out, void *workspace, size_t workspace_bytes, int B, int P, int C,
                    int dtype, void *stream);

/* In place y[b,p,c] += v[b,c] (v fp32 [B,C]): the broadcast add of the pooled branch, conv_block.py:49,
 * and its mirror in the backward (the gradient of the mean, conv_block.py:46). */
int pdw_add_rowbias(void *y, const float *v, int B, int P, int C, int dtype, void *stream);

/* Pooled branch of the block, forward (conv_block.py:46-47 plus the bias of :44): per image b,
 *   m[b,:]       = mean over the P positions of x[b,:,:]            (rounded to the element type, kept for backward)
 *   rowbias[b,o] = sum_c m[b,c] * w_pool[o,c] + b_pool[o] + b_out[o] (fp32; b_pool / b_out may be NULL)
 * rowbias is what pdw_dense_fwd / pdw_add_rowbias then broadcast over the positions (conv_block.py:49). */
size_t pdw_pool_branch_workspace_bytes(int B, int P, int D);
int pdw_pool_branch_fwd(const void *x, const void *w_pool, const void *b_pool, const void *b_out, void *m,
                        float *rowbias, void *workspace, size_t workspace_bytes, int B, int P, int D, int dtype,
                        void *stream);
/* Its backward from gy[B,P,D]: gbias[o] = sum over all positions of gy (the gradient of both biases; gbias2,
 * if not null, receives a second copy so that each bias owns its gradient tensor),
 * gw_pool[o,c] = sum_b gs[b,o] * m[b,c] with gs the per-image column sums of gy, and
 * dmean[b,c] = (1/P) * sum_o gs[b,o] * w_pool[o,c] (fp32), the per-image term that the mean's gradient
 * adds to every position of dx. */
int pdw_pool_branch_bwd(const void *gy, const void *m, const void *w_pool, void *gbias, void *gbias2, void *gw_pool,
                        float *dmean, void *workspace, size_t workspace_bytes, int B, int P, int D, int dtype,
                        void *stream);

/* The same two steps from per-chunk column sums the caller already has (parts[B][nparts][D], fp32, chunks of
 * equal or unequal length covering the P positions of an image), e.g. from pdw_dense_fwd_colsum: x / gy is not
 * read again.  pdw_pool_branch_bwd_parts still takes the workspace of pdw_pool_branch_workspace_bytes. */
int pdw_pool_branch_fwd_parts(const float *parts, int nparts, const void *w_pool, const void *b_pool,
                              const void *b_out, void *m, float *rowbias, int B, int P, int D, int dtype,
                              void *stream);
int pdw_pool_branch_bwd_parts(const float *parts, int nparts, const void *m, const void *w_pool, void *gbias,
                              void *gbias2, void *gw_pool, float *dmean, void *workspace, size_t workspace_bytes,
                              int B, int P, int D, int dtype, void *stream);

/* The middle of a two-scale block as one launch each way: pdw_gate_pair_fwd together with
 * pdw_pool_branch_fwd_parts, and pdw_gate_pair_bwd together with pdw_pool_branch_bwd_parts (same arguments, same
 * results; the mean branch is a handful of latency-bound workgroups that ride in the gate kernel's grid).  When
 * the combination is not covered (fp32, D > 128, unaligned slices) the two kernels are launched one after the
 * other.  P = positions per image of the tensor whose chunk sums `parts` holds (conv_block.py:40-49).  Between
 * pdw_reduce_defer_begin and the flush, pdw_block_mid_bwd leaves gw_pool, gbias and gbias2 to the deferred work
 * (they are sums over the images of values it writes into `workspace`, which must stay in place until then). */
int pdw_block_mid_fwd(const void *xf, const void *xh, void *y, int B, int H, int W, int h, int w, int I, int ldy,
                      const float *parts, int nparts, const void *w_pool, const void *b_pool, const void *b_out,
                      void *m, float *rowbias, int P, int D, int dtype, void *stream);
int pdw_block_mid_bwd(const void *gy, const void *xf, const void *xh, void *gxf, void *gxh, int B, int H, int W,
                      int h, int w, int I, int ldgy, const float *parts, int nparts, const void *m,
                      const void *w_pool, void *gbias, void *gbias2, void *gw_pool, float *dmean, void *workspace,
                      size_t workspace_bytes, int P, int D, int dtype, void *stream);
/* The middle of the two-scale block at inference: the gated half-resolution scale xh[B,h,w,G] upsampled
 * (pdw_bilinear_fwd) into y[..., :G] with pixel stride ldy (its slice of the concatenation), together with
 * pdw_pool_branch_fwd_parts, in one launch where the combination is covered and one after the other otherwise.
 * conv_block.py:20-21, :46-49. */
int pdw_block_mid_infer(const void *xh, void *y, int B, int H, int W, int h, int w, int G, int ldy,
                        const float *parts, int nparts, const void *w_pool, const void *b_pool, const void *b_out,
                        void *m, float *rowbias, int P, int D, int dtype, void *stream);

/* Dense layers of the block on the matrix cores.  bf16/fp16 with K <= 128, NO <= 128, K % 8 == 0, NO % 8 == 0 run the
 * tiled kernels (persistent workgroups, weights in LDS, a 32-row tile per wavefront over all features); fp32 and
 * every other width with K % 4 == 0, NO % 4 == 0, K <= 256 run one 32 x 32 result tile per wavefront
 * (v_mfma_f32_32x32x2_f32 in fp32), forward, input gradient and weight gradient alike.  pdw_dense_supported says
 * whether a shape is covered - callers use a library GEMM otherwise.
 *   y[n,o] = sum_k x[n,k] * W(o,k) + bias[o] + rowbias[n / P][o]        x[N,K] -> y[N,NO]
 * W(o,k) = w[o*K + k] (w_kmajor == 0, the nn.Linear layout) or w[k*NO + o] (w_kmajor != 0, which gives the
 * input gradient of a layer from its own weight without a transpose).  bias (element type) and rowbias
 * (fp32 [ceil(N/P), NO]) may be NULL.  Replaces nn.Linear at conv_block.py:37 and :44 together with the
 * broadcast add of conv_block.py:49, and the matching input-gradient GEMMs of the backward. */
int pdw_dense_supported(int K, int NO, int dtype);
int pdw_dense_fwd(const void *x, const void *w, int w_kmajor, const void *bias, const float *rowbias, void *y,
                  long long N, int K, int NO, int P, int dtype, void *stream);

/* pdw_dense_fwd that also writes colsum[t][k] = sum of x[n,k] over the rows n of the t-th group of R rows (fp32,
 * ceil(N/R) x K, R = pdw_dense_colsum_rows(), the kernel's row tile): with R | P these are per-chunk sums of each
 * image, which pdw_pool_branch_fwd_parts /
 * _bwd_parts take in place of a second pass over x (the x.mean of conv_block.py:46 and its gradient ride on
 * conv_up, conv_block.py:37, and on the input gradient of conv_out, conv_block.py:44).  K = 64 or 128 only:
 * pdw_dense_colsum_supported. */
int pdw_dense_colsum_supported(int K, int NO, int dtype);
int pdw_dense_colsum_rows(void);
int pdw_dense_fwd_colsum(const void *x, const void *w, int w_kmajor, const void *bias, const float *rowbias, void *y,
                         float *colsum, long long N, int K, int NO, int P, int dtype, void *stream);

/* pdw_dense_fwd_colsum for the pixels of x[B,H,W,K] (no rowbias) that also writes the 2x2 average pool of y,
 * pool[B,H/2,W/2,NO] = what pdw_avgpool_fwd makes of y (conv_block.py:37 together with the pooling of conv_block.py:16
 * for the second scale: the convolutions of both scales can then start together, pdw_dwconv_fwd2).  The kernel's row
 * tiles are blocks of 4 image rows x 8 columns, so colsum[t] are the sums of x over such blocks (still H*W/32 per
 * image, image after image).  Status 3 (nothing launched) where not covered: 16-bit types, (K, NO) = (128, 64),
 * (96, 48) or (64, 32), H % 4 == 0, W % 8 == 0 only. */
int pdw_dense_fwd_colsum_pool(const void *x, const void *w, const void *bias, void *y, float *colsum, void *pool, int B,
                              int H, int W, int K, int NO, int dtype, void *stream);

/* The output layer of a two-scale block on rows made where they are multiplied (conv_block.py:18-21, 41-44 and :44
 * as one launch): y[b,i,j,:] = [ gate(cf[b,i,j]) | bilinear resize to H x W of gate(ch[b]) at (i,j) ] w^T + bias +
 * rowbias[b], with cf[B,H,W,I] and ch[B,H/2,W/2,I] the convolution outputs of the two scales, gate(v) = v[:I/2] *
 * v[I/2:] * sqrt(I/2) rounded to `dtype`, w[D][I], bias[D] or NULL, rowbias fp32 [B][D] or NULL.  cat[B,H,W,I] (or
 * NULL) receives the rows, which the backward pass reads again.  Bitwise what pdw_gate_pair_fwd (or pdw_block_mid_fwd)
 * followed by pdw_dense_fwd produce; the gated tensor is not read back from memory.  ldf > 0 (inference, after
 * pdw_dwconv_fwd2_gate): both scales arrive gated, cf[B,H,W,I/2] at a pixel stride of ldf values and ch[B,H/2,W/2,I/2],
 * only the resize is left to do and cat must be NULL.  Status 3 (nothing launched) where not covered
 * (pdw_dense_fwd_gated_supported says so beforehand): 16-bit types, H % 4 == 0, W % 8 == 0, I a multiple of 16 up to 64,
 * D a multiple of 8 up to 128 with D + 8 >= 1.5 I (I = 64, D = 128 runs the variant with compile-time extents). */
int pdw_dense_fwd_gated_supported(int H, int W, int I, int D, int dtype);
int pdw_dense_fwd_gated(const void *cf, const void *ch, void *cat, const void *w, const void *bias,
                        const float *rowbias, void *y, int B, int H, int W, int I, int D, int ldf, int dtype,
                        void *stream);

/* Weight gradient of such a layer: dw[m,o] = sum_n a[n,m] * b[n,o]  (a[N,M], b[N,NO] -> dw[M,NO]), fp32
 * accumulation, two deterministic passes through `workspace` (no atomics). */
size_t pdw_dense_wgrad_workspace_bytes(long long N, int M, int NO);
int pdw_dense_wgrad(const void *a, const void *b, void *dw, void *workspace, size_t workspace_bytes, long long N,
                    int M, int NO, int dtype, void *stream);

/* Both gradients of a dense layer y = x W^T (W[O][I]) that need gy, in one launch: dx[N,I] = gy W
 * (+ rowbias[n / P], fp32 [ceil(N/P), I], may be NULL; P >= 32) and dw[O,I] = gy^T x (workspace and summation as pdw_dense_wgrad, size pdw_dense_wgrad_workspace_bytes(N, O, I)); with
 * colsum != NULL also the sums of gy over groups of pdw_dense_colsum_rows() rows, as pdw_dense_fwd_colsum.  The two
 * products share the chip instead of following each other (each alone leaves half of it waiting on memory).
 * Covered (pdw_dense_bwd_pair_supported): 16-bit types and the widths pdw_dense_fwd and pdw_dense_wgrad both cover
 * (multiples of 8 up to 128, at most 8 tiles of 32 x 32 in dW); (O, I) = (128, 64), (64, 128), (64, 32), (32, 64) -
 * the backward of conv_out and conv_up, conv_block.py:44 and :37, in ConvBlock(128) and ConvBlock(64) - run with
 * the extents as compile-time constants; colsum where pdw_dense_bwd_pair_colsum_supported says so (the widths
 * pdw_dense_fwd_colsum covers); other shapes take pdw_dense_fwd(w_kmajor) and pdw_dense_wgrad.  Unlike pdw_dense_wgrad it carries no recorded summations along. */
int pdw_dense_bwd_pair_supported(int O, int I, int dtype);
int pdw_dense_bwd_pair_colsum_supported(int O, int I, int dtype); /* ... with the tile sums (`colsum` != NULL) */
int pdw_dense_bwd_pair(const void *gy, const void *w, const void *x, void *dx, float *colsum, void *dw, void *workspace,
                       size_t workspace_bytes, const float *rowbias, int P, long long N, int O, int I, int dtype,
                       void *stream);

/* The whole block of conv_block.py:25-49 (scales (1, 1/2), conv_up without bias) as one host call each way: the
 * launch sequence of the entry points above (forward: conv_up with the pool of its result, the convolutions of both
 * scales with the mean branch, conv_out on rows it makes from their outputs, writing cat: 3 launches for D = 128,
 * I = 64, H % 4 == 0, W % 8 == 0; other widths that pdw_dense_fwd_gated covers pool in a launch of their own; else the
 * gates and the mean branch are one launch before conv_out; backward: 5
 * launches and one summation launch)
 * without a host interpreter between them.  Covered when pdw_convblock_supported: 16-bit dtype, even H, W >= 4 with
 * H*W a multiple of pdw_dense_colsum_rows(), layer widths D (block), I (inner, a multiple of 16) that the dense
 * kernels and pdw_dense_bwd_pair cover (multiples of 8 up to 128; D = 128, 96 and 64 with I = D / 2 run variants with
 * compile-time extents), odd K.  All tensors channels-last and contiguous, all
 * parameters in `dtype`: x, y[B,H,W,D]; w_up[I,D]; w_dw0, w_dw1[K,K,I]; w_pool[D,D]; w_out[D,I]; b_pool, b_out[D] or
 * NULL.  The forward writes what the backward reads again: a = conv_up(x), c0 = conv(a), xp = pool(a)[B,H/2,W/2,I],
 * c1 = conv(xp), cat[B,H,W,I] (the gated scales), m[B,D] (per-image mean of x).  The backward overwrites dx and the
 * parameter gradients (gb_pool, gb_out may be NULL).  Workspaces: device scratch of the stated size, free for reuse
 * when the call's work on `stream` is done.  Results are bitwise those of the calls listed above made one by one.
 * Replaces the Python-level sequence of ConvBlock.forward, conv_block.py:36-49, and its autograd backward. */
int pdw_convblock_supported(int B, int H, int W, int D, int I, int K, int dtype);
/* Inference forward of the same block (same coverage): y only.  conv_up (which also pools its result for the second
 * scale where its kernel can, pdw_dense_fwd_colsum_pool); then, where pdw_dense_fwd_gated covers the widths and
 * extents, the convolutions of both scales with the mean branch in their launch (pdw_dwconv_fwd2_mean) and conv_out on
 * rows it makes itself from their outputs: three launches, no gated or concatenated tensor in memory.  Elsewhere, for
 * filters up to 13, each
 * scale's convolution with the gate applied in its store (both as one launch, pdw_dwconv_fwd2_gate, or
 * pdw_dwconv_fwd_gate twice, the full-resolution one then pooling its input), the half-resolution gate upsampled into
 * its slice of the concatenation with the mean branch (pdw_block_mid_infer), conv_out: neither convolution output is
 * written to HBM; larger filters at those widths run the launches of pdw_convblock_fwd on workspace tensors (measured
 * faster than the gated store of their 8-channel slices).  Every intermediate lives in `workspace`
 * (pdw_convblock_infer_workspace_bytes).  Same arithmetic as
 * pdw_convblock_fwd.  Replaces ConvBlock.forward under torch.no_grad(), conv_block.py:36-49 with :13-22. */
size_t pdw_convblock_infer_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype);
int pdw_convblock_infer(const void *x, const void *w_up, const void *w_dw0, const void *w_dw1, const void *w_pool,
                        const void *b_pool, const void *w_out, const void *b_out, void *y, void *workspace,
                        size_t workspace_bytes, int B, int H, int W, int D, int I, int K, int dtype, void *stream);
size_t pdw_convblock_fwd_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype);
int pdw_convblock_fwd(const void *x, const void *w_up, const void *w_dw0, const void *w_dw1, const void *w_pool,
                      const void *b_pool, const void *w_out, const void *b_out, void *a, void *c0, void *xp, void *c1,
                      void *cat, void *m, void *y, void *workspace, size_t workspace_bytes, int B, int H, int W,
                      int D, int I, int K, int dtype, void *stream);
size_t pdw_convblock_bwd_workspace_bytes(int B, int H, int W, int D, int I, int K, int dtype);
int pdw_convblock_bwd(const void *gy, const void *x, const void *a, const void *c0, const void *xp, const void *c1,
                      const void *cat, const void *m, const void *w_up, const void *w_dw0, const void *w_dw1,
                      const void *w_pool, const void *w_out, void *dx, void *gw_up, void *gw_dw0, void *gw_dw1,
                      void *gw_pool, void *gb_pool, void *gw_out, void *gb_out, void *workspace,
                      size_t workspace_bytes, int B, int H, int W, int D, int I, int K, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PDW_H_ */
