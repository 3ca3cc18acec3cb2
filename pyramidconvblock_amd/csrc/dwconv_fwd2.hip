// Dispatch of the block's two forward convolution launches as one (dwconv_fwd2.h) by filter size.
#include <cmath>

#include "common.h"
#include "kernels.h"
#include "pool_branch.h"

namespace pdw {

#define PDW_FWD2_DECL(K)                                                                                              \
    int dwconv_fwd2_k##K(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H, \
                         int W, int C, int dtype, hipStream_t s, const TzGate* gate0, const TzGate* gate1,   \
                         const PoolFwdJob* mean);
PDW_FWD2_DECL(3) PDW_FWD2_DECL(5) PDW_FWD2_DECL(7) PDW_FWD2_DECL(9) PDW_FWD2_DECL(11) PDW_FWD2_DECL(13) PDW_FWD2_DECL(15)
PDW_FWD2_DECL(17)
#undef PDW_FWD2_DECL

// Whether dwconv_fwd2_launch takes the case (aligned tensors assumed): what a caller checks before it pools the
// input with a launch of its own instead of letting the full scale's convolution write the pool.
bool dwconv_fwd2_covers(int B, int H, int W, int C, int K, int dtype) {
    if (tune_env("PDW_NO_FWD2")) return false;
    if (dtype == kF32 || K < 3 || K > 17 || !(K & 1) || C % 8 != 0 || (H & 1) || (W & 1) || B < 1 || H < 2 || W < 2) return false;
    const long long pad16 = (long long)cdiv(W, 64) * 64 * B, pad8 = (long long)cdiv(W, 32) * 32 * cdiv(B, 2) * 2;
    return pad16 <= pad8 && (long long)H * W * C * 2 <= 0x1fffffffLL;
}

// -1: not covered (the caller makes the two launches).  ldy0 > 0: both convolutions with the gate applied in the store
// (y[..., ych + c] = conv[..., c] * conv[..., C/2 + c] * sqrt(C/2) at a pixel stride of ldy channels).
// mean (optional): the block's mean branch in mean->B more workgroups of the same launch.
int dwconv_fwd2_launch(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H,
                       int W, int C, int K, int dtype, hipStream_t s, int ldy0, int ych0, int ldy1, int ych1,
                       const PoolFwdJob* mean) {
    if (tune_env("PDW_NO_FWD2")) return -1;
    const bool gated = ldy0 > 0;
    if (gated && C % 16 != 0) return -1;
    const TzGate g0{ldy0, ych0, sqrtf((float)(C / 2))}, g1{ldy1, ych1, sqrtf((float)(C / 2))};
    const TzGate *gate0 = gated ? &g0 : nullptr, *gate1 = gated ? &g1 : nullptr;
    switch (K) {
#define PDW_FWD2_CASE(KK) \
    case KK: return dwconv_fwd2_k##KK(x0, w0, y0, x1, w1, y1, B, H, W, C, dtype, s, gate0, gate1, mean);
        PDW_FWD2_CASE(3) PDW_FWD2_CASE(5) PDW_FWD2_CASE(7) PDW_FWD2_CASE(9) PDW_FWD2_CASE(11) PDW_FWD2_CASE(13)
        PDW_FWD2_CASE(15) PDW_FWD2_CASE(17)
#undef PDW_FWD2_CASE
        default: return -1;
    }
}

}  // namespace pdw
