// Dispatch of the block's three independent backward convolution launches as one (dwconv_bwd3.h) by filter size.
#include "common.h"
#include "kernels.h"

namespace pdw {

#define PDW_BWD3_DECL(K)                                                                                               \
    int dwconv_bwd3_k##K(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0, \
                         const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int dtype,     \
                         hipStream_t s, int* plan_out);
PDW_BWD3_DECL(3) PDW_BWD3_DECL(5) PDW_BWD3_DECL(7) PDW_BWD3_DECL(9) PDW_BWD3_DECL(11) PDW_BWD3_DECL(13) PDW_BWD3_DECL(15)
PDW_BWD3_DECL(17)
#undef PDW_BWD3_DECL

// -1: not covered (the caller makes the three launches).  With plan_out the launch is only planned: the band counts
// of the input gradient, the full and the half scale's weight gradient go to plan_out[0..2], no pointer is looked at
// and nothing is launched.
int dwconv_bwd3_launch(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0,
                       const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int K, int dtype,
                       hipStream_t s, int* plan_out) {
    if (tune_env("PDW_NO_BWD3")) return -1;
    switch (K) {
#define PDW_BWD3_CASE(KK) \
    case KK: return dwconv_bwd3_k##KK(gyf, w0, addp, dx, x0, dw0, ws0, x1, gy1, dw1, ws1, B, H, W, C, dtype, s, plan_out);
        PDW_BWD3_CASE(3) PDW_BWD3_CASE(5) PDW_BWD3_CASE(7) PDW_BWD3_CASE(9) PDW_BWD3_CASE(11) PDW_BWD3_CASE(13)
        PDW_BWD3_CASE(15) PDW_BWD3_CASE(17)
#undef PDW_BWD3_CASE
        default: return -1;
    }
}

}  // namespace pdw
