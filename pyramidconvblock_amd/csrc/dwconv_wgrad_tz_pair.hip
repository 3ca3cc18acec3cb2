// Depthwise-convolution weight gradients of two problems with the same filter size, batch and channel count in one
// launch of the dense matrix-core kernel (dwconv_wgrad_tz.h): the instantiations by the row groups an operand spans
// and the tile widths of the two problems (a wide first problem with a wide or a narrow second one), and the launcher.
#include "dwconv_wgrad_tz.h"

#include "reduce_parts.h"

namespace pdw {

template <typename T>
static int wgrad_tz_pair_go(const WgTzPlan& p0, const void* x0, const void* gy0, void* ws0, const WgTzPlan& p1,
                            const void* x1, const void* gy1, void* ws1, hipStream_t s) {
    const int nga = wgrad_tz_nga(p0.g.K);
#define PDW_TZP(NGA_, NB_)                                                                          \
    return p1.ncb == 8 ? launch_wgrad_tz_pair<T, NGA_, 8, 8, NB_>(p0, x0, gy0, ws0, p1, x1, gy1, ws1, s) \
                       : launch_wgrad_tz_pair<T, NGA_, 8, 5, NB_>(p0, x0, gy0, ws0, p1, x1, gy1, ws1, s);
    if (p0.g.K == 17) { PDW_TZP(5, 3) }
    switch (nga) {
        case 2: PDW_TZP(2, 2)
        case 3: PDW_TZP(3, 2)
        case 4: PDW_TZP(4, 2)
        case 5: PDW_TZP(5, 2)
        default: return -1;
    }
#undef PDW_TZP
}

// -1: not covered (the caller runs the two problems one by one).  Problem 0 is the wider one.
int dwconv_wgrad_tz_pair_launch(const void* x0, const void* gy0, void* dw0, void* ws0, int H0, int W0, const void* x1,
                                const void* gy1, void* dw1, void* ws1, int H1, int W1, int B, int C, int K, int PH, int PW,
                                int dtype, hipStream_t s) {
    if (dtype == kF32) return -1;
    for (const void* p : {x0, gy0, (const void*)ws0, x1, gy1, (const void*)ws1})
        if ((reinterpret_cast<uintptr_t>(p) & 15) != 0) return -1;
    const WgTzPlan p0 = wgrad_tz_plan(B, H0, W0, C, K, PH, PW), p1 = wgrad_tz_plan(B, H1, W1, C, K, PH, PW);
    if (!p0.ok || !p1.ok || p0.ncb != 8) return -1;
    const int r = dtype == kF16 ? wgrad_tz_pair_go<f16_t>(p0, x0, gy0, ws0, p1, x1, gy1, ws1, s)
                                : wgrad_tz_pair_go<bf16_t>(p0, x0, gy0, ws0, p1, x1, gy1, ws1, s);
    if (r != 0) return r;
    const int n0 = B * p0.g.nbands * p0.g.ncolt, n1 = B * p1.g.nbands * p1.g.ncolt;
    if (dtype == kF16) {
        if (int e = wgrad_reduce_launch<f16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
        return wgrad_reduce_launch<f16_t>((const float*)ws1, dw1, n1, K * K * C, s);
    }
    if (int e = wgrad_reduce_launch<bf16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
    return wgrad_reduce_launch<bf16_t>((const float*)ws1, dw1, n1, K * K * C, s);
}

}  // namespace pdw
