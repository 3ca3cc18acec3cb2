// Depthwise-convolution weight gradient on the dense matrix cores (dwconv_wgrad_tz.h): the instantiations of the
// kernel template (filter sizes 1..17 by the row groups an operand spans, two tile widths, two 16-bit types), the workspace query
// and the launcher.
#include "dwconv_wgrad_tz.h"

#include "reduce_parts.h"

namespace pdw {

size_t dwconv_wgrad_tz_workspace(int B, int H, int W, int C, int K, int PH, int PW, int dtype) {
    if (dtype == kF32) return 0;
    return wgrad_tz_workspace(B, H, W, C, K, PH, PW);
}

template <typename T>
static int wgrad_tz_go(const WgTzPlan& p, const void* x, const void* gy, void* ws, hipStream_t s) {
    const int nga = wgrad_tz_nga(p.g.K);
#define PDW_TZ(NGA_, NB_)                                                            \
    return p.ncb == 8 ? launch_wgrad_tz<T, NGA_, 8, NB_>(p, x, gy, ws, s) : launch_wgrad_tz<T, NGA_, 5, NB_>(p, x, gy, ws, s);
    if (p.g.K == 17) { PDW_TZ(5, 3) }
    switch (nga) {
        case 2: PDW_TZ(2, 2)
        case 3: PDW_TZ(3, 2)
        case 4: PDW_TZ(4, 2)
        case 5: PDW_TZ(5, 2)
        default: return -1;
    }
#undef PDW_TZ
}

// -1: not covered (the caller falls back to the other weight-gradient kernels).
int dwconv_wgrad_tz_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int K, int PH,
                           int PW, int dtype, hipStream_t s) {
    if (dtype == kF32) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(gy) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(ws) & 15) != 0)
        return -1;
    const WgTzPlan p = wgrad_tz_plan(B, H, W, C, K, PH, PW);
    if (!p.ok) return -1;
    const int r = dtype == kF16 ? wgrad_tz_go<f16_t>(p, x, gy, ws, s) : wgrad_tz_go<bf16_t>(p, x, gy, ws, s);
    if (r != 0) return r;
    const int nparts = B * p.g.nbands * p.g.ncolt;
    if (dtype == kF16) return wgrad_reduce_launch<f16_t>((const float*)ws, dw, nparts, K * K * C, s);
    return wgrad_reduce_launch<bf16_t>((const float*)ws, dw, nparts, K * K * C, s);
}

}  // namespace pdw
