// The block's three independent backward convolution launches as one (dwconv_bwd3.h), 5x5 filter: one translation
// unit per size so the build compiles them in parallel.
#include "dwconv_bwd3.h"

namespace pdw {

int dwconv_bwd3_k5(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0,
                     const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int dtype,
                     hipStream_t s, int* plan_out) {
    return launch_bwd3<5>(gyf, w0, addp, dx, x0, dw0, ws0, x1, gy1, dw1, ws1, B, H, W, C, dtype, s, plan_out);
}

}  // namespace pdw
