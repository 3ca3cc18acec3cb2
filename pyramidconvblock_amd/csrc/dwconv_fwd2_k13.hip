// The forward convolutions of both scales of a two-scale block as one launch (dwconv_fwd2.h), 13x13 filter: one
// translation unit per size so the build compiles them in parallel.
#include "dwconv_fwd2.h"

namespace pdw {

int dwconv_fwd2_k13(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H, int W,
                    int C, int dtype, hipStream_t s, const TzGate* gate0, const TzGate* gate1,
                    const PoolFwdJob* mean) {
    return launch_fwd2<13>(x0, w0, y0, x1, w1, y1, B, H, W, C, dtype, s, gate0, gate1, mean);
}

}  // namespace pdw
