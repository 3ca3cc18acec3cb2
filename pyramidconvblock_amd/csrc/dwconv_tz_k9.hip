// Block-Toeplitz depthwise convolution on the dense matrix cores (forward / input gradient), 9x9 filter: the
// instantiations of the kernel template in dwconv_tz.h for this size, one translation unit per size so the build
// compiles them in parallel.
#include "dwconv_tz.h"

namespace pdw {

int dwconv_tz_k9(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s) {
    return launch_tz_dtype<9>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
}

}  // namespace pdw
