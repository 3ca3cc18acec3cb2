// LDS-tiled depthwise convolution (forward / input gradient), filter width 3: the
// instantiations of the kernel template in dwconv_tiled.h for this width, one translation
// unit per width so the build compiles them in parallel.
#include "dwconv_tiled.h"

namespace pdw {

int dwconv_tiled_kw3(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s) {
    return launch_dtype<3>(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
}

}  // namespace pdw
