// LDS-tiled depthwise-convolution weight gradient, 15x15 filter: the instantiations of the
// kernel template in dwconv_wgrad_tiled.h for this size (one translation unit per size so the
// build compiles them in parallel).
#include "dwconv_wgrad_tiled.h"

namespace pdw {

size_t dwconv_wgrad_tiled_ws_k15(int B, int H, int W, int C, int PH, int PW, int dtype) {
    return wgrad_tiled_workspace_k<15>(B, H, W, C, PH, PW, dtype);
}

int dwconv_wgrad_tiled_k15(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s) {
    return wgrad_tiled_launch_k<15>(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
}

}  // namespace pdw
