// LDS-tiled depthwise-convolution weight gradient, 13x13 filter: the instantiations of the
// kernel template in dwconv_wgrad_tiled.h for this size (one translation unit per size so the
// build compiles them in parallel).
#include "dwconv_wgrad_tiled.h"

namespace pdw {

size_t dwconv_wgrad_tiled_ws_k13(int B, int H, int W, int C, int PH, int PW, int dtype) {
    return wgrad_tiled_workspace_k<13>(B, H, W, C, PH, PW, dtype);
}

int dwconv_wgrad_tiled_k13(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s) {
    return wgrad_tiled_launch_k<13>(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
}

}  // namespace pdw
