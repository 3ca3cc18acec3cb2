// Matrix-core depthwise-convolution weight gradient, 5x5 filter: the instantiations of the kernel
// template in dwconv_wgrad_mfma.h for this size (one translation unit per size so the build compiles
// them in parallel).
#include "dwconv_wgrad_mfma.h"

namespace pdw {

size_t dwconv_wgrad_mfma_ws_k5(int B, int H, int W, int C, int PH, int PW, int dtype) {
    if (dtype == kF16) return wgrad_mfma_workspace_t<f16_t, 5>(B, H, W, C, PH, PW);
    if (dtype == kBF16) return wgrad_mfma_workspace_t<bf16_t, 5>(B, H, W, C, PH, PW);
    return 0;
}

int dwconv_wgrad_mfma_k5(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s) {
    if (dtype == kF16) return wgrad_mfma_launch_t<f16_t, 5>(x, gy, dw, ws, B, H, W, C, PH, PW, s);
    if (dtype == kBF16) return wgrad_mfma_launch_t<bf16_t, 5>(x, gy, dw, ws, B, H, W, C, PH, PW, s);
    return -1;
}

int dwconv_wgrad_mfma_pair_k5(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s) {
    if (dtype == kF16)
        return wgrad_mfma_pair_launch_t<f16_t, 5>(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, s);
    if (dtype == kBF16)
        return wgrad_mfma_pair_launch_t<bf16_t, 5>(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, s);
    return -1;
}

}  // namespace pdw
