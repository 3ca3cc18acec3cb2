// Dispatch of the LDS-tiled depthwise-convolution weight gradient (stride 1, dilation 1, odd
// square filters up to 17x17) by filter size.  The kernel template and its description live in
// dwconv_wgrad_tiled.h; each size is instantiated in its own translation unit.
#include <stdlib.h>

#include "common.h"
#include "kernels.h"

namespace pdw {

size_t dwconv_wgrad_tiled_ws_k3(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k3(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k5(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k5(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k7(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k7(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k9(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k9(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k11(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k11(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k13(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k13(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k15(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k15(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_tiled_ws_k17(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_tiled_k17(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                           int PW, int dtype, hipStream_t s);

size_t dwconv_wgrad_mfma_ws_k3(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k3(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k5(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k5(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k7(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k7(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k9(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k9(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k11(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k11(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k13(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k13(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k15(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k15(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);
size_t dwconv_wgrad_mfma_ws_k17(int B, int H, int W, int C, int PH, int PW, int dtype);
int dwconv_wgrad_mfma_k17(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int PH,
                            int PW, int dtype, hipStream_t s);

int dwconv_wgrad_mfma_pair_k3(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k5(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k7(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k9(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k11(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k13(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k15(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);
int dwconv_wgrad_mfma_pair_k17(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                               const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int PH, int PW,
                               int dtype, hipStream_t s);

// dwconv_wgrad_tz.hip: dense matrix-core kernel (16-bit types, C % 8 == 0, K <= 17)
size_t dwconv_wgrad_tz_workspace(int B, int H, int W, int C, int K, int PH, int PW, int dtype);
int dwconv_wgrad_tz_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int K, int PH,
                           int PW, int dtype, hipStream_t s);
int dwconv_wgrad_tz_pair_launch(const void* x0, const void* gy0, void* dw0, void* ws0, int H0, int W0, const void* x1,
                                const void* gy1, void* dw1, void* ws1, int H1, int W1, int B, int C, int K, int PH, int PW,
                                int dtype, hipStream_t s);
static bool wgrad_tz_enabled() {
    const char* e = tune_env("PDW_WGRAD_TZ");
    return !(e && atoi(e) == 0);
}

// Matrix-core variant (16-bit types): workspace bytes (0 = not covered) and launch (-1 = not covered).
static bool wgrad_mfma_enabled(int dtype) {
    if (dtype == kF32) return false;
    const char* e = tune_env("PDW_MFMA");
    return !(e && atoi(e) == 0);
}
static size_t wgrad_mfma_workspace(int B, int H, int W, int C, int K, int PH, int PW, int dtype) {
    if (!wgrad_mfma_enabled(dtype)) return 0;
    switch (K) {
        case 3: return dwconv_wgrad_mfma_ws_k3(B, H, W, C, PH, PW, dtype);
        case 5: return dwconv_wgrad_mfma_ws_k5(B, H, W, C, PH, PW, dtype);
        case 7: return dwconv_wgrad_mfma_ws_k7(B, H, W, C, PH, PW, dtype);
        case 9: return dwconv_wgrad_mfma_ws_k9(B, H, W, C, PH, PW, dtype);
        case 11: return dwconv_wgrad_mfma_ws_k11(B, H, W, C, PH, PW, dtype);
        case 13: return dwconv_wgrad_mfma_ws_k13(B, H, W, C, PH, PW, dtype);
        case 15: return dwconv_wgrad_mfma_ws_k15(B, H, W, C, PH, PW, dtype);
        case 17: return dwconv_wgrad_mfma_ws_k17(B, H, W, C, PH, PW, dtype);
        default: return 0;
    }
}
static int wgrad_mfma_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int K, int PH,
                             int PW, int dtype, hipStream_t s) {
    if (!wgrad_mfma_enabled(dtype)) return -1;
    switch (K) {
        case 3: return dwconv_wgrad_mfma_k3(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 5: return dwconv_wgrad_mfma_k5(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 7: return dwconv_wgrad_mfma_k7(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 9: return dwconv_wgrad_mfma_k9(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 11: return dwconv_wgrad_mfma_k11(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 13: return dwconv_wgrad_mfma_k13(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 15: return dwconv_wgrad_mfma_k15(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 17: return dwconv_wgrad_mfma_k17(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        default: return -1;
    }
}

// Two weight gradients of the same filter size, batch and channel count in one matrix-core launch (stride 1,
// dilation 1, square filter); -1 when that kernel does not cover both, and the caller runs them one by one.
int dwconv_wgrad_pair_launch(const void* xa, const void* gya, void* dwa, void* wsa, int Ha, int Wa, const void* xb,
                             const void* gyb, void* dwb, void* wsb, int Hb, int Wb, int B, int C, int K, int PH, int PW,
                             int dtype, hipStream_t s) {
    if (!wgrad_mfma_enabled(dtype) || tune_env("PDW_NO_WGRAD_PAIR")) return -1;
    if (wgrad_tz_enabled() && dwconv_wgrad_tz_workspace(B, Ha, Wa, C, K, PH, PW, dtype) &&
        dwconv_wgrad_tz_workspace(B, Hb, Wb, C, K, PH, PW, dtype)) {
        // the dense matrix-core kernel covers both: as one launch of it, else as two (which beat the shared launch of
        // the kernel below)
        if (tune_env("PDW_NO_TZ_PAIR")) return -1;
        return dwconv_wgrad_tz_pair_launch(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, K, PH, PW, dtype, s);
    }
    switch (K) {
        case 3: return dwconv_wgrad_mfma_pair_k3(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 5: return dwconv_wgrad_mfma_pair_k5(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 7: return dwconv_wgrad_mfma_pair_k7(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 9: return dwconv_wgrad_mfma_pair_k9(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 11: return dwconv_wgrad_mfma_pair_k11(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 13: return dwconv_wgrad_mfma_pair_k13(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 15: return dwconv_wgrad_mfma_pair_k15(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        case 17: return dwconv_wgrad_mfma_pair_k17(xa, gya, dwa, wsa, Ha, Wa, xb, gyb, dwb, wsb, Hb, Wb, B, C, PH, PW, dtype, s);
        default: return -1;
    }
}

// Bytes of fp32 workspace the tiled weight gradient needs (the larger of its two variants); 0 when it does not
// cover the case.
size_t dwconv_wgrad_tiled_workspace(int B, int H, int W, int C, int KH, int KW, int PH, int PW, int dtype) {
    if (KH != KW) return 0;
    size_t wm = wgrad_mfma_workspace(B, H, W, C, KH, PH, PW, dtype);
    const size_t wz = wgrad_tz_enabled() ? dwconv_wgrad_tz_workspace(B, H, W, C, KH, PH, PW, dtype) : 0;
    if (wz > wm) wm = wz;
    size_t wt = 0;
    switch (KH) {
        case 3: wt = dwconv_wgrad_tiled_ws_k3(B, H, W, C, PH, PW, dtype); break;
        case 5: wt = dwconv_wgrad_tiled_ws_k5(B, H, W, C, PH, PW, dtype); break;
        case 7: wt = dwconv_wgrad_tiled_ws_k7(B, H, W, C, PH, PW, dtype); break;
        case 9: wt = dwconv_wgrad_tiled_ws_k9(B, H, W, C, PH, PW, dtype); break;
        case 11: wt = dwconv_wgrad_tiled_ws_k11(B, H, W, C, PH, PW, dtype); break;
        case 13: wt = dwconv_wgrad_tiled_ws_k13(B, H, W, C, PH, PW, dtype); break;
        case 15: wt = dwconv_wgrad_tiled_ws_k15(B, H, W, C, PH, PW, dtype); break;
        case 17: wt = dwconv_wgrad_tiled_ws_k17(B, H, W, C, PH, PW, dtype); break;
        default: return 0;
    }
    return wt > wm ? wt : wm;
}

// Returns -1 when the case is not covered (the caller then uses the direct kernel).
int dwconv_wgrad_tiled_launch(const void* x, const void* gy, void* dw, void* ws, int B, int H, int W, int C, int KH,
                              int KW, int PH, int PW, int dtype, hipStream_t s) {
    if (KH != KW) return -1;
    if (wgrad_tz_enabled()) {
        const int r = dwconv_wgrad_tz_launch(x, gy, dw, ws, B, H, W, C, KH, PH, PW, dtype, s);
        if (r != -1) return r;
    }
    {
        const int r = wgrad_mfma_launch(x, gy, dw, ws, B, H, W, C, KH, PH, PW, dtype, s);
        if (r != -1) return r;
    }
    switch (KH) {
        case 3: return dwconv_wgrad_tiled_k3(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 5: return dwconv_wgrad_tiled_k5(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 7: return dwconv_wgrad_tiled_k7(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 9: return dwconv_wgrad_tiled_k9(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 11: return dwconv_wgrad_tiled_k11(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 13: return dwconv_wgrad_tiled_k13(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 15: return dwconv_wgrad_tiled_k15(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        case 17: return dwconv_wgrad_tiled_k17(x, gy, dw, ws, B, H, W, C, PH, PW, dtype, s);
        default: return -1;
    }
}

}  // namespace pdw
