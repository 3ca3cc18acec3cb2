// Dispatch of the LDS-tiled depthwise convolution (stride 1, dilation 1) by filter width.
// The kernel template and its description live in dwconv_tiled.h; each width is instantiated
// in its own translation unit (dwconv_tiled_kw*.hip).
#include <stdlib.h>

#include "common.h"
#include "kernels.h"

namespace pdw {

int dwconv_tiled_kw3(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw5(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw7(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw9(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw11(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw13(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw15(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);
int dwconv_tiled_kw17(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int PH, int PW,
                      bool flip, int dtype, hipStream_t s);

int dwconv_mfma_k3(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k5(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k7(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k9(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k11(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k13(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k15(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);
int dwconv_mfma_k17(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                    bool flip, int dtype, hipStream_t s);

int dwconv_tz_k3(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k5(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k7(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k9(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k11(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k13(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k15(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);
int dwconv_tz_k17(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int PH, int PW,
                   bool flip, int dtype, const TzGate* gate, hipStream_t s);

// Block-Toeplitz kernel on the dense matrix cores (dwconv_tz.h): square odd filters, 16-bit types, C % 8 == 0.
static int dwconv_tz_launch(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int KH,
                            int KW, int PH, int PW, bool flip, int dtype, hipStream_t s, const TzGate* gate = nullptr) {
    if (KH != KW || dtype == kF32) return -1;
    const char* e = tune_env("PDW_TZ");
    if (e && atoi(e) == 0) return -1;
    switch (KW) {
        case 3: return dwconv_tz_k3(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 5: return dwconv_tz_k5(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 7: return dwconv_tz_k7(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 9: return dwconv_tz_k9(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 11: return dwconv_tz_k11(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 13: return dwconv_tz_k13(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 15: return dwconv_tz_k15(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        case 17: return dwconv_tz_k17(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, gate, s);
        default: return -1;
    }
}

// Matrix-core kernel for square filters and 16-bit types; -1 when it does not cover the case.
static int dwconv_mfma_launch(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C, int KH,
                              int KW, int PH, int PW, bool flip, int dtype, hipStream_t s) {
    if (KH != KW || dtype == kF32) return -1;
    const char* e = tune_env("PDW_MFMA");
    if (e && atoi(e) == 0) return -1;
    switch (KW) {
        case 3: return dwconv_mfma_k3(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 5: return dwconv_mfma_k5(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 7: return dwconv_mfma_k7(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 9: return dwconv_mfma_k9(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 11: return dwconv_mfma_k11(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 13: return dwconv_mfma_k13(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 15: return dwconv_mfma_k15(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        case 17: return dwconv_mfma_k17(x, w, add, pool, y, B, H, W, C, PH, PW, flip, dtype, s);
        default: return -1;
    }
}

// Returns -1 when the tiled kernel does not cover the case (the caller then uses the direct
// kernel), otherwise the launch status.  With flip the 180-degree rotated filter is used: the
// caller passes gy as x with padding k-1-p, which yields the input gradient.
int dwconv_tiled_launch(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW, int PH,
                        int PW, bool flip, int dtype, hipStream_t s, const void* add, void* pool) {
    if (KH > 31 || H + 2 * PH - KH + 1 < 1 || W + 2 * PW - KW + 1 < 1) return -1;
    {
        const int r = dwconv_tz_launch(x, w, add, pool, y, B, H, W, C, KH, KW, PH, PW, flip, dtype, s);
        if (r != -1) return r;
    }
    {
        const int r = dwconv_mfma_launch(x, w, add, pool, y, B, H, W, C, KH, KW, PH, PW, flip, dtype, s);
        if (r != -1 || add || pool) return r;   // only the matrix-core kernel has the fused forms
    }
    if (dtype == kF32) {   // fp32 matrix cores (square odd filters 5 .. 17, C % 4 == 0)
        const int r = dwconv_f32m_launch(x, w, y, B, H, W, C, KH, KW, PH, PW, flip, s);
        if (r != -1) return r;
    }
    switch (KW) {
        case 3: return dwconv_tiled_kw3(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 5: return dwconv_tiled_kw5(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 7: return dwconv_tiled_kw7(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 9: return dwconv_tiled_kw9(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 11: return dwconv_tiled_kw11(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 13: return dwconv_tiled_kw13(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 15: return dwconv_tiled_kw15(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        case 17: return dwconv_tiled_kw17(x, w, y, B, H, W, C, KH, PH, PW, flip, dtype, s);
        default: return -1;
    }
}

int dwconv_gate_launch(const void* x, const void* w, void* y, void* pool, int B, int H, int W, int C, int K, int PH,
                       int PW, int ldy, int ych, int dtype, hipStream_t s) {
    if (K < 1 || H + 2 * PH - K + 1 < 1 || W + 2 * PW - K + 1 < 1 || C % 16 != 0) return -1;
    const TzGate gate{ldy, ych, sqrtf((float)(C / 2))};
    return dwconv_tz_launch(x, w, nullptr, pool, y, B, H, W, C, K, K, PH, PW, false, dtype, s, &gate);
}

}  // namespace pdw
