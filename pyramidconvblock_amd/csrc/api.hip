// C ABI of libpdw.so (declared in include/pdw.h): argument validation and dispatch to
// the kernel launchers.  No allocation, no synchronisation; the only state is the per-thread
// error text here, the per-thread list of deferred summations (dwconv_direct.hip), the
// once-per-process LDS-limit set-up next to each large kernel's launcher, the bounded per-shape
// launch-plan caches of the shared conv launches (dwconv_fwd2.h, dwconv_bwd3.h: a std::map behind a
// mutex each, emptied at kPlanCacheMax entries) and the per-device address of the static scratch array.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "../../include/pdw.h"
#include "common.h"
#include "kernels.h"
#include "pool_branch.h"
#include "reduce_parts.h"

namespace pdw {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return 2;
    }
    return 0;
}

static bool valid_dtype(int dtype) { return dtype == kF32 || dtype == kF16 || dtype == kBF16; }

static int check_conv(const char* fn, const void* a, const void* b, const void* c, int B, int H, int W, int C, int KH,
                      int KW, int SH, int SW, int PH, int PW, int DH, int DW, int dtype) {
    if (!valid_dtype(dtype)) return set_error("%s: unknown dtype %d", fn, dtype), 1;
    if (B < 0 || H < 1 || W < 1 || C < 1 || KH < 1 || KW < 1)
        return set_error("%s: bad extents B=%d H=%d W=%d C=%d KH=%d KW=%d", fn, B, H, W, C, KH, KW), 1;
    if (SH < 1 || SW < 1 || DH < 1 || DW < 1 || PH < 0 || PW < 0)
        return set_error("%s: bad stride/padding/dilation (%d,%d)/(%d,%d)/(%d,%d)", fn, SH, SW, PH, PW, DH, DW), 1;
    if (B > 0 && (!a || !b || !c)) return set_error("%s: null pointer", fn), 1;
    return 0;
}

static int check_resample(const char* fn, const void* a, const void* b, int B, int H, int W, int C, int h, int w,
                          int dtype) {
    if (!valid_dtype(dtype)) return set_error("%s: unknown dtype %d", fn, dtype), 1;
    if (B < 0 || H < 1 || W < 1 || C < 1 || h < 1 || w < 1)
        return set_error("%s: bad extents B=%d H=%d W=%d C=%d h=%d w=%d", fn, B, H, W, C, h, w), 1;
    if (B > 0 && (!a || !b)) return set_error("%s: null pointer", fn), 1;
    if ((long long)H * h >= 0x7fffffffLL || (long long)W * w >= 0x7fffffffLL)
        return set_error("%s: extents too large", fn), 1;
    return 0;
}

// Scratch of the entry point that allocates nothing (pdw_dwconv_wgrad_static): one copy of this array lives on every
// device the library is loaded on, at that device's own address.  The name is a host-side stand-in; device
// code and HIP calls get the address hipGetSymbolAddress returns for the current device.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device, looked up once per device (with that device current).
static int static_scratch(const char* fn, void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error("%s: hipGetDevice: %s", fn, hipGetErrorString(e)), 2;
    if (dev < 0 || dev >= kMaxDevices) return set_error("%s: device index %d not supported", fn, dev), 2;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return set_error("%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e)), 2;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace pdw

using namespace pdw;

extern "C" {

int pdw_version(void) { return 5; }

const char* pdw_last_error(void) { return g_err; }

int pdw_conv_out_size(int in, int k, int stride, int pad, int dil) {
    if (in < 1 || k < 1 || stride < 1 || dil < 1 || pad < 0) return 0;
    return conv_out_size(in, k, stride, pad, dil);
}

int pdw_dwconv_fwd(const void* x, const void* w, void* y, int B, int H, int W, int C, int KH, int KW, int SH, int SW,
                   int PH, int PW, int DH, int DW, int dtype, void* stream) {
    if (int e = check_conv("pdw_dwconv_fwd", x, w, y, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype)) return e;
    if (B == 0 || conv_out_size(H, KH, SH, PH, DH) == 0 || conv_out_size(W, KW, SW, PW, DW) == 0) return 0;
    if (SH == 1 && SW == 1 && DH == 1 && DW == 1) {
        const int r = dwconv_tiled_launch(x, w, y, B, H, W, C, KH, KW, PH, PW, false, dtype, (hipStream_t)stream);
        if (r != -1) return r;
    }
    return dwconv_fwd_direct_launch(x, w, y, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype, (hipStream_t)stream);
}

int pdw_dwconv_fwd_pool(const void* x, const void* w, void* y, void* xp, int B, int H, int W, int C, int KH, int KW,
                        int SH, int SW, int PH, int PW, int DH, int DW, int h, int wp, int dtype, void* stream) {
    if (int e = check_conv("pdw_dwconv_fwd_pool", x, w, y, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype)) return e;
    if (int e = check_resample("pdw_dwconv_fwd_pool", x, xp, B, H, W, C, h, wp, dtype)) return e;
    if (B == 0) return 0;
    const int OH = conv_out_size(H, KH, SH, PH, DH), OW = conv_out_size(W, KW, SW, PW, DW);
    if (OH > 0 && OW > 0 && SH == 1 && SW == 1 && DH == 1 && DW == 1 && H == 2 * h && W == 2 * wp) {
        const int r = dwconv_tiled_launch(x, w, y, B, H, W, C, KH, KW, PH, PW, false, dtype, (hipStream_t)stream, nullptr,
                                          xp);
        if (r != -1) return r;
    }
    if (int e = pdw_dwconv_fwd(x, w, y, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype, stream)) return e;
    return avgpool_fwd_launch(x, xp, B, H, W, C, h, wp, dtype, (hipStream_t)stream);
}

int pdw_dwconv_fwd_gate(const void* x, const void* w, void* y, void* xp, int B, int H, int W, int C, int K, int pad,
                        int ldy, int ych, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dwconv_fwd_gate: unknown dtype %d", dtype), 1;
    if (B < 0 || H < 1 || W < 1 || C < 2 || K < 1 || pad < 0)
        return set_error("pdw_dwconv_fwd_gate: bad extents B=%d H=%d W=%d C=%d K=%d pad=%d", B, H, W, C, K, pad), 1;
    if (ldy == 0) ldy = C / 2;
    if ((C & 1) || ych < 0 || ldy < ych + C / 2)
        return set_error("pdw_dwconv_fwd_gate: need even C and ych + C/2 <= ldy (C=%d ldy=%d ych=%d)", C, ldy, ych), 1;
    if (B > 0 && (!x || !w || !y)) return set_error("pdw_dwconv_fwd_gate: null pointer"), 1;
    if (B == 0) return 0;
    const int r = dwconv_gate_launch(x, w, y, xp, B, H, W, C, K, pad, pad, ldy, ych, dtype, (hipStream_t)stream);
    if (r == -1)
        return set_error("pdw_dwconv_fwd_gate: B=%d H=%d W=%d C=%d K=%d pad=%d dtype=%d not covered by the fused kernel", B,
                         H, W, C, K, pad, dtype), 3;
    return r;
}

int pdw_dwconv_dgrad(const void* gy, const void* w, void* dx, int B, int H, int W, int C, int KH, int KW, int SH,
                     int SW, int PH, int PW, int DH, int DW, int dtype, void* stream) {
    if (int e = check_conv("pdw_dwconv_dgrad", gy, w, dx, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype)) return e;
    if (B == 0) return 0;
    if (SH == 1 && SW == 1 && DH == 1 && DW == 1 && PH <= KH - 1 && PW <= KW - 1) {
        // dx = correlation of gy with the 180-degree rotated filter at padding k-1-p
        const int OH = conv_out_size(H, KH, 1, PH, 1), OW = conv_out_size(W, KW, 1, PW, 1);
        if (OH > 0 && OW > 0) {
            const int r = dwconv_tiled_launch(gy, w, dx, B, OH, OW, C, KH, KW, KH - 1 - PH, KW - 1 - PW, true, dtype,
                                              (hipStream_t)stream);
            if (r != -1) return r;
        }
    }
    return dwconv_dgrad_direct_launch(gy, w, dx, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype,
                                      (hipStream_t)stream);
}

int pdw_dwconv_dgrad_addpool(const void* gy, const void* w, const void* gp, void* dx, int B, int H, int W, int C, int KH,
                             int KW, int SH, int SW, int PH, int PW, int DH, int DW, int h, int wp, int dtype,
                             void* stream) {
    if (int e = check_conv("pdw_dwconv_dgrad_addpool", gy, w, dx, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype))
        return e;
    if (int e = check_resample("pdw_dwconv_dgrad_addpool", gp, dx, B, H, W, C, h, wp, dtype)) return e;
    if (B == 0) return 0;
    if (SH == 1 && SW == 1 && DH == 1 && DW == 1 && PH <= KH - 1 && PW <= KW - 1 && H == 2 * h && W == 2 * wp) {
        const int OH = conv_out_size(H, KH, 1, PH, 1), OW = conv_out_size(W, KW, 1, PW, 1);
        if (OH > 0 && OW > 0) {
            const int r = dwconv_tiled_launch(gy, w, dx, B, OH, OW, C, KH, KW, KH - 1 - PH, KW - 1 - PW, true, dtype,
                                              (hipStream_t)stream, gp);
            if (r != -1) return r;
        }
    }
    if (int e = pdw_dwconv_dgrad(gy, w, dx, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype, stream)) return e;
    return avgpool_bwd_launch(gp, dx, B, H, W, C, h, wp, 1, dtype, (hipStream_t)stream);
}

int pdw_sum_parts(const float* parts, void* out, int nparts, long long n, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_sum_parts: unknown dtype %d", dtype), 1;
    if (nparts < 1 || n < 0 || n > 0x7fffffffLL) return set_error("pdw_sum_parts: bad extents nparts=%d n=%lld", nparts, n), 1;
    if (n == 0) return 0;
    if (!parts || !out) return set_error("pdw_sum_parts: null pointer"), 1;
    switch (dtype) {
        case kF32: return wgrad_reduce_launch<float>(parts, out, nparts, (int)n, (hipStream_t)stream);
        case kF16: return wgrad_reduce_launch<f16_t>(parts, out, nparts, (int)n, (hipStream_t)stream);
        default: return wgrad_reduce_launch<bf16_t>(parts, out, nparts, (int)n, (hipStream_t)stream);
    }
}

int pdw_reduce_defer_begin(void) { return reduce_defer_begin(); }

int pdw_reduce_defer_flush(void* stream) { return reduce_defer_flush((hipStream_t)stream); }

size_t pdw_dwconv_wgrad_workspace_bytes(int B, int H, int W, int C, int KH, int KW, int SH, int SW, int PH, int PW,
                                        int DH, int DW, int dtype) {
    if (check_conv("pdw_dwconv_wgrad_workspace_bytes", "", "", "", B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype))
        return 0;
    size_t need = dwconv_wgrad_direct_workspace(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW);
    if (SH == 1 && SW == 1 && DH == 1 && DW == 1) {
        const size_t t = dwconv_wgrad_tiled_workspace(B, H, W, C, KH, KW, PH, PW, dtype);
        if (t > need) need = t;
    }
    return need;
}

int pdw_dwconv_wgrad(const void* x, const void* gy, void* dw, void* workspace, size_t workspace_bytes, int B, int H,
                     int W, int C, int KH, int KW, int SH, int SW, int PH, int PW, int DH, int DW, int dtype,
                     void* stream) {
    if (int e = check_conv("pdw_dwconv_wgrad", x, gy, dw, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype)) return e;
    if (!dw) return set_error("pdw_dwconv_wgrad: null dw"), 1;
    const size_t need = pdw_dwconv_wgrad_workspace_bytes(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype);
    if (!workspace || workspace_bytes < need)
        return set_error("pdw_dwconv_wgrad: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    if (B > 0 && SH == 1 && SW == 1 && DH == 1 && DW == 1) {
        const int r = dwconv_wgrad_tiled_launch(x, gy, dw, workspace, B, H, W, C, KH, KW, PH, PW, dtype,
                                                (hipStream_t)stream);
        if (r != -1) return r;
    }
    return dwconv_wgrad_direct_launch(x, gy, dw, workspace, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype,
                                      (hipStream_t)stream);
}

size_t pdw_static_scratch_bytes(void) { return kStaticScratchBytes; }

int pdw_static_scratch_init(void) {
    void* p = nullptr;
    return static_scratch("pdw_static_scratch_init", &p);
}

int pdw_dwconv_wgrad_static(const void* x, const void* gy, void* dw, int B, int H, int W, int C, int KH, int KW, int SH,
                            int SW, int PH, int PW, int DH, int DW, int dtype, void* stream) {
    if (int e = check_conv("pdw_dwconv_wgrad_static", x, gy, dw, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype))
        return e;
    if (reduce_deferring())
        return set_error("pdw_dwconv_wgrad_static: not available between pdw_reduce_defer_begin and the flush (the "
                         "shared scratch would have to stay untouched until then)"), 1;
    const size_t need = pdw_dwconv_wgrad_workspace_bytes(B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype);
    if (need > kStaticScratchBytes)
        return set_error("pdw_dwconv_wgrad_static: these extents need %zu bytes of scratch, the static buffer holds "
                         "%zu; use pdw_dwconv_wgrad with a workspace", need, kStaticScratchBytes), 1;
    void* ws = nullptr;
    if (int e = static_scratch("pdw_dwconv_wgrad_static", &ws)) return e;
    return pdw_dwconv_wgrad(x, gy, dw, ws, kStaticScratchBytes, B, H, W, C, KH, KW, SH, SW, PH, PW, DH, DW, dtype, stream);
}

int pdw_dwconv_wgrad_pair(const void* x0, const void* gy0, void* dw0, void* workspace0, size_t workspace0_bytes, int H0,
                          int W0, const void* x1, const void* gy1, void* dw1, void* workspace1, size_t workspace1_bytes,
                          int H1, int W1, int B, int C, int K, int dtype, void* stream) {
    const int P = K / 2;
    if (int e = check_conv("pdw_dwconv_wgrad_pair", x0, gy0, dw0, B, H0, W0, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (int e = check_conv("pdw_dwconv_wgrad_pair", x1, gy1, dw1, B, H1, W1, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (!(K & 1)) return set_error("pdw_dwconv_wgrad_pair: odd filter size needed (K=%d)", K), 1;
    if (!dw0 || !dw1) return set_error("pdw_dwconv_wgrad_pair: null dw"), 1;
    const size_t need0 = pdw_dwconv_wgrad_workspace_bytes(B, H0, W0, C, K, K, 1, 1, P, P, 1, 1, dtype);
    const size_t need1 = pdw_dwconv_wgrad_workspace_bytes(B, H1, W1, C, K, K, 1, 1, P, P, 1, 1, dtype);
    if (!workspace0 || workspace0_bytes < need0 || !workspace1 || workspace1_bytes < need1)
        return set_error("pdw_dwconv_wgrad_pair: workspaces of %zu and %zu bytes given, %zu and %zu needed",
                         workspace0_bytes, workspace1_bytes, need0, need1), 1;
    if (B > 0) {
        const int r = dwconv_wgrad_pair_launch(x0, gy0, dw0, workspace0, H0, W0, x1, gy1, dw1, workspace1, H1, W1, B, C,
                                               K, P, P, dtype, (hipStream_t)stream);
        if (r != -1) return r;
    }
    if (int e = pdw_dwconv_wgrad(x0, gy0, dw0, workspace0, workspace0_bytes, B, H0, W0, C, K, K, 1, 1, P, P, 1, 1, dtype,
                                 stream))
        return e;
    return pdw_dwconv_wgrad(x1, gy1, dw1, workspace1, workspace1_bytes, B, H1, W1, C, K, K, 1, 1, P, P, 1, 1, dtype,
                            stream);
}

int pdw_dwconv_bwd3(const void* gy0, const void* w0, const void* gp, void* dx, const void* x0, void* dw0, void* workspace0,
                    size_t workspace0_bytes, const void* x1, const void* gy1, void* dw1, void* workspace1,
                    size_t workspace1_bytes, int B, int H, int W, int C, int K, int dtype, void* stream) {
    const int P = K / 2;
    if (!(K & 1)) return set_error("pdw_dwconv_bwd3: odd filter size needed (K=%d)", K), 1;
    if ((H & 1) || (W & 1)) return set_error("pdw_dwconv_bwd3: even extents needed (H=%d W=%d)", H, W), 1;
    if (int e = check_conv("pdw_dwconv_bwd3", x0, gy0, dw0, B, H, W, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (int e = check_conv("pdw_dwconv_bwd3", x1, gy1, dw1, B, H / 2, W / 2, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (!w0 || !gp || !dx || !dw0 || !dw1) return set_error("pdw_dwconv_bwd3: null pointer"), 1;
    const size_t need0 = pdw_dwconv_wgrad_workspace_bytes(B, H, W, C, K, K, 1, 1, P, P, 1, 1, dtype);
    const size_t need1 = pdw_dwconv_wgrad_workspace_bytes(B, H / 2, W / 2, C, K, K, 1, 1, P, P, 1, 1, dtype);
    if (!workspace0 || workspace0_bytes < need0 || !workspace1 || workspace1_bytes < need1)
        return set_error("pdw_dwconv_bwd3: workspaces of %zu and %zu bytes given, %zu and %zu needed", workspace0_bytes,
                         workspace1_bytes, need0, need1), 1;
    if (B == 0) return 0;
    const int r = dwconv_bwd3_launch(gy0, w0, gp, dx, x0, dw0, workspace0, x1, gy1, dw1, workspace1, B, H, W, C, K, dtype,
                                     (hipStream_t)stream);
    if (r == -1) return set_error("pdw_dwconv_bwd3: case not covered (B=%d H=%d W=%d C=%d K=%d dtype=%d)", B, H, W, C, K, dtype), 3;
    return r;
}

int pdw_dwconv_bwd3_plan(int B, int H, int W, int C, int K, int dtype, int* bands) {
    if (!bands || !valid_dtype(dtype) || B < 1 || H < 2 || W < 2 || C < 1 || K < 1 || !(K & 1) || (H & 1) || (W & 1))
        return set_error("pdw_dwconv_bwd3_plan: bad arguments (B=%d H=%d W=%d C=%d K=%d dtype=%d)", B, H, W, C, K, dtype), 1;
    const int r = dwconv_bwd3_launch(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                                     nullptr, nullptr, B, H, W, C, K, dtype, nullptr, bands);
    if (r == -1) return set_error("pdw_dwconv_bwd3_plan: case not covered"), 3;
    return r;
}

int pdw_dwconv_fwd2_supported(int B, int H, int W, int C, int K, int dtype) {
    return valid_dtype(dtype) && dwconv_fwd2_covers(B, H, W, C, K, dtype) ? 1 : 0;
}

int pdw_dwconv_fwd2(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H, int W,
                    int C, int K, int dtype, void* stream) {
    const int P = K / 2;
    if (!(K & 1)) return set_error("pdw_dwconv_fwd2: odd filter size needed (K=%d)", K), 1;
    if ((H & 1) || (W & 1)) return set_error("pdw_dwconv_fwd2: even extents needed (H=%d W=%d)", H, W), 1;
    if (int e = check_conv("pdw_dwconv_fwd2", x0, w0, y0, B, H, W, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (int e = check_conv("pdw_dwconv_fwd2", x1, w1, y1, B, H / 2, W / 2, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (B == 0) return 0;
    const int r = dwconv_fwd2_launch(x0, w0, y0, x1, w1, y1, B, H, W, C, K, dtype, (hipStream_t)stream);
    if (r == -1) return set_error("pdw_dwconv_fwd2: case not covered (B=%d H=%d W=%d C=%d K=%d dtype=%d)", B, H, W, C, K, dtype), 3;
    return r;
}

int pdw_dwconv_fwd2_mean(const void* x0, const void* w0, void* y0, int ldy0, int ych0, const void* x1, const void* w1,
                         void* y1, int ldy1, int ych1, int B, int H, int W, int C, int K, const float* parts, int nparts,
                         const void* w_pool, const void* b_pool, const void* b_out, void* m, float* rowbias, int P, int D,
                         int dtype, void* stream) {
    const int Pd = K / 2;
    if (!(K & 1)) return set_error("pdw_dwconv_fwd2_mean: odd filter size needed (K=%d)", K), 1;
    if ((H & 1) || (W & 1)) return set_error("pdw_dwconv_fwd2_mean: even extents needed (H=%d W=%d)", H, W), 1;
    if (int e = check_conv("pdw_dwconv_fwd2_mean", x0, w0, y0, B, H, W, C, K, K, 1, 1, Pd, Pd, 1, 1, dtype)) return e;
    if (int e = check_conv("pdw_dwconv_fwd2_mean", x1, w1, y1, B, H / 2, W / 2, C, K, K, 1, 1, Pd, Pd, 1, 1, dtype)) return e;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_dwconv_fwd2_mean: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!parts || !w_pool || !m || !rowbias) return set_error("pdw_dwconv_fwd2_mean: null pointer"), 1;
    if ((ldy0 > 0) != (ldy1 > 0) || ldy0 < 0 || ldy1 < 0 || ych0 < 0 || ych1 < 0 ||
        (ldy0 > 0 && ((C & 1) || ldy0 < ych0 + C / 2 || ldy1 < ych1 + C / 2)))
        return set_error("pdw_dwconv_fwd2_mean: gated stores need even C and ych + C/2 <= ldy for both scales (C=%d ldy=%d,%d "
                         "ych=%d,%d)", C, ldy0, ldy1, ych0, ych1), 1;
    int r = -1;
    if (pool_branch_v8_ok(w_pool, m, parts, B, D, dtype) && !(reinterpret_cast<uintptr_t>(rowbias) & 15)) {
        const PoolFwdJob job{parts, nparts, B, D, 1.f / (float)P, w_pool, b_pool, b_out, m, rowbias};
        r = dwconv_fwd2_launch(x0, w0, y0, x1, w1, y1, B, H, W, C, K, dtype, (hipStream_t)stream, ldy0, ych0, ldy1, ych1,
                               &job);
    }
    if (r == -1)
        return set_error("pdw_dwconv_fwd2_mean: case not covered (B=%d H=%d W=%d C=%d K=%d D=%d dtype=%d)", B, H, W, C, K, D,
                         dtype), 3;
    return r;
}

int pdw_dwconv_fwd2_gate(const void* x0, const void* w0, void* y0, int ldy0, int ych0, const void* x1, const void* w1,
                         void* y1, int ldy1, int ych1, int B, int H, int W, int C, int K, int dtype, void* stream) {
    const int P = K / 2;
    if (!(K & 1)) return set_error("pdw_dwconv_fwd2_gate: odd filter size needed (K=%d)", K), 1;
    if ((H & 1) || (W & 1)) return set_error("pdw_dwconv_fwd2_gate: even extents needed (H=%d W=%d)", H, W), 1;
    if (int e = check_conv("pdw_dwconv_fwd2_gate", x0, w0, y0, B, H, W, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (int e = check_conv("pdw_dwconv_fwd2_gate", x1, w1, y1, B, H / 2, W / 2, C, K, K, 1, 1, P, P, 1, 1, dtype)) return e;
    if (ldy0 == 0) ldy0 = C / 2;
    if (ldy1 == 0) ldy1 = C / 2;
    if ((C & 1) || ych0 < 0 || ych1 < 0 || ldy0 < ych0 + C / 2 || ldy1 < ych1 + C / 2)
        return set_error("pdw_dwconv_fwd2_gate: need even C and ych + C/2 <= ldy (C=%d ldy=%d,%d ych=%d,%d)", C, ldy0, ldy1,
                         ych0, ych1), 1;
    if (B == 0) return 0;
    const int r = dwconv_fwd2_launch(x0, w0, y0, x1, w1, y1, B, H, W, C, K, dtype, (hipStream_t)stream, ldy0, ych0, ldy1, ych1);
    if (r == -1)
        return set_error("pdw_dwconv_fwd2_gate: case not covered (B=%d H=%d W=%d C=%d K=%d dtype=%d)", B, H, W, C, K, dtype), 3;
    return r;
}

int pdw_avgpool_fwd(const void* x, void* y, int B, int H, int W, int C, int h, int w, int dtype, void* stream) {
    if (int e = check_resample("pdw_avgpool_fwd", x, y, B, H, W, C, h, w, dtype)) return e;
    return avgpool_fwd_launch(x, y, B, H, W, C, h, w, dtype, (hipStream_t)stream);
}

int pdw_avgpool_bwd(const void* gy, void* gx, int B, int H, int W, int C, int h, int w, int accumulate, int dtype,
                    void* stream) {
    if (int e = check_resample("pdw_avgpool_bwd", gy, gx, B, H, W, C, h, w, dtype)) return e;
    return avgpool_bwd_launch(gy, gx, B, H, W, C, h, w, accumulate ? 1 : 0, dtype, (hipStream_t)stream);
}

int pdw_bilinear_fwd(const void* x, void* y, int B, int h, int w, int C, int H, int W, int ldy, int dtype,
                     void* stream) {
    if (int e = check_resample("pdw_bilinear_fwd", x, y, B, H, W, C, h, w, dtype)) return e;
    if (ldy == 0) ldy = C;
    if (ldy < C) return set_error("pdw_bilinear_fwd: ldy=%d smaller than C=%d", ldy, C), 1;
    return bilinear_fwd_launch(x, y, B, h, w, C, H, W, ldy, dtype, (hipStream_t)stream);
}

int pdw_bilinear_bwd(const void* gy, void* gx, int B, int h, int w, int C, int H, int W, int ldgy, int dtype,
                     void* stream) {
    if (int e = check_resample("pdw_bilinear_bwd", gy, gx, B, H, W, C, h, w, dtype)) return e;
    if (ldgy == 0) ldgy = C;
    if (ldgy < C) return set_error("pdw_bilinear_bwd: ldgy=%d smaller than C=%d", ldgy, C), 1;
    return bilinear_bwd_launch(gy, gx, B, h, w, C, H, W, ldgy, dtype, (hipStream_t)stream);
}

int pdw_gate_fwd(const void* x, void* y, long long M, int I, int ldy, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_gate_fwd: unknown dtype %d", dtype), 1;
    if (M < 0 || I < 2 || (I & 1)) return set_error("pdw_gate_fwd: need M >= 0 and even I >= 2 (M=%lld I=%d)", M, I), 1;
    if (M > 0 && (!x || !y)) return set_error("pdw_gate_fwd: null pointer"), 1;
    if (ldy == 0) ldy = I / 2;
    if (ldy < I / 2) return set_error("pdw_gate_fwd: ldy=%d smaller than I/2=%d", ldy, I / 2), 1;
    return gate_fwd_launch(x, y, M, I, ldy, dtype, (hipStream_t)stream);
}

int pdw_gate_bwd(const void* x, const void* gy, void* gx, long long M, int I, int ldgy, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_gate_bwd: unknown dtype %d", dtype), 1;
    if (M < 0 || I < 2 || (I & 1)) return set_error("pdw_gate_bwd: need M >= 0 and even I >= 2 (M=%lld I=%d)", M, I), 1;
    if (M > 0 && (!x || !gy || !gx)) return set_error("pdw_gate_bwd: null pointer"), 1;
    if (ldgy == 0) ldgy = I / 2;
    if (ldgy < I / 2) return set_error("pdw_gate_bwd: ldgy=%d smaller than I/2=%d", ldgy, I / 2), 1;
    return gate_bwd_launch(x, gy, gx, M, I, ldgy, dtype, (hipStream_t)stream);
}

int pdw_gate_bilinear_fwd(const void* x, void* y, int B, int h, int w, int I, int H, int W, int ldy, int dtype,
                          void* stream) {
    if (int e = check_resample("pdw_gate_bilinear_fwd", x, y, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_gate_bilinear_fwd: need even I >= 2 (I=%d)", I), 1;
    if (ldy == 0) ldy = I / 2;
    if (ldy < I / 2) return set_error("pdw_gate_bilinear_fwd: ldy=%d smaller than I/2=%d", ldy, I / 2), 1;
    return gate_bilinear_fwd_launch(x, y, B, h, w, I, H, W, ldy, dtype, (hipStream_t)stream);
}

int pdw_bilinear_gate_bwd(const void* gy, const void* x, void* gx, int B, int h, int w, int I, int H, int W, int ldgy,
                          int dtype, void* stream) {
    if (int e = check_resample("pdw_bilinear_gate_bwd", gy, gx, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_bilinear_gate_bwd: need even I >= 2 (I=%d)", I), 1;
    if (H != 2 * h || W != 2 * w || h < 2 || w < 2)
        return set_error("pdw_bilinear_gate_bwd: needs H = 2h, W = 2w, h,w >= 2 (h=%d w=%d H=%d W=%d); use "
                         "pdw_bilinear_bwd + pdw_gate_bwd", h, w, H, W), 1;
    if ((long long)B * h * w > 0 && !x) return set_error("pdw_bilinear_gate_bwd: null pointer"), 1;
    if (ldgy == 0) ldgy = I / 2;
    if (ldgy < I / 2) return set_error("pdw_bilinear_gate_bwd: ldgy=%d smaller than I/2=%d", ldgy, I / 2), 1;
    return bilinear_gate_bwd_launch(gy, x, gx, B, h, w, I, H, W, ldgy, dtype, (hipStream_t)stream);
}

int pdw_gate_pair_fwd(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                      int dtype, void* stream) {
    if (int e = check_resample("pdw_gate_pair_fwd", xh, y, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_gate_pair_fwd: need even I >= 2 (I=%d)", I), 1;
    if (B > 0 && !xf) return set_error("pdw_gate_pair_fwd: null pointer"), 1;
    if (ldy == 0) ldy = I;
    if (ldy < I) return set_error("pdw_gate_pair_fwd: ldy=%d smaller than I=%d", ldy, I), 1;
    return gate_pair_fwd_launch(xf, xh, y, B, H, W, h, w, I, ldy, dtype, (hipStream_t)stream);
}

int pdw_gate_pair_bwd(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                      int w, int I, int ldgy, int dtype, void* stream) {
    if (int e = check_resample("pdw_gate_pair_bwd", gy, gxh, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_gate_pair_bwd: need even I >= 2 (I=%d)", I), 1;
    if (B > 0 && (!xf || !xh || !gxf)) return set_error("pdw_gate_pair_bwd: null pointer"), 1;
    if (ldgy == 0) ldgy = I;
    if (ldgy < I) return set_error("pdw_gate_pair_bwd: ldgy=%d smaller than I=%d", ldgy, I), 1;
    const int r = gate_pair_bwd_launch(gy, xf, xh, gxf, gxh, B, H, W, h, w, I, ldgy, dtype, (hipStream_t)stream);
    if (r == -1) return set_error("pdw_gate_pair_bwd: case not covered (B=%d H=%d W=%d h=%d w=%d)", B, H, W, h, w), 3;
    return r;
}

size_t pdw_spatial_sum_workspace_bytes(int B, int P, int C) {
    if (B < 1 || P < 1 || C < 1) return 0;
    return spatial_sum_workspace(B, P, C);
}

int pdw_spatial_sum(const void* x, float* out, void* workspace, size_t workspace_bytes, int B, int P, int C, int dtype,
                    void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_spatial_sum: unknown dtype %d", dtype), 1;
    if (B < 0 || P < 1 || C < 1) return set_error("pdw_spatial_sum: bad extents B=%d P=%d C=%d", B, P, C), 1;
    if (B == 0) return 0;
    if (!x || !out) return set_error("pdw_spatial_sum: null pointer"), 1;
    const size_t need = spatial_sum_workspace(B, P, C);
    if (!workspace || workspace_bytes < need)
        return set_error("pdw_spatial_sum: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    return spatial_sum_launch(x, out, (float*)workspace, B, P, C, dtype, (hipStream_t)stream);
}

int pdw_add_rowbias(void* y, const float* v, int B, int P, int C, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_add_rowbias: unknown dtype %d", dtype), 1;
    if (B < 0 || P < 0 || C < 1) return set_error("pdw_add_rowbias: bad extents B=%d P=%d C=%d", B, P, C), 1;
    if (B == 0 || P == 0) return 0;
    if (!y || !v) return set_error("pdw_add_rowbias: null pointer"), 1;
    return add_rowbias_launch(y, v, B, P, C, dtype, (hipStream_t)stream);
}

size_t pdw_pool_branch_workspace_bytes(int B, int P, int D) {
    if (B < 1 || P < 1 || D < 1) return 0;
    return pool_branch_workspace(B, P, D);
}

int pdw_pool_branch_fwd(const void* x, const void* w_pool, const void* b_pool, const void* b_out, void* m,
                        float* rowbias, void* workspace, size_t workspace_bytes, int B, int P, int D, int dtype,
                        void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_pool_branch_fwd: unknown dtype %d", dtype), 1;
    if (B < 0 || P < 1 || D < 1) return set_error("pdw_pool_branch_fwd: bad extents B=%d P=%d D=%d", B, P, D), 1;
    if (B == 0) return 0;
    if (!x || !w_pool || !m || !rowbias) return set_error("pdw_pool_branch_fwd: null pointer"), 1;
    if (!workspace || workspace_bytes < pool_branch_workspace(B, P, D))
        return set_error("pdw_pool_branch_fwd: workspace too small"), 1;
    return pool_branch_fwd_launch(x, w_pool, b_pool, b_out, m, rowbias, (float*)workspace, B, P, D, dtype,
                                  (hipStream_t)stream);
}

int pdw_pool_branch_bwd(const void* gy, const void* m, const void* w_pool, void* gbias, void* gbias2, void* gw_pool,
                        float* dmean, void* workspace, size_t workspace_bytes, int B, int P, int D, int dtype,
                        void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_pool_branch_bwd: unknown dtype %d", dtype), 1;
    if (B < 1 || P < 1 || D < 1) return set_error("pdw_pool_branch_bwd: bad extents B=%d P=%d D=%d", B, P, D), 1;
    if (!gy || !m || !w_pool || !gbias || !gw_pool || !dmean) return set_error("pdw_pool_branch_bwd: null pointer"), 1;
    if (!workspace || workspace_bytes < pool_branch_workspace(B, P, D))
        return set_error("pdw_pool_branch_bwd: workspace too small"), 1;
    return pool_branch_bwd_launch(gy, m, w_pool, gbias, gbias2, gw_pool, dmean, (float*)workspace, B, P, D, dtype,
                                  (hipStream_t)stream);
}

int pdw_pool_branch_fwd_parts(const float* parts, int nparts, const void* w_pool, const void* b_pool, const void* b_out,
                              void* m, float* rowbias, int B, int P, int D, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_pool_branch_fwd_parts: unknown dtype %d", dtype), 1;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_pool_branch_fwd_parts: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!parts || !w_pool || !m || !rowbias) return set_error("pdw_pool_branch_fwd_parts: null pointer"), 1;
    return pool_branch_fwd_launch(nullptr, w_pool, b_pool, b_out, m, rowbias, nullptr, B, P, D, dtype,
                                  (hipStream_t)stream, parts, nparts);
}

int pdw_pool_branch_bwd_parts(const float* parts, int nparts, const void* m, const void* w_pool, void* gbias,
                              void* gbias2, void* gw_pool, float* dmean, void* workspace, size_t workspace_bytes, int B,
                              int P, int D, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_pool_branch_bwd_parts: unknown dtype %d", dtype), 1;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_pool_branch_bwd_parts: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!parts || !m || !w_pool || !gbias || !gw_pool || !dmean)
        return set_error("pdw_pool_branch_bwd_parts: null pointer"), 1;
    if (!workspace || workspace_bytes < pool_branch_workspace(B, P, D))
        return set_error("pdw_pool_branch_bwd_parts: workspace too small"), 1;
    return pool_branch_bwd_launch(nullptr, m, w_pool, gbias, gbias2, gw_pool, dmean, (float*)workspace, B, P, D, dtype,
                                  (hipStream_t)stream, parts, nparts);
}

int pdw_block_mid_infer(const void* xh, void* y, int B, int H, int W, int h, int w, int G, int ldy, const float* parts,
                        int nparts, const void* w_pool, const void* b_pool, const void* b_out, void* m, float* rowbias,
                        int P, int D, int dtype, void* stream) {
    if (int e = check_resample("pdw_block_mid_infer", xh, y, B, H, W, G, h, w, dtype)) return e;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_block_mid_infer: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!parts || !w_pool || !m || !rowbias) return set_error("pdw_block_mid_infer: null pointer"), 1;
    if (ldy == 0) ldy = G;
    if (ldy < G) return set_error("pdw_block_mid_infer: ldy=%d smaller than G=%d", ldy, G), 1;
    const int r = bilinear_pool_fwd_launch(xh, y, B, h, w, G, H, W, ldy, parts, nparts, w_pool, b_pool, b_out, m, rowbias,
                                           P, D, dtype, (hipStream_t)stream);
    if (r != -1) return r;
    if (int e = bilinear_fwd_launch(xh, y, B, h, w, G, H, W, ldy, dtype, (hipStream_t)stream)) return e;
    return pool_branch_fwd_launch(nullptr, w_pool, b_pool, b_out, m, rowbias, nullptr, B, P, D, dtype,
                                  (hipStream_t)stream, parts, nparts);
}

int pdw_block_mid_fwd(const void* xf, const void* xh, void* y, int B, int H, int W, int h, int w, int I, int ldy,
                      const float* parts, int nparts, const void* w_pool, const void* b_pool, const void* b_out, void* m,
                      float* rowbias, int P, int D, int dtype, void* stream) {
    if (int e = check_resample("pdw_block_mid_fwd", xh, y, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_block_mid_fwd: need even I >= 2 (I=%d)", I), 1;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_block_mid_fwd: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!xf || !parts || !w_pool || !m || !rowbias) return set_error("pdw_block_mid_fwd: null pointer"), 1;
    if (ldy == 0) ldy = I;
    if (ldy < I) return set_error("pdw_block_mid_fwd: ldy=%d smaller than I=%d", ldy, I), 1;
    const int r = block_mid_fwd_launch(xf, xh, y, B, H, W, h, w, I, ldy, parts, nparts, w_pool, b_pool, b_out, m,
                                       rowbias, P, D, dtype, (hipStream_t)stream);
    if (r != -1) return r;
    if (int e = gate_pair_fwd_launch(xf, xh, y, B, H, W, h, w, I, ldy, dtype, (hipStream_t)stream)) return e;
    return pool_branch_fwd_launch(nullptr, w_pool, b_pool, b_out, m, rowbias, nullptr, B, P, D, dtype,
                                  (hipStream_t)stream, parts, nparts);
}

int pdw_block_mid_bwd(const void* gy, const void* xf, const void* xh, void* gxf, void* gxh, int B, int H, int W, int h,
                      int w, int I, int ldgy, const float* parts, int nparts, const void* m, const void* w_pool,
                      void* gbias, void* gbias2, void* gw_pool, float* dmean, void* workspace, size_t workspace_bytes,
                      int P, int D, int dtype, void* stream) {
    if (int e = check_resample("pdw_block_mid_bwd", gy, gxh, B, H, W, I, h, w, dtype)) return e;
    if (I < 2 || (I & 1)) return set_error("pdw_block_mid_bwd: need even I >= 2 (I=%d)", I), 1;
    if (B < 1 || P < 1 || D < 1 || nparts < 1)
        return set_error("pdw_block_mid_bwd: bad extents B=%d P=%d D=%d nparts=%d", B, P, D, nparts), 1;
    if (!xf || !xh || !gxf || !parts || !m || !w_pool || !gbias || !gw_pool || !dmean)
        return set_error("pdw_block_mid_bwd: null pointer"), 1;
    if (H != 2 * h || W != 2 * w || h < 2 || w < 2)
        return set_error("pdw_block_mid_bwd: needs H = 2h, W = 2w, h,w >= 2 (h=%d w=%d H=%d W=%d)", h, w, H, W), 1;
    if (!workspace || workspace_bytes < pool_branch_workspace(B, P, D))
        return set_error("pdw_block_mid_bwd: workspace too small"), 1;
    if (ldgy == 0) ldgy = I;
    if (ldgy < I) return set_error("pdw_block_mid_bwd: ldgy=%d smaller than I=%d", ldgy, I), 1;
    const int r = block_mid_bwd_launch(gy, xf, xh, gxf, gxh, B, H, W, h, w, I, ldgy, parts, nparts, m, w_pool, gbias,
                                       gbias2, gw_pool, dmean, (float*)workspace, P, D, dtype, (hipStream_t)stream);
    if (r != -1) return r;
    if (int e = gate_pair_bwd_launch(gy, xf, xh, gxf, gxh, B, H, W, h, w, I, ldgy, dtype, (hipStream_t)stream)) return e;
    return pool_branch_bwd_launch(nullptr, m, w_pool, gbias, gbias2, gw_pool, dmean, (float*)workspace, B, P, D, dtype,
                                  (hipStream_t)stream, parts, nparts);
}

int pdw_dense_colsum_supported(int K, int NO, int dtype) {
    return (dense_colsum_supported(K, NO, dtype) && dense_wgrad_supported(K, NO, dtype)) ? 1 : 0;
}

int pdw_dense_colsum_rows(void) { return dense_colsum_rows(); }

int pdw_dense_fwd_colsum(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                         float* colsum, long long N, int K, int NO, int P, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_fwd_colsum: unknown dtype %d", dtype), 1;
    if (N < 0 || K < 1 || NO < 1) return set_error("pdw_dense_fwd_colsum: bad extents N=%lld K=%d NO=%d", N, K, NO), 1;
    if (N > 0 && (!x || !w || !y || !colsum)) return set_error("pdw_dense_fwd_colsum: null pointer"), 1;
    if (rowbias && P < 1) return set_error("pdw_dense_fwd_colsum: rowbias needs P >= 1"), 1;
    const int r = dense_rows_launch(x, w, w_kmajor ? 1 : 0, bias, rowbias, y, N, K, NO, P, dtype, (hipStream_t)stream,
                                    colsum);
    if (r == -1)
        return set_error("pdw_dense_fwd_colsum: K=%d NO=%d dtype=%d not supported (see pdw_dense_colsum_supported)", K,
                         NO, dtype), 3;
    return r;
}

int pdw_dense_fwd_colsum_pool(const void* x, const void* w, const void* bias, void* y, float* colsum, void* pool, int B,
                              int H, int W, int K, int NO, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_fwd_colsum_pool: unknown dtype %d", dtype), 1;
    if (B < 0 || H < 2 || W < 2 || (H & 1) || (W & 1) || K < 1 || NO < 1)
        return set_error("pdw_dense_fwd_colsum_pool: bad extents B=%d H=%d W=%d K=%d NO=%d", B, H, W, K, NO), 1;
    if (B > 0 && (!x || !w || !y || !colsum || !pool)) return set_error("pdw_dense_fwd_colsum_pool: null pointer"), 1;
    if (B == 0) return 0;
    const int r = dense_rows_pool_launch(x, w, bias, y, colsum, pool, B, H, W, K, NO, dtype, (hipStream_t)stream);
    if (r == -1)
        return set_error("pdw_dense_fwd_colsum_pool: case not covered (B=%d H=%d W=%d K=%d NO=%d dtype=%d)", B, H, W, K, NO,
                         dtype), 3;
    return r;
}

int pdw_dense_fwd_gated_supported(int H, int W, int I, int D, int dtype) {
    return valid_dtype(dtype) && H > 0 && W > 0 && I > 0 && D > 0 ? dense_mid_rows_supported(H, W, I, D, dtype) : 0;
}

int pdw_dense_fwd_gated(const void* cf, const void* ch, void* cat, const void* w, const void* bias, const float* rowbias,
                        void* y, int B, int H, int W, int I, int D, int ldf, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_fwd_gated: unknown dtype %d", dtype), 1;
    if (B < 0 || H < 2 || W < 2 || (H & 1) || (W & 1) || I < 2 || (I & 1) || D < 1)
        return set_error("pdw_dense_fwd_gated: bad extents B=%d H=%d W=%d I=%d D=%d", B, H, W, I, D), 1;
    if (B > 0 && (!cf || !ch || !w || !y)) return set_error("pdw_dense_fwd_gated: null pointer"), 1;
    if (ldf < 0 || (ldf > 0 && (ldf < I / 2 || cat)))
        return set_error("pdw_dense_fwd_gated: gated inputs need ldf >= I/2 and no cat (ldf=%d I=%d)", ldf, I), 1;
    if (B == 0) return 0;
    const int r = dense_mid_rows_launch(cf, ch, cat, w, bias, rowbias, y, B, H, W, I, D, dtype, (hipStream_t)stream, ldf);
    if (r == -1)
        return set_error("pdw_dense_fwd_gated: case not covered (B=%d H=%d W=%d I=%d D=%d dtype=%d)", B, H, W, I, D, dtype), 3;
    return r;
}

int pdw_dense_supported(int K, int NO, int dtype) {
    return (dense_rows_supported(K, NO, dtype) && dense_wgrad_supported(K, NO, dtype)) ? 1 : 0;
}

int pdw_dense_fwd(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                  long long N, int K, int NO, int P, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_fwd: unknown dtype %d", dtype), 1;
    if (N < 0 || K < 1 || NO < 1) return set_error("pdw_dense_fwd: bad extents N=%lld K=%d NO=%d", N, K, NO), 1;
    if (N > 0 && (!x || !w || !y)) return set_error("pdw_dense_fwd: null pointer"), 1;
    if (rowbias && P < 1) return set_error("pdw_dense_fwd: rowbias needs P >= 1"), 1;
    const int r = dense_rows_launch(x, w, w_kmajor ? 1 : 0, bias, rowbias, y, N, K, NO, P, dtype, (hipStream_t)stream);
    if (r == -1) return set_error("pdw_dense_fwd: K=%d NO=%d dtype=%d not supported (see pdw_dense_supported)", K, NO, dtype), 3;
    return r;
}

int pdw_dense_fwd_flush(const void* x, const void* w, int w_kmajor, const void* bias, const float* rowbias, void* y,
                        long long N, int K, int NO, int P, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_fwd_flush: unknown dtype %d", dtype), 1;
    if (N < 0 || K < 1 || NO < 1) return set_error("pdw_dense_fwd_flush: bad extents N=%lld K=%d NO=%d", N, K, NO), 1;
    if (N > 0 && (!x || !w || !y)) return set_error("pdw_dense_fwd_flush: null pointer"), 1;
    if (rowbias && P < 1) return set_error("pdw_dense_fwd_flush: rowbias needs P >= 1"), 1;
    ReduceJobs jobs;
    const bool ride = N > 0 && dense_rows_supported(K, NO, dtype) && reduce_defer_take(&jobs) > 0;
    const int r = dense_rows_launch(x, w, w_kmajor ? 1 : 0, bias, rowbias, y, N, K, NO, P, dtype, (hipStream_t)stream,
                                    nullptr, ride ? &jobs : nullptr);
    if (r == -1) {
        if (ride) (void)reduce_jobs_launch(jobs, (hipStream_t)stream);  // the reductions still run, on their own
        return set_error("pdw_dense_fwd_flush: K=%d NO=%d dtype=%d not supported (see pdw_dense_supported)", K, NO, dtype), 3;
    }
    return r;
}

size_t pdw_dense_wgrad_workspace_bytes(long long N, int M, int NO) {
    if (N < 0 || M < 1 || NO < 1) return 0;
    return dense_wgrad_workspace(N, M, NO);
}

int pdw_dense_wgrad(const void* a, const void* b, void* dw, void* workspace, size_t workspace_bytes, long long N, int M,
                    int NO, int dtype, void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_wgrad: unknown dtype %d", dtype), 1;
    if (N < 0 || M < 1 || NO < 1) return set_error("pdw_dense_wgrad: bad extents N=%lld M=%d NO=%d", N, M, NO), 1;
    if (!dw || (N > 0 && (!a || !b))) return set_error("pdw_dense_wgrad: null pointer"), 1;
    const size_t need = dense_wgrad_workspace(N, M, NO);
    if (!workspace || workspace_bytes < need)
        return set_error("pdw_dense_wgrad: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    const int r = dense_wgrad_launch(a, b, dw, workspace, N, M, NO, dtype, (hipStream_t)stream);
    if (r == -1) return set_error("pdw_dense_wgrad: M=%d NO=%d dtype=%d not supported", M, NO, dtype), 3;
    return r;
}

int pdw_dense_bwd_pair_supported(int O, int I, int dtype) {
    return valid_dtype(dtype) ? dense_bwd_pair_supported(O, I, dtype) : 0;
}

int pdw_dense_bwd_pair_colsum_supported(int O, int I, int dtype) {
    return valid_dtype(dtype) ? dense_bwd_pair_colsum_supported(O, I, dtype) : 0;
}

int pdw_dense_bwd_pair(const void* gy, const void* w, const void* x, void* dx, float* colsum, void* dw, void* workspace,
                       size_t workspace_bytes, const float* rowbias, int P, long long N, int O, int I, int dtype,
                       void* stream) {
    if (!valid_dtype(dtype)) return set_error("pdw_dense_bwd_pair: unknown dtype %d", dtype), 1;
    if (N < 1 || O < 1 || I < 1) return set_error("pdw_dense_bwd_pair: bad extents N=%lld O=%d I=%d", N, O, I), 1;
    if (!gy || !w || !x || !dx || !dw) return set_error("pdw_dense_bwd_pair: null pointer"), 1;
    const size_t need = dense_wgrad_workspace(N, O, I);
    if (!workspace || workspace_bytes < need)
        return set_error("pdw_dense_bwd_pair: workspace of %zu bytes given, %zu needed", workspace_bytes, need), 1;
    if (rowbias && P < 1) return set_error("pdw_dense_bwd_pair: rowbias needs P >= 1"), 1;
    const int r = dense_bwd_pair_launch(gy, w, x, dx, colsum, dw, workspace, rowbias, P, N, O, I, dtype,
                                        (hipStream_t)stream);
    if (r == -1)
        return set_error("pdw_dense_bwd_pair: O=%d I=%d dtype=%d (P=%d) not covered (see pdw_dense_bwd_pair_supported)",
                         O, I, dtype, P), 3;
    return r;
}

}  // extern "C"
