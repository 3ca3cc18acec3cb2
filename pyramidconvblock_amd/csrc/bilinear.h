// Source rows / columns, weights and the four-tap mix of the bilinear resize (F.interpolate(mode="bilinear",
// align_corners=False), conv_block.py:21), shared by every kernel that resizes so that all of them produce the same bits.
#pragma once
#include "common.h"

namespace pdw {

// src = max(scale*(dst+0.5)-0.5, 0), i0 = floor(src), i1 = min(i0+1, in-1), lam = src - i0 (fp32, as ATen does
// for every element type up to float).
__device__ __forceinline__ void bl_src(int dst, float scale, int in, int& i0, int& i1, float& lam) {
    float src = scale * ((float)dst + 0.5f) - 0.5f;
    src = src < 0.f ? 0.f : src;
    int lo = (int)src;
    lo = lo > in - 1 ? in - 1 : lo;
    i0 = lo;
    i1 = lo + (lo < in - 1 ? 1 : 0);
    lam = src - (float)lo;
}

// One resized value from its four taps (row y0: g00, g01; row y1: g10, g11) and bl_src's weights.  The order of the
// operations and the fused multiply-adds are spelled out and the result is an fp32 value of its own (see gate_f32),
// so that every kernel that resizes produces the same bits whatever the compiler would contract.
__device__ __forceinline__ float bl_mix(float g00, float g01, float g10, float g11, float ly, float lx) {
    const float hy = 1.f - ly, hx = 1.f - lx;
    const float t0 = __fmaf_rn(lx, g01, __fmul_rn(hx, g00));
    const float t1 = __fmaf_rn(lx, g11, __fmul_rn(hx, g10));
    float r = __fmaf_rn(ly, t1, __fmul_rn(hy, t0));
    asm volatile("" : "+v"(r));
    return r;
}

}  // namespace pdw
