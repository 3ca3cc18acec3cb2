// Shared device helpers for the gfx950 kernels: element types, fp32 conversion,
// channel-vector loads/stores and launch-status plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

namespace pdw {

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

enum : int { kF32 = 0, kF16 = 1, kBF16 = 2 };

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v) {
    return (T)v;  // round-to-nearest-even (v_cvt_f16_f32 / v_cvt_pk_bf16_f32)
}

// a * b * s as an fp32 value of its own.  Without the barrier the compiler may fuse the second multiplication with
// a following conversion to a 16-bit type (one rounding instead of two), in some kernels and element positions and
// not in others: results that differ in the last bit for about one value in 20 000.
__device__ __forceinline__ float gate_f32(float a, float b, float s) {
    float q = a * b * s;
    asm volatile("" : "+v"(q));
    return q;
}

// N consecutive channels moved as one naturally aligned access of N*sizeof(T) bytes.
template <typename T, int N>
struct alignas(sizeof(T) * N) ChanVec {
    T v[N];
};

template <typename T, int N>
__device__ __forceinline__ void load_f32(const T* __restrict__ p, float (&out)[N]) {
    ChanVec<T, N> r = *reinterpret_cast<const ChanVec<T, N>*>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_f32(r.v[i]);
}

template <typename T, int N>
__device__ __forceinline__ void store_f32(T* __restrict__ p, const float (&in)[N]) {
    ChanVec<T, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = from_f32<T>(in[i]);
    *reinterpret_cast<ChanVec<T, N>*>(p) = r;
}

// Widest channel vector (in elements, <= 16 bytes) that keeps every pixel's channel run
// aligned: requires C % N == 0 and an N*sizeof(T)-aligned base pointer.
inline int pick_vec(int C, size_t elem, const void* const* ptrs, int nptrs) {
    int n = (int)(16 / elem);
    while (n > 1) {
        bool ok = (C % n) == 0;
        for (int i = 0; ok && i < nptrs; ++i)
            ok = (reinterpret_cast<uintptr_t>(ptrs[i]) % (n * elem)) == 0;
        if (ok) break;
        n >>= 1;
    }
    return n;
}

inline int cdiv(long long a, long long b) { return (int)((a + b - 1) / b); }

// Entries a per-shape launch-plan cache may hold before it is emptied (a plan costs microseconds to redo).
constexpr size_t kPlanCacheMax = 256;

// Planner overrides for experiments (PDW_* environment variables): read only in a build with -DPDW_TUNE.
// The shipped library never looks at the environment; every planner then takes its own choice.
#ifdef PDW_TUNE
inline const char* tune_env(const char* name) { return getenv(name); }
#else
inline const char* tune_env(const char*) { return nullptr; }
#endif

// Thread-local last-error text returned through the C ABI.
void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace pdw
