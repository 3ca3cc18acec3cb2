// The forward convolutions of both scales of a two-scale block as one launch: y0 = conv(x0, w0) at the full scale and
// y1 = conv(x1, w1) at half the extents (x1 being the 2x2 average pool of x0, made before the launch), neither
// depending on the other.  A compute unit holds one workgroup of these kernels at a time and a band costs a start-up
// that does not depend on its height, so a launch of its own cuts a problem into enough bands to fill the chip; here
// the full scale runs as whole-image bands on half of the compute units while the half scale's workgroups run on the
// others (14.8 us against 13.9 + 7.9 us and a launch gap at [32,56,56,64], K = 13).
// The kernel template and its per-filter-size launcher; dwconv_fwd2_k<K>.hip instantiate it, one file per size.
#pragma once
#include <algorithm>
#include <map>
#include <queue>
#include <tuple>
#include <vector>

#include "dwconv_tz.h"
#include "pool_branch.h"

namespace pdw {

struct Fwd2Args {
    const void *x0, *w0, *x1, *w1;
    void *y0, *y1;
    TzGeom g0, g1;
    int s0, n0, s1, n1;   // first workgroup and number of workgroups of each problem
    PoolFwdJob mean;      // workgroups behind both problems (one per image, mean.B of them): the block's mean branch
};

// MODE 0: the convolutions; 4: each with the gate applied in its store (dwconv_tz.h).
template <typename T, int K, int CS, int NPC1, int MODE>
__global__ __launch_bounds__(512, 1) void dwconv_fwd2_k(const Fwd2Args a) {
    const unsigned blk = blockIdx.x;
    if (blk - (unsigned)a.s0 < (unsigned)a.n0)
        dwconv_tz_body<T, K, 16, CS, MODE>((const T*)a.x0, (const T*)a.w0, nullptr, nullptr, (T*)a.y0, a.g0, (int)blk - a.s0,
                                           a.n0);
    else if (blk - (unsigned)a.s1 < (unsigned)a.n1)
        dwconv_tz_body<T, K, NPC1, CS, MODE>((const T*)a.x1, (const T*)a.w1, nullptr, nullptr, (T*)a.y1, a.g1,
                                             (int)blk - a.s1, a.n1);
    else {
        // The mean branch (per-image mean -> conv_pool -> the row added to every output row of the image) needs a
        // launch whose memory system is not saturated, and its inputs are ready when this one starts: last in the
        // grid, its short workgroups go to compute units the convolutions leave free or have finished with.
        extern __shared__ uint32_t smem[];
        pool_branch_fwd_v8_body<T>(a.mean.part, a.mean.nchunks, a.mean.D, a.mean.inv_p, (const T*)a.mean.wp,
                                   (const T*)a.mean.bp, (const T*)a.mean.bo, (T*)a.mean.m, a.mean.rowbias,
                                   (int)blk - a.n0 - a.n1, reinterpret_cast<float*>(smem));
    }
}

// Workgroups dealt in grid order to the earliest free of 256 compute units: the time the last one ends.
inline double tz_makespan(int nproblems, const double* cost, const long long* count, const int* ord) {
    constexpr int kCU = 256;
    std::priority_queue<double, std::vector<double>, std::greater<double>> free_at;
    for (int c = 0; c < kCU; ++c) free_at.push(0.0);
    double end = 0;
    for (int o = 0; o < nproblems; ++o)
        for (long long n = 0; n < count[ord[o]]; ++n) {
            const double t = free_at.top() + cost[ord[o]];
            free_at.pop();
            free_at.push(t);
            end = std::max(end, t);
        }
    return end;
}

struct Fwd2Plan {
    int nb[2];    // bands of the full and of the half scale
    int first;    // problem whose workgroups come first in the grid
};

// Band costs in microseconds fitted to traces at [32,56,56,64]: a 64-column band of one image 9.6 + 0.045 per row
// (K = 13), a 32-column band of two images 3.7 + 0.175 per row.
template <int K, int CS, int NPC1>
static Fwd2Plan fwd2_plan(int B, const TzGeom& g0, const TzGeom& g1) {
    static std::mutex mu;
    struct Key {
        int B, H, W, C;
        bool operator<(const Key& o) const { return std::tie(B, H, W, C) < std::tie(o.B, o.H, o.W, o.C); }
    };
    static std::map<Key, Fwd2Plan> cache;
    const Key key{B, g0.OH, g0.OW, g0.C};
    std::lock_guard<std::mutex> lock(mu);
    if (auto it = cache.find(key); it != cache.end()) return it->second;
    const int oh[2] = {g0.OH, g1.OH};
    const long long per_band[2] = {(long long)cdiv(B, TzShape<K, 16, CS>::NI) * g0.ncolt * g0.nslices,
                                   (long long)cdiv(B, TzShape<K, NPC1, CS>::NI) * g1.ncolt * g1.nslices};
    const int standalone[2] = {g0.nbands, g1.nbands};
    const double work = TzShape<K, 16, CS>::NM / 8.0;
    auto band_cost = [&](int i, int br) {
        if (i == 0 || NPC1 == 16) return (CS == 16 ? 9.6 : 7.0) + 0.045 * br * work;
        return (CS == 16 ? 3.7 : 3.0) + 0.175 * br * work;
    };
    Fwd2Plan best{{standalone[0], standalone[1]}, 0};
    double best_t = 0;
    const bool plenty = per_band[0] + per_band[1] > 1536;   // the chip is full whatever the cut: fewest start-ups
    const int cand[4] = {1, 2, 4, 0};                       // 0: the stand-alone planner's count
    for (int a = 0; a < 4; ++a)
        for (int b = 0; b < 4; ++b) {
            if (plenty && (a | b) != 0) continue;
            const int pick[2] = {cand[a], cand[b]};
            int nb[2];
            double cost[2];
            long long count[2];
            bool ok = true;
            for (int i = 0; i < 2; ++i) {
                nb[i] = pick[i] ? pick[i] : standalone[i];
                if (pick[i] && nb[i] > std::max(1, oh[i] / 4)) ok = false;
                const int br = (cdiv(oh[i], nb[i]) + 3) / 4 * 4;
                nb[i] = cdiv(oh[i], br);
                cost[i] = band_cost(i, br), count[i] = per_band[i] * nb[i];
            }
            if (!ok) continue;
            const int ord[2] = {cost[0] >= cost[1] ? 0 : 1, cost[0] >= cost[1] ? 1 : 0};   // longest first
            const double t = plenty ? 1.0 : tz_makespan(2, cost, count, ord);
            if (best_t == 0 || t < best_t - 1e-9) best_t = t, best = Fwd2Plan{{nb[0], nb[1]}, ord[0]};
        }
    if (cache.size() >= kPlanCacheMax) cache.clear();   // callers with ever-changing shapes: a plan is cheap to redo
    cache[key] = best;
    return best;
}

// -1: not covered (the caller makes the two launches).  16-bit types, C % 8 == 0, padding K / 2, the second scale
// exactly half the first, the full scale in the wide tile.
// gate0, gate1 (both or neither): the gate in the store of each scale, y0 / y1 then being the gated tensors with the
// strides and channel offsets the gates name.
template <int K>
static int launch_fwd2(const void* x0, const void* w0, void* y0, const void* x1, const void* w1, void* y1, int B, int H,
                       int W, int C, int dtype, hipStream_t s, const TzGate* gate0 = nullptr,
                       const TzGate* gate1 = nullptr, const PoolFwdJob* mean = nullptr) {
    constexpr int CS = (2 * 4 * TzShape<K, 16, 16>::NM + 2 * 4 * TzShape<K, 16, 16>::RING) <= 160 ? 16 : 8;
    if (dtype == kF32 || C % 8 != 0 || (H & 1) || (W & 1) || B < 1 || H < 2 || W < 2) return -1;
    if ((gate0 != nullptr) != (gate1 != nullptr)) return -1;
    const int P = K / 2, h = H / 2, wd = W / 2;
    for (const void* p : {x0, w0, (const void*)y0, x1, w1, (const void*)y1})
        if (!p || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    auto wide = [&](int ow) {
        const long long pad16 = (long long)cdiv(ow, 64) * 64 * B, pad8 = (long long)cdiv(ow, 32) * 32 * cdiv(B, 2) * 2;
        return pad16 <= pad8;
    };
    if (!wide(W)) return -1;
    const bool wide1 = wide(wd);
    Fwd2Args a;
    long long n0, n1;
    if (!tz_make_geom<K, 16, CS>(a.g0, n0, false, B, H, W, C, P, P, false, gate0)) return -1;
    if (!(wide1 ? tz_make_geom<K, 16, CS>(a.g1, n1, false, B, h, wd, C, P, P, false, gate1)
                : tz_make_geom<K, 8, CS>(a.g1, n1, false, B, h, wd, C, P, P, false, gate1)))
        return -1;
    Fwd2Plan plan = wide1 ? fwd2_plan<K, CS, 16>(B, a.g0, a.g1) : fwd2_plan<K, CS, 8>(B, a.g0, a.g1);
    if (const char* e = tune_env("PDW_FWD2_BANDS")) {   // "bands of the full scale, of the half scale, first problem"
        if (sscanf(e, "%d,%d,%d", &plan.nb[0], &plan.nb[1], &plan.first) != 3) return -1;
    }
    if (tune_env("PDW_FWD2_PRINT"))
        fprintf(stderr, "fwd2 plan B=%d H=%d W=%d C=%d K=%d: bands %d %d first %d\n", B, H, W, C, K, plan.nb[0], plan.nb[1], plan.first);
    auto rows_of = [](int oh, int nb) { return (cdiv(oh, nb) + 3) / 4 * 4; };
    a.g0.BR = rows_of(a.g0.OH, plan.nb[0]), a.g0.nbands = cdiv(a.g0.OH, a.g0.BR);
    a.g1.BR = rows_of(a.g1.OH, plan.nb[1]), a.g1.nbands = cdiv(a.g1.OH, a.g1.BR);
    n0 = (long long)cdiv(B, TzShape<K, 16, CS>::NI) * a.g0.nbands * a.g0.ncolt * a.g0.nslices;
    n1 = (long long)cdiv(B, wide1 ? TzShape<K, 16, CS>::NI : TzShape<K, 8, CS>::NI) * a.g1.nbands * a.g1.ncolt * a.g1.nslices;
    const int nmean = mean ? mean->B : 0;
    if (n0 + n1 + nmean > 0x7fffffffLL) return -1;
    a.mean = mean ? *mean : PoolFwdJob{};
    a.x0 = x0, a.w0 = w0, a.y0 = y0, a.x1 = x1, a.w1 = w1, a.y1 = y1;
    a.n0 = (int)n0, a.n1 = (int)n1;
    a.s0 = plan.first == 0 ? 0 : a.n1, a.s1 = plan.first == 0 ? a.n0 : 0;
    size_t lds = TzShape<K, 16, CS>::lds_bytes;
    if (!wide1 && TzShape<K, 8, CS>::lds_bytes > lds) lds = TzShape<K, 8, CS>::lds_bytes;
    if (nmean > 0 && lds < (size_t)9 * mean->D * sizeof(float)) lds = (size_t)9 * mean->D * sizeof(float);
    const unsigned grid = (unsigned)(n0 + n1 + nmean);
    static std::once_flag once[8];
#define PDW_FWD2_GO(T, NPC1, MODE, SLOT)                                                                              \
    {                                                                                                                 \
        auto kern = dwconv_fwd2_k<T, K, CS, NPC1, MODE>;                                                              \
        std::call_once(once[SLOT], [&] {                                                                              \
            (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);     \
        });                                                                                                           \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, s, a);                                                   \
    }
    if (gate0) {
        if (dtype == kF16) {
            if (wide1) PDW_FWD2_GO(f16_t, 16, 4, 4) else PDW_FWD2_GO(f16_t, 8, 4, 5)
        } else {
            if (wide1) PDW_FWD2_GO(bf16_t, 16, 4, 6) else PDW_FWD2_GO(bf16_t, 8, 4, 7)
        }
    } else if (dtype == kF16) {
        if (wide1) PDW_FWD2_GO(f16_t, 16, 0, 0) else PDW_FWD2_GO(f16_t, 8, 0, 1)
    } else {
        if (wide1) PDW_FWD2_GO(bf16_t, 16, 0, 2) else PDW_FWD2_GO(bf16_t, 8, 0, 3)
    }
#undef PDW_FWD2_GO
    return check_launch("dwconv_fwd2");
}

}  // namespace pdw
