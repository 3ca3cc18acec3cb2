// The three convolution launches at the end of a two-scale block's backward pass that do not depend on one another
// (the full-scale input gradient with the pooled branch's gradient added, and the weight gradients of both scales) as
// one launch: on a compute unit a band of each runs back to back, without two drains and launch gaps in between.
// The kernel template and its per-filter-size launcher; dwconv_bwd3_k<K>.hip instantiate it, one file per size.
#pragma once
#include "dwconv_tz.h"
#include "dwconv_wgrad_tz.h"
#include <algorithm>
#include <map>
#include <queue>
#include <tuple>
#include <vector>

#include "reduce_parts.h"

namespace pdw {

struct Bwd3Args {
    const void *gy, *w, *add;   // input gradient: dx = conv^T(gy, w) + add / 4 (2x2 blocks)
    void* dx;
    const void *x0, *gy0, *x1, *gy1;   // weight gradients
    float *part0, *part1;
    TzGeom gd;
    WgTzGeom g0, g1;
    int sd, nd, s1, n1, s0, n0;   // first workgroup and number of workgroups of the input gradient, the half scale's
                                  // and the full scale's weight gradient
};

// Each problem's workgroups are a contiguous range of the grid, in the order the launcher chose.
template <typename T, int K, int CS, int NGA, int NCB1, int NB>
__global__ __launch_bounds__(512, 1) void dwconv_bwd3_k(const Bwd3Args a) {
    const unsigned blk = blockIdx.x;
    if (blk - (unsigned)a.sd < (unsigned)a.nd)
        dwconv_tz_body<T, K, 16, CS, 1>((const T*)a.gy, (const T*)a.w, (const T*)a.add, nullptr, (T*)a.dx, a.gd,
                                        (int)blk - a.sd, a.nd);
    else if (blk - (unsigned)a.s1 < (unsigned)a.n1)
        dwconv_wgrad_tz_body<T, NGA, NCB1, NB>((const T*)a.x1, (const T*)a.gy1, a.part1, a.g1, (int)blk - a.s1, a.n1);
    else
        dwconv_wgrad_tz_body<T, NGA, 8, NB>((const T*)a.x0, (const T*)a.gy0, a.part0, a.g0, (int)blk - a.s0, a.n0);
}

// Band heights and grid order of the three problems.  A compute unit holds one workgroup of this launch at a time, and a
// band costs a start-up (first windows, operand set-up) that does not depend on its height, so unlike a launch of its
// own, which has to fill the chip, a problem here is best cut into as few bands as the other problems leave room for:
// each candidate (1, 2, 4 or the stand-alone planner's number of bands per problem) is priced by dealing its
// workgroups, longest problem first (the grid order), to the earliest free of 256 compute units.  Band costs in
// microseconds, fitted to traces of this launch at [32,56,56,64] (whole-image bands for all three: 28.7 us against
// 37.4 us with the bands of the separate launches at K = 13, 30.3 against 38.5 at K = 9, 50.0 against 60.2 at K = 17).
struct Bwd3Plan {
    int nb[3];        // bands of the input gradient, the full scale's and the half scale's weight gradient
    char order[4];    // 'D', 'F', 'H' in grid order
};

inline double bwd3_makespan(const double (&cost)[3], const long long (&count)[3], const int (&ord)[3]) {
    constexpr int kCU = 256;
    std::priority_queue<double, std::vector<double>, std::greater<double>> free_at;   // earliest free unit on top
    for (int c = 0; c < kCU; ++c) free_at.push(0.0);
    double end = 0;
    for (int o = 0; o < 3; ++o)
        for (long long n = 0; n < count[ord[o]]; ++n) {
            const double t = free_at.top() + cost[ord[o]];
            free_at.pop();
            free_at.push(t);
            end = std::max(end, t);
        }
    return end;
}

template <int K, int CS>
static Bwd3Plan bwd3_plan(int B, const TzGeom& gd, const WgTzPlan& p0, const WgTzPlan& p1) {
    static std::mutex mu;
    struct Key {
        int B, H, W, C;
        bool operator<(const Key& o) const { return std::tie(B, H, W, C) < std::tie(o.B, o.H, o.W, o.C); }
    };
    static std::map<Key, Bwd3Plan> cache;
    const Key key{B, gd.OH, gd.OW, gd.C};
    std::lock_guard<std::mutex> lock(mu);
    if (auto it = cache.find(key); it != cache.end()) return it->second;
    const int oh[3] = {gd.OH, p0.g.OH, p1.g.OH};
    const long long per_band[3] = {(long long)cdiv(B, TzShape<K, 16, CS>::NI) * gd.ncolt * gd.nslices,
                                   (long long)B * p0.g.ncolt * p0.g.nslices, (long long)B * p1.g.ncolt * p1.g.nslices};
    const int standalone[3] = {gd.nbands, p0.g.nbands, p1.g.nbands};
    constexpr int nmf = K == 17 ? 2 : 1;
    auto band_rows = [&](int i, int nb) { return (cdiv(oh[i], nb) + 3) / 4 * 4; };
    auto band_cost = [&](int i, int br) {
        if (i == 0) return (CS == 16 ? 9.6 : 7.0) + 0.045 * br * (TzShape<K, 16, CS>::NM / 8.0);
        const int ncb = i == 1 ? p0.ncb : p1.ncb;
        return 3.0 + 1.5 * nmf * (ncb == 8 ? 1.0 : 0.9) * ((br + 4) / 4);
    };
    // the fallback when no candidate survives: every problem cut as its stand-alone launch cuts it
    Bwd3Plan best{{std::max(1, standalone[0]), std::max(1, standalone[1]), std::max(1, standalone[2])}, "DFH"};
    double best_t = 0;
    // with many times more whole-image bands than compute units the chip is full whatever the cut: fewest start-ups
    const bool plenty = per_band[0] + per_band[1] + per_band[2] > 1536;
    const int cand[4] = {1, 2, 4, 0};   // 0: the stand-alone planner's count
    for (int a = 0; a < 4; ++a)
        for (int b = 0; b < 4; ++b)
            for (int c = 0; c < 4; ++c) {
                const int pick[3] = {cand[a], cand[b], cand[c]};
                if (plenty && (a | b | c) != 0) continue;
                int nb[3];
                double cost[3];
                long long count[3];
                bool ok = true;
                for (int i = 0; i < 3; ++i) {
                    nb[i] = pick[i] ? pick[i] : standalone[i];
                    // a weight gradient's partials must fit the workspace sized for the stand-alone plan
                    if (pick[i] && (nb[i] > std::max(1, oh[i] / 4) || (i > 0 && nb[i] > standalone[i]))) ok = false;
                    const int br = band_rows(i, nb[i]);
                    nb[i] = cdiv(oh[i], br);
                    cost[i] = band_cost(i, br), count[i] = per_band[i] * nb[i];
                }
                if (!ok) continue;
                int ord[3] = {0, 1, 2};
                // longest first; the input gradient ahead of a weight gradient of similar length (its band is mostly
                // start-up, memory latency that overlaps best with the other problems' arithmetic: 29.1 against 30.2 us)
                auto rank = [&](int x) { return cost[x] * (x == 0 ? 1.25 : 1.0); };
                std::sort(ord, ord + 3, [&](int x, int y) { return rank(x) > rank(y); });
                const double t = plenty ? 1.0 : bwd3_makespan(cost, count, ord);
                if (best_t == 0 || t < best_t - 1e-9) {
                    best_t = t;
                    for (int i = 0; i < 3; ++i) best.nb[i] = nb[i], best.order[i] = "DFH"[ord[i]];
                    best.order[3] = 0;
                }
            }
    if (cache.size() >= kPlanCacheMax) cache.clear();   // callers with ever-changing shapes: a plan is cheap to redo
    cache[key] = best;
    return best;
}

// -1: not covered (the caller makes the three launches).  16-bit types, C % 16 == 0, padding K / 2, the second scale
// exactly half the first, the full scale in the wide tiles of both kernels.
template <int K>
static int launch_bwd3(const void* gyf, const void* w0, const void* addp, void* dx, const void* x0, void* dw0, void* ws0,
                       const void* x1, const void* gy1, void* dw1, void* ws1, int B, int H, int W, int C, int dtype,
                       hipStream_t s, int* plan_out) {
    constexpr int CS = (2 * 4 * TzShape<K, 16, 16>::NM + 2 * 4 * TzShape<K, 16, 16>::RING) <= 160 ? 16 : 8;
    constexpr int NGA0 = (4 + 2 * ((K - 1) / 2) + 3) / 4, NGA = NGA0 < 2 ? 2 : NGA0, NB = K == 17 ? 3 : 2;
    if (dtype == kF32 || C % 16 != 0 || (H & 1) || (W & 1) || B < 1) return -1;
    const int P = K / 2, h = H / 2, wd = W / 2;
    if (!plan_out)
        for (const void* p : {gyf, w0, addp, (const void*)dx, x0, (const void*)ws0, x1, gy1, (const void*)ws1})
            if (!p || (reinterpret_cast<uintptr_t>(p) & 15)) return -1;
    const long long pad16 = (long long)cdiv(W, 64) * 64 * B, pad8 = (long long)cdiv(W, 32) * 32 * cdiv(B, 2) * 2;
    if (pad16 > pad8) return -1;   // the input gradient's wide tile only
    Bwd3Args a;
    long long nd;
    if (!tz_make_geom<K, 16, CS>(a.gd, nd, true, B, H, W, C, K - 1 - P, K - 1 - P, true, nullptr)) return -1;
    WgTzPlan p0 = wgrad_tz_plan(B, H, W, C, K, P, P), p1 = wgrad_tz_plan(B, h, wd, C, K, P, P);
    if (!p0.ok || !p1.ok) return -1;
    Bwd3Plan plan = bwd3_plan<K, CS>(B, a.gd, p0, p1);
    if (const char* e = tune_env("PDW_BWD3_BANDS")) {   // e.g. "2,2,1,DHF": bands of D, F, H and the grid order
        if (sscanf(e, "%d,%d,%d,%3s", &plan.nb[0], &plan.nb[1], &plan.nb[2], plan.order) != 4) return -1;
    }
    if (tune_env("PDW_BWD3_PRINT"))
        fprintf(stderr, "bwd3 plan B=%d H=%d W=%d C=%d K=%d: bands D %d F %d H %d order %s\n", B, H, W, C, K, plan.nb[0],
                plan.nb[1], plan.nb[2], plan.order);
    if (plan.nb[0] < 1 || plan.nb[1] < 1 || plan.nb[2] < 1) return -1;
    auto rows_of = [](int oh, int nb) { return (cdiv(oh, nb) + 3) / 4 * 4; };
    a.gd.BR = rows_of(a.gd.OH, plan.nb[0]), a.gd.nbands = cdiv(a.gd.OH, a.gd.BR);
    nd = (long long)cdiv(B, TzShape<K, 16, CS>::NI) * a.gd.nbands * a.gd.ncolt * a.gd.nslices;
    p0.g.BR = rows_of(p0.g.OH, plan.nb[1]), p0.g.nbands = cdiv(p0.g.OH, p0.g.BR);
    p0.nblocks = (long long)B * p0.g.nslices * p0.g.ncolt * p0.g.nbands;
    p1.g.BR = rows_of(p1.g.OH, plan.nb[2]), p1.g.nbands = cdiv(p1.g.OH, p1.g.BR);
    p1.nblocks = (long long)B * p1.g.nslices * p1.g.ncolt * p1.g.nbands;
    if (!p0.ok || !p1.ok || p0.ncb != 8 || wgrad_tz_nga(K) != NGA) return -1;
    if (nd + p0.nblocks + p1.nblocks > 0x7fffffffLL) return -1;
    if (plan_out) {
        plan_out[0] = a.gd.nbands, plan_out[1] = p0.g.nbands, plan_out[2] = p1.g.nbands;
        return 0;
    }
    a.gy = gyf, a.w = w0, a.add = addp, a.dx = dx;
    a.x0 = x0, a.gy0 = gyf, a.x1 = x1, a.gy1 = gy1, a.part0 = (float*)ws0, a.part1 = (float*)ws1;
    a.g0 = p0.g, a.g1 = p1.g, a.nd = (int)nd, a.n1 = (int)p1.nblocks, a.n0 = (int)p0.nblocks;
    {
        // order of the three problems in the grid: a permutation of D (input gradient), H (half scale), F (full scale)
        const char* ord = plan.order;
        int at = 0;
        for (int i = 0; i < 3; ++i) {
            if (ord[i] == 'D') a.sd = at, at += a.nd;
            if (ord[i] == 'H') a.s1 = at, at += a.n1;
            if (ord[i] == 'F') a.s0 = at, at += a.n0;
        }
    }
    size_t lds = TzShape<K, 16, CS>::lds_bytes;
    if (WgTzShape<NGA, 8, NB>::lds_bytes > lds) lds = WgTzShape<NGA, 8, NB>::lds_bytes;
    if (WgTzShape<NGA, 5, NB>::lds_bytes > lds) lds = WgTzShape<NGA, 5, NB>::lds_bytes;
    const unsigned grid = (unsigned)(nd + p0.nblocks + p1.nblocks);
    static std::once_flag once[4];
#define PDW_BWD3_GO(T, NCB1, SLOT)                                                                                        \
    {                                                                                                                     \
        auto kern = dwconv_bwd3_k<T, K, CS, NGA, NCB1, NB>;                                                               \
        std::call_once(once[SLOT], [&] {                                                                                  \
            (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);         \
        });                                                                                                               \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, s, a);                                                       \
    }
    if (dtype == kF16) {
        if (p1.ncb == 8) PDW_BWD3_GO(f16_t, 8, 0) else PDW_BWD3_GO(f16_t, 5, 1)
    } else {
        if (p1.ncb == 8) PDW_BWD3_GO(bf16_t, 8, 2) else PDW_BWD3_GO(bf16_t, 5, 3)
    }
#undef PDW_BWD3_GO
    if (int e = check_launch("dwconv_bwd3")) return e;
    const int n0 = B * p0.g.nbands * p0.g.ncolt, n1 = B * p1.g.nbands * p1.g.ncolt;
    if (dtype == kF16) {
        if (int e = wgrad_reduce_launch<f16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
        return wgrad_reduce_launch<f16_t>((const float*)ws1, dw1, n1, K * K * C, s);
    }
    if (int e = wgrad_reduce_launch<bf16_t>((const float*)ws0, dw0, n0, K * K * C, s)) return e;
    return wgrad_reduce_launch<bf16_t>((const float*)ws1, dw1, n1, K * K * C, s);
}

}  // namespace pdw
