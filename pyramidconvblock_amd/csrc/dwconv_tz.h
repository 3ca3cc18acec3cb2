// Depthwise convolution as a block-Toeplitz product on the dense matrix cores: forward and input gradient for
// 16-bit types, stride 1, dilation 1, odd square filters up to 17 (the input gradient is the same kernel run on gy
// with the 180-degree rotated filter and padding k-1-p).
//
// For one channel, a patch of 4 x 4 outputs is a product of the filter, spread out as a 16 x (K+3)(K+3) matrix
//     A[(di,dj)][(r,s)] = w[r - di][s - dj]          (zero where the tap falls outside the filter)
// with the patch's (K+3) x (K+3) input window as a vector.  v_mfma_f32_16x16x32_{bf16,f16} computes
// D[m][n] += sum_k A[m][k] B[k][n] with m = one of the patch's 16 outputs, n = one of 16 patches and k running over
// 32 window positions per instruction: 4 "k groups" of 8 consecutive columns of one window row, which is what one
// lane holds (lane = n + 16 * group for B, m + 16 * group for A).  A window row is ICB = ceil((K+3)/8) groups wide,
// so a patch takes NM = ceil((K+3) * ICB / 4) instructions (8 at K = 13: 169 of every 256 multiply-adds fall on a
// real tap, on the pipe that runs at four times the rate of the 4x4x4 block form).  A depends on the channel only:
// each wavefront owns CPW channels and keeps their A operands in registers for the whole kernel.
//
// The 16 patches of an instruction lie side by side (4 columns apart) in NI = 16 / NPC images, and a wavefront
// walks down the rows four at a time.  Moving down by 4 rows shifts every B operand by ICB instructions, so the
// operands live in a register ring: a step reads only the 4 new window rows from LDS (ICB operands of 16 bytes per
// lane) for NM instructions.  That is what makes the kernel a stream: per step and channel 2 LDS reads, 8 MFMAs.
//
// A workgroup (8 wavefronts, CS = 8 CPW channels) owns a band of BR output rows x 4 NPC columns of NI images.  Its
// input window is staged once in LDS, channel-major: xl[image][channel][row][column] as 16-bit values, so that 8
// consecutive columns of a channel are 16 contiguous bytes.  Threads load 2 x 2 pixels x 8 channels (four 16-byte
// loads), interleave column pairs with byte permutes and write dwords; the passes of this copy are requested two
// ahead and committed only as far as the next step needs, so steps start while the lower rows are still on their
// way and the loads, the MFMAs and the stores of a band overlap.  Results are rounded once, transposed through a
// small double-buffered LDS tile (pixel-major, one dword of padding per 4 pixels keeps the 4-byte scatter free of
// bank conflicts) and leave as 16-byte stores, one step behind the MFMAs.
//
// MODE is a set of bits.
// 1 (input gradient of a tensor that was also average-pooled 2x2): y += add[i/2, j/2] / 4 in the store.
// 2 (forward): the 2x2 average pool of x is written to `pool` by the staging threads, which hold exactly the
// four pixels of a pool window in registers (needs even padding, so that windows do not straddle threads).
// 4 (forward, inference): the gate of conv_block.py:18-19 in the store.  A workgroup's 16 channels are 8 of the first
// half and the matching 8 of the second half of C, and the two store threads of a pixel multiply four channel pairs
// each (the rounded convolution outputs, as the stand-alone gate kernel does): y[..., c] = conv[c] * conv[C/2 + c] * gs,
// C/2 channels wide, written with a pixel stride of YC channels from channel `ych` on (into the concatenation).
// With 8 channels per workgroup (filters from 15 on) the slice is 4 channels of each half: every 16-byte load of the
// staging and of the filter becomes two 8-byte loads C bytes apart, and a pixel's one store thread gates the two
// halves of its piece.
//
// Zero entries of A multiply real pixels of the window (and the window is wider than K+3 where (K+3) % 8 != 0), so a
// non-finite input value reaches outputs up to 3 + 8 ICB - (K+3) pixels beyond its K x K footprint as NaN.
#pragma once
#include <mutex>

#include "common.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

typedef float tz_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ tz_f32x4 mfma16(uint4 a, uint4 b, tz_f32x4 c, bf16_t) {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
}
__device__ __forceinline__ tz_f32x4 mfma16(uint4 a, uint4 b, tz_f32x4 c, f16_t) {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
}

template <int K, int NPC, int CS>
struct TzShape {
    static constexpr int NT = 512, NWV = 8;
    static constexpr int IC = K + 3;                  // window columns (and rows) of a 4 x 4 patch
    static constexpr int ICB = (IC + 7) / 8;          // k groups per window row
    static constexpr int NKG = IC * ICB;              // k groups of a patch
    static constexpr int NM = (NKG + 3) / 4;          // MFMAs per patch (group of 16) and channel
    static constexpr int PER = (NM + ICB - 1) / ICB;  // row groups (of 4 rows) an operand ring spans
    static constexpr int RING = PER * ICB;            // operands in the ring
    static constexpr int NI = 16 / NPC;               // images side by side in one instruction
    static constexpr int TW = 4 * NPC;                // output columns of a workgroup
    static constexpr int NH = CS / 8;                 // 8-channel pieces per pixel
    static constexpr int CPW = CS / 8;                // channels per wavefront
    static constexpr int WCOLS = 4 * (NPC - 1) + 8 * ICB;  // window columns the operands touch
    static constexpr int RP = (2 * WCOLS + 7) / 8 * 8;     // bytes per window row of a channel
    static constexpr int OPX = 2 * CS;                     // bytes per pixel of the result tile
    static constexpr int OROWP = TW * OPX + NPC * 4;       // bytes per row of the result tile (4 per 4 pixels padding)
    static constexpr int OLB = NI * 4 * OROWP;             // one result tile: 4 rows of every image
    static constexpr int WTH = 4 * PER + 3, WTW = 8 * ICB + 4;  // zero-bordered filter table [channel][WTH][WTW]
    static constexpr int WTB = CS * WTH * WTW * 2;
    static constexpr int R2B = (4 * OLB > 2 * WTB ? 4 * OLB : 2 * WTB + 15) / 16 * 16;  // 4 result tiles / two filter tables (shared)
    static_assert(K % 2 == 1 && K >= 3 && K <= 17, "odd filters up to 17");
    static_assert(NPC == 16 || NPC == 8, "patches per image row");
    static_assert(CS == 8 || CS == 16, "channels per workgroup");
    static constexpr int win_rows(int BR) { return BR + 4 * (PER - 1); }  // window rows of a band; BR % 4 == 0
    // The window lives in LDS as a ring of NR row groups (of 4 rows), window row r at ring row r % NRR: a step reads
    // the two row groups it adds to the operand registers while the next step's two are being written, and the
    // first step needs PER + 1 row groups in place before it starts.
    static constexpr int NR = PER + 1 > 4 ? PER + 1 : 4;
    static constexpr int NRR = 4 * NR;
    static constexpr int CHP = NRR * RP % 16 == 8 ? NRR * RP : NRR * RP + 8;  // bytes per channel plane, = 8 mod 16
    static constexpr size_t lds_bytes = (size_t)NI * CS * CHP + R2B;
    static_assert(lds_bytes <= 160 * 1024, "LDS");
};

struct TzGeom {
    int B, H, W, C;    // input extents
    int OH, OW;        // output extents
    int PH, PW;        // padding
    int BR;            // output rows of a band (multiple of 4)
    int nbands, ncolt, nslices;
    int flip;          // 1: 180-degree rotated filter (input gradient)
    int AH, AW;        // extents of the half-resolution addend / pooled output
    int YC, ych;       // output pixel stride in channels, first output channel
    float gs;          // gate factor (MODE & 4)
};

// 8 values of T: a + b / 4, rounded once more (what an accumulating pool gradient does to a stored tensor).
template <typename T>
__device__ __forceinline__ uint4 tz_add_quarter(uint4 a, uint4 b) {
    union U {
        uint4 u;
        T t[8];
    } ua, ub, uo;
    ua.u = a, ub.u = b;
#pragma unroll
    for (int i = 0; i < 8; ++i) uo.t[i] = from_f32<T>(to_f32(ua.t[i]) + 0.25f * to_f32(ub.t[i]));
    return uo.u;
}

// 4 values of T: a * b * s, rounded once (the arithmetic of the stand-alone gate kernel).
template <typename T>
__device__ __forceinline__ uint2 tz_gate(uint2 a, uint2 b, float s) {
    union U {
        uint2 u;
        T t[4];
    } ua, ub, uo;
    ua.u = a, ub.u = b;
#pragma unroll
    for (int i = 0; i < 4; ++i) uo.t[i] = from_f32<T>(gate_f32(to_f32(ua.t[i]), to_f32(ub.t[i]), s));
    return uo.u;
}

// One workgroup's band: `blk` of the problem's `nblk` workgroups.
template <typename T, int K, int NPC, int CS, int MODE>
__device__ __forceinline__ void dwconv_tz_body(const T* __restrict__ x, const T* __restrict__ w,
                                               const T* __restrict__ add, T* __restrict__ pool, T* __restrict__ y,
                                               const TzGeom& g, int blk, int nblk) {
    using Sh = TzShape<K, NPC, CS>;
    constexpr int NT = Sh::NT, ICB = Sh::ICB, NKG = Sh::NKG, NM = Sh::NM, PER = Sh::PER, RING = Sh::RING;
    constexpr int NI = Sh::NI, TW = Sh::TW, NH = Sh::NH, CPW = Sh::CPW, RP = Sh::RP, OPX = Sh::OPX, OROWP = Sh::OROWP;
    constexpr int OLB = Sh::OLB, WTH = Sh::WTH, WTW = Sh::WTW, NR = Sh::NR, NRR = Sh::NRR, CHP = Sh::CHP;
    constexpr bool ADD = (MODE & 1) != 0, POOL = (MODE & 2) != 0, GATE = (MODE & 4) != 0;
    static_assert(!GATE || !ADD, "the gate is a forward mode");
    // the gate pairs channel c with channel C/2 + c: a 16-channel slice is 8 channels of each half of C (its two
    // 8-channel pieces), an 8-channel slice 4 of each (the halves of its one piece, moved as two 8-byte accesses)
    constexpr bool G8 = GATE && CS == 8;
    static_assert(!(G8 && POOL), "the pool's stores assume 8 contiguous channels");
    extern __shared__ uint32_t smem[];
    char* const xl = reinterpret_cast<char*>(smem);        // [NI][CS] planes of CHP bytes: [ring row][column] of T
    char* const r2 = xl + NI * CS * CHP;                 // filter table, then the two result tiles

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int bid = xcd_remap(blk, nblk);
    const int sl = bid % g.nslices;
    bid /= g.nslices;
    const int ct = bid % g.ncolt;
    bid /= g.ncolt;
    const int band = bid % g.nbands, ig = bid / g.nbands;
    const int c0 = sl * CS, ocol0 = ct * TW, orow0 = band * g.BR, b0 = ig * NI;
    const int rows_valid = min(g.BR, g.OH - orow0), cols_valid = min(TW, g.OW - ocol0);
    const int nsteps = (rows_valid + 3) >> 2;
    const int NROWS = 4 * (nsteps + PER - 1);              // window rows the steps read
    const int WCP = (4 * ((cols_valid + 3) / 4 - 1) + 8 * ICB) / 2;  // column pairs the used patches read
    const long long img_in = (long long)g.H * g.W * g.C, img_out = (long long)g.OH * g.OW * g.YC;
    // first channel of the slice's 8-channel piece h
    auto chof = [&](int h) { return G8 ? 4 * sl : GATE ? 8 * sl + h * (g.C >> 1) : c0 + 8 * h; };

    // ---- filter slice, 8 channels of a tap per load: requested before the window, so that waiting for it leaves
    // the window's loads in flight
    constexpr int NWL = (K * K * NH + NT - 1) / NT;
    uint4 wval[NWL];
#pragma unroll
    for (int i = 0; i < NWL; ++i) {
        const int idx = min(tid + i * NT, K * K * NH - 1);
        if constexpr (G8) {
            const T* wp = w + idx * g.C + 4 * sl;
            const uint2 lo = *reinterpret_cast<const uint2*>(wp), hi = *reinterpret_cast<const uint2*>(wp + (g.C >> 1));
            wval[i] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        } else {
            wval[i] = *reinterpret_cast<const uint4*>(w + (idx / NH) * g.C + min(chof(idx % NH), g.C - 8));
        }
    }

    // ---- staging.  The window arrives in passes, requested two ahead into two register buffers.  Passes 0 and 1
    // are halves of the PER + 1 row groups (of 4 rows) the first step reads, every later pass the two row groups the
    // next step adds, so step f is preceded by the commit of pass f + 1.  A thread's item is (row pair of the pass,
    // image, column pair cp, 8-channel piece h), h fastest, the same in every pass.
    constexpr int RP01 = PER + 1;                                // row pairs of pass 0 and of pass 1
    constexpr int RPMAX = RP01 > 4 ? RP01 : 4;
    constexpr int NLD = (RPMAX * NI * (Sh::WCOLS / 2) * NH + NT - 1) / NT;  // items per thread and pass
    constexpr int UNRF = PER % 4 == 0 ? PER / 2 : (PER % 2 == 0 ? PER : 2 * PER);  // steps per trip: even, PER | 2 UNRF
    auto first_rowpair = [&](int pass) { return pass < 2 ? pass * RP01 : 2 * RP01 + 4 * (pass - 2); };
    auto rowpair_count = [&](int pass) { return pass < 2 ? RP01 : 4; };
    // Loads go through a buffer descriptor over the workgroup's images: an offset past its end (an image beyond the
    // batch, or one of the markers for a row / column / channel outside the tensor) reads as zero and moves no
    // data, which is the zero padding.  NI * H * W * C < 2^29 elements (guarded on the host), so valid byte
    // offsets stay below 2^30 and any sum with a marker stays past the end.
    constexpr uint32_t kNoCol = 0x40000000u, kNoRow = 0x80000000u;
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(x + (long long)b0 * img_in), (short)0, (int)(min(NI, g.B - b0) * img_in * 2), 0x00020000);
    auto xload_from = [&](const __amdgpu_buffer_rsrc_t& r, uint32_t off) {
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
        return make_uint4(v.x, v.y, v.z, v.w);
    };
    auto xload = [&](uint32_t off) {
        if constexpr (G8) {   // 4 channels of each half of C (C bytes apart); a marker offset stays past the end
            typedef unsigned v2u __attribute__((ext_vector_type(2)));
            const v2u lo = __builtin_amdgcn_raw_buffer_load_b64(xrsrc, (int)off, 0, 0);
            const v2u hi = __builtin_amdgcn_raw_buffer_load_b64(xrsrc, (int)(off + (uint32_t)g.C), 0, 0);
            return make_uint4(lo.x, lo.y, hi.x, hi.y);
        } else {
            return xload_from(xrsrc, off);
        }
    };
    uint32_t icol[NLD][2];  // byte offsets of the item's two columns (image and channel piece included), or kNoCol
    int irpw[NLD];          // row pair within a pass
    int idst[NLD];          // LDS byte offset of the item's plane and column pair
#pragma unroll
    for (int l = 0; l < NLD; ++l) {
        const int idx = tid + l * NT;
        const int h = idx % NH, cp = (idx / NH) % WCP, img = (idx / NH / WCP) % NI, rpw = idx / NH / WCP / NI;
        irpw[l] = rpw;
        const int ic = ocol0 - g.PW + 2 * cp;
        const bool any = (G8 || chof(h) < g.C) && rpw < RPMAX;
        const uint32_t ioff = (uint32_t)img * (uint32_t)img_in + (uint32_t)chof(h);
        icol[l][0] = any && ic >= 0 && ic < g.W ? (ioff + (uint32_t)(ic * g.C)) * 2u : kNoCol;
        icol[l][1] = any && ic + 1 >= 0 && ic + 1 < g.W ? (ioff + (uint32_t)((ic + 1) * g.C)) * 2u : kNoCol;
        idst[l] = (img * CS + 8 * h) * CHP + 4 * cp;
    }
    // the 2x2 average pool of x (MODE 2) leaves through a buffer descriptor as well: a store past its end is dropped
    __amdgpu_buffer_rsrc_t prsrc = xrsrc;
    if constexpr (POOL)
        prsrc = __builtin_amdgcn_make_buffer_rsrc(pool + (long long)b0 * g.AH * g.AW * g.C, (short)0,
                                                  (int)((long long)min(NI, g.B - b0) * g.AH * g.AW * g.C * 2), 0x00020000);
    uint4 buf[2][NLD][4];
    auto issue = [&](uint4 (&bf)[NLD][4], int pass) {  // rows beyond the pass or the window read nothing
        const int wr0 = 2 * first_rowpair(pass), nrp = rowpair_count(pass);
#pragma unroll
        for (int l = 0; l < NLD; ++l) {
            const int wr = wr0 + 2 * irpw[l];  // window row
            const int ir = orow0 - g.PH + wr;
            const bool ok = irpw[l] < nrp && wr < NROWS;
            const uint32_t r0 = ok && ir >= 0 && ir < g.H ? (uint32_t)(ir * g.W * g.C) * 2u : kNoRow;
            const uint32_t r1 = ok && ir + 1 >= 0 && ir + 1 < g.H ? (uint32_t)((ir + 1) * g.W * g.C) * 2u : kNoRow;
            bf[l][0] = xload(r0 + icol[l][0]);
            bf[l][1] = xload(r0 + icol[l][1]);
            bf[l][2] = xload(r1 + icol[l][0]);
            bf[l][3] = xload(r1 + icol[l][1]);
        }
    };
    auto commit = [&](const uint4 (&bf)[NLD][4], int pass) {
        const int wr0 = 2 * first_rowpair(pass), nrp = rowpair_count(pass);
#pragma unroll
        for (int l = 0; l < NLD; ++l) {
            const int wr = wr0 + 2 * irpw[l];
            if (irpw[l] < nrp && wr < NROWS) {
                const uint32_t a0[4] = {bf[l][0].x, bf[l][0].y, bf[l][0].z, bf[l][0].w};
                const uint32_t a1[4] = {bf[l][1].x, bf[l][1].y, bf[l][1].z, bf[l][1].w};
                const uint32_t a2[4] = {bf[l][2].x, bf[l][2].y, bf[l][2].z, bf[l][2].w};
                const uint32_t a3[4] = {bf[l][3].x, bf[l][3].y, bf[l][3].z, bf[l][3].w};
                int rr = wr0 % NRR + 2 * irpw[l];   // ring row of the item's first row (a pair never wraps: both even)
                rr -= rr >= NRR ? NRR : 0;
                char* dst = xl + idst[l] + rr * RP;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // column pair of channels 2j and 2j+1, the item's two rows
                    *reinterpret_cast<uint32_t*>(dst + (2 * j) * CHP) = __builtin_amdgcn_perm(a1[j], a0[j], 0x05040100u);
                    *reinterpret_cast<uint32_t*>(dst + (2 * j + 1) * CHP) = __builtin_amdgcn_perm(a1[j], a0[j], 0x07060302u);
                    *reinterpret_cast<uint32_t*>(dst + (2 * j) * CHP + RP) = __builtin_amdgcn_perm(a3[j], a2[j], 0x05040100u);
                    *reinterpret_cast<uint32_t*>(dst + (2 * j + 1) * CHP + RP) = __builtin_amdgcn_perm(a3[j], a2[j], 0x07060302u);
                }
            }
            if constexpr (POOL) {
                // the thread holds one window of the 2x2 pool (H, W, PH, PW even): the band that owns these rows writes it
                const int idx = tid + l * NT;
                const int h = idx % NH, cp = (idx / NH) % WCP, img = (idx / NH / WCP) % NI;
                const int ir = orow0 - g.PH + wr, ic = ocol0 - g.PW + 2 * cp;
                const bool mine = irpw[l] < nrp && chof(h) < g.C && ir >= orow0 && ir < orow0 + rows_valid && ic >= ocol0 &&
                                  ic < ocol0 + cols_valid;
                union U {
                    uint4 u;
                    T t[8];
                } p0, p1, p2, p3, o;
                p0.u = bf[l][0], p1.u = bf[l][1], p2.u = bf[l][2], p3.u = bf[l][3];
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    o.t[e] = from_f32<T>((((to_f32(p0.t[e]) + to_f32(p1.t[e])) + to_f32(p2.t[e])) + to_f32(p3.t[e])) * 0.25f);
                const uint32_t off = mine ? (uint32_t)(((img * g.AH + (ir >> 1)) * g.AW + (ic >> 1)) * g.C + chof(h)) * 2u : kNoRow;
                typedef unsigned v4u __attribute__((ext_vector_type(4)));
                __builtin_amdgcn_raw_buffer_store_b128(v4u{o.u.x, o.u.y, o.u.z, o.u.w}, prsrc, (int)off, 0, 0);
            }
        }
    };
    issue(buf[0], 0);
    issue(buf[1], 1);

    // LDS accesses of this wavefront complete, then the workgroup barrier; global loads and stores stay in flight
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // ---- filter table wt[copy][channel][3 + u][3 + v] (rotated for the input gradient), zero elsewhere; copy 1 is
    // the same table one element to the left, so that a run of 8 values that starts at an odd index is dword
    // aligned in it
    constexpr int WTC = CS * WTH * WTW;  // elements per copy
    unsigned short* const wt = reinterpret_cast<unsigned short*>(r2);
    {
        uint4* wz = reinterpret_cast<uint4*>(r2);
        for (int i = tid; i < (2 * Sh::WTB + 15) / 16; i += NT) wz[i] = make_uint4(0u, 0u, 0u, 0u);
        lds_barrier();
#pragma unroll
        for (int i = 0; i < NWL; ++i) {
            const int idx = tid + i * NT;
            const int h = idx % NH, uv = idx / NH;
            const int u = uv / K, v = uv - u * K;
            if (idx < K * K * NH && (G8 || chof(h) < g.C)) {
                const uint32_t d[4] = {wval[i].x, wval[i].y, wval[i].z, wval[i].w};
                const int uu = g.flip ? K - 1 - u : u, vv = g.flip ? K - 1 - v : v;
                unsigned short* wp = wt + ((8 * h) * WTH + 3 + uu) * WTW + 3 + vv;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const unsigned short val = (unsigned short)((d[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                    wp[e * WTH * WTW] = val;
                    wp[WTC + e * WTH * WTW - 1] = val;
                }
            }
        }
        // (the table is read after the barrier that also publishes the window's first passes)
    }
    const int ln = lane & 15, kg = lane >> 4;
    // ---- per-lane addresses
    // B operands: lane = (patch n = image * NPC + pc, k group kg); operand a = ICB * rowgroup + i covers window rows
    // 4 rowgroup + (4i + kg) / ICB, column block (4i + kg) % ICB
    const int pimg = ln / NPC, pc = ln % NPC;
    const char* xb[CPW][ICB];
#pragma unroll
    for (int q = 0; q < CPW; ++q)
#pragma unroll
        for (int i = 0; i < ICB; ++i)
            xb[q][i] = xl + (pimg * CS + wv * CPW + q) * CHP + ((4 * i + kg) / ICB) * RP + ((4 * i + kg) % ICB) * 16 + pc * 8;
    // results: register r of a lane is output (row kg, column 4 pc + r) of patch n
    char* const olw = r2 + (pimg * 4 + kg) * OROWP + (4 * pc) * OPX + pc * 4 + 2 * (wv * CPW);
    // store phase: one 16-byte piece (image, row, column, h) of each 4-row result tile per thread, through buffer
    // descriptors (an offset past the end: nothing stored / zero loaded), so that no vector memory instruction of the
    // kernel sits behind a branch and the in-flight counts the staging waits rely on stay exact
    const int sh = tid % NH, scol = (tid / NH) % TW, srow = (tid / NH / TW) % 4, simg = tid / NH / TW / 4;
    const bool s_ok = simg < NI && scol < cols_valid && (GATE || c0 + 8 * sh < g.C);
    const char* const olr = r2 + (min(simg, NI - 1) * 4 + srow) * OROWP + scol * OPX + (scol >> 2) * 4 + 16 * sh;
    const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(
        y + (long long)b0 * img_out, (short)0, (int)(min(NI, g.B - b0) * img_out * 2), 0x00020000);
    const uint32_t ycol = (uint32_t)simg * (uint32_t)img_out +
                          (uint32_t)((ocol0 + scol) * g.YC + g.ych + (G8 ? 4 * sl : GATE ? 8 * sl + 4 * sh : c0 + 8 * sh));
    __amdgpu_buffer_rsrc_t arsrc = xrsrc;
    if constexpr (ADD)
        arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(add + (long long)b0 * g.AH * g.AW * g.C), (short)0,
                                                  (int)((long long)min(NI, g.B - b0) * g.AH * g.AW * g.C * 2), 0x00020000);
    uint4 addv[2] = {make_uint4(0u, 0u, 0u, 0u), make_uint4(0u, 0u, 0u, 0u)};
    auto add_fetch = [&](int f) {   // the addends of step f's two tiles
        if constexpr (ADD) {
#pragma unroll
            for (int gi = 0; gi < 2; ++gi) {
                const int row = 4 * (2 * f + gi) + srow;
                const bool ok = s_ok && row < rows_valid;
                const uint32_t off = ok ? (uint32_t)(((simg * g.AH + ((orow0 + row) >> 1)) * g.AW + ((ocol0 + scol) >> 1)) * g.C + c0 + 8 * sh) * 2u : kNoRow;
                addv[gi] = xload_from(arsrc, off);
            }
        }
    };
    auto store = [&](int f) {   // f = -1: nothing
#pragma unroll
        for (int gi = 0; gi < 2; ++gi) {
            const char* src = olr + (2 * (f & 1) + gi) * OLB;
            uint4 v;
            v.x = *reinterpret_cast<const uint32_t*>(src), v.y = *reinterpret_cast<const uint32_t*>(src + 4);
            v.z = *reinterpret_cast<const uint32_t*>(src + 8), v.w = *reinterpret_cast<const uint32_t*>(src + 12);
            if constexpr (ADD) v = tz_add_quarter<T>(v, addv[gi]);
            const int row = 4 * (2 * f + gi) + srow;
            const bool ok = s_ok && f >= 0 && row < rows_valid;
            const uint32_t off = ok ? (ycol + (uint32_t)((orow0 + row) * g.OW * g.YC)) * 2u : kNoRow;
            if constexpr (GATE) {
                // the thread gates 4 channel pairs of the pixel: values 4 sh .. 4 sh + 3 of both 8-channel pieces, or
                // the two halves of an 8-channel slice's one piece
                const char* sg = G8 ? src : src - 8 * sh;   // (src points 16 sh into the pixel)
                constexpr int PB = G8 ? 8 : 16;             // bytes between a pair's two values
                const uint2 a = make_uint2(*reinterpret_cast<const uint32_t*>(sg), *reinterpret_cast<const uint32_t*>(sg + 4));
                const uint2 b = make_uint2(*reinterpret_cast<const uint32_t*>(sg + PB), *reinterpret_cast<const uint32_t*>(sg + PB + 4));
                const uint2 o = tz_gate<T>(a, b, g.gs);
                typedef unsigned v2u __attribute__((ext_vector_type(2)));
                __builtin_amdgcn_raw_buffer_store_b64(v2u{o.x, o.y}, yrsrc, (int)off, 0, 0);
            } else {
                typedef unsigned v4u __attribute__((ext_vector_type(4)));
                __builtin_amdgcn_raw_buffer_store_b128(v4u{v.x, v.y, v.z, v.w}, yrsrc, (int)off, 0, 0);
            }
        }
    };

    uint4 ring[CPW][RING];
    auto read16 = [&](const char* p) {
        const uint2 lo = *reinterpret_cast<const uint2*>(p), hi = *reinterpret_cast<const uint2*>(p + 8);
        return make_uint4(lo.x, lo.y, hi.x, hi.y);
    };
    auto load_group = [&](int slotgroup, int byteoff) {  // window rows byteoff / RP .. + 3 -> ICB operands per channel
#pragma unroll
        for (int q = 0; q < CPW; ++q)
#pragma unroll
            for (int i = 0; i < ICB; ++i) ring[q][slotgroup * ICB + i] = read16(xb[q][i] + byteoff);
    };
    // the passes the first step reads, then the ring's first PER - 1 row groups
    commit(buf[0], 0);
    issue(buf[0], 2);
    commit(buf[1], 1);
    issue(buf[1], 3);
    lds_barrier();
    // ---- this wavefront's A operands: lane = (m = 4 di + dj, k group kg); operand t covers k groups 4t .. 4t+3
    uint4 A[CPW][NM];
    {
        const int di = ln >> 2, dj = ln & 3;
#pragma unroll
        for (int q = 0; q < CPW; ++q) {
#pragma unroll
            for (int t = 0; t < NM; ++t) {
                const int kap = 4 * t + kg;
                const int r = kap / ICB, cb = kap - r * ICB;
                const int v0 = 8 * cb - dj + 3;  // first of the lane's 8 table columns
                const uint32_t* wp = reinterpret_cast<const uint32_t*>(
                    wt + (v0 & 1) * WTC + ((wv * CPW + q) * WTH + r - di + 3) * WTW + (v0 & ~1));
                const bool real = kap < NKG;
                A[q][t] = make_uint4(real ? wp[0] : 0u, real ? wp[1] : 0u, real ? wp[2] : 0u, real ? wp[3] : 0u);
            }
        }
    }

#pragma unroll
    for (int j = 0; j < PER - 1; ++j) load_group(j, 4 * j * RP);
    // A step is two row groups (8 output rows).  Trips of UNRF steps (the ring's period in steps), left after the
    // band's last step by a uniform exit between steps.  Besides its products a step
    // stores the previous step's tiles and commits the pass the NEXT step needs; the wavefronts 0-3 do the products
    // first and the others last, so that of the two wavefronts a SIMD holds one feeds the matrix pipe while the
    // other moves data (both make the same memory requests in the same order: the in-flight counts stay exact).
    const int nfat = (nsteps + 1) >> 1;
    int fdone = 0;
    bool left = false;
    auto stage_step = [&](int jf, int f) {
        store(f - 1);
        add_fetch(f);
        commit(buf[jf % 2], f + 2);   // pass f + 2 sits in buffer f % 2 = jf % 2 (UNRF is even)
        issue(buf[jf % 2], f + 4);
    };
    auto compute_step = [&](int jf, int f) {
        // the two row groups this step adds to the ring; the second goes to the slot of the step's own first
        // group, which the first tile still reads, so it waits in registers until the products are issued
        load_group((2 * jf + PER - 1) % PER, ((2 * f + PER - 1) % NR) * (4 * RP));
        const int late_off = ((2 * f + PER) % NR) * (4 * RP);
        uint4 late[CPW][ICB];
#pragma unroll
        for (int q = 0; q < CPW; ++q)
#pragma unroll
            for (int i = 0; i < ICB; ++i) late[q][i] = read16(xb[q][i] + late_off);
        tz_f32x4 acc[2][CPW];
#pragma unroll
        for (int gi = 0; gi < 2; ++gi)
#pragma unroll
            for (int q = 0; q < CPW; ++q) acc[gi][q] = tz_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < NM; ++t)
#pragma unroll
            for (int q = 0; q < CPW; ++q) {
                acc[0][q] = mfma16(A[q][t], ring[q][(ICB * 2 * jf + t) % RING], acc[0][q], T());
                const uint4 b1 = t < ICB * (PER - 1) ? ring[q][(ICB * (2 * jf + 1) + t) % RING] : late[q][t - ICB * (PER - 1) < ICB ? t - ICB * (PER - 1) : 0];
                acc[1][q] = mfma16(A[q][t], b1, acc[1][q], T());
            }
#pragma unroll
        for (int q = 0; q < CPW; ++q)
#pragma unroll
            for (int i = 0; i < ICB; ++i) ring[q][((2 * jf) % PER) * ICB + i] = late[q][i];
#pragma unroll
        for (int gi = 0; gi < 2; ++gi) {
            char* dst = olw + (2 * (f & 1) + gi) * OLB;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if constexpr (CPW == 2) {
                    union {
                        T t[2];
                        uint32_t u;
                    } o;
                    o.t[0] = from_f32<T>(acc[gi][0][r]), o.t[1] = from_f32<T>(acc[gi][1][r]);
                    *reinterpret_cast<uint32_t*>(dst + r * OPX) = o.u;
                } else {
                    *reinterpret_cast<T*>(dst + r * OPX) = from_f32<T>(acc[gi][0][r]);
                }
            }
        }
    };
    for (int f0 = 0; f0 < nfat; f0 += UNRF) {
#pragma unroll
        for (int jf = 0; jf < UNRF; ++jf) {
            const int f = f0 + jf;
            lds_barrier();  // the previous step's tiles are complete, its window reads done
            if (wv < 4) {
                if (f < nfat) compute_step(jf, f);
                stage_step(jf, f);
            } else {
                stage_step(jf, f);
                if (f < nfat) compute_step(jf, f);
            }
            if (f + 1 >= nfat) {   // the band's last step (uniform): its tiles are stored after the loop
                left = true;
                fdone = f + 1;
                break;
            }
        }
        if (left) break;
        fdone = f0 + UNRF;
    }
    lds_barrier();
    store(fdone - 1);
}

template <typename T, int K, int NPC, int CS, int MODE>
__global__ __launch_bounds__(512, 1) void dwconv_tz_k(const T* __restrict__ x, const T* __restrict__ w,
                                                      const T* __restrict__ add, T* __restrict__ pool,
                                                      T* __restrict__ y, const TzGeom g) {
    dwconv_tz_body<T, K, NPC, CS, MODE>(x, w, add, pool, y, g, blockIdx.x, gridDim.x);
}

// ------------------------------------------------------------------------------------------------
// Host side

// Band height: the choice with the shortest estimated run, rounds of workgroups over 256 compute units times the
// rows a workgroup moves (window rows plus a fixed cost of about 8 rows' worth).
template <int K, int NPC, int CS>
static int tz_pick_band(int B, int OH, int OW, int C) {
    using Sh = TzShape<K, NPC, CS>;
    const long long per_band = (long long)cdiv(B, Sh::NI) * cdiv(C, CS) * cdiv(OW, Sh::TW);
    if (const char* e = tune_env("PDW_TZ_BR")) return atoi(e);
    int best = 0;
    double best_cost = 0;
    for (int br = 4; br <= ((OH + 3) / 4) * 4; br += 4) {
        const long long wgs = per_band * cdiv(OH, br);
        const double cost = (double)cdiv(wgs, 256) * (Sh::win_rows(br) + 8);
        if (best == 0 || cost <= best_cost) best = br, best_cost = cost;
    }
    return best;
}

// The geometry of a launch (false: not covered) and its number of workgroups.
template <int K, int NPC, int CS>
static bool tz_make_geom(TzGeom& g, long long& nblocks, bool add, int B, int H, int W, int C, int PH, int PW, bool flip,
                         const TzGate* gate) {
    using Sh = TzShape<K, NPC, CS>;
    g.B = B, g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW, g.flip = flip ? 1 : 0;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    g.AH = add ? g.OH / 2 : H / 2, g.AW = add ? g.OW / 2 : W / 2;
    g.YC = gate ? gate->ldy : C, g.ych = gate ? gate->ych : 0, g.gs = gate ? gate->gs : 1.f;
    if (gate && (add || flip || C % 16 != 0 || gate->ldy < gate->ych + C / 2 || (gate->ldy | gate->ych) % 8 != 0)) return false;
    if ((long long)H * W * C * Sh::NI > 0x1fffffffLL || (long long)g.OH * g.OW * g.YC * Sh::NI > 0x1fffffffLL) return false;
    g.BR = tz_pick_band<K, NPC, CS>(B, g.OH, g.OW, C);
    if (g.BR < 4) return false;
    g.nbands = cdiv(g.OH, g.BR), g.ncolt = cdiv(g.OW, Sh::TW), g.nslices = cdiv(C, CS);
    nblocks = (long long)cdiv(B, Sh::NI) * g.nbands * g.ncolt * g.nslices;
    return nblocks <= 0x7fffffffLL;
}

template <typename T, int K, int NPC, int CS>
static int launch_tz(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C,
                     int PH, int PW, bool flip, const TzGate* gate, hipStream_t s) {
    using Sh = TzShape<K, NPC, CS>;
    TzGeom g;
    long long nblocks;
    if (!tz_make_geom<K, NPC, CS>(g, nblocks, add != nullptr, B, H, W, C, PH, PW, flip, gate)) return -1;
    const size_t lds = Sh::lds_bytes;
    const int mode = (add ? 1 : 0) | (pool ? 2 : 0) | (gate ? 4 : 0);
    auto kern = dwconv_tz_k<T, K, NPC, CS, 0>;
    if (mode == 1) kern = dwconv_tz_k<T, K, NPC, CS, 1>;
    if (mode == 2) kern = dwconv_tz_k<T, K, NPC, CS, 2>;
    if (mode == 4) kern = dwconv_tz_k<T, K, NPC, CS, 4>;
    if constexpr (CS == 16) {
        if (mode == 6) kern = dwconv_tz_k<T, K, NPC, CS, 6>;
    }
    if (mode == 3 || mode == 5 || mode == 7 || (mode == 6 && CS != 16)) return -1;
    static std::once_flag attr_once[8];
    std::call_once(attr_once[mode], [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(Sh::NT), lds, s, (const T*)x, (const T*)w, (const T*)add,
                       (T*)pool, (T*)y, g);
    return check_launch("dwconv_tz");
}

// -1: not covered (the caller falls back to the other kernels).
template <typename T, int K>
static int launch_tz_best(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C,
                          int PH, int PW, bool flip, const TzGate* gate, hipStream_t s) {
    const int OH = H + 2 * PH - K + 1, OW = W + 2 * PW - K + 1;
    if (OH < 1 || OW < 1 || C % 8 != 0 || B < 1) return -1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(w) & 15) != 0)
        return -1;
    if (add && ((OH | OW) & 1 || (reinterpret_cast<uintptr_t>(add) & 15) != 0)) return -1;
    if (pool && (add || flip || OH != H || OW != W || ((H | W | PH | PW) & 1) || (reinterpret_cast<uintptr_t>(pool) & 15) != 0))
        return -1;
    // patches per image row: the width whose padding of (columns x images) is smaller, wider on ties
    const long long pad16 = (long long)cdiv(OW, 64) * 64 * B, pad8 = (long long)cdiv(OW, 32) * 32 * cdiv(B, 2) * 2;
    const bool wide_tile = pad16 <= pad8;
    // 16 channels per workgroup (two per wavefront) while the operand registers allow it, else 8
    constexpr int CS = (2 * 4 * TzShape<K, 16, 16>::NM + 2 * 4 * TzShape<K, 16, 16>::RING) <= 160 ? 16 : 8;
    if (wide_tile) return launch_tz<T, K, 16, CS>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, gate, s);
    return launch_tz<T, K, 8, CS>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, gate, s);
}

template <int K>
static int launch_tz_dtype(const void* x, const void* w, const void* add, void* pool, void* y, int B, int H, int W, int C,
                           int PH, int PW, bool flip, int dtype, const TzGate* gate, hipStream_t s) {
    switch (dtype) {
        case kF16: return launch_tz_best<f16_t, K>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, gate, s);
        case kBF16: return launch_tz_best<bf16_t, K>(x, w, add, pool, y, B, H, W, C, PH, PW, flip, gate, s);
        default: return -1;
    }
}

}  // namespace pdw
