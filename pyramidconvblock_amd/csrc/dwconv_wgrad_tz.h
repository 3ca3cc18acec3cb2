// Depthwise-convolution weight gradient on the dense matrix cores (16-bit types, stride 1, dilation 1, square
// filters up to 17):     dw[u,v,c] = sum_{b,i,j} gy[b,i,j,c] * xw[b, i+u, j+v, c],   xw[r][s] = x[r-PH][s-PW].
//
// With u = 2a + du, v = 8b + dv and the position p = (i + du, j + dv) the sum for one channel is
//     dw[2a+du][8b+dv] = sum_p  xw[p + (2a, 8b)] * gy[p - (du, dv)],
// which is one v_mfma_f32_16x16x32_{bf16,f16} product D[m][n] += sum_k A[m][k] B[k][n] with m = (a, b) = 2a + b,
// n = (du, dv) = 8 du + dv and k running over a block of 4 rows x 8 columns of positions (a lane holds 8 consecutive
// columns of one row: lane = m + 16 * row for A, n + 16 * row for B):
//     A[(a,b)][(kr,e)]   = xw[R + kr + 2a][Cc + e + 8b]
//     B[(kr,e)][(du,dv)] = gy[R + kr - du][Cc + e - dv]        (zero outside the band's own rows and columns)
// One accumulator of 4 registers holds all 16 x 16 taps of a channel (169 of 256 used at K = 13), and a band of
// BR x 56 positions takes ceil((BR+1)/4) x 8 instructions per channel.  K = 17 has 9 x 3 tap blocks (a, b): they are
// numbered a * NB + b over two instructions that share the gy operand.  Both operands are data, so nothing is kept
// per channel but the accumulator: a wavefront owns 2 of the workgroup's 16 channels for the whole band and
// writes their taps to the fp32 partial of the band at the end; the partials are summed in a fixed order by
// wgrad_reduce_parts (no atomics: bit-reproducible).
//
// The kernel is bound by LDS reads (two 1 KB operands per instruction, no reuse).  Aligned 16-byte reads run at
// twice the rate of narrower ones on this part (measured: 256 against 128 bytes per clock), which is why the
// column offsets of the xw operand are multiples of 8 elements: it is one ds_read_b128.  The fine offsets (du, dv)
// shift gy by single elements, so gy is staged twice, the second copy one element to the left, and a lane reads
// whichever copy makes its run of 8 values dword aligned (two ds_read2_b32).  A gy staging item is 4 consecutive
// columns of one row (x an 8-channel piece), so that both copies are written as 8-byte stores: the second copy's last
// pair takes the first column of the item to the right through a lane shift (a window row sits in one wavefront).
//
// Staging is the streamed scheme of dwconv_tz.h: both tensors arrive in passes of 8 rows, requested two ahead
// into two register buffers each and committed to LDS one step before they are read; the LDS windows are rings of
// row groups (of 4 rows), channel-major ([channel][row][column] of 16-bit values), so their size does not depend
// on the band height.
#pragma once
#include <mutex>

#include "common.h"
#include "dwconv_tz.h"
#include "kernels.h"
#include "tile_common.h"

namespace pdw {

// NGA: row groups (of 4 rows) the xw operand of a step spans (rows kr + 2a, a <= (K-1)/2); NCB: column blocks of 8
// positions per band row (8: bands of 56 columns, 5: of 32); NB: tap column blocks (2: K <= 16, 3: K = 17).
template <int NGA, int NCB, int NB>
struct WgTzShape {
    static constexpr int NT = 512, CS = 16, CPW = 2, NH = 2;
    static constexpr int TWG = 8 * NCB - 8;                 // gy columns of a workgroup: TWG + 7 <= 8 NCB positions
    static constexpr int NMF = NB == 3 ? 2 : 1;             // instructions per position block and channel
    static constexpr int WCX = 8 * NCB + 8 * (NB - 1);      // xw window columns the operands touch
    static constexpr int WCG = 8 * NCB + 8;                 // gy window columns: 8 of padding on the left
    // LDS pitches, chosen by measurement of the operands' access patterns on this part.  xw (ds_read_b128, lane (a, b, kr)
    // at row kr + 2a, byte 16 b): rows 32 bytes (mod 128) apart run at the full rate (3.9 cycles per instruction against
    // 6.1 with rows 16 bytes (mod 128) apart).  gy (ds_read2_b32): a pass reads 3 consecutive rows x 5 dwords from
    // each copy (dwords 1..5 of the first, 0..4 of the second); with rows 10 banks apart and the second copy 6 banks
    // further the six runs start at banks 1, 6, 11, 16, 23, 28: no two share a bank.
    static constexpr int RPX = (2 * WCX - 32 + 127) / 128 * 128 + 32;
    static constexpr int RPG = (2 * WCG - 40 + 127) / 128 * 128 + 40;
    // ring slots (row groups).  xw: the NGA groups a step reads and the two the pass committed meanwhile covers; even,
    // so that a pass never wraps.  gy: a step reads groups t-1 and t while a whole pass (groups t+1, t+2) is committed;
    // where LDS is short (NGA = 5) a step commits only group t+1, one half of a pass, and 3 slots do.
    static constexpr int NSX = NGA + 2 + (NGA % 2), NSG = NGA == 5 ? 3 : 4;
    static constexpr int GBX = 4 * RPX, GBG = 4 * RPG;      // bytes per row group of a channel
    static constexpr int CHPX = NSX * GBX + 16, CHPG = NSG * GBG + 8;   // channel planes
    static constexpr int XHALF = 64;                        // channels 8..15 sit 16 banks further: the two 8-channel
                                                            // pieces of a staging pass write different banks
    static constexpr int XB = CS * CHPX + XHALF, GCB = (CS * CHPG + 127) / 128 * 128 + 24;  // xw window; one gy copy
    static constexpr size_t lds_bytes = (size_t)XB + 2 * GCB;
    static_assert(NGA >= 2 && NGA <= 5 && (NCB == 8 || NCB == 5) && (NB == 2 || NB == 3), "row groups spanned, column blocks");
    static_assert(RPX % 128 == 32 && RPX >= 2 * WCX && RPG % 128 == 40 && RPG >= 2 * WCG && CHPX % 16 == 0 && GCB % 128 == 24,
                  "operand alignment / bank spread");
    // gy staging item: 4 consecutive columns of one window row x an 8-channel piece; a window row is GLPR consecutive
    // lanes of one wavefront (the item to the right is NH lanes up: its first column completes the second copy's
    // last pair), GRPW whole rows per wavefront
    static constexpr int GLPR = (WCG / 4) * NH, GRPW = 64 / GLPR;
    static_assert(4 * (WCX / 2) * NH <= NT && GRPW >= 1 && (8 + GRPW - 1) / GRPW <= NT / 64 && WCG % 4 == 0,
                  "a pass is at most one item per thread");
    static_assert(lds_bytes <= 160 * 1024, "LDS");
};

struct WgTzGeom {
    int B, H, W, C;     // x extents
    int OH, OW;         // gy extents
    int PH, PW, K;
    int BR;             // gy rows of a band (multiple of 4)
    int nbands, ncolt, nslices;
};

// One workgroup's band: `blk` of the problem's `nblk` workgroups.
template <typename T, int NGA, int NCB, int NB>
__device__ __forceinline__ void dwconv_wgrad_tz_body(const T* __restrict__ x, const T* __restrict__ gy,
                                                     float* __restrict__ part, const WgTzGeom& g, int blk, int nblk) {
    using Sh = WgTzShape<NGA, NCB, NB>;
    constexpr int NT = Sh::NT, CS = Sh::CS, CPW = Sh::CPW, NH = Sh::NH, TWG = Sh::TWG, RPX = Sh::RPX, RPG = Sh::RPG, NMF = Sh::NMF;
    constexpr int NSX = Sh::NSX, NSG = Sh::NSG, GBX = Sh::GBX, GBG = Sh::GBG, CHPX = Sh::CHPX, CHPG = Sh::CHPG;
    constexpr int WCPX = Sh::WCX / 2;
    extern __shared__ uint32_t smem[];
    char* const xl = reinterpret_cast<char*>(smem);   // [CS] planes of CHPX bytes: [slot][row][column]
    char* const gl = xl + Sh::XB;                     // two copies of [CS] planes of CHPG bytes

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int bid = xcd_remap(blk, nblk);
    const int sl = bid % g.nslices;
    bid /= g.nslices;
    const int ct = bid % g.ncolt;
    bid /= g.ncolt;
    const int band = bid % g.nbands, b = bid / g.nbands;
    const int chunk = (b * g.nbands + band) * g.ncolt + ct;
    const int c0 = sl * CS, j0 = ct * TWG, i0 = band * g.BR;
    const int rows_valid = min(g.BR, g.OH - i0), cols_valid = min(TWG, g.OW - j0);
    const int nsteps = (rows_valid + 1 + 3) >> 2;      // position rows i0 .. i0 + rows_valid, four per step
    const int NGX = nsteps + NGA - 1;                  // xw row groups read
    const int amax = (g.K - 1) >> 1;                   // tap row blocks in use: a <= amax
    const long long img_x = (long long)g.H * g.W * g.C, img_g = (long long)g.OH * g.OW * g.C;

    // ---- staging (see dwconv_tz.h): buffer loads, offsets past the end read as zero without moving data
    constexpr uint32_t kNoCol = 0x40000000u, kNoRow = 0x80000000u;
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x + b * img_x), (short)0, (int)(img_x * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t grsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(gy + b * img_g), (short)0, (int)(img_g * 2), 0x00020000);
    auto bload = [&](const __amdgpu_buffer_rsrc_t& r, uint32_t off) {
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
        return make_uint4(v.x, v.y, v.z, v.w);
    };
    // item of a pass: (row pair 0..3, column pair, 8-channel piece h), h fastest
    const int ih = tid % NH;
    const bool chok = c0 + 8 * ih < g.C;
    uint32_t xcol[2], gcol[4];
    int xrp, grow, xdst, gdst;
    bool gact;
    {
        const int cp = (tid / NH) % WCPX, rp = tid / NH / WCPX;
        xrp = rp < 4 ? rp : -1;
        const int ic = j0 - g.PW + 2 * cp;
        const bool any = chok && rp < 4;
        xcol[0] = any && ic >= 0 && ic < g.W ? (uint32_t)(ic * g.C + c0 + 8 * ih) * 2u : kNoCol;
        xcol[1] = any && ic + 1 >= 0 && ic + 1 < g.W ? (uint32_t)((ic + 1) * g.C + c0 + 8 * ih) * 2u : kNoCol;
        xdst = (8 * ih) * CHPX + ih * Sh::XHALF + (2 * min(rp, 3)) * RPX + 4 * cp;
    }
    {
        grow = wv * Sh::GRPW + lane / Sh::GLPR;          // row of the pass
        const int q = (lane % Sh::GLPR) / NH;            // columns 4 q .. 4 q + 3 of the window
        gact = chok && lane < Sh::GRPW * Sh::GLPR && grow < 8;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int jc = 4 * q + p - 8;   // column relative to j0: the band's own columns are 0 .. cols_valid-1
            gcol[p] = gact && jc >= 0 && jc < cols_valid ? (uint32_t)((j0 + jc) * g.C + c0 + 8 * ih) * 2u : kNoCol;
        }
        grow = min(grow, 7);
        gdst = (8 * ih) * CHPG + (grow & 3) * RPG + 8 * q;   // within the row group (grow >> 2) of the pass
    }
    uint4 bx[2][4], bg[2][4];
    auto issue_x = [&](uint4 (&bf)[4], int pass) {   // xw rows 8 pass .. 8 pass + 7 (window row 0 = x row i0 - PH)
        const int wr = 8 * pass + 2 * max(xrp, 0);
        const int ir = i0 - g.PH + wr;
        const bool ok = wr < 4 * NGX;
        const uint32_t r0 = ok && ir >= 0 && ir < g.H ? (uint32_t)(ir * g.W * g.C) * 2u : kNoRow;
        const uint32_t r1 = ok && ir + 1 >= 0 && ir + 1 < g.H ? (uint32_t)((ir + 1) * g.W * g.C) * 2u : kNoRow;
        bf[0] = bload(xrsrc, r0 + xcol[0]);
        bf[1] = bload(xrsrc, r0 + xcol[1]);
        bf[2] = bload(xrsrc, r1 + xcol[0]);
        bf[3] = bload(xrsrc, r1 + xcol[1]);
    };
    auto issue_g = [&](uint4 (&bf)[4], int pass) {   // gy rows i0 + 8 pass .. + 7, the band's own rows only
        const int wr = 8 * pass + grow;
        const uint32_t r0 = wr < rows_valid ? (uint32_t)((i0 + wr) * g.OW * g.C) * 2u : kNoRow;
#pragma unroll
        for (int p = 0; p < 4; ++p) bf[p] = bload(grsrc, r0 + gcol[p]);   // lanes without an item read zeros
    };
    auto commit_x = [&](const uint4 (&bf)[4], int pass) {
        if (xrp < 0) return;
        const uint32_t a0[4] = {bf[0].x, bf[0].y, bf[0].z, bf[0].w}, a1[4] = {bf[1].x, bf[1].y, bf[1].z, bf[1].w};
        const uint32_t a2[4] = {bf[2].x, bf[2].y, bf[2].z, bf[2].w}, a3[4] = {bf[3].x, bf[3].y, bf[3].z, bf[3].w};
        char* dst = xl + xdst + ((2 * pass) % NSX) * GBX;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint32_t*>(dst + (2 * j) * CHPX) = __builtin_amdgcn_perm(a1[j], a0[j], 0x05040100u);
            *reinterpret_cast<uint32_t*>(dst + (2 * j + 1) * CHPX) = __builtin_amdgcn_perm(a1[j], a0[j], 0x07060302u);
            *reinterpret_cast<uint32_t*>(dst + (2 * j) * CHPX + RPX) = __builtin_amdgcn_perm(a3[j], a2[j], 0x05040100u);
            *reinterpret_cast<uint32_t*>(dst + (2 * j + 1) * CHPX + RPX) = __builtin_amdgcn_perm(a3[j], a2[j], 0x07060302u);
        }
    };
    // the value of the lane NH up (the next item of the row; zeros behind the row's last item: no item or no column)
    auto from_right = [&](uint32_t v) {
        static_assert(NH == 2, "two single-lane wavefront shifts");
        v = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x130, 0xf, 0xf, true);   // wave_shl:1: lane i takes lane i + 1
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x130, 0xf, 0xf, true);
    };
    auto commit_g = [&](const uint4 (&bf)[4], int pass, int half) {   // half 0 / 1: one row group of the pass; -1: both
        const uint32_t a0[4] = {bf[0].x, bf[0].y, bf[0].z, bf[0].w}, a1[4] = {bf[1].x, bf[1].y, bf[1].z, bf[1].w};
        const uint32_t a2[4] = {bf[2].x, bf[2].y, bf[2].z, bf[2].w}, a3[4] = {bf[3].x, bf[3].y, bf[3].z, bf[3].w};
        uint32_t a4[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) a4[j] = from_right(a0[j]);   // every lane takes part in the shift
        if (!gact || (half >= 0 && (grow >> 2) != half)) return;
        char* dst = gl + gdst + ((2 * pass + (grow >> 2)) % NSG) * GBG;
#pragma unroll
        for (int j = 0; j < 4; ++j) {   // channels 2 j (low halves) and 2 j + 1 (high halves) of the piece
            char* d0 = dst + (2 * j) * CHPG;
            char* d1 = dst + (2 * j + 1) * CHPG;
            *reinterpret_cast<uint2*>(d0) = make_uint2(__builtin_amdgcn_perm(a1[j], a0[j], 0x05040100u),
                                                       __builtin_amdgcn_perm(a3[j], a2[j], 0x05040100u));
            *reinterpret_cast<uint2*>(d1) = make_uint2(__builtin_amdgcn_perm(a1[j], a0[j], 0x07060302u),
                                                       __builtin_amdgcn_perm(a3[j], a2[j], 0x07060302u));
            // second copy, one element to the left: column c goes to index c - 1 (columns 4 q + 1 .. 4 q + 4 here)
            *reinterpret_cast<uint2*>(d0 + Sh::GCB) = make_uint2(__builtin_amdgcn_perm(a2[j], a1[j], 0x05040100u),
                                                                 __builtin_amdgcn_perm(a4[j], a3[j], 0x05040100u));
            *reinterpret_cast<uint2*>(d1 + Sh::GCB) = make_uint2(__builtin_amdgcn_perm(a2[j], a1[j], 0x07060302u),
                                                                 __builtin_amdgcn_perm(a4[j], a3[j], 0x07060302u));
        }
    };
    issue_x(bx[0], 0);
    issue_g(bg[0], 0);
    issue_x(bx[1], 1);
    issue_g(bg[1], 1);

    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // gy row group -1 (the rows above the band, read by the first step) is ring slot NSG-1: zero in both copies
    for (int i = tid; i < 2 * CS * (GBG / 4); i += NT) {
        const int cpy = i / (CS * (GBG / 4)), rem = i % (CS * (GBG / 4));
        const int ch = rem / (GBG / 4), d = rem % (GBG / 4);
        *reinterpret_cast<uint32_t*>(gl + cpy * Sh::GCB + ch * CHPG + (NSG - 1) * GBG + 4 * d) = 0u;
    }

    // ---- per-lane operand addresses
    const int ln = lane & 15, kr = lane >> 4;
    // A: tap block (a, b) = (i / NB, i % NB) of instruction f, i = ln + 16 f; blocks beyond the filter read valid data
    int la[NMF];
    const char* xlane[NMF];
#pragma unroll
    for (int f = 0; f < NMF; ++f) {
        la[f] = min((ln + 16 * f) / NB, amax);
        xlane[f] = xl + (wv * CPW) * CHPX + ((wv * CPW) >> 3) * Sh::XHALF + (8 * ((ln + 16 * f) % NB)) * 2;
    }
    const int ldu = ln >> 3, ldv = ln & 7;            // B: fine offset (du, dv)
    const char* const glane = gl + (ldv & 1) * Sh::GCB + (wv * CPW) * CHPG + ((8 - ldv) & ~1) * 2;

    tz_f32x4 acc[CPW][NMF];
#pragma unroll
    for (int q = 0; q < CPW; ++q)
#pragma unroll
        for (int f = 0; f < NMF; ++f) acc[q][f] = tz_f32x4{0.f, 0.f, 0.f, 0.f};

    // the passes the first step reads: xw groups 0 .. NGA-1, gy group 0
    constexpr int P0X = (NGA + 1) / 2;
#pragma unroll
    for (int p = 0; p < P0X; ++p) {
        commit_x(bx[p % 2], p);
        issue_x(bx[p % 2], p + 2);
        if (p == 0) {
            if constexpr (NSG == 4) {
                commit_g(bg[0], 0, -1);
                issue_g(bg[0], 2);
            } else {
                commit_g(bg[0], 0, 0);
            }
        }
    }
    auto read_a = [&](const char* p) { return *reinterpret_cast<const uint4*>(p); };   // 16-byte aligned
    // Steps in trips of 4, left after the band's last step (a uniform exit between steps: the loads of passes past the
    // band's end, requested on the way, move nothing).  A step first commits what the NEXT step adds to the windows (an
    // 8-row pass of xw or of gy on alternating steps; with 3 gy slots one row group of gy every step, the pass's
    // registers being requested again once both of its groups are in LDS), behind the barrier that ends the previous step's reads of the ring slots it
    // overwrites; no condition depends on data, so the loads keep their exact in-flight counts.
    constexpr int UNR = 4;
    for (int s0 = 0; s0 < nsteps; s0 += UNR) {
#pragma unroll
        for (int j = 0; j < UNR; ++j) {
            const int t = s0 + j;
            lds_barrier();
            if ((j + NGA) % 2 == 0) {   // xw row group t + NGA opens a pass (j is unrolled)
                const int bi = ((j + NGA) / 2) % 2, pass = (t + NGA) / 2;
                commit_x(bx[bi], pass);
                issue_x(bx[bi], pass + 2);
            }
            if constexpr (NSG == 4) {
                if (j % 2 == 1) {       // gy row group t + 1 opens a pass
                    const int bi = ((j + 1) / 2) % 2, pass = (t + 1) / 2;
                    commit_g(bg[bi], pass, -1);
                    issue_g(bg[bi], pass + 2);
                }
            } else {                    // gy row group t + 1: half (t + 1) % 2 of pass (t + 1) / 2
                const int bi = ((j + 1) / 2) % 2, pass = (t + 1) / 2;
                commit_g(bg[bi], pass, (j + 1) % 2);
                if ((j + 1) % 2 == 1) issue_g(bg[bi], pass + 2);
            }
            // A: xw rows 4 t + kr + 2 a;  B: gy rows 4 t + kr - du (relative to the band): group t, or t - 1 for row -1
            const char* xa[NMF];
#pragma unroll
            for (int f = 0; f < NMF; ++f) {
                const int ra = 4 * (t % NSX) + kr + 2 * la[f];      // row within the ring, before wrapping
                xa[f] = xlane[f] + (ra >= 4 * NSX ? ra - 4 * NSX : ra) * RPX;
            }
            const int st = t % NSG, sp = (t + NSG - 1) % NSG;
            const char* gb = glane + (kr < ldu ? sp * GBG + 3 * RPG : st * GBG + (kr - ldu) * RPG);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int q = 0; q < CPW; ++q) {
                    const uint32_t* gp = reinterpret_cast<const uint32_t*>(gb + q * CHPG + 16 * cb);
                    const uint4 bop = make_uint4(gp[0], gp[1], gp[2], gp[3]);
#pragma unroll
                    for (int f = 0; f < NMF; ++f) acc[q][f] = mfma16(read_a(xa[f] + q * CHPX + 16 * cb), bop, acc[q][f], T());
                }
            if (t + 1 >= nsteps) {   // the band's last step (uniform): the rest of the trip would multiply zeros
                s0 = nsteps;
                break;
            }
        }
    }
    // ---- this band's partial.  Lane (n = (du, dv), row block kr) holds in register r of instruction f the tap block
    // i = 4 kr + r + 16 f = (a, b) = (i / NB, i % NB) of its two channels; the taps go through LDS ([tap][channel], 20 floats apart) so that a tap's 16
    // channels leave as four 16-byte stores.
    lds_barrier();
    float* const ep = reinterpret_cast<float*>(smem);
    constexpr int EPP = 20;
#pragma unroll
    for (int q = 0; q < CPW; ++q)
#pragma unroll
        for (int f = 0; f < NMF; ++f)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * kr + r + 16 * f;
                const int u = 2 * (i / NB) + ldu, v = 8 * (i % NB) + ldv;
                if (u < g.K && v < g.K) ep[(u * g.K + v) * EPP + wv * CPW + q] = acc[q][f][r];
            }
    __syncthreads();
    float* pc = part + (long long)chunk * g.K * g.K * g.C;
    for (int i = tid; i < g.K * g.K * (CS / 4); i += NT) {
        const int tap = i / (CS / 4), c4 = 4 * (i % (CS / 4));
        if (c0 + c4 < g.C) *reinterpret_cast<float4*>(pc + (long long)tap * g.C + c0 + c4) = *reinterpret_cast<const float4*>(ep + tap * EPP + c4);
    }
}

template <typename T, int NGA, int NCB, int NB>
__global__ __launch_bounds__(512, 1) void dwconv_wgrad_tz_k(const T* __restrict__ x, const T* __restrict__ gy,
                                                            float* __restrict__ part, const WgTzGeom g) {
    dwconv_wgrad_tz_body<T, NGA, NCB, NB>(x, gy, part, g, blockIdx.x, gridDim.x);
}

// Two problems of the same filter size in one launch (the two scales of a block): the second problem's nblk1
// workgroups come first in the grid.  With one workgroup per compute unit and two problems that each fill the chip
// once, a compute unit runs one band of each back to back, without the drain and the launch between two kernels.
template <typename T, int NGA, int NCB0, int NCB1, int NB>
__global__ __launch_bounds__(512, 1) void dwconv_wgrad_tz_pair_k(const T* __restrict__ x0, const T* __restrict__ gy0,
                                                                 float* __restrict__ part0, const WgTzGeom g0,
                                                                 const T* __restrict__ x1, const T* __restrict__ gy1,
                                                                 float* __restrict__ part1, const WgTzGeom g1, int nblk1) {
    if ((int)blockIdx.x < nblk1)
        dwconv_wgrad_tz_body<T, NGA, NCB1, NB>(x1, gy1, part1, g1, blockIdx.x, nblk1);
    else
        dwconv_wgrad_tz_body<T, NGA, NCB0, NB>(x0, gy0, part0, g0, blockIdx.x - nblk1, gridDim.x - nblk1);
}

// ------------------------------------------------------------------------------------------------
// Host side

inline int wgrad_tz_nga(int K) { return (4 + 2 * ((K - 1) / 2) + 3) / 4 < 2 ? 2 : (4 + 2 * ((K - 1) / 2) + 3) / 4; }

struct WgTzPlan {
    bool ok = false;
    int ncb = 0;
    WgTzGeom g;
    long long nblocks = 0;
};

// Covered: 16-bit types (the caller checks), C % 8 == 0, K <= 17, 16-byte aligned tensors.
inline WgTzPlan wgrad_tz_plan(int B, int H, int W, int C, int K, int PH, int PW) {
    WgTzPlan p;
    WgTzGeom& g = p.g;
    g.B = B, g.H = H, g.W = W, g.C = C, g.PH = PH, g.PW = PW, g.K = K;
    g.OH = H + 2 * PH - K + 1, g.OW = W + 2 * PW - K + 1;
    if (K < 1 || K > 17 || C % 8 != 0 || B < 1 || g.OH < 1 || g.OW < 1) return p;
    if ((long long)H * W * C > 0x1fffffffLL || (long long)g.OH * g.OW * C > 0x1fffffffLL) return p;
    p.ncb = g.OW <= 32 ? 5 : 8;
    const int twg = 8 * p.ncb - 8, ta = wgrad_tz_nga(K);
    g.ncolt = cdiv(g.OW, twg), g.nslices = cdiv(C, 16);
    // band height: shortest estimated run, rounds of workgroups over 256 compute units times the rows one moves
    const long long per_band = (long long)B * g.nslices * g.ncolt;
    int best = 0;
    double best_cost = 0;
    for (int br = 4; br <= ((g.OH + 3) / 4) * 4; br += 4) {
        const long long wgs = per_band * cdiv(g.OH, br);
        const double cost = (double)cdiv(wgs, 256) * (br + 1 + 4 * (ta - 1) + 8);
        if (best == 0 || cost <= best_cost) best = br, best_cost = cost;
    }
    g.BR = best;
    g.nbands = cdiv(g.OH, g.BR);
    p.nblocks = per_band * g.nbands;
    if (p.nblocks > 0x7fffffffLL || (long long)B * g.nbands * g.ncolt > 0x7fffffffLL) return p;
    p.ok = true;
    return p;
}

inline size_t wgrad_tz_workspace(int B, int H, int W, int C, int K, int PH, int PW) {
    const WgTzPlan p = wgrad_tz_plan(B, H, W, C, K, PH, PW);
    return p.ok ? (size_t)B * p.g.nbands * p.g.ncolt * K * K * C * sizeof(float) : 0;
}

template <typename T, int NGA, int NCB, int NB>
static int launch_wgrad_tz(const WgTzPlan& p, const void* x, const void* gy, void* ws, hipStream_t s) {
    using Sh = WgTzShape<NGA, NCB, NB>;
    auto kern = dwconv_wgrad_tz_k<T, NGA, NCB, NB>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nblocks), dim3(Sh::NT), Sh::lds_bytes, s, (const T*)x, (const T*)gy, (float*)ws, p.g);
    return check_launch("dwconv_wgrad_tz");
}

template <typename T, int NGA, int NCB0, int NCB1, int NB>
static int launch_wgrad_tz_pair(const WgTzPlan& p0, const void* x0, const void* gy0, void* ws0, const WgTzPlan& p1,
                                const void* x1, const void* gy1, void* ws1, hipStream_t s) {
    using Sh0 = WgTzShape<NGA, NCB0, NB>;
    using Sh1 = WgTzShape<NGA, NCB1, NB>;
    auto kern = dwconv_wgrad_tz_pair_k<T, NGA, NCB0, NCB1, NB>;
    static std::once_flag attr_once;
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    if (p0.nblocks + p1.nblocks > 0x7fffffffLL) return -1;
    const size_t lds = Sh0::lds_bytes > Sh1::lds_bytes ? Sh0::lds_bytes : Sh1::lds_bytes;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p0.nblocks + p1.nblocks)), dim3(Sh0::NT), lds, s, (const T*)x0, (const T*)gy0,
                       (float*)ws0, p0.g, (const T*)x1, (const T*)gy1, (float*)ws1, p1.g, (int)p1.nblocks);
    return check_launch("dwconv_wgrad_tz_pair");
}

}  // namespace pdw
