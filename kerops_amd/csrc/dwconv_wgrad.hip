// Depthwise 3x3x3 weight gradient for [N][H][W][D][C] fp16 (gfx950), fp32 end to end.
//
//   gw[kh,kw,kd,c] = sum_{n,h,w,d} g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]
//
// Same march as the forward kernel: a workgroup owns a (TW x TD) patch of the (W, D)
// plane for a slab of CG*8 channels and walks a chunk of rows along H.  Each x plane
// hp (with its halo) is staged through LDS once; a thread owns 2 channels of a few pairs
// of D-adjacent patch positions (d, d+1), reads the in-plane neighbours of x from LDS and
// multiplies them with the three rows of g that see this plane (g[hp+1] for kh=0, g[hp]
// for kh=1, g[hp-1] for kh=2).  Both factors of a pair are packed per channel into one
// dword with a byte permute, so one 2-way fp16 dot instruction adds the contributions of
// both positions to a tap's fp32 accumulator: 54 dots + 20 permutes per pair and plane
// instead of 108 multiply-adds.  g needs no halo: it is read straight from global memory,
// one row ahead, and kept (packed) in registers for three steps.  The 27*2 fp32
// accumulators of a thread live for the whole march; at the end lanes that own the same channels are
// combined with wavefront shuffles, wavefronts through LDS, and the workgroup writes
// one partial [27][slab] to the workspace.  A second kernel adds the partials in a
// fixed order, so the result is deterministic (no atomics).
#include <cstdlib>

#include "common.hpp"
#include "dwconv_wgrad.hpp"

namespace kerops {

template <int CG_, int TW_, int TD_, int NT_>
struct WgCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_;
    static constexpr int CL = 2;               // channels per lane: one dword of fp16
    static constexpr int SC = CG * 8;          // channels in the slab
    static constexpr int NCL = SC / CL;        // lane groups per voxel
    static constexpr int PW = TW + 2, PD = TD + 2;
    static constexpr int NPAIR = TW * (TD / 2) * NCL;  // (d, d+1) position pairs per plane
    static constexpr int PP = NPAIR / NT;              // pairs per thread per plane
    static constexpr bool STRAIGHT = (PP <= 2);        // branch-free march (see the kernel); needs spare registers
    static constexpr int NCH = PW * PD * CG;   // staged c8 chunks per plane
    static constexpr int NLD = (NCH + NT - 1) / NT;
    static constexpr int NWAVE = NT / kWave;
    static constexpr int STAGE_BYTES = 2 * (NCH + 1) * 16;  // +1: dump slot, see the forward kernel
    static constexpr int RED_BYTES = NWAVE * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    static_assert(NPAIR % NT == 0, "patch must divide evenly over the threads");
    static_assert(NT % NCL == 0 && kWave % NCL == 0, "lane groups tile a wavefront");
    static_assert((TD & (TD - 1)) == 0 && TD >= 2, "TD power of two");
};


__device__ __forceinline__ half2_t pack_lo(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(b, a, 0x05040100u));  // (a.lo, b.lo)
}
__device__ __forceinline__ half2_t pack_hi(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(b, a, 0x07060302u));  // (a.hi, b.hi)
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, (Cfg::NT >= 512 || Cfg::STRAIGHT) ? 4 : 3) void dwconv_wgrad_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, PP = Cfg::PP, NLD = Cfg::NLD, NCH = Cfg::NCH;
    constexpr int PD = Cfg::PD, CL = Cfg::CL, NCL = Cfg::NCL, SC = Cfg::SC;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half8_t* stage = reinterpret_cast<half8_t*>(smem);

    uint32_t L = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (L >= a.nblocks) return;
    const uint32_t ws_slot = L;
    const int slab = L % a.n_slab;
    L /= a.n_slab;
    const int dt = L % a.n_dt;
    L /= a.n_dt;
    const int wt_i = L % a.n_wt;
    L /= a.n_wt;
    const int hc = L % a.n_hc;
    const int n = L / a.n_hc;

    const int t = threadIdx.x;
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    const int w0 = wt_i * Cfg::TW, d0 = dt * TD;
    const int hs = hc * a.h_chunk;
    const int he = min(hs + a.h_chunk, H);
    const int cslab = slab * SC;
    const int64_t plane_stride = (int64_t)W * D * C;
    const half_t* xn = a.x + (int64_t)n * H * plane_stride;
    const half_t* gn_ptr = a.g + (int64_t)n * H * plane_stride;

    // staging assignment (c8 chunks of the halo patch); every lane loads and writes
    // unconditionally, lanes with nothing to stage use the plane's first chunk and a dump slot
    uint32_t goff[NLD];
    int ldst[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const int q = t + j * NT;
        const int wq = q / (PD * CG);
        const int r = q - wq * (PD * CG);
        const int dq = r / CG;
        const int cq = r - dq * CG;
        const int w = w0 - 1 + wq, d = d0 - 1 + dq;
        const bool ok = (q < NCH) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
        goff[j] = ok ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
        ldst[j] = ok ? q : NCH;
        if (q < NCH && !ok) {
            const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
            stage[q] = z;
            stage[(NCH + 1) + q] = z;
        }
    }

    // this thread's (d, d+1) position pairs
    const int cl = t % NCL;
    int lbase[PP];        // LDS offset (halves) of x[w-1][d-1] for the pair
    uint32_t poff[PP];    // byte offset of g[w][d] inside a plane
    bool pv0[PP], pv1[PP];
#pragma unroll
    for (int k = 0; k < PP; ++k) {
        const int i = t + k * NT;
        const int dp = (i / NCL) % (TD / 2);
        const int wl = i / (NCL * (TD / 2));
        const int dl = 2 * dp;
        lbase[k] = ((wl * PD + dl) * CG) * 8 + cl * CL;
        const int w = w0 + wl, d = d0 + dl;
        pv0[k] = (w < W) && (d < D);
        pv1[k] = (w < W) && (d + 1 < D);
        poff[k] = pv0[k] ? (uint32_t)(((w * D + d) * C + cslab + cl * CL) * 2) : 0u;
    }

    float acc[27][CL];
#pragma unroll
    for (int tap = 0; tap < 27; ++tap)
#pragma unroll
        for (int c = 0; c < CL; ++c) acc[tap][c] = 0.0f;

    // Straight march: only the x planes that exist are visited (planes -1 and H are all zero and contribute
    // nothing), so a step has no branch around its memory operations; the compiler's wait-count bookkeeping
    // is only exact on branch-free paths. It costs about 18 more live registers, so the configurations with
    // four position pairs per lane keep the branching march, which tests every plane instead.
    constexpr bool ST = Cfg::STRAIGHT;
    const int hp_lo = ST ? max(hs - 1, 0) : hs - 1, hp_hi = ST ? min(he, H - 1) : he;
    half8_t pre[NLD];
    auto prefetch_x = [&](int hp) {
        if (ST || ((hp >= 0) && (hp < H))) {
            const char* xplane = reinterpret_cast<const char*>(xn + hp * plane_stride);
#pragma unroll
            for (int j = 0; j < NLD; ++j) pre[j] = *reinterpret_cast<const half8_t*>(xplane + goff[j]);
        }
    };
    // g of one row for every pair: raw dwords (c0,c1) at d and d+1.  The loads are unconditional and
    // nothing looks at the values until they are packed one step later (a select right behind the
    // load would force a wait on every load in flight): rows outside the chunk are replaced by zeros
    // at packing time, positions outside the volume are masked with a precomputed per-lane AND mask.
    uint32_t gmask[PP][2];
#pragma unroll
    for (int k = 0; k < PP; ++k) {
        gmask[k][0] = pv0[k] ? 0xffffffffu : 0u;
        gmask[k][1] = pv1[k] ? 0xffffffffu : 0u;
    }
    auto load_g = [&](int h, uint32_t(&graw)[PP][2]) {
        const int hc_row = min(max(h, hs), he - 1);  // any valid row: the values of other rows are dropped
        const char* gplane = reinterpret_cast<const char*>(gn_ptr + hc_row * plane_stride);
        const uint32_t dstep = (uint32_t)C * 2u;
#pragma unroll
        for (int k = 0; k < PP; ++k) {
            // g is read exactly once: streaming hint, it should not displace the x halo rows in L2
            graw[k][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(gplane + poff[k]));
            graw[k][1] = __builtin_nontemporal_load(
                reinterpret_cast<const uint32_t*>(gplane + poff[k] + (pv1[k] ? dstep : 0u)));
        }
    };
    // packed (g[d][c], g[d+1][c]) per pair and channel for the rows hp-1, hp, hp+1
    half2_t gm[PP][CL], gc[PP][CL], gnx[PP][CL];
    auto pack_g = [&](half2_t(&dst)[PP][CL], const uint32_t(&graw)[PP][2], int h) {
        const bool inb = (h >= hs) && (h < he);  // wavefront-uniform
#pragma unroll
        for (int k = 0; k < PP; ++k) {
            const uint32_t a0 = inb ? (graw[k][0] & gmask[k][0]) : 0u;
            const uint32_t a1 = inb ? (graw[k][1] & gmask[k][1]) : 0u;
            dst[k][0] = pack_lo(a0, a1);
            dst[k][1] = pack_hi(a0, a1);
        }
    };
    // g rows are fetched two steps before they are packed, so their latency is hidden behind
    // a whole plane of arithmetic: ga holds row hp+2 (in flight or landed), gb receives row hp+3
    uint32_t ga[PP][2], gb[PP][2];
    load_g(hp_lo - 1, ga);
    pack_g(gm, ga, hp_lo - 1);
    load_g(hp_lo, ga);
    pack_g(gc, ga, hp_lo);
    load_g(hp_lo + 1, ga);
    pack_g(gnx, ga, hp_lo + 1);
    load_g(hp_lo + 2, ga);

    int parity = 0;
    prefetch_x(hp_lo);
    __syncthreads();  // one-off zero fill of out-of-volume halo chunks
    for (int hp = hp_lo; hp <= hp_hi; ++hp) {
        const bool inb = ST || ((hp >= 0) && (hp < H));
        half8_t* buf = stage + parity * (NCH + 1);
        parity ^= 1;
        if (inb) {
#pragma unroll
            for (int j = 0; j < NLD; ++j) buf[ldst[j]] = pre[j];
        }
        __syncthreads();
        if (ST) {
            prefetch_x(min(hp + 1, hp_hi));  // the last one re-reads the current plane (cache hit) and is dropped
        } else if (hp + 1 <= he) {
            prefetch_x(hp + 1);
        }
        load_g(hp + 3, gb);
        // scheduling fences: the loads stay ahead of the arithmetic that hides their latency
        if (ST) __builtin_amdgcn_sched_barrier(0);
        if (inb) {
            const half_t* plane = reinterpret_cast<const half_t*>(buf);
#pragma unroll
            for (int k = 0; k < PP; ++k) {
#pragma unroll
                for (int kw = 0; kw < 3; ++kw) {
                    uint32_t xv[4];  // x[w+kw-1][d-1 .. d+2], two channels each
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        xv[e] = *reinterpret_cast<const uint32_t*>(plane + lbase[k] + ((kw * PD + e) * CG) * 8);
#pragma unroll
                    for (int kd = 0; kd < 3; ++kd) {
                        const half2_t x0 = pack_lo(xv[kd], xv[kd + 1]);  // channel 0 at (d+kd-1, d+kd)
                        const half2_t x1 = pack_hi(xv[kd], xv[kd + 1]);  // channel 1
                        const int t0 = (0 * 3 + kw) * 3 + kd, t1 = (1 * 3 + kw) * 3 + kd, t2 = (2 * 3 + kw) * 3 + kd;
                        acc[t0][0] = __builtin_amdgcn_fdot2(gnx[k][0], x0, acc[t0][0], false);
                        acc[t0][1] = __builtin_amdgcn_fdot2(gnx[k][1], x1, acc[t0][1], false);
                        acc[t1][0] = __builtin_amdgcn_fdot2(gc[k][0], x0, acc[t1][0], false);
                        acc[t1][1] = __builtin_amdgcn_fdot2(gc[k][1], x1, acc[t1][1], false);
                        acc[t2][0] = __builtin_amdgcn_fdot2(gm[k][0], x0, acc[t2][0], false);
                        acc[t2][1] = __builtin_amdgcn_fdot2(gm[k][1], x1, acc[t2][1], false);
                    }
                }
            }
        }
        if (ST) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < PP; ++k)
#pragma unroll
            for (int c = 0; c < CL; ++c) {
                gm[k][c] = gc[k][c];
                gc[k][c] = gnx[k][c];
            }
        pack_g(gnx, ga, hp + 2);
#pragma unroll
        for (int k = 0; k < PP; ++k) {
            ga[k][0] = gb[k][0];
            ga[k][1] = gb[k][1];
        }
    }

    // ---- combine: lanes with equal cl inside a wavefront, then wavefronts via LDS ----
#pragma unroll
    for (int tap = 0; tap < 27; ++tap)
#pragma unroll
        for (int c = 0; c < CL; ++c) acc[tap][c] = wave_sum_stride<NCL>(acc[tap][c]);

    __syncthreads();  // staging buffers are dead from here on
    float* red = reinterpret_cast<float*>(smem);  // [NWAVE][27][SC]
    const int lane = t % kWave, wave = t / kWave;
    if (lane < NCL) {
#pragma unroll
        for (int tap = 0; tap < 27; ++tap)
#pragma unroll
            for (int c = 0; c < CL; ++c) red[(wave * 27 + tap) * SC + lane * CL + c] = acc[tap][c];
    }
    __syncthreads();
    float* out = a.ws + (int64_t)ws_slot * 27 * SC;
    for (int o = t; o < 27 * SC; o += NT) {
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < Cfg::NWAVE; ++wv) s += red[wv * 27 * SC + o];
        out[o] = s;
    }
}

// ---------------------------------------------------------------------------------------------
// Matrix-core variant (lane_channels = 16).
//
// v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4 blocks, D_b[i][j] += sum_k A_b[i][k] * B_b[k][j];
// lane 4b+i holds row i of A_b as four fp16 (k = 0..3), lane 4b+j holds column j of B_b, and lane 4b+j
// receives column j of D_b in four fp32 registers (i = 0..3).  A depthwise weight gradient has no
// reduction over channels, so a block is one channel and the reduction index k runs over four
// D-adjacent positions d0..d0+3 of one (h, w) row:
//
//   A_b[i][k] = x[hp][w][d0 + k + i - 1][c_b]          (the window of lane i starts i-1 positions in: kd = i)
//   B_b[k][j] = g[hp + 1 - j][w - kw + 1][d0 + k][c_b]  (lane j takes the g plane that sees x plane hp at kh = j)
//   D_b[i][j] accumulates gw[kh = j][kw][kd = i][c_b]   (one accumulator tile per kw)
//
// Row i = 3 and column j = 3 compute nothing useful and are ignored (9 of 16 outputs, 576 of 1024
// multiply-adds per instruction are useful); the meaning of a lane's accumulators never changes, so
// three accumulator tiles are chained through the whole march.  Per g row, four positions and
// 16 channels the cost is 3 matrix instructions instead of 54 dot + 20 permute vector instructions
// per 2 positions x 2 channels: the arithmetic drops to a fraction of the memory time.
//
// Operands come from LDS as dwords (two channels per lane and position) and are split into the even
// and the odd channel's operand by two byte permutes each.  The last four g planes stay in LDS (a
// ring): lane j simply reads its plane's slot, so no operand is kept in registers across steps, and
// the g operand of a row is gathered once per step and used by the three x rows around it.
//
// LDS layout: a position occupies PB = 2*SC bytes; inside it the channel offset is rotated by 32 bytes
// per position (rot) so that the three distinct positions read by half a wavefront fall into disjoint
// banks; g slots are 32 bytes apart modulo 128 for the same reason (lanes j read different slots).
template <int CG_, int TW_, int TD_, int NT_>
struct WmCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_, NWAVE = NT_ / 64;
    static constexpr int SC = CG * 8;                      // channels in the slab
    static constexpr int PB = SC * 2;                      // bytes of one position
    static constexpr int NQ = SC >= 32 ? 16 : SC / 2;      // channel pairs per matrix instruction
    static constexpr int NSUB = 16 / NQ;                   // groups of 4 positions per instruction
    static constexpr int NHALF = SC / (2 * NQ);            // 32-channel halves of the slab
    static constexpr int NPART = NWAVE / NHALF;            // wavefronts that share a half split the patch
    static constexpr int GD = TD / (4 * NSUB);             // position groups along D, one per wavefront
    static constexpr int RSPLIT = NPART / GD;              // ... and row ranges along W
    static constexpr int RG = TW / RSPLIT;                 // g rows per wavefront (it reads RG + 2 x rows)
    static constexpr int R = TW + 2;                       // x rows incl. halo
    static constexpr int PDP = (TD + 2 + 3) / 4 * 4;       // x positions per row incl. halo, padded to 4
    static constexpr int XSLOT = R * PDP * PB;
    // lanes j read different slots: shift their banks apart (with 8 channels a half wavefront reads two
    // position groups 16 banks apart, so the shift is 4 banks there, 8 otherwise)
    static constexpr int GSLOT = TW * TD * PB + (SC == 8 ? 16 : 32);
    static constexpr int XOFF = 4 * GSLOT;                 // [4 g slots][2 x slots][dump]
    static constexpr int DUMP = XOFF + 2 * XSLOT;
    static constexpr int STAGE_BYTES = DUMP + 16;
    static constexpr int NXCH = R * (TD + 2) * CG, NGCH = TW * TD * CG;
    static constexpr int NLDX = (NXCH + NT - 1) / NT, NLDG = (NGCH + NT - 1) / NT;
    static constexpr int RED_BYTES = NPART * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    static_assert(TD % (4 * NSUB) == 0, "a row splits into whole position groups");
    static_assert(NPART % GD == 0 && NPART >= GD, "one position group per wavefront");
    static_assert(TW % RSPLIT == 0, "rows split evenly");
    static_assert(STAGE_BYTES % 16 == 0, "16-byte chunks");
    __device__ static constexpr int swz(int p, int cb) { return lds_swizzle<PB>(p, cb); }
};

// NTI: loads of x chunks no other workgroup reads carry the streaming hint (a compile-time choice: a run-time branch
// next to the loads would make the compiler wait for every load in flight)
template <class Cfg, bool NTI>
__global__ __launch_bounds__(Cfg::NT, Cfg::NT >= 512 ? 4 : 3) void dwconv_wgrad_mfma_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RG = Cfg::RG, XSLOT = Cfg::XSLOT, GSLOT = Cfg::GSLOT;
    constexpr int NLDX = Cfg::NLDX, NLDG = Cfg::NLDG;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];

    const uint32_t ws_slot = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (ws_slot >= a.nblocks) return;
    const int H = a.H, W = a.W, D = a.D, C = a.C;

    // operand gathering: lane = (block b, index rr); block = (channel pair q, position group sub)
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int half = wave % Cfg::NHALF, part = wave / Cfg::NHALF;
    const int gd = part % Cfg::GD, ra = (part / Cfg::GD) * RG;  // this wavefront: position group, first g row
    const int b = lane / 4, rr = lane % 4;
    const int q = b % NQ, sub = b / NQ;
    const int r2 = min(rr, 2);  // index 3 repeats index 2: its results are never used
    // ... and its operands are made zero by the byte selectors of the operand split: the quarter of the multipliers
    // that works for index 3 of either operand then does not toggle (measured: 1738 -> 1765 MHz sustained core clock
    // under this kernel and 2.5 % less time; the kernel follows the core clock, which the power management lowers
    // under matrix-core load)
    const uint32_t sel_e = rr < 3 ? 0x05040100u : 0x0c0c0c0cu, sel_o = rr < 3 ? 0x07060302u : 0x0c0c0c0cu;
    const int cb = half * 64 + q * 4;
    const int pgrp = (gd * NSUB + sub) * 4;  // first position of the lane's group inside a row
    int aoff[4], boff[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        aoff[k] = Cfg::XOFF + Cfg::swz(ra * PDP + pgrp + r2 + k, cb);  // x row ra (patch row ra-1), window r2
        boff[k] = Cfg::swz(ra * TD + pgrp + k, cb);                     // g row ra; the slot is added per step
    }

    // the sums run over every segment of the workgroup: all its tiles belong to the same slab
    float4_t acc[3][2];
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
        for (int e = 0; e < 2; ++e) acc[kw][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // Work of this workgroup: one (tile, row range) segment with uniform chunks, or, in the balanced split, its
    // group's contiguous share [u, u_end) of the (bundle of bal_group tiles, row) sequence (see pick_balanced).
    const bool balanced = a.bal_group > 0;
    uint32_t u = 0, u_end = 0, member = 0;  // wavefront-uniform, kept in scalar registers
    uint32_t ws_row = ws_slot;  // the workgroup's row of partial sums; row % slabs is its slab
    if (balanced) {
        const uint32_t group = ws_slot / a.bal_group;
        member = ws_slot - group * a.bal_group;
        u = __builtin_amdgcn_readfirstlane(group * a.bal_q + min(group, a.bal_r));
        u_end = __builtin_amdgcn_readfirstlane(u + a.bal_q + (group < a.bal_r ? 1u : 0u));
        // Two slabs (128 channels): the first half of a group's members takes slab 0 of the bundle's patches, the
        // second half slab 1, instead of alternating: each half then holds whole patch rows of one slab, which share
        // their halo voxels in the L2 (measured on the forward kernel: 1.56 -> 1.52 ms).
        if (a.n_slab == 2 && a.bal_group % 2 == 0) {
            const uint32_t halfg = a.bal_group / 2;
            member = (member % halfg) * 2 + member / halfg;
            ws_row = group * a.bal_group + member;
        }
    }
    for (bool first = true;; first = false) {
        // the thread index is made opaque per segment: the staging assignment derived from it is then computed inside
        // the segment instead of being hoisted out of this loop and held in registers across the march
        int t = threadIdx.x;
        asm volatile("" : "+v"(t));
        uint32_t L;
        int hs, he;
        if (balanced) {
            if (u >= u_end) break;
            const uint32_t bundle = u / (uint32_t)H;
            hs = (int)(u - bundle * (uint32_t)H);
            he = (int)min((uint32_t)H, hs + (u_end - u));
            u += he - hs;
            L = bundle * a.bal_group + member;
            if (L >= a.n_tiles) continue;  // a partly filled last bundle
            if (!first) __syncthreads();   // the previous segment's last plane has been read by every wavefront
        } else {
            if (!first) break;
            L = ws_slot;
        }
        const int slab = L % a.n_slab;
        L /= a.n_slab;
        const int dt = L % a.n_dt;
        L /= a.n_dt;
        const int wt_i = L % a.n_wt;
        L /= a.n_wt;
        int n;
        if (balanced) {
            n = L;
        } else {
            const int hc = L % a.n_hc;
            n = L / a.n_hc;
            hs = hc * a.h_chunk;
            he = min(hs + a.h_chunk, H);
        }
        const int w0 = wt_i * Cfg::TW, d0 = dt * TD;
        const int cslab = slab * SC;
        const int64_t plane_stride = (int64_t)W * D * C;
        const half_t* xn = a.x + (int64_t)n * H * plane_stride;
        const half_t* gn_ptr = a.g + (int64_t)n * H * plane_stride;

        // everything that staging never writes must read as zero: positions outside the volume and the
        // g planes before the chunk
        const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int o = t * 16; o < Cfg::STAGE_BYTES; o += NT * 16) *reinterpret_cast<half8_t*>(smem + o) = z8;

        // staging assignment, 16-byte chunks (8 channels of one position); lanes without a chunk inside the
        // volume load the plane's first chunk and write it to the dump slot
        uint32_t xgo[NLDX], ggo[NLDG];
        int xls[NLDX], gls[NLDG];
        typedef HaloOrder<Cfg::TW, TD, CG> Order;  // chunks shared with neighbouring patches first, interior last
    #pragma unroll
        for (int j = 0; j < NLDX; ++j) {
            const int ch = t + j * NT;
            int wq, dq, cq;
            Order::decode(ch, wq, dq, cq);
            const int w = w0 - 1 + wq, d = d0 - 1 + dq;
            const bool ok = (ch < Cfg::NXCH) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
            xgo[j] = ok ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
            xls[j] = ok ? Cfg::swz(wq * PDP + dq, cq * 16) : -1;
        }
    #pragma unroll
        for (int j = 0; j < NLDG; ++j) {
            const int ch = t + j * NT;
            const int wq = ch / (TD * CG);
            const int rem = ch - wq * (TD * CG);
            const int dq = rem / CG, cq = rem - dq * CG;
            const int w = w0 + wq, d = d0 + dq;
            const bool ok = (ch < Cfg::NGCH) && (w < W) && (d < D);
            ggo[j] = ok ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
            gls[j] = ok ? Cfg::swz(wq * TD + dq, cq * 16) : -1;
        }

        // Global loads run two planes ahead of the arithmetic, into two register sets used alternately.
        // They are unconditional (plane indices are clamped, values of planes that do not exist or lie
        // outside the chunk are never used): the compiler's wait-count bookkeeping is exact only on
        // branch-free paths, and a conservative wait would also wait for the newer set.
        half8_t xpre0[NLDX], xpre1[NLDX], gpre0[NLDG], gpre1[NLDG];
        auto prefetch = [&](int hp, half8_t(&xpre)[NLDX], half8_t(&gpre)[NLDG]) {  // x plane hp, g plane hp+1
            const char* xplane = reinterpret_cast<const char*>(xn + min(max(hp, 0), H - 1) * plane_stride);
            const char* gplane = reinterpret_cast<const char*>(gn_ptr + min(max(hp + 1, hs), he - 1) * plane_stride);
    #pragma unroll
            for (int j = 0; j < NLDX; ++j) {
                // nobody else reads the interior chunks: with the hint they do not push shared lines out of the L2
                if (NTI && Order::interior_only(j * NT))
                    xpre[j] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(xplane + xgo[j]));
                else
                    xpre[j] = *reinterpret_cast<const half8_t*>(xplane + xgo[j]);
            }
    #pragma unroll
            for (int j = 0; j < NLDG; ++j)
                gpre[j] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(gplane + ggo[j]));
        };

        int parity = 0;
        // step hp: x plane hp meets the g planes hp+1 (kh = 0), hp (kh = 1), hp-1 (kh = 2)
        auto step = [&](int hp, half8_t(&xpre)[NLDX], half8_t(&gpre)[NLDG], bool live) {
            const bool xin = live && (hp >= 0) && (hp < H);  // wavefront-uniform
            const bool gin = hp + 1 < he;
            unsigned char* xbuf = smem + Cfg::XOFF + parity * XSLOT;
            unsigned char* gslot = smem + ((hp + 1) & 3) * GSLOT;
    #pragma unroll
            for (int j = 0; j < NLDX; ++j) {
                unsigned char* dst = xls[j] >= 0 ? xbuf + xls[j] : smem + Cfg::DUMP;
                *reinterpret_cast<half8_t*>(dst) = xpre[j];
            }
            // g planes past the chunk read as zero; the slot held a plane that is no longer needed
    #pragma unroll
            for (int j = 0; j < NLDG; ++j) {
                unsigned char* dst = gls[j] >= 0 ? gslot + gls[j] : smem + Cfg::DUMP;
                *reinterpret_cast<half8_t*>(dst) = gin ? gpre[j] : z8;
            }
            __syncthreads();
            prefetch(hp + 2, xpre, gpre);
            __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the arithmetic that hides their latency
            if (xin) {
                const int xo = parity * XSLOT;
                const int go = ((hp + 1 - r2) & 3) * GSLOT;  // lane j reads the slot of plane hp+1-j
                half4_t G[RG][2];
    #pragma unroll
                for (int xr = 0; xr < RG + 2; ++xr) {
                    if (xr < RG) {  // the g row first needed by this x row
                        uint32_t r[4];
    #pragma unroll
                        for (int k = 0; k < 4; ++k)
                            r[k] = *reinterpret_cast<const uint32_t*>(smem + go + boff[k] + xr * TD * PB);
                        split_operands_sel(r, sel_e, sel_o, G[xr][0], G[xr][1]);
                    }
                    uint32_t r[4];
    #pragma unroll
                    for (int k = 0; k < 4; ++k)
                        r[k] = *reinterpret_cast<const uint32_t*>(smem + xo + aoff[k] + xr * PDP * PB);
                    half4_t A[2];
                    split_operands_sel(r, sel_e, sel_o, A[0], A[1]);
    #pragma unroll
                    for (int kw = 0; kw < 3; ++kw) {
                        // x patch row ra-1+xr meets g row ra+xr-kw at tap kw
                        if (xr - kw >= 0 && xr - kw < RG) {
    #pragma unroll
                            for (int e = 0; e < 2; ++e) {
                                acc[kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(A[e], G[xr - kw][e], acc[kw][e], 0, 0, 0);
                            }
                        }
                    }
                }
            }
            parity ^= 1;
        };

        prefetch(hs - 1, xpre0, gpre0);
        prefetch(hs, xpre1, gpre1);
        __syncthreads();  // the one-off zero fill is complete before staging writes anything
        // The steps hp = hs-1 .. he run in pairs, one per register set, in a loop whose only exit is at its end: an
        // exit between the two steps would give the loop a second way into its first step, on which the newer set
        // is the older one, and the compiler's wait before that step's staging writes would cover both sets.  An odd
        // count ends with a step that stages planes nobody reads and computes nothing.
        for (int hp = hs - 1; hp <= he; hp += 2) {
            step(hp, xpre0, gpre0, true);
            step(hp + 1, xpre1, gpre1, hp + 1 <= he);
        }
    }  // segments

    const int t = threadIdx.x;
    // ---- combine: position groups inside a wavefront, then the wavefronts of a half via LDS ----
    if (NSUB > 1) {
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    float v = acc[kw][e][i];
#pragma unroll
                    for (int off = 4 * NQ; off < kWave; off <<= 1) v += __shfl_xor(v, off, kWave);
                    acc[kw][e][i] = v;
                }
    }
    __syncthreads();  // staging buffers are dead from here on
    float* red = reinterpret_cast<float*>(smem);  // [NPART][27][SC]
    if (sub == 0 && rr < 3) {
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    red[(part * 27 + (rr * 3 + kw) * 3 + i) * SC + half * 32 + 2 * q + e] = acc[kw][e][i];
    }
    __syncthreads();
    float* out = a.ws + (int64_t)ws_row * 27 * SC;
    for (int o = t; o < 27 * SC; o += NT) {
        float sacc = 0.0f;
#pragma unroll
        for (int pt = 0; pt < Cfg::NPART; ++pt) sacc += red[pt * 27 * SC + o];
        out[o] = sacc;
    }
}

// ---------------------------------------------------------------------------------------------
// Fused backward: input gradient and weight gradient in one pass over x and g.
//
//   dx[n,h,w,d,c] = sum_{kh,kw,kd} g[n,h-kh+1,w-kw+1,d-kd+1,c] * wt[kh,kw,kd,c]   (= DWConv(g, wt flipped))
//   gw[kh,kw,kd,c] = sum g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]
//
// Run separately the two products read g twice (8.8 GB at C=64 with the halos); here a workgroup stages
// every g plane of its patch once, with halo, into a ring of four LDS slots and uses it twice: as the
// scattered operand of the forward scheme (weights flipped, accumulator registers = the dx planes
// p+1, p, p-1 of g plane p) and as the window operand of the weight-gradient scheme.  The weight gradient is
// summed over the x positions of the patch, gw[kh,kw,kd] = sum x[h+kh-1,w,d] * g[h,w-kw+1,d-kd+1] (the same sum
// with the shifts along W and D moved to g; positions of g outside the volume contribute nothing), so x is read
// without a halo along W and D: one tensor with halo instead of two.  x planes live in a ring of four patch-sized
// slots; g plane P is multiplied with the x planes P-1, P, P+1 (lane j takes the slot of plane P+j-1) once plane
// P+1 of x has arrived.  The g planes next to the chunk are real data for dx but belong to other chunks for gw:
// those steps are skipped by the weight-gradient role.
//
// The two products run on different wavefronts: all 8 wavefronts of a workgroup stage the planes of x and g
// into LDS, then wavefronts 0-3 run the input-gradient scheme (and store dx) while wavefronts 4-7
// run the weight-gradient scheme on the same LDS data, each role in its own loop with the same sequence of
// workgroup barriers.  A role keeps only its own accumulators: 123-128 registers and 42-62 KB of LDS, so two
// workgroups (16 wavefronts) are resident per CU, where running both schemes in every wavefront needs ~190
// registers and holds 8 wavefronts.  An 8x8 patch with 16 wavefronts re-reads less halo but leaves one
// workgroup per CU, whose per-plane barriers are then fully exposed.
template <int CG_, int TW_, int TD_, int NT_>
struct BsCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_, RWAVES = NT_ / 128;  // wavefronts per role
    static constexpr int SC = CG * 8, PB = SC * 2;
    static constexpr int NQ = SC >= 32 ? 16 : SC / 2, NSUB = 16 / NQ, NHALF = SC / (2 * NQ);
    static constexpr int NPART = RWAVES / NHALF, GD = TD / (4 * NSUB), RSPLIT = NPART / GD, RO = TW / RSPLIT;
    static constexpr int R = TW + 2, PDP = (TD + 3 + 3) / 4 * 4, GSLOT = R * PDP * PB;  // a g plane with its halo
    static constexpr int NPOS = TW * TD;
    // an x plane of the patch alone; lanes j of the weight-gradient role read different slots: shift their banks apart
    static constexpr int XSLOT = NPOS * PB + (SC == 8 ? 16 : 32);
    static constexpr int XOFF = 4 * GSLOT;
    // dx leaves through two LDS output tiles as 16-byte chunks (whole lines, one store per thread and plane)
    static constexpr int OT_BYTES = NPOS * PB, OT_OFF = XOFF + 4 * XSLOT;
    static constexpr int DUMP = OT_OFF + 2 * OT_BYTES, STAGE_BYTES = DUMP + 16;
    static constexpr int NCH = R * (TD + 2) * CG;  // 16-byte chunks of a staged g plane: one per thread, t < NCH
    static constexpr int NXCH = NPOS * CG;         // ... of a staged x plane: t < NXCH
    static constexpr int RED_BYTES = NPART * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    static_assert(NCH <= NT && NXCH <= NT && RO == 4 && TD % (4 * NSUB) == 0 && NPART % GD == 0 && TW % RSPLIT == 0,
                  "even split");
    static_assert(NPOS * CG == RWAVES * 64, "the dx role stores the tile: one 16-byte chunk per thread");
    static_assert(STAGE_BYTES % 16 == 0, "16-byte chunks");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 4) void dwconv_bwd_split_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RO = Cfg::RO, GSLOT = Cfg::GSLOT, XSLOT = Cfg::XSLOT;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];

    const uint32_t ws_slot = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (ws_slot >= a.nblocks) return;
    const int t = threadIdx.x;
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    const int64_t plane_stride = (int64_t)W * D * C;
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};

    const int lane = t % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
    const int role = wave / Cfg::RWAVES, rwave = wave % Cfg::RWAVES;  // 0: input gradient, 1: weight gradient
    const int half = rwave % Cfg::NHALF, part = rwave / Cfg::NHALF;
    const int gd = part % Cfg::GD, ra = (part / Cfg::GD) * RO;
    // every tile of a workgroup belongs to the same slab (uniform chunks: one tile; balanced split: the group
    // size is a multiple of the slab count)

    // Work of this workgroup: one (tile, row range) segment with uniform chunks, or, in the balanced split, its
    // group's contiguous share [u, u_end) of the (bundle of bal_group tiles, row) sequence (see pick_balanced).
    // Both roles walk the same segments with the same sequence of workgroup barriers.
    const bool balanced = a.bal_group > 0;
    uint32_t u = 0, u_end = 0, member = 0;  // wavefront-uniform, kept in scalar registers
    uint32_t ws_row = ws_slot;  // the workgroup's row of partial sums; row % slabs is its slab
    if (balanced) {
        const uint32_t group = ws_slot / a.bal_group;
        member = ws_slot - group * a.bal_group;
        u = __builtin_amdgcn_readfirstlane(group * a.bal_q + min(group, a.bal_r));
        u_end = __builtin_amdgcn_readfirstlane(u + a.bal_q + (group < a.bal_r ? 1u : 0u));
        // two slabs: slab-major member order, see dwconv_wgrad_mfma_kernel
        if (a.n_slab == 2 && a.bal_group % 2 == 0) {
            const uint32_t halfg = a.bal_group / 2;
            member = (member % halfg) * 2 + member / halfg;
            ws_row = group * a.bal_group + member;
        }
    }
    const int cslab = (int)(ws_row % (uint32_t)a.n_slab) * SC;
    bool first = true;
    // the segment in hand
    int hs = 0, he = 0, w0 = 0, d0 = 0;
    const half_t* xn = a.x;
    const half_t* gn_ptr = a.g;
    half_t* dxn = a.dx;
    uint32_t go = 0, xgo = 0;  // staging: thread t owns chunk t of the g patch with halo and chunk t of the x patch;
    int ls = -1, xls = -1;     // threads without a chunk inside the volume load the plane's first chunk and write
                               // it to the dump slot
    auto next_segment = [&]() -> bool {  // workgroup-uniform
        uint32_t L;
        for (;;) {
            if (balanced) {
                if (u >= u_end) return false;
                const uint32_t bundle = u / (uint32_t)H;
                hs = (int)(u - bundle * (uint32_t)H);
                he = (int)min((uint32_t)H, hs + (u_end - u));
                u += he - hs;
                L = bundle * a.bal_group + member;
                if (L >= a.n_tiles) continue;  // a partly filled last bundle
            } else {
                if (!first) return false;
                L = ws_slot;
            }
            break;
        }
        first = false;
        L /= a.n_slab;
        const int dt = L % a.n_dt;
        L /= a.n_dt;
        const int wt_i = L % a.n_wt;
        L /= a.n_wt;
        int n;
        if (balanced) {
            n = L;
        } else {
            const int hc = L % a.n_hc;
            n = L / a.n_hc;
            hs = hc * a.h_chunk;
            he = min(hs + a.h_chunk, H);
        }
        // the decoded values are wavefront-uniform but come out of vector divisions: back to scalar registers
        n = __builtin_amdgcn_readfirstlane(n);
        hs = __builtin_amdgcn_readfirstlane(hs);
        he = __builtin_amdgcn_readfirstlane(he);
        w0 = __builtin_amdgcn_readfirstlane(wt_i * Cfg::TW);
        d0 = __builtin_amdgcn_readfirstlane(dt * TD);
        xn = a.x + (int64_t)n * H * plane_stride;
        gn_ptr = a.g + (int64_t)n * H * plane_stride;
        dxn = a.dx + (int64_t)n * H * plane_stride;
        // what staging never writes must read as zero (positions outside the volume, g planes before the chunk); the
        // previous segment's barrier after its last plane makes the buffers free.  The output tiles behind the
        // staging buffers are left alone: the other role may still be storing the last one.
        for (int o = t * 16; o < Cfg::OT_OFF; o += NT * 16) *reinterpret_cast<half8_t*>(smem + o) = z8;
        // an opaque copy of the thread index keeps this assignment from being hoisted out of the segment loop
        int ts = t;
        asm volatile("" : "+v"(ts));
        const int wq = ts / ((TD + 2) * CG);
        const int rem = ts - wq * ((TD + 2) * CG);
        const int dq = rem / CG, cq = rem - dq * CG;
        const int w = w0 - 1 + wq, d = d0 - 1 + dq;
        const bool ok = (ts < Cfg::NCH) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
        go = ok ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
        ls = ok ? lds_swizzle<PB>(wq * PDP + dq, cq * 16) : -1;
        // x: the patch alone (the weight gradient is summed over the x positions of the patch against the g
        // positions around them, so that only one of the two tensors is read with a halo)
        const int xwq = ts / (TD * CG);
        const int xrem = ts - xwq * (TD * CG);
        const int xdq = xrem / CG, xcq = xrem - xdq * CG;
        const bool xok = (ts < Cfg::NXCH) && (w0 + xwq < W) && (d0 + xdq < D);
        xgo = xok ? (uint32_t)((((w0 + xwq) * D + d0 + xdq) * C + cslab + xcq * 8) * 2) : 0u;
        xls = xok ? lds_swizzle<PB>(xwq * TD + xdq, xcq * 16) : -1;
        return true;
    };

    // loads run two steps ahead in two register sets; unconditional (clamped plane indices)
    half8_t xpre0, xpre1, gpre0, gpre1;
    auto prefetch = [&](int p, half8_t& xpre, half8_t& gpre) {  // planes p of x and g
        const int64_t poff = min(max(p, 0), H - 1) * plane_stride;
        xpre = *reinterpret_cast<const half8_t*>(reinterpret_cast<const char*>(xn + poff) + xgo);
        gpre = *reinterpret_cast<const half8_t*>(reinterpret_cast<const char*>(gn_ptr + poff) + go);
    };
    int parity = 0;  // output tile in use (input-gradient role)
    // Planes outside the volume or beyond the chunk arrive as copies of a clamped plane and are staged as they
    // are: the input-gradient role skips the step of such a g plane, the weight-gradient role never takes a g
    // plane outside its chunk and zeroes the operand of a lane whose x plane lies outside the volume.
    auto stage = [&](int p, const half8_t& xpre, const half8_t& gpre) {
        unsigned char* xslot = smem + Cfg::XOFF + (p & 3) * XSLOT;
        unsigned char* gslot = smem + (p & 3) * GSLOT;
        unsigned char* xd = xls >= 0 ? xslot + xls : smem + Cfg::DUMP;
        unsigned char* gdst = ls >= 0 ? gslot + ls : smem + Cfg::DUMP;
        *reinterpret_cast<half8_t*>(xd) = xpre;
        *reinterpret_cast<half8_t*>(gdst) = gpre;
    };

    if (role == 0) {
        // ---- input gradient: flipped weight operands, (kd' = 0, 1, 2, -) of one kh' per lane.  The four registers
        // of an accumulator tile form a ring: dx plane h lives in register (h - hs + 1) % 4 for the three steps
        // that add to it, so nothing is moved between steps.  At step s (g plane p = hs - 1 + s) register i takes
        // kh' = (s + 1 - i) % 4 (3 = none: zero weights), i.e. every step each lane hands its weights to the next
        // lane of its quad; a march of 4n steps leaves them where they started. ----
        half4_t wA[3][2];
        {
            const int r0 = (1 - lane % 4) & 3, c0 = cslab + half * 32 + 2 * ((lane / 4) % NQ);
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    half4_t v = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
                    if (r0 < 3) {
#pragma unroll
                        for (int kd = 0; kd < 3; ++kd)
                            v[kd] = a.wt[(((2 - r0) * 3 + (2 - kw)) * 3 + (2 - kd)) * C + c0 + e];
                    }
                    wA[kw][e] = v;
                }
        }
        auto ot_swz = [](int pos, int cbyte) {
            return PB == 128 ? pos * PB + ((cbyte + 64 * (pos & 1)) & 127) : pos * PB + cbyte;
        };
        while (next_segment()) {
            // lane constants from an opaque copy of the thread index: computed per segment, so that what only the
            // segment's set-up needs is not held in registers across the march
            int tl = t;
            asm volatile("" : "+v"(tl));
            const int lane = tl % kWave;
            const int b = lane / 4, rr = lane % 4;
            const int q = b % NQ, sub = b / NQ;
            const int cb = half * 64 + q * 4;
            const int pgrp = (gd * NSUB + sub) * 4;
            int dboff[3];
    #pragma unroll
            for (int k = 0; k < 3; ++k) dboff[k] = lds_swizzle<PB>(ra * PDP + pgrp + rr + k, cb);
            int owr[RO];
    #pragma unroll
            for (int o = 0; o < RO; ++o) owr[o] = ot_swz((ra + o) * TD + pgrp + rr, cb);
            // the threads of this role store the output tile, one 16-byte chunk each
            const int opos = tl / CG, ocq = tl % CG;
            const int ord = ot_swz(opos, ocq * 16);
            const int ow = w0 + opos / TD, odd = d0 + opos % TD;
            const bool ovalid = (ow < W) && (odd < D);
            const uint32_t ogo = ovalid ? (uint32_t)(((ow * D + odd) * C + cslab + ocq * 8) * 2) : 0u;
            parity = 0;
            prefetch(hs - 1, xpre0, gpre0);
            prefetch(hs, xpre1, gpre1);
            __syncthreads();  // the zero fill is complete before staging writes anything
            int pending_row = -1;
            auto flush_row = [&](int par) {
                if (pending_row >= 0) {  // workgroup-uniform
                    const half8_t o8 = *reinterpret_cast<const half8_t*>(smem + Cfg::OT_OFF + par * Cfg::OT_BYTES + ord);
                    if (ovalid)
                        __builtin_nontemporal_store(
                            o8, reinterpret_cast<half8_t*>(reinterpret_cast<char*>(dxn + pending_row * plane_stride) + ogo));
                }
            };
            float4_t T[RO][2];  // dx tiles, four planes in a ring of registers
    #pragma unroll
            for (int o = 0; o < RO; ++o)
    #pragma unroll
                for (int e = 0; e < 2; ++e) T[o][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

            auto step = [&](auto ring, int p, half8_t& xpre, half8_t& gpre, bool live) {
                constexpr int DONE = (decltype(ring)::value + 3) & 3;  // register of dx plane p-1, complete after this step
                const bool gin = live && (p >= 0) && (p < H) && (p <= he);
                unsigned char* gslot = smem + (p & 3) * GSLOT;
                stage(p, xpre, gpre);
                __syncthreads();
                flush_row(parity ^ 1);
                prefetch(p + 2, xpre, gpre);
                __builtin_amdgcn_sched_barrier(0);
                if (gin) {
    #pragma unroll
                    for (int xr = 0; xr < RO + 2; ++xr) {
                        uint32_t r[3];
    #pragma unroll
                        for (int k = 0; k < 3; ++k)
                            r[k] = *reinterpret_cast<const uint32_t*>(gslot + dboff[k] + xr * PDP * PB);
                        half4_t B[2];
                        split_operands3(r, B[0], B[1]);
    #pragma unroll
                        for (int kw = 0; kw < 3; ++kw) {
                            if (xr - kw >= 0 && xr - kw < RO) {
    #pragma unroll
                                for (int e = 0; e < 2; ++e)
                                    T[xr - kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(wA[kw][e], B[e], T[xr - kw][e], 0, 0, 0);
                            }
                        }
                    }
                }
                const int ho = p - 1;
                const bool store = live && (ho >= hs) && (ho < he);
                pending_row = store ? ho : -1;
                if (store) {
                    unsigned char* otile = smem + Cfg::OT_OFF + parity * Cfg::OT_BYTES;
    #pragma unroll
                    for (int o = 0; o < RO; ++o) {
                        half2_t v;
    #pragma unroll
                        for (int e = 0; e < 2; ++e) v[e] = (half_t)T[o][e][DONE];
                        *reinterpret_cast<half2_t*>(otile + owr[o]) = v;
                    }
                }
                // the finished register rests for one step (its lane has zero weights then) and starts its next
                // plane from zero; the weights move on by one lane
    #pragma unroll
                for (int o = 0; o < RO; ++o)
    #pragma unroll
                    for (int e = 0; e < 2; ++e) T[o][e][DONE] = 0.0f;
    #pragma unroll
                for (int kw = 0; kw < 3; ++kw)
    #pragma unroll
                    for (int e = 0; e < 2; ++e) wA[kw][e] = quad_rotate_up(wA[kw][e]);
                parity ^= 1;
            };
            // groups of four steps (the ring's period), register sets alternating, and a single exit (see
            // dwconv_wgrad_mfma_kernel); both roles run the same number of steps, so their barriers match
            for (int p = hs - 1; p <= he + 1; p += 4) {
                step(std::integral_constant<int, 0>{}, p, xpre0, gpre0, true);
                step(std::integral_constant<int, 1>{}, p + 1, xpre1, gpre1, p + 1 <= he + 1);
                step(std::integral_constant<int, 2>{}, p + 2, xpre0, gpre0, p + 2 <= he + 1);
                step(std::integral_constant<int, 3>{}, p + 3, xpre1, gpre1, p + 3 <= he + 1);
            }
            __syncthreads();  // the last tile is written, every wavefront is done with the staging buffers
            flush_row(parity ^ 1);
        }  // segments
        __syncthreads();  // (the other role: staging buffers are dead)
        __syncthreads();  // (the other role: partial sums are in LDS)
    } else {
        // ---- weight gradient, summed over the x positions of the patch: gw[kh][kw][kd] = sum x[P+kh-1][w][d] *
        // g[P][w-kw+1][d-kd+1].  Operand A (lane i = kd): the window of g plane P, halo row ra + t, that starts kd
        // positions to the left; operand B (lane j = kh): four positions of x row ra + o in the slot of plane
        // P + j - 1.  Planes of x next to the chunk are real data, g planes next to it belong to other chunks: the
        // step with such a P is skipped as a whole. ----
        int aoff[4], boff[4], r2s = 0;  // set per segment (see the other role)
        float4_t acc[3][2];  // one tile per kw: D[i = kd][j = kh]
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int e = 0; e < 2; ++e) acc[kw][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

        // byte selectors that split a dword pair into the even / odd channel's operand; all-zero operands
        // (selector 0x0c0c0c0c) for index 3, which no result uses, and for a lane whose x plane is outside the volume
        uint32_t sel_e = 0x05040100u, sel_o = 0x07060302u;
        auto step = [&](int p, half8_t& xpre, half8_t& gpre, bool live) {
            const int P = p - 1;  // g plane P meets the x planes P-1, P, P+1 = p, the newest one staged
            const bool on = live && (P >= hs) && (P < he);
            stage(p, xpre, gpre);
            __syncthreads();
            prefetch(p + 2, xpre, gpre);
            __builtin_amdgcn_sched_barrier(0);
            if (on) {
                const unsigned char* gsl = smem + (P & 3) * GSLOT;
                const int xp = P - 1 + r2s;  // the lane's x plane
                const unsigned char* xsl = smem + Cfg::XOFF + (xp & 3) * XSLOT;
                const bool xv = (unsigned)xp < (unsigned)H;
                const uint32_t se = xv ? sel_e : 0x0c0c0c0cu, so = xv ? sel_o : 0x0c0c0c0cu;
                half4_t X[RO][2];
#pragma unroll
                for (int o = 0; o < RO; ++o) {
                    uint32_t r[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) r[k] = *reinterpret_cast<const uint32_t*>(xsl + boff[k] + o * TD * PB);
                    split_operands_sel(r, se, so, X[o][0], X[o][1]);
                }
#pragma unroll
                for (int tr = 0; tr < RO + 2; ++tr) {
                    uint32_t r[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) r[k] = *reinterpret_cast<const uint32_t*>(gsl + aoff[k] + tr * PDP * PB);
                    half4_t A[2];
                    split_operands(r, A[0], A[1]);
#pragma unroll
                    for (int kw = 0; kw < 3; ++kw) {
                        if (tr + kw - 2 >= 0 && tr + kw - 2 < RO) {
#pragma unroll
                            for (int e = 0; e < 2; ++e)
                                acc[kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(A[e], X[tr + kw - 2][e], acc[kw][e], 0, 0, 0);
                        }
                    }
                }
            }
        };
        while (next_segment()) {
            {
                int tl = t;
                asm volatile("" : "+v"(tl));
                const int ln = tl % kWave;
                const int bb = ln / 4;
                const int qq = bb % NQ, ss = bb / NQ;
                const int cbs = half * 64 + qq * 4, pg = (gd * NSUB + ss) * 4;
                r2s = min(ln % 4, 2);
                sel_e = ln % 4 < 3 ? 0x05040100u : 0x0c0c0c0cu;
                sel_o = ln % 4 < 3 ? 0x07060302u : 0x0c0c0c0cu;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    aoff[k] = lds_swizzle<PB>(ra * PDP + pg + 2 - r2s + k, cbs);
                    boff[k] = lds_swizzle<PB>(ra * TD + pg + k, cbs);
                }
            }
            parity = 0;
            prefetch(hs - 1, xpre0, gpre0);
            prefetch(hs, xpre1, gpre1);
            __syncthreads();  // the zero fill is complete before staging writes anything
            for (int p = hs - 1; p <= he + 1; p += 4) {  // four steps per round, as in the other role
                step(p, xpre0, gpre0, true);
                step(p + 1, xpre1, gpre1, p + 1 <= he + 1);
                step(p + 2, xpre0, gpre0, p + 2 <= he + 1);
                step(p + 3, xpre1, gpre1, p + 3 <= he + 1);
            }
            __syncthreads();  // (the other role: the last tile is written); the staging buffers are free
        }
        if (NSUB > 1) {  // position groups inside the wavefront
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                for (int e = 0; e < 2; ++e)
#pragma unroll
                    for (int i = 0; i < 3; ++i) {
                        float v = acc[kw][e][i];
#pragma unroll
                        for (int off = 4 * NQ; off < kWave; off <<= 1) v += __shfl_xor(v, off, kWave);
                        acc[kw][e][i] = v;
                    }
        }
        __syncthreads();  // staging buffers are dead from here on
        float* red = reinterpret_cast<float*>(smem);  // [NPART][27][SC]
        const int rr = lane % 4, q = (lane / 4) % NQ, sub = (lane / 4) / NQ;
        if (sub == 0 && rr < 3) {
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                for (int e = 0; e < 2; ++e)
#pragma unroll
                    for (int i = 0; i < 3; ++i)
                        red[(part * 27 + (rr * 3 + kw) * 3 + i) * SC + half * 32 + 2 * q + e] = acc[kw][e][i];
        }
        __syncthreads();
    }
    const float* red = reinterpret_cast<const float*>(smem);
    float* out = a.ws + (int64_t)ws_row * 27 * SC;
    for (int o = t; o < 27 * SC; o += NT) {
        float sacc = 0.0f;
#pragma unroll
        for (int pt = 0; pt < Cfg::NPART; ++pt) sacc += red[pt * 27 * SC + o];
        out[o] = sacc;
    }
}

// Second pass, fixed summation order (deterministic).  The workspace holds one row per (n, h-chunk, w-patch,
// d-patch) of width RW = slabs*27*SC floats.  A workgroup owns 16 columns, its 64 row slices sum interleaved rows
// (four loads in flight), the slices are combined in LDS in a fixed order and the result is scattered to the
// [27][C] layout.  One launch: at 128^3-class shapes a second small launch was 5 % of the whole op.
// OutT: fp32, or fp16 = the sum rounded once (what a cast of the fp32 result gives, without its launch).
template <class OutT>
__global__ __launch_bounds__(1024) void wgrad_reduce_kernel(const float* __restrict__ ws, OutT* __restrict__ gw,
                                                            int n_rows, int RW, int SC, int C)
{
    __shared__ float part[64][17];
    const int cl = threadIdx.x % 16, slice = threadIdx.x / 16;
    const int col = blockIdx.x * 16 + cl;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (col < RW) {
        int r = slice;
        for (; r + 192 < n_rows; r += 256) {
            s0 += ws[(int64_t)r * RW + col];
            s1 += ws[(int64_t)(r + 64) * RW + col];
            s2 += ws[(int64_t)(r + 128) * RW + col];
            s3 += ws[(int64_t)(r + 192) * RW + col];
        }
        for (; r < n_rows; r += 64) s0 += ws[(int64_t)r * RW + col];
    }
    part[slice][cl] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int w = 32; w > 0; w >>= 1) {
        if (slice < w) part[slice][cl] += part[slice + w][cl];
        __syncthreads();
    }
    if (slice == 0 && col < RW) {
        const int slab = col / (27 * SC), rem = col % (27 * SC);
        const int tap = rem / SC, cs = rem % SC;
        gw[tap * C + slab * SC + cs] = (OutT)part[0][cl];
    }
}

struct WgPlan {
    int cg, tile_w, tile_d, cl, h_chunk, n_wt, n_dt, n_hc, n_slab, n_xcd = 8;
    int64_t nblocks;
    uint32_t bal_group = 0, bal_q = 0, bal_r = 0, n_tiles = 0;  // balanced split (bal_group > 0), see pick_balanced
};

static int plan_wgrad(int N, int H, int W, int D, int C, int tile_w, int tile_d, int h_chunk, int lane_channels,
                      WgPlan* p)
{
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwconv_wgrad: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if (!(C == 8 || C == 16 || C == 32 || C == 64 || C == 128)) {
        set_error("dwconv_wgrad: unsupported channel count %d", C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    if (plane_exceeds_i32(W, D, C)) {
        set_error("dwconv_wgrad: one (W,D,C) plane must stay below 2^31 elements");
        return KEROPS_E_BADARG;
    }
    p->cg = C >= 64 ? 8 : C / 8;
    if (tile_w == 0 && tile_d == 0 && lane_channels == 0) {
        // measured best on MI355X at (1, C, 350, 350, 128): the matrix-core kernels with LDS-direct staging,
        // 256-thread workgroups on patches of 512 16-byte chunks
        switch (p->cg) {
            case 1: tile_w = 8; tile_d = 64; break;
            case 2: tile_w = 8; tile_d = 32; break;
            case 4: tile_w = 8; tile_d = 16; break;
            default: tile_w = 8; tile_d = 8; break;
        }
        lane_channels = 32;
    }
    // only the all-zero triple selects the built-in shape; anything else must name a positive patch
    // (checked before the extents are divided by it) and is matched against the built kernels at launch
    if (tile_w <= 0 || tile_d <= 0 || tile_w > 1024 || tile_d > 1024 || lane_channels <= 0) {
        set_error("dwconv_wgrad: no kernel built for C=%d tile_w=%d tile_d=%d lane_channels=%d", C, tile_w, tile_d,
                  lane_channels);
        return KEROPS_E_BADARG;
    }
    p->cl = lane_channels;
    p->tile_w = tile_w;
    p->tile_d = tile_d;
    p->n_slab = C / (p->cg * 8);
    p->n_wt = ceil_div(W, tile_w);
    p->n_dt = ceil_div(D, tile_d);
    // 256 CUs hold 2 workgroups of 512 threads or 4 of 256 each; every workgroup also leaves one partial
    const int64_t per_plane = (int64_t)N * p->n_wt * p->n_dt * p->n_slab;
    // patches of 512 or more 16-byte chunks: two workgroups per compute unit (512 threads each when staged through
    // registers; the LDS-direct kernels run 256 threads and are held to two by their staging rings)
    const bool big_wg = lane_channels >= 16 ? tile_w * tile_d * p->cg >= 512 : (p->cg == 8 && tile_w * tile_d >= 64);
    const DeviceGeometry geo = device_geometry();
    p->n_xcd = geo.xcds;
    const int slots = geo.resident_workgroups(big_wg ? 512 : 256);
    p->bal_group = 0;
    // h_chunk 0: balanced split with the group size of the cost model (-g: groups of g workgroups; matrix-core
    // kernels only); > 0: uniform chunks of that many rows
    if (lane_channels >= 16 && h_chunk <= 0) {
        if (h_chunk < 0 && (-h_chunk) % p->n_slab != 0) {
            set_error("dwconv_wgrad: the group size of the balanced split must be a multiple of the slab count %d",
                      p->n_slab);
            return KEROPS_E_BADARG;
        }
        const BalancedSplit b = h_chunk < 0 ? make_balanced(H, per_plane, slots, -h_chunk)
                                            : pick_balanced(H, per_plane, p->n_dt * p->n_slab, slots, 8, p->n_slab,
                                                            geo.xcds);
        const bool fits = b.units < (1LL << 31) && per_plane + b.group < (1LL << 31);  // 32-bit counters in the kernel
        if (!fits && h_chunk < 0) {
            set_error("dwconv_wgrad: too many plane steps for the balanced split");
            return KEROPS_E_BADARG;
        }
        if (fits) {
            p->bal_group = b.group;
            p->bal_q = (uint32_t)(b.units / b.ngroups);
            p->bal_r = (uint32_t)(b.units % b.ngroups);
            p->n_tiles = (uint32_t)per_plane;
            p->h_chunk = H;
            p->n_hc = 1;
            p->nblocks = (int64_t)b.group * b.ngroups;
            return KEROPS_OK;
        }
    }
    if (h_chunk <= 0) h_chunk = pick_h_chunk(H, per_plane, slots, 8);
    p->h_chunk = std::min(h_chunk, H);
    p->n_hc = ceil_div(H, p->h_chunk);
    p->nblocks = (int64_t)N * p->n_hc * p->n_wt * p->n_dt * p->n_slab;
    if (p->nblocks > 0x7fffff00LL) {
        set_error("dwconv_wgrad: too many workgroups (%lld)", (long long)p->nblocks);
        return KEROPS_E_BADARG;
    }
    return KEROPS_OK;
}

// per-workgroup partials
static int64_t wgrad_ws_bytes(const WgPlan& p)
{
    const int64_t sc = p.cg * 8;
    return p.nblocks * 27 * sc * (int64_t)sizeof(float);
}

// the two reduction kernels over the per-workgroup partials [nblocks][27][SC] at the start of ws
// where the reduced gradient goes: an fp32 [27][C] array, or an fp16 one (KEROPS_DTYPE_F16)
struct GwOut {
    void* p;
    int dtype;
    GwOut(float* f) : p(f), dtype(KEROPS_DTYPE_F32) {}
    GwOut(void* q, int dt) : p(q), dtype(dt) {}
};

static int reduce_partials(float* ws, const WgPlan& p, int SC, int C, GwOut gw, hipStream_t stream)
{
    const int n_rows = (int)(p.nblocks / p.n_slab);
    const int RW = p.n_slab * 27 * SC;
    if (gw.dtype == KEROPS_DTYPE_F16)
        hipLaunchKernelGGL(wgrad_reduce_kernel<half_t>, dim3(ceil_div(RW, 16)), dim3(1024), 0, stream, ws, (half_t*)gw.p,
                           n_rows, RW, SC, C);
    else
        hipLaunchKernelGGL(wgrad_reduce_kernel<float>, dim3(ceil_div(RW, 16)), dim3(1024), 0, stream, ws, (float*)gw.p,
                           n_rows, RW, SC, C);
    return check_launch("dwconv_wgrad_reduce");
}

static int check_gw_dtype(const char* op, int32_t gw_dtype)
{
    if (gw_dtype == KEROPS_DTYPE_F32 || gw_dtype == KEROPS_DTYPE_F16) return KEROPS_OK;
    set_error("%s: gw_dtype must be KEROPS_DTYPE_F32 or KEROPS_DTYPE_F16", op);
    return KEROPS_E_BADARG;
}

template <class Cfg, class KernelT>
static int launch_wgrad_cfg(KernelT kernel, const WgArgs& base, const WgPlan& p, GwOut gw, hipStream_t stream)
{
    WgArgs a = base;
    a.n_wt = p.n_wt;
    a.n_dt = p.n_dt;
    a.n_hc = p.n_hc;
    a.n_slab = p.n_slab;
    a.h_chunk = p.h_chunk;
    a.nblocks = (uint32_t)p.nblocks;
    a.bal_group = p.bal_group;
    a.bal_q = p.bal_q;
    a.bal_r = p.bal_r;
    a.n_tiles = p.n_tiles;
    a.n_xcd = (uint32_t)p.n_xcd;
    hipLaunchKernelGGL(kernel, dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, stream, a);
    int rc = check_launch("dwconv_wgrad");
    if (rc != KEROPS_OK) return rc;
    return reduce_partials(a.ws, p, Cfg::SC, a.C, gw, stream);
}

template <int CG, int TW, int TD, int NT>
static int launch_wgrad(const WgArgs& base, const WgPlan& p, GwOut gw, hipStream_t stream)
{
    using Cfg = WgCfg<CG, TW, TD, NT>;
    return launch_wgrad_cfg<Cfg>(dwconv_wgrad_kernel<Cfg>, base, p, gw, stream);
}

template <int CG, int TW, int TD, int NT>
static int launch_wgrad_mfma(const WgArgs& base, const WgPlan& p, GwOut gw, hipStream_t stream)
{
    using Cfg = WmCfg<CG, TW, TD, NT>;
    if (base.stream_interior) return launch_wgrad_cfg<Cfg>(dwconv_wgrad_mfma_kernel<Cfg, true>, base, p, gw, stream);
    return launch_wgrad_cfg<Cfg>(dwconv_wgrad_mfma_kernel<Cfg, false>, base, p, gw, stream);
}

// fused backward: one patch shape per channel count, two workgroups of 512 threads per CU
// KEROPS_BWD_STAGING=registers selects the register-staged kernel (kept as a tested alternative) instead of the
// LDS-direct one; the two use different patch shapes, so the choice is part of the plan
static bool bwd_staged_in_registers()
{
    static const bool v = [] {
        const char* e = getenv("KEROPS_BWD_STAGING");
        return e && e[0] == 'r';
    }();
    return v;
}

static int plan_bwd(int N, int H, int W, int D, int C, int h_chunk, WgPlan* p)
{
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwconv_bwd: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if (!(C == 8 || C == 16 || C == 32 || C == 64 || C == 128)) {
        set_error("dwconv_bwd: unsupported channel count %d", C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    if (plane_exceeds_i32(W, D, C)) {
        set_error("dwconv_bwd: one (W,D,C) plane must stay below 2^31 elements");
        return KEROPS_E_BADARG;
    }
    p->cg = C >= 64 ? 8 : C / 8;
    p->cl = 16;
    if (bwd_staged_in_registers()) {
        p->tile_w = p->cg == 8 ? 4 : 8;
        p->tile_d = p->cg >= 4 ? 8 : p->cg == 2 ? 16 : 32;
    } else {  // patches of 512 16-byte chunks: a wavefront of either role owns four rows
        p->tile_w = 8;
        p->tile_d = 64 / p->cg;
    }
    p->n_slab = C / (p->cg * 8);
    p->n_wt = ceil_div(W, p->tile_w);
    p->n_dt = ceil_div(D, p->tile_d);
    const int64_t per_plane = (int64_t)N * p->n_wt * p->n_dt * p->n_slab;
    const DeviceGeometry geo = device_geometry();
    p->n_xcd = geo.xcds;
    const int slots = geo.resident_workgroups(512);  // two workgroups of 512 threads per compute unit
    p->bal_group = 0;
    // h_chunk 0: balanced split with the group size of the cost model (-g: groups of g workgroups); > 0: uniform
    // chunks of that many rows
    if (h_chunk <= 0) {
        if (h_chunk < 0 && (-h_chunk) % p->n_slab != 0) {
            set_error("dwconv_bwd: the group size of the balanced split must be a multiple of the slab count %d",
                      p->n_slab);
            return KEROPS_E_BADARG;
        }
        const BalancedSplit b = h_chunk < 0 ? make_balanced(H, per_plane, slots, -h_chunk)
                                            : pick_balanced(H, per_plane, p->n_dt * p->n_slab, slots, 8, p->n_slab,
                                                            geo.xcds);
        const bool fits = b.units < (1LL << 31) && per_plane + b.group < (1LL << 31);  // 32-bit counters in the kernel
        if (!fits && h_chunk < 0) {
            set_error("dwconv_bwd: too many plane steps for the balanced split");
            return KEROPS_E_BADARG;
        }
        if (fits) {
            p->bal_group = b.group;
            p->bal_q = (uint32_t)(b.units / b.ngroups);
            p->bal_r = (uint32_t)(b.units % b.ngroups);
            p->n_tiles = (uint32_t)per_plane;
            p->h_chunk = H;
            p->n_hc = 1;
            p->nblocks = (int64_t)b.group * b.ngroups;
            return KEROPS_OK;
        }
        h_chunk = pick_h_chunk(H, per_plane, slots, 8);
    }
    p->h_chunk = std::min(h_chunk, H);
    p->n_hc = ceil_div(H, p->h_chunk);
    p->nblocks = (int64_t)N * p->n_hc * p->n_wt * p->n_dt * p->n_slab;
    if (p->nblocks > 0x7fffff00LL) {
        set_error("dwconv_bwd: too many workgroups (%lld)", (long long)p->nblocks);
        return KEROPS_E_BADARG;
    }
    return KEROPS_OK;
}

}  // namespace kerops

using namespace kerops;

extern "C" int64_t kerops_dwconv_bwd_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                                     int32_t h_chunk)
{
    WgPlan p;
    int rc = plan_bwd(N, H, W, D, C, h_chunk, &p);
    if (rc != KEROPS_OK) return rc;
    return wgrad_ws_bytes(p);
}

extern "C" int kerops_dwconv_bwd_f16(const void* x, const void* g, const void* wt, void* dx, float* gw,
                                     void* workspace, int64_t workspace_bytes, int32_t N, int32_t H, int32_t W,
                                     int32_t D, int32_t C, int32_t h_chunk, void* stream)
{
    return kerops_dwconv_bwd_f16_out(x, g, wt, dx, gw, KEROPS_DTYPE_F32, workspace, workspace_bytes, N, H, W, D, C,
                                     h_chunk, stream);
}

extern "C" int kerops_dwconv_bwd_f16_out(const void* x, const void* g, const void* wt, void* dx, void* gw_out,
                                         int32_t gw_dtype, void* workspace, int64_t workspace_bytes, int32_t N,
                                         int32_t H, int32_t W, int32_t D, int32_t C, int32_t h_chunk, void* stream)
{
    if (check_gw_dtype("dwconv_bwd", gw_dtype) != KEROPS_OK) return KEROPS_E_BADARG;
    const GwOut gw(gw_out, gw_dtype);
    if (!x || !g || !wt || !dx || !gw_out || !aligned16(x) || !aligned16(g) || !aligned16(wt) || !aligned16(dx) ||
        !aligned16(gw_out)) {
        set_error("dwconv_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    WgPlan p;
    int rc = plan_bwd(N, H, W, D, C, h_chunk, &p);
    if (rc != KEROPS_OK) return rc;
    const int64_t need = wgrad_ws_bytes(p);
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("dwconv_bwd: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    WgArgs a{};
    a.x = (const half_t*)x;
    a.g = (const half_t*)g;
    a.wt = (const half_t*)wt;
    a.dx = (half_t*)dx;
    a.ws = (float*)workspace;
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    a.stream_interior = (int64_t)N * H * W * D * C * 2 >= kStreamInteriorMinBytes;
    hipStream_t s = (hipStream_t)stream;
    WgArgs b = a;
    b.n_wt = p.n_wt;
    b.n_dt = p.n_dt;
    b.n_hc = p.n_hc;
    b.n_slab = p.n_slab;
    b.h_chunk = p.h_chunk;
    b.nblocks = (uint32_t)p.nblocks;
    b.bal_group = p.bal_group;
    b.bal_q = p.bal_q;
    b.bal_r = p.bal_r;
    b.n_tiles = p.n_tiles;
    b.n_xcd = (uint32_t)p.n_xcd;
    if (!bwd_staged_in_registers() && launch_bwd_dma(b, p.cg, p.tile_w, p.tile_d, s) == 0) {
        rc = check_launch("dwconv_bwd");
        if (rc != KEROPS_OK) return rc;
        return reduce_partials(b.ws, p, p.cg * 8, b.C, gw, s);
    }
#define KEROPS_BS_GO(CGv, TWv, TDv)                                                                                  \
    {                                                                                                                \
        using Cfg = BsCfg<CGv, TWv, TDv, 512>;                                                                       \
        hipLaunchKernelGGL(dwconv_bwd_split_kernel<Cfg>, dim3(xcd_padded_grid(b.nblocks, b.n_xcd)), dim3(Cfg::NT), 0, s, b); \
    }
    switch (p.cg) {
        case 1: KEROPS_BS_GO(1, 8, 32) break;
        case 2: KEROPS_BS_GO(2, 8, 16) break;
        case 4: KEROPS_BS_GO(4, 8, 8) break;
        default: KEROPS_BS_GO(8, 4, 8) break;
    }
#undef KEROPS_BS_GO
    rc = check_launch("dwconv_bwd");
    if (rc != KEROPS_OK) return rc;
    return reduce_partials(b.ws, p, p.cg * 8, b.C, gw, s);
}

extern "C" int64_t kerops_dwconv_wgrad_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                                       int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                                                       int32_t lane_channels)
{
    WgPlan p;
    int rc = plan_wgrad(N, H, W, D, C, tile_w, tile_d, h_chunk, lane_channels, &p);
    if (rc != KEROPS_OK) return rc;
    return wgrad_ws_bytes(p);
}

extern "C" int kerops_dwconv_wgrad_f16(const void* x, const void* g, float* gw, void* workspace,
                                       int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                       int32_t tile_w, int32_t tile_d, int32_t h_chunk, int32_t lane_channels,
                                       void* stream)
{
    return kerops_dwconv_wgrad_f16_out(x, g, gw, KEROPS_DTYPE_F32, workspace, workspace_bytes, N, H, W, D, C, tile_w,
                                       tile_d, h_chunk, lane_channels, stream);
}

extern "C" int kerops_dwconv_wgrad_f16_out(const void* x, const void* g, void* gw_out, int32_t gw_dtype,
                                           void* workspace, int64_t workspace_bytes, int32_t N, int32_t H, int32_t W,
                                           int32_t D, int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                                           int32_t lane_channels, void* stream)
{
    if (check_gw_dtype("dwconv_wgrad", gw_dtype) != KEROPS_OK) return KEROPS_E_BADARG;
    const GwOut gw(gw_out, gw_dtype);
    if (!x || !g || !gw_out || !aligned16(x) || !aligned16(g) || !aligned16(gw_out)) {
        set_error("dwconv_wgrad: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    WgPlan p;
    int rc = plan_wgrad(N, H, W, D, C, tile_w, tile_d, h_chunk, lane_channels, &p);
    if (rc != KEROPS_OK) return rc;
    const int64_t need = wgrad_ws_bytes(p);
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("dwconv_wgrad: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    WgArgs a{};
    a.x = (const half_t*)x;
    a.g = (const half_t*)g;
    a.ws = (float*)workspace;
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    a.stream_interior = (int64_t)N * H * W * D * C * 2 >= kStreamInteriorMinBytes;
    hipStream_t s = (hipStream_t)stream;
    // (channel groups of 8, patch W, patch D, threads)
#define KEROPS_WG_CASE(CGv, TWv, TDv, NTv)                                 \
    if (p.cg == CGv && p.tile_w == TWv && p.tile_d == TDv && p.cl == 2) \
        return launch_wgrad<CGv, TWv, TDv, NTv>(a, p, gw, s);
    KEROPS_WG_CASE(1, 16, 32, 256)
    KEROPS_WG_CASE(1, 8, 32, 256)
    KEROPS_WG_CASE(2, 8, 32, 256)
    KEROPS_WG_CASE(2, 8, 16, 256)
    KEROPS_WG_CASE(4, 8, 16, 256)
    KEROPS_WG_CASE(4, 4, 16, 256)
    KEROPS_WG_CASE(8, 8, 8, 512)
    KEROPS_WG_CASE(8, 4, 16, 256)
    KEROPS_WG_CASE(8, 4, 8, 256)
#undef KEROPS_WG_CASE
    // matrix-core kernels: (channel groups of 8, patch W, patch D, threads)
#define KEROPS_WM_CASE(CGv, TWv, TDv, NTv)                                   \
    if (p.cg == CGv && p.tile_w == TWv && p.tile_d == TDv && p.cl == 16) \
        return launch_wgrad_mfma<CGv, TWv, TDv, NTv>(a, p, gw, s);
    KEROPS_WM_CASE(1, 8, 32, 256)
    KEROPS_WM_CASE(2, 8, 16, 256)
    KEROPS_WM_CASE(4, 4, 16, 256)
    KEROPS_WM_CASE(1, 8, 64, 512)
    KEROPS_WM_CASE(2, 8, 32, 512)
    KEROPS_WM_CASE(4, 8, 16, 512)
    KEROPS_WM_CASE(8, 4, 8, 256)
    KEROPS_WM_CASE(8, 8, 8, 512)
    KEROPS_WM_CASE(8, 4, 16, 512)
#undef KEROPS_WM_CASE
    // LDS-direct matrix-core kernels: lane_channels 32 (built-in planes ahead), 33 / 34 / 35 = (1,1) / (2,2) / (1,2)
    if (p.cl >= 32 && p.cl <= 35) {
        WgArgs b = a;
        b.n_wt = p.n_wt;
        b.n_dt = p.n_dt;
        b.n_hc = p.n_hc;
        b.n_slab = p.n_slab;
        b.h_chunk = p.h_chunk;
        b.nblocks = (uint32_t)p.nblocks;
        b.bal_group = p.bal_group;
        b.bal_q = p.bal_q;
        b.bal_r = p.bal_r;
        b.n_tiles = p.n_tiles;
        b.n_xcd = (uint32_t)p.n_xcd;
        const int depth = p.cl == 32 ? 0 : p.cl == 33 ? 11 : p.cl == 34 ? 22 : 12;
        if (launch_wgrad_dma(b, p.cg, p.tile_w, p.tile_d, depth, s) == 0) {
            rc = check_launch("dwconv_wgrad");
            if (rc != KEROPS_OK) return rc;
            return reduce_partials(b.ws, p, p.cg * 8, b.C, gw, s);
        }
    }
    set_error("dwconv_wgrad: no kernel built for C=%d tile_w=%d tile_d=%d lane_channels=%d", C, p.tile_w, p.tile_d,
              p.cl);
    return KEROPS_E_BADARG;
}
