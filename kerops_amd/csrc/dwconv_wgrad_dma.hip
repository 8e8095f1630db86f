// Depthwise 3x3x3 weight gradient, matrix-core kernel with LDS-direct staging (gfx950).
//
// This file is compiled without the load/store optimizer (see kerops_amd/build.py): that pass fuses pairs of
// 8-byte LDS reads into ds_read2_b64, which gfx950 executes in 8 clocks or more (16 with the operand patterns
// below) where two ds_read_b64 take 2.4 each.
#include "dwconv_wgrad.hpp"
// Measurement switches (both 1 in the library): -DKEROPS_WD_COMPUTE=0 builds the kernel without its arithmetic (the
// time of its memory traffic alone, 0.588 ms at (1,64,350,350,128)), -DKEROPS_WD_LOADS=0 without the plane loads of
// the march (the time of its LDS reads and matrix instructions alone, 0.406 ms); neither variant computes the result.
#ifndef KEROPS_WD_COMPUTE
#define KEROPS_WD_COMPUTE 1
#endif
#ifndef KEROPS_WD_LOADS
#define KEROPS_WD_LOADS 1
#endif

namespace kerops {

// Matrix-core weight gradient with LDS-direct staging (lane_channels = 32).
//
// Same product scheme as dwconv_wgrad_mfma_kernel.  Two things differ:
//
//  * Operand reads are 8 bytes wide (4 channels per lane and position).  An LDS read instruction of a wavefront
//    costs the same issue slots for 4 and for 8 bytes per lane (measured on gfx950: 2.4 clocks per ds_read_b32 and
//    per ds_read_b64, 4.6 per ds_read_b128; addresses that are not multiples of the access width take 64), so the
//    8-byte form fetches the operands of twice as many channels per slot; a wavefront then covers all 64
//    channels of a slab and owns two g rows of the patch instead of four.
//  * Planes go from global memory straight into LDS (global_load_lds_dwordx4): no staging registers, no LDS store
//    instructions, and the planes in flight are limited by LDS space instead of registers.  One such instruction
//    of a wavefront writes 1024 consecutive bytes of LDS, lane l the 16 bytes at M0 + 16*l, so the layout is
//    expressed by the choice of the global chunk each lane asks for: a block of 1024 bytes holds 1024/PB
//    consecutive positions of the staged plane, and inside a position the chunk slots are rotated as the operand
//    reads want them.  Lanes whose position lies outside the volume (or in the padding of the last block) are
//    switched off in EXEC for the instruction: their LDS bytes keep the zeros written once per segment.
//    The compiler does not know these loads (they are inline assembly, so its own wait-count bookkeeping neither
//    sees nor delays them); the waits are placed by hand: every wavefront issues the same number of loads per step,
//    in the same order, and `s_waitcnt vmcnt(n)` before the step's barrier leaves exactly the loads of later steps
//    in flight.  The kernel uses M0 for nothing else.
//
// Ring of AX + 1 x slots and AG + 3 g slots: step hp reads x plane hp and g planes hp - 1, hp, hp + 1, while x
// plane hp + AX and g plane hp + 1 + AG are on their way.  g planes outside the chunk are zeroed at the consumer
// (byte selectors of the operand split), so every step loads real planes (indices clamped into the volume).
template <int CG_, int TW_, int TD_, int NT_, int AX_, int AG_>
struct WdCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_, NWAVE = NT_ / 64, AX = AX_, AG = AG_;
    static constexpr int CPL = 4;
    static constexpr int SC = CG * 8, PB = SC * 2;
    static constexpr int NQ = SC / CPL >= 16 ? 16 : SC / CPL, NSUB = 16 / NQ, NHALF = SC / (CPL * NQ);
    static constexpr int NPART = NWAVE / NHALF, GD = TD / (4 * NSUB), RSPLIT = NPART / GD, RG = TW / RSPLIT;
    static constexpr int R = TW + 2, PDP = TD + 2;   // staged x rows and positions per row (dense)
    static constexpr int PPB = 1024 / PB;            // positions per block = per load instruction of a wavefront
    static constexpr int NXB = (R * PDP + PPB - 1) / PPB, NGB = (TW * TD + PPB - 1) / PPB;
    static constexpr int NXI = (NXB + NWAVE - 1) / NWAVE, NGI = (NGB + NWAVE - 1) / NWAVE;  // loads per wavefront
    static constexpr int NXS = AX + 1, NGS = AG + 3;
    static constexpr int XSLOT = NXB * 1024;
    static constexpr int GPAD = PB >= 64 ? 64 : PB;  // lanes j read different slots: shift their banks apart
    static constexpr int GSLOT = NGB * 1024 + GPAD;
    static constexpr int XOFF = NGS * GSLOT;
    static constexpr int STAGE_BYTES = XOFF + NXS * XSLOT;
    static constexpr int RED_BYTES = NPART * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    // loads that may stay in flight at a step's wait: those of later steps.  Issue order inside a step: x, then g;
    // with the streaming split every x block takes two instructions.
    template <bool NTI>
    static constexpr int inflight()
    {
        constexpr int per_step = (NTI ? 2 : 1) * NXI + NGI;
        return AX == AG ? (AX - 1) * per_step : (AX - 1) * per_step + NGI;
    }
    static_assert(AX == AG || (AX == 1 && AG == 2), "planes ahead: (1,1), (2,2) or x 1 / g 2");
    static_assert(TD % (4 * NSUB) == 0 && NPART % GD == 0 && NPART >= GD && TW % RSPLIT == 0, "even split");
    static_assert(1024 % PB == 0 && STAGE_BYTES % 16 == 0 && GSLOT % 16 == 0, "whole positions per block");
    // half a wavefront reads 64 bytes at each of three consecutive positions of a row: at 64 channels positions are
    // 128 bytes apart, so every second pair of positions has its chunk slots rotated by 64 bytes (d, d + 1, d + 2
    // then fall into disjoint quarters of the 256 bytes of banks); narrower slabs need none
    __device__ static constexpr int rot(int dq) { return PB == 128 ? 64 * ((dq >> 1) & 1) : 0; }
};

// NTI: the x chunks that no other workgroup reads (the patch without its border ring) are loaded by instructions
// of their own that carry the streaming hint, so that they do not push the shared halo lines out of the L2; a
// compile-time choice made on the host by tensor size (streaming loads bypass the memory-side cache as well)
template <class Cfg, bool NTI>
__global__ __launch_bounds__(Cfg::NT, 4) void dwconv_wgrad_dma_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, TW = Cfg::TW, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RG = Cfg::RG, XSLOT = Cfg::XSLOT, GSLOT = Cfg::GSLOT, CPL = Cfg::CPL;
    constexpr int NXI = Cfg::NXI, NGI = Cfg::NGI, NXS = Cfg::NXS, NGS = Cfg::NGS, AX = Cfg::AX, AG = Cfg::AG;
    constexpr int NWAVE = Cfg::NWAVE, PPB = Cfg::PPB;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(void __attribute__((address_space(3)))*)smem;

    const uint32_t ws_slot = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (ws_slot >= a.nblocks) return;
    const int H = a.H, W = a.W, D = a.D, C = a.C;

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int half = wave % Cfg::NHALF, part = wave / Cfg::NHALF;
    const int gd = part % Cfg::GD, ra = (part / Cfg::GD) * RG;  // this wavefront: position group, first g row
    const int b = lane / 4, rr = lane % 4;
    const int q = b % NQ, sub = b / NQ;
    const int r2 = min(rr, 2);  // index 3 repeats index 2; its operands are zeroed by the selectors, its results unused
    const uint32_t sel_e = rr < 3 ? 0x05040100u : 0x0c0c0c0cu, sel_o = rr < 3 ? 0x07060302u : 0x0c0c0c0cu;
    const int cb = (half * NQ + q) * (CPL * 2);
    const int pgrp = (gd * NSUB + sub) * 4;  // first position of the lane's group inside a patch row
    int aoff[4], boff[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int dx = pgrp + r2 + k, dg = pgrp + k;  // position inside the staged x row / the g row
        aoff[k] = Cfg::XOFF + (ra * PDP + dx) * PB + ((cb + Cfg::rot(dx)) & (PB - 1));
        boff[k] = (ra * TD + dg) * PB + ((cb + Cfg::rot(dg)) & (PB - 1));
    }

    float4_t acc[3][CPL];
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
        for (int e = 0; e < CPL; ++e) acc[kw][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    auto gather = [&](const unsigned char* base, const int (&off)[4], uint32_t se, uint32_t so, half4_t(&dst)[CPL]) {
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const u32x2_t r = *reinterpret_cast<const u32x2_t*>(base + off[k]);
            lo[k] = r[0];
            hi[k] = r[1];
        }
        split_operands_sel(lo, se, so, dst[0], dst[1]);
        split_operands_sel(hi, se, so, dst[2], dst[3]);
    };

    const bool balanced = a.bal_group > 0;
    uint32_t u = 0, u_end = 0, member = 0;
    uint32_t ws_row = ws_slot;
    if (balanced) {
        const uint32_t group = ws_slot / a.bal_group;
        member = ws_slot - group * a.bal_group;
        u = __builtin_amdgcn_readfirstlane(group * a.bal_q + min(group, a.bal_r));
        u_end = __builtin_amdgcn_readfirstlane(u + a.bal_q + (group < a.bal_r ? 1u : 0u));
        if (a.n_slab == 2 && a.bal_group % 2 == 0) {
            const uint32_t halfg = a.bal_group / 2;
            member = (member % halfg) * 2 + member / halfg;
            ws_row = group * a.bal_group + member;
        }
    }
    for (bool first = true;; first = false) {
        uint32_t L;
        int hs, he;
        if (balanced) {
            if (u >= u_end) break;
            const uint32_t bundle = u / (uint32_t)H;
            hs = __builtin_amdgcn_readfirstlane((int)(u - bundle * (uint32_t)H));
            he = (int)min((uint32_t)H, hs + (u_end - u));
            u += he - hs;
            L = __builtin_amdgcn_readfirstlane(bundle * a.bal_group + member);
            if (L >= a.n_tiles) continue;  // a partly filled last bundle
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
        const int w0 = wt_i * TW, d0 = dt * TD;
        const int cslab = slab * SC;
        const int64_t plane_stride = (int64_t)W * D * C;
        const char* xn = reinterpret_cast<const char*>(a.x + (int64_t)n * H * plane_stride);
        const char* gn = reinterpret_cast<const char*>(a.g + (int64_t)n * H * plane_stride);

        // every load of the previous segment has landed and every wavefront has read its last plane
        wait_loads_in_flight<0>();
        __syncthreads();
        // positions outside the volume are never loaded: they read as the zeros written here
        {
            const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int o = threadIdx.x * 16; o < Cfg::STAGE_BYTES; o += NT * 16) *reinterpret_cast<half8_t*>(smem + o) = z8;
        }
        // this lane's chunk in each block its wavefront loads: lane l fills chunk slot l % CG of position
        // (block * PPB + l / CG); the global chunk is the one that the rotation puts into that slot
        uint32_t xvo[NXI], gvo[NGI];
        uint64_t xmask[NXI], xmask_in[NXI], gmask[NGI];
        uint32_t xlds[NXI], glds[NGI];
#pragma unroll
        for (int i = 0; i < NXI; ++i) {
            const int blk = wave + i * NWAVE;
            const int P = blk * PPB + lane / CG, cs = lane % CG;
            const int wq = P / PDP, dq = P - wq * PDP;
            const int w = w0 - 1 + wq, d = d0 - 1 + dq;
            const bool ok = (blk < Cfg::NXB) && (wq < Cfg::R) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
            const int cbyte = (cs * 16 - Cfg::rot(dq)) & (PB - 1);
            xvo[i] = ok ? (uint32_t)(((w * D + d) * C + cslab) * 2 + cbyte) : 0u;
            const bool interior = NTI && (wq >= 2) && (wq <= TW - 1) && (dq >= 2) && (dq <= TD - 1);
            xmask[i] = __ballot(ok && !interior);
            xmask_in[i] = __ballot(ok && interior);
            xlds[i] = lds0 + Cfg::XOFF + (blk < Cfg::NXB ? blk : 0) * 1024;
        }
#pragma unroll
        for (int i = 0; i < NGI; ++i) {
            const int blk = wave + i * NWAVE;
            const int P = blk * PPB + lane / CG, cs = lane % CG;
            const int wq = P / TD, dq = P - wq * TD;
            const int w = w0 + wq, d = d0 + dq;
            const bool ok = (blk < Cfg::NGB) && (wq < TW) && (w < W) && (d < D);
            const int cbyte = (cs * 16 - Cfg::rot(dq)) & (PB - 1);
            gvo[i] = ok ? (uint32_t)(((w * D + d) * C + cslab) * 2 + cbyte) : 0u;
            gmask[i] = __ballot(ok);
            glds[i] = lds0 + (blk < Cfg::NGB ? blk : 0) * 1024;
        }
        auto load_x = [&](int hp, int slot) {  // x plane hp (clamped into the volume) into x slot `slot`
            const char* plane = uniform_ptr(xn + (int64_t)min(max(hp, 0), H - 1) * plane_stride * 2);
#pragma unroll
            for (int i = 0; i < NXI; ++i) {
                lds_direct_load16<false>(plane, xvo[i], xlds[i] + slot * XSLOT, xmask[i]);
                if (NTI) lds_direct_load16<true>(plane, xvo[i], xlds[i] + slot * XSLOT, xmask_in[i]);
            }
        };
        auto load_g = [&](int hp, int slot) {  // g is read exactly once: streaming hint
            const char* plane = uniform_ptr(gn + (int64_t)min(max(hp, 0), H - 1) * plane_stride * 2);
#pragma unroll
            for (int i = 0; i < NGI; ++i) lds_direct_load16<true>(plane, gvo[i], glds[i] + slot * GSLOT, gmask[i]);
        };
        __syncthreads();  // the zero fill is complete before any load writes LDS

        // ring positions: x plane hp lives in slot xs, g plane hp + 1 in slot gs (both advance by one per step)
        int xs = 0, gs = 1;
        // pipeline fill, in the order the steps would have issued them (see inflight())
        if (AX == AG) {
#pragma unroll
            for (int i = 0; i < AX; ++i) {
                load_x(hs - 1 + i, i % NXS);
                load_g(hs + i, (1 + i) % NGS);
            }
        } else {
            load_x(hs - 1, 0);
            load_g(hs, 1);
            load_g(hs + 1, 2);
        }
        int xs_load = AX % NXS, gs_load = (1 + AG) % NGS;  // slots of the planes loaded by the next step
        // lane j reads the g slot of plane hp + 1 - j: its slot index runs one step behind lane j - 1's
        int gslot_lane = (1 + NGS - r2) % NGS;
        for (int hp = hs - 1; hp <= he; ++hp) {
            wait_loads_in_flight<KEROPS_WD_LOADS ? Cfg::template inflight<NTI>() : 0>();
            __syncthreads();
            if (KEROPS_WD_LOADS) {
                load_x(hp + AX, xs_load);
                load_g(hp + 1 + AG, gs_load);
            }
            xs_load = xs_load + 1 == NXS ? 0 : xs_load + 1;
            gs_load = gs_load + 1 == NGS ? 0 : gs_load + 1;
            if (KEROPS_WD_COMPUTE && hp >= 0 && hp < H) {  // wavefront-uniform
                const unsigned char* xbase = smem + xs * XSLOT;
                const unsigned char* gbase = smem + gslot_lane * GSLOT;
                // g planes outside the chunk belong to other segments: zero operands
                const int pj = hp + 1 - r2;
                const bool gok = (pj >= hs) && (pj < he);
                const uint32_t gsel_e = gok ? sel_e : 0x0c0c0c0cu, gsel_o = gok ? sel_o : 0x0c0c0c0cu;
                half4_t G[RG][CPL];
#pragma unroll
                for (int xr = 0; xr < RG + 2; ++xr) {
                    if (xr < RG) gather(gbase + xr * TD * PB, boff, gsel_e, gsel_o, G[xr]);
                    half4_t A[CPL];
                    gather(xbase + xr * PDP * PB, aoff, sel_e, sel_o, A);
#pragma unroll
                    for (int kw = 0; kw < 3; ++kw) {
                        // x patch row ra-1+xr meets g row ra+xr-kw at tap kw
                        if (xr - kw >= 0 && xr - kw < RG) {
#pragma unroll
                            for (int e = 0; e < CPL; ++e)
                                acc[kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(A[e], G[xr - kw][e], acc[kw][e], 0, 0, 0);
                        }
                    }
                }
            }
            xs = xs + 1 == NXS ? 0 : xs + 1;
            gslot_lane = gslot_lane + 1 == NGS ? 0 : gslot_lane + 1;
        }
    }  // segments
    wait_loads_in_flight<0>();

    const int t = threadIdx.x;
    // ---- combine: position groups inside a wavefront, then the wavefronts of a half via LDS ----
    if (NSUB > 1) {
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int e = 0; e < CPL; ++e)
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
            for (int e = 0; e < CPL; ++e)
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    red[(part * 27 + (rr * 3 + kw) * 3 + i) * SC + (half * NQ + q) * CPL + e] = acc[kw][e][i];
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


namespace {
template <int CG, int TW, int TD, int NT, int AX, int AG>
void launch_shape(const WgArgs& a, hipStream_t stream)
{
    using Cfg = WdCfg<CG, TW, TD, NT, AX, AG>;
    const dim3 grid(xcd_padded_grid(a.nblocks, a.n_xcd)), block(Cfg::NT);
    if (a.stream_interior)
        hipLaunchKernelGGL((dwconv_wgrad_dma_kernel<Cfg, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((dwconv_wgrad_dma_kernel<Cfg, false>), grid, block, 0, stream, a);
}
template <int CG, int TW, int TD, int NT>
void launch_depth(const WgArgs& a, int depth, hipStream_t stream)
{
    // measured at (1, C, 350, 350, 128), C = 8..128: one plane of each ahead is as fast as or faster than the deeper
    // rings (more planes in flight cost L2 space that the shared halo lines need; five g slots cannot be kept
    // in disjoint banks for every three consecutive ones)
    if (depth == 22)
        launch_shape<CG, TW, TD, NT, 2, 2>(a, stream);
    else if (depth == 12)
        launch_shape<CG, TW, TD, NT, 1, 2>(a, stream);
    else
        launch_shape<CG, TW, TD, NT, 1, 1>(a, stream);  // the built-in choice
}
}  // namespace

int launch_wgrad_dma(const WgArgs& a, int cg, int tile_w, int tile_d, int depth, hipStream_t stream)
{
#define KEROPS_WD_CASE(CGv, TWv, TDv, NTv)                    \
    if (cg == CGv && tile_w == TWv && tile_d == TDv) {        \
        launch_depth<CGv, TWv, TDv, NTv>(a, depth, stream);   \
        return 0;                                             \
    }
    // 8-row patches on four wavefronts: each owns four g rows and gathers six x rows for them (ten operand
    // gathers per 48 matrix instructions; eight wavefronts with two rows each need six per 24), measured 3-8 %
    // faster at every channel count although half as many wavefronts are resident
    KEROPS_WD_CASE(8, 8, 8, 256)
    KEROPS_WD_CASE(4, 8, 16, 256)
    KEROPS_WD_CASE(2, 8, 32, 256)
    KEROPS_WD_CASE(1, 8, 64, 256)
    KEROPS_WD_CASE(8, 4, 8, 256)
    KEROPS_WD_CASE(4, 4, 16, 256)
    KEROPS_WD_CASE(2, 4, 32, 256)
    KEROPS_WD_CASE(1, 4, 64, 256)
#undef KEROPS_WD_CASE
    return 1;
}

}  // namespace kerops
