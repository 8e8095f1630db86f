// Fused backward of the depthwise 3x3x3 convolution with LDS-direct staging (gfx950): input gradient and weight
// gradient in one pass over x and g.
//
//   dx[n,h,w,d,c] = sum_{kh,kw,kd} g[n,h-kh+1,w-kw+1,d-kd+1,c] * wt[kh,kw,kd,c]   (= DWConv(g, wt flipped))
//   gw[kh,kw,kd,c] = sum x[n,h+kh-1,w,d,c] * g[n,h,w-kw+1,d-kd+1,c]               (summed over the positions of x)
//
// The scheme is that of dwconv_bwd_split_kernel (dwconv_wgrad.hip): a workgroup owns a patch, every plane of g is
// staged once with its halo, every plane of x without one; the first half of its wavefronts runs the input-gradient
// product (weights as the A operand, a ring of four accumulator registers per tile), the second half the weight
// gradient on the same LDS planes, each role in its own loop with the same sequence of workgroup barriers.
// What differs:
//
//  * planes go from global memory straight into LDS (global_load_lds_dwordx4, see common.hpp): no staging registers,
//    no LDS store instructions; lanes whose position lies outside the volume are switched off for the instruction
//    and their LDS bytes keep the zeros written once per segment;
//  * operand reads are 8 bytes wide (4 channels per lane and position: the LDS read path moves twice the bytes per
//    issue slot), so a wavefront covers every channel of the slab;
//  * a wavefront that covers the whole slab writes whole 128-byte lines when every lane stores its 8 bytes of dx
//    directly, so there is no output tile in LDS: the dx planes leave through hand-issued streaming stores, which are
//    counted by the hand-placed waits like the loads.
//
// Rings: g planes p - 1, p, p + 1 (three slots: the input-gradient role reads plane p, the weight-gradient role plane
// p - 1, plane p + 1 is on its way), x planes p - 2 .. p + 1 (four slots).
//
// This file is compiled without the load/store optimizer (see kerops_amd/build.py): that pass fuses pairs of
// 8-byte LDS reads into ds_read2_b64, which gfx950 executes at a fraction of the rate of two ds_read_b64.
#include "dwconv_wgrad.hpp"

namespace kerops {

template <int CG_, int TW_, int TD_>
struct BdCfg {
    // two wavefronts per role: each covers every row of an 8-row patch (ten operand gathers per 96 matrix
    // instructions), measured 2-15 % faster than four per role with half the rows each
    static constexpr int CG = CG_, TW = TW_, TD = TD_, RWAVES = 2, NWAVE = 2 * RWAVES, NT = 64 * NWAVE;
    static constexpr int CPL = 4;
    static constexpr int SC = CG * 8, PB = SC * 2;
    static constexpr int NQ = SC / CPL >= 16 ? 16 : SC / CPL, NSUB = 16 / NQ;
    static constexpr int GD = TD / (4 * NSUB), RSPLIT = RWAVES / GD, RO = TW / RSPLIT;
    static constexpr int R = TW + 2, PDP = TD + 2;   // staged g rows and positions per row (dense)
    static constexpr int NPOS = TW * TD;
    static constexpr int PPB = 1024 / PB;            // positions per block = per load instruction of a wavefront
    static constexpr int NGB = (R * PDP + PPB - 1) / PPB, NXB = (NPOS + PPB - 1) / PPB;
    static constexpr int NGI = (NGB + NWAVE - 1) / NWAVE, NXI = (NXB + NWAVE - 1) / NWAVE;  // loads per wavefront
    static constexpr int NGS = 3, NXS = 4;
    static constexpr int GSLOT = NGB * 1024;
    static constexpr int XPAD = PB >= 64 ? 64 : PB;  // lanes j read different x slots: shift their banks apart
    static constexpr int XSLOT = NXB * 1024 + XPAD;
    static constexpr int XOFF = NGS * GSLOT;
    static constexpr int STAGE_BYTES = XOFF + NXS * XSLOT;
    static constexpr int RED_BYTES = RWAVES * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    static_assert(TD % (4 * NSUB) == 0 && RWAVES % GD == 0 && RWAVES >= GD && TW % RSPLIT == 0, "even split");
    static_assert(1024 % PB == 0 && STAGE_BYTES % 16 == 0 && XSLOT % 16 == 0, "whole positions per block");
    // chunk-slot rotation inside a position, see WdCfg in dwconv_wgrad_dma.hip
    __device__ static constexpr int rot(int dq) { return PB == 128 ? 64 * ((dq >> 1) & 1) : 0; }
};

// 8-byte streaming store of the lanes in `mask` to sbase + voff, counted by the hand-placed waits like the loads
__device__ __forceinline__ void masked_store8_stream(void* sbase, uint32_t voff, u32x2_t data, uint64_t mask)
{
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\tglobal_store_dwordx2 %2, %3, %1 nt\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "s"(sbase), "v"(voff), "v"(data), "s"(mask)
                 : "memory");
}

template <class Cfg, bool NTI>
// two workgroups per compute unit (their staging rings fill the LDS): two wavefronts per SIMD, 256 registers each
__global__ __launch_bounds__(Cfg::NT, 2) void dwconv_bwd_dma_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, TW = Cfg::TW, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RO = Cfg::RO, GSLOT = Cfg::GSLOT, XSLOT = Cfg::XSLOT, CPL = Cfg::CPL;
    constexpr int NGI = Cfg::NGI, NXI = Cfg::NXI, NGS = Cfg::NGS, NXS = Cfg::NXS, NWAVE = Cfg::NWAVE, PPB = Cfg::PPB;
    // vector memory instructions a wavefront issues per step: the plane loads (g blocks twice when their interior
    // chunks take the streaming hint), then, in the input-gradient role, one store per output row
    constexpr int LOADS = (NTI ? 2 : 1) * NGI + NXI;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(void __attribute__((address_space(3)))*)smem;

    const uint32_t ws_slot = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (ws_slot >= a.nblocks) return;
    const int t = threadIdx.x;
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    const int64_t plane_bytes = (int64_t)W * D * C * 2;

    const int lane = t % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
    const int role = wave / Cfg::RWAVES, rwave = wave % Cfg::RWAVES;  // 0: input gradient, 1: weight gradient
    const int gd = rwave % Cfg::GD, ra = (rwave / Cfg::GD) * RO;
    const int b = lane / 4, rr = lane % 4;
    const int q = b % NQ, sub = b / NQ;
    const int cb = q * (CPL * 2);            // byte offset of the lane's four channels inside a position
    const int pgrp = (gd * NSUB + sub) * 4;  // first position of the lane's group inside a patch row

    // segments of the H march, as in dwconv_bwd_split_kernel
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
    const int cslab = (int)(ws_row % (uint32_t)a.n_slab) * SC;
    bool first = true;
    int hs = 0, he = 0, w0 = 0, d0 = 0;
    const char* xn = reinterpret_cast<const char*>(a.x);
    const char* gn = reinterpret_cast<const char*>(a.g);
    char* dxn = reinterpret_cast<char*>(a.dx);
    // this lane's chunk in each block its wavefront loads (see dwconv_wgrad_dma_kernel)
    uint32_t gvo[NGI], xvo[NXI], glds[NGI], xlds[NXI];
    uint64_t gmask[NGI], gmask_in[NGI], xmask[NXI];
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
        n = __builtin_amdgcn_readfirstlane(n);
        hs = __builtin_amdgcn_readfirstlane(hs);
        he = __builtin_amdgcn_readfirstlane(he);
        w0 = __builtin_amdgcn_readfirstlane(wt_i * TW);
        d0 = __builtin_amdgcn_readfirstlane(dt * TD);
        xn = reinterpret_cast<const char*>(a.x) + (int64_t)n * H * plane_bytes;
        gn = reinterpret_cast<const char*>(a.g) + (int64_t)n * H * plane_bytes;
        dxn = reinterpret_cast<char*>(a.dx) + (int64_t)n * H * plane_bytes;
        // every load and store of the previous segment has completed, every wavefront has read its last plane
        wait_loads_in_flight<0>();
        __syncthreads();
        // positions outside the volume are never loaded: they read as the zeros written here
        const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int o = t * 16; o < Cfg::STAGE_BYTES; o += NT * 16) *reinterpret_cast<half8_t*>(smem + o) = z8;
#pragma unroll
        for (int i = 0; i < NGI; ++i) {
            const int blk = wave + i * NWAVE;
            const int P = blk * PPB + lane / CG, cs = lane % CG;
            const int wq = P / PDP, dq = P - wq * PDP;
            const int w = w0 - 1 + wq, d = d0 - 1 + dq;
            const bool ok = (blk < Cfg::NGB) && (wq < Cfg::R) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
            const int cbyte = (cs * 16 - Cfg::rot(dq)) & (PB - 1);
            gvo[i] = ok ? (uint32_t)(((w * D + d) * C + cslab) * 2 + cbyte) : 0u;
            // chunks no other workgroup reads (the patch without its border ring) take the streaming hint
            const bool interior = NTI && (wq >= 2) && (wq <= TW - 1) && (dq >= 2) && (dq <= TD - 1);
            gmask[i] = __ballot(ok && !interior);
            gmask_in[i] = __ballot(ok && interior);
            glds[i] = lds0 + (blk < Cfg::NGB ? blk : 0) * 1024;
        }
#pragma unroll
        for (int i = 0; i < NXI; ++i) {
            const int blk = wave + i * NWAVE;
            const int P = blk * PPB + lane / CG, cs = lane % CG;
            const int wq = P / TD, dq = P - wq * TD;
            const int w = w0 + wq, d = d0 + dq;
            const bool ok = (blk < Cfg::NXB) && (wq < TW) && (w < W) && (d < D);
            const int cbyte = (cs * 16 - Cfg::rot(dq)) & (PB - 1);
            xvo[i] = ok ? (uint32_t)(((w * D + d) * C + cslab) * 2 + cbyte) : 0u;
            xmask[i] = __ballot(ok);
            xlds[i] = lds0 + Cfg::XOFF + (blk < Cfg::NXB ? blk : 0) * 1024;
        }
        __syncthreads();  // the zero fill is complete before any load writes LDS
        return true;
    };
    // planes p of x and g (clamped into the volume; copies of a clamped plane are never used) into their ring slots
    auto load_planes = [&](int p, int gs, int xs) {
        const int64_t off = (int64_t)min(max(p, 0), H - 1) * plane_bytes;
        const char* gplane = uniform_ptr(gn + off);
        const char* xplane = uniform_ptr(xn + off);
#pragma unroll
        for (int i = 0; i < NGI; ++i) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(glds[i] + gs * GSLOT);
            lds_direct_load16<false>(gplane, gvo[i], dst, gmask[i]);
            if (NTI) lds_direct_load16<true>(gplane, gvo[i], dst, gmask_in[i]);
        }
        // x is read by this workgroup alone: streaming hint
#pragma unroll
        for (int i = 0; i < NXI; ++i)
            lds_direct_load16<true>(xplane, xvo[i], __builtin_amdgcn_readfirstlane(xlds[i] + xs * XSLOT), xmask[i]);
    };

    // The loads of a step at raised wave priority: the memory instructions of the wavefronts of a compute unit share
    // one issue path, and without it the loads queue behind the 8-byte stores of the wavefronts that write dx and
    // reach memory late (measured at C = 64: 1.138 -> 1.055 ms; raising the stores as well gives 1.133).
    auto load_planes_first = [&](int p, int gs, int xs) {
        __builtin_amdgcn_s_setprio(3);
        load_planes(p, gs, xs);
        __builtin_amdgcn_s_setprio(0);
    };

    if (role == 0) {
        // ---- input gradient: flipped weight operands, (kd' = 0, 1, 2, -) of one kh' per lane; the four registers of
        // an accumulator tile form a ring (see dwconv_fwd_mfma_segment): every step each lane hands its weights to the
        // next lane of its quad ----
        half4_t wA[3][CPL];
        {
            const int r0 = (1 - rr) & 3, c0 = cslab + q * CPL;
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                for (int e = 0; e < CPL; ++e) {
                    half4_t v = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
                    if (r0 < 3) {
#pragma unroll
                        for (int kd = 0; kd < 3; ++kd)
                            v[kd] = a.wt[(((2 - r0) * 3 + (2 - kw)) * 3 + (2 - kd)) * C + c0 + e];
                    }
                    wA[kw][e] = v;
                }
        }
        // g operand: lane rr = j reads the staged positions pgrp + j + k, k = 0..2
        int boff[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int dq = pgrp + rr + k;
            boff[k] = (ra * PDP + dq) * PB + ((cb + Cfg::rot(dq)) & (PB - 1));
        }
        while (next_segment()) {
            // the lane's 8 bytes (four channels) of position pgrp + rr in the output rows ra .. ra + RO - 1: the 16
            // lanes that share a position write one whole 128-byte line between them (permuting the values across
            // the wavefront first, so that consecutive lanes store consecutive bytes, changed nothing measurable)
            uint32_t ooff[RO];
            uint64_t omask[RO];
#pragma unroll
            for (int o = 0; o < RO; ++o) {
                const int w = w0 + ra + o, d = d0 + pgrp + rr;
                const bool ok = (w < W) && (d < D);
                ooff[o] = ok ? (uint32_t)(((w * D + d) * C + cslab) * 2 + cb) : 0u;
                omask[o] = __ballot(ok);
            }
            float4_t T[RO][CPL];  // dx tiles, four planes in a ring of registers
#pragma unroll
            for (int o = 0; o < RO; ++o)
#pragma unroll
                for (int e = 0; e < CPL; ++e) T[o][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            int gs = 0, gs_load = 1, xs_load = 1;  // ring slots of g plane p / of the planes loaded next
            load_planes(hs - 1, 0, 0);
            // the waits count RO stores behind every step's loads
#pragma unroll
            for (int o = 0; o < RO; ++o) masked_store8_stream(dxn, 0u, u32x2_t{0u, 0u}, 0);

            auto step = [&](auto ring, int p, bool live) {
                constexpr int DONE = (decltype(ring)::value + 3) & 3;  // register of dx plane p-1, complete after this step
                const bool gin = live && (p >= 0) && (p < H) && (p <= he);
                wait_loads_in_flight<RO>();  // this step's planes have landed; the stores behind them may be in flight
                __syncthreads();
                load_planes_first(p + 1, gs_load, xs_load);
                gs_load = gs_load + 1 == NGS ? 0 : gs_load + 1;
                xs_load = xs_load + 1 == NXS ? 0 : xs_load + 1;
                if (gin) {
                    const unsigned char* gslot = smem + gs * GSLOT;
#pragma unroll
                    for (int xr = 0; xr < RO + 2; ++xr) {
                        uint32_t lo[3], hi[3];
#pragma unroll
                        for (int k = 0; k < 3; ++k) {
                            const u32x2_t r = *reinterpret_cast<const u32x2_t*>(gslot + boff[k] + xr * PDP * PB);
                            lo[k] = r[0];
                            hi[k] = r[1];
                        }
                        half4_t B[CPL];
                        split_operands3(lo, B[0], B[1]);
                        split_operands3(hi, B[2], B[3]);
#pragma unroll
                        for (int kw = 0; kw < 3; ++kw) {
                            if (xr - kw >= 0 && xr - kw < RO) {
#pragma unroll
                                for (int e = 0; e < CPL; ++e)
                                    T[xr - kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(wA[kw][e], B[e], T[xr - kw][e], 0, 0, 0);
                            }
                        }
                    }
                }
                const int ho = p - 1;
                const bool store = live && (ho >= hs) && (ho < he);
                char* dplane = const_cast<char*>(uniform_ptr(dxn + (int64_t)max(ho, 0) * plane_bytes));
#pragma unroll
                for (int o = 0; o < RO; ++o) {
                    half4_t v;
#pragma unroll
                    for (int e = 0; e < CPL; ++e) v[e] = (half_t)T[o][e][DONE];
                    masked_store8_stream(dplane, ooff[o], __builtin_bit_cast(u32x2_t, v), store ? omask[o] : 0);
                }
                // the finished register rests for one step (its lane has zero weights then) and starts its next
                // plane from zero; the weights move on by one lane
#pragma unroll
                for (int o = 0; o < RO; ++o)
#pragma unroll
                    for (int e = 0; e < CPL; ++e) T[o][e][DONE] = 0.0f;
#pragma unroll
                for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                    for (int e = 0; e < CPL; ++e) wA[kw][e] = quad_rotate_up(wA[kw][e]);
                gs = gs + 1 == NGS ? 0 : gs + 1;
            };
            // groups of four steps (the ring's period); both roles run the same number of steps, so their barriers match
            for (int p = hs - 1; p <= he + 1; p += 4) {
                step(std::integral_constant<int, 0>{}, p, true);
                step(std::integral_constant<int, 1>{}, p + 1, p + 1 <= he + 1);
                step(std::integral_constant<int, 2>{}, p + 2, p + 2 <= he + 1);
                step(std::integral_constant<int, 3>{}, p + 3, p + 3 <= he + 1);
            }
        }  // segments
        wait_loads_in_flight<0>();
        __syncthreads();  // (the other role: staging buffers are dead)
        __syncthreads();  // (the other role: partial sums are in LDS)
    } else {
        // ---- weight gradient, summed over the x positions of the patch.  Operand A (lane i = kd): the window of g
        // plane P, halo row ra + tr, that starts kd positions to the left; operand B (lane j = kh): four positions of
        // x row ra + o in the slot of plane P + j - 1. ----
        const int r2 = min(rr, 2);
        const uint32_t sel_e = rr < 3 ? 0x05040100u : 0x0c0c0c0cu, sel_o = rr < 3 ? 0x07060302u : 0x0c0c0c0cu;
        int aoff[4], boff[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int dg = pgrp + 2 - r2 + k, dx_ = pgrp + k;  // position inside the staged g row / the x row
            aoff[k] = (ra * PDP + dg) * PB + ((cb + Cfg::rot(dg)) & (PB - 1));
            boff[k] = Cfg::XOFF + (ra * TD + dx_) * PB + ((cb + Cfg::rot(dx_)) & (PB - 1));
        }
        float4_t acc[3][CPL];  // one tile per kw: D[i = kd][j = kh]
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
        while (next_segment()) {
            int gs_prev = NGS - 1, gs_load = 1, xs_load = 1;  // slot of g plane p - 1 / of the planes loaded next
            // lane j reads the x slot of plane P + j - 1 = p - 2 + j: its slot index runs behind the newest plane's
            int xslot_lane = (NXS + r2 - 2) % NXS;
            load_planes(hs - 1, 0, 0);
            // as many steps as the other role runs (groups of four), so that the barriers match
            const int nsteps = (he - hs + 3 + 3) / 4 * 4;
            for (int i = 0; i < nsteps; ++i) {
                const int p = hs - 1 + i;
                const int P = p - 1;  // g plane P meets the x planes P-1, P, P+1 = p, the newest one staged
                const bool on = (p <= he + 1) && (P >= hs) && (P < he);
                wait_loads_in_flight<0>();
                __syncthreads();
                load_planes_first(p + 1, gs_load, xs_load);
                gs_load = gs_load + 1 == NGS ? 0 : gs_load + 1;
                xs_load = xs_load + 1 == NXS ? 0 : xs_load + 1;
                if (on) {
                    const unsigned char* gsl = smem + gs_prev * GSLOT;
                    const unsigned char* xsl = smem + xslot_lane * XSLOT;
                    const int xp = P - 1 + r2;  // the lane's x plane
                    const bool xv = (unsigned)xp < (unsigned)H;
                    const uint32_t se = xv ? sel_e : 0x0c0c0c0cu, so = xv ? sel_o : 0x0c0c0c0cu;
                    half4_t X[RO][CPL];
#pragma unroll
                    for (int o = 0; o < RO; ++o) gather(xsl + o * TD * PB, boff, se, so, X[o]);
#pragma unroll
                    for (int tr = 0; tr < RO + 2; ++tr) {
                        half4_t A[CPL];
                        gather(gsl + tr * PDP * PB, aoff, sel_e, sel_o, A);  // (index 3 repeats index 2: zero operands)
#pragma unroll
                        for (int kw = 0; kw < 3; ++kw) {
                            if (tr + kw - 2 >= 0 && tr + kw - 2 < RO) {
#pragma unroll
                                for (int e = 0; e < CPL; ++e)
                                    acc[kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(A[e], X[tr + kw - 2][e], acc[kw][e], 0, 0, 0);
                            }
                        }
                    }
                }
                gs_prev = gs_prev + 1 == NGS ? 0 : gs_prev + 1;
                xslot_lane = xslot_lane + 1 == NXS ? 0 : xslot_lane + 1;
            }
        }
        wait_loads_in_flight<0>();
        if (NSUB > 1) {  // position groups inside the wavefront
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
        float* red = reinterpret_cast<float*>(smem);  // [RWAVES][27][SC]
        if (sub == 0 && rr < 3) {
#pragma unroll
            for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                for (int e = 0; e < CPL; ++e)
#pragma unroll
                    for (int i = 0; i < 3; ++i)
                        red[(rwave * 27 + (rr * 3 + kw) * 3 + i) * SC + q * CPL + e] = acc[kw][e][i];
        }
        __syncthreads();
    }
    const float* red = reinterpret_cast<const float*>(smem);
    float* out = a.ws + (int64_t)ws_row * 27 * SC;
    for (int o = t; o < 27 * SC; o += NT) {
        float sacc = 0.0f;
#pragma unroll
        for (int pt = 0; pt < Cfg::RWAVES; ++pt) sacc += red[pt * 27 * SC + o];
        out[o] = sacc;
    }
}

namespace {
template <int CG, int TW, int TD>
void launch_shape(const WgArgs& a, hipStream_t stream)
{
    using Cfg = BdCfg<CG, TW, TD>;
    const dim3 grid(xcd_padded_grid(a.nblocks, a.n_xcd)), block(Cfg::NT);
    if (a.stream_interior)
        hipLaunchKernelGGL((dwconv_bwd_dma_kernel<Cfg, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((dwconv_bwd_dma_kernel<Cfg, false>), grid, block, 0, stream, a);
}
}  // namespace

int launch_bwd_dma(const WgArgs& a, int cg, int tile_w, int tile_d, hipStream_t stream)
{
#define KEROPS_BD_CASE(CGv, TWv, TDv)                     \
    if (cg == CGv && tile_w == TWv && tile_d == TDv) {    \
        launch_shape<CGv, TWv, TDv>(a, stream);           \
        return 0;                                         \
    }
    KEROPS_BD_CASE(8, 8, 8)
    KEROPS_BD_CASE(4, 8, 16)
    KEROPS_BD_CASE(2, 8, 32)
    KEROPS_BD_CASE(1, 8, 64)
#undef KEROPS_BD_CASE
    return 1;
}

}  // namespace kerops
