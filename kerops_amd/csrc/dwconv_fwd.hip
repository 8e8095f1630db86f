// Depthwise 3x3x3 forward for [N][H][W][D][C] fp16 (gfx950).
//
// Work decomposition.  A workgroup owns a (TW x TD) patch of the (W, D) plane for a
// slab of CG*8 channels and marches along H over a chunk of rows.  For every input
// plane hp it stages the (TW+2) x (TD+2) halo patch through LDS once (global -> regs
// one plane ahead, regs -> LDS, one barrier per plane, two LDS buffers) and every
// thread *scatters* that plane into three rotating fp32 accumulator sets: output rows
// hp-1 (weight row kh=2, finishing), hp (kh=1) and hp+1 (kh=0, starting).  Each input
// voxel is therefore read from LDS 9 times instead of 27 and from HBM/L2 once per
// patch; the finished row is rounded once (RNE) and stored as 16-byte chunks.
//
// Lane mapping.  One thread = one c8 chunk (8 channels, 16 bytes) of one voxel;
// consecutive lanes take consecutive chunks in memory order (channel group fastest,
// then D), so global loads/stores of a wavefront are contiguous 1 KiB runs and LDS
// reads are consecutive words (conflict free).  The weights of the thread's channels stay
// packed as fp16 pairs in registers; products are formed by the 2-way fp16 dot
// instruction and mixed-precision FMA, both accumulating in fp32.
#include <type_traits>

#include "common.hpp"

namespace kerops {

template <int CG_, int TW_, int TD_, int CL_, int NT_, int WPE_>
struct FwdCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, CL = CL_, NT = NT_;
    static constexpr int WPE = WPE_;           // wavefronts per SIMD the register budget is held to
    // Branch-free march with deferred stores (see dwconv_fwd_body). It needs a few more live registers, so
    // only the configurations with room under their register budget use it.
    static constexpr bool STRAIGHT = (WPE_ == 4);
    static constexpr int SC = CG * 8;          // channels in the slab
    static constexpr int NCL = SC / CL;        // lane groups (CL channels each) per voxel
    static constexpr int PW = TW + 2, PD = TD + 2;
    static constexpr int NPOS = TW * TD * NCL;  // output pieces per plane
    static constexpr int P = NPOS / NT;         // output pieces per thread per plane
    static constexpr int NCH = PW * PD * CG;    // staged c8 chunks per plane
    static constexpr int NLD = (NCH + NT - 1) / NT;
    static_assert(NPOS % NT == 0, "patch must divide evenly over the threads");
    static_assert(NT % NCL == 0, "a thread keeps one lane group");
    static_assert((TD & (TD - 1)) == 0, "TD power of two");
    static_assert(CL == 2 || CL == 4 || CL == 8, "2, 4 or 8 channels per lane");
};

template <int CL>
struct HalfN {
    typedef _Float16 type __attribute__((ext_vector_type(CL)));
};

struct FwdArgs {
    const half_t* x;
    const half_t* wt;
    half_t* y;
    const float* scale;  // optional fused epilogue y = max(acc * scale[c] + shift[c], 0)
    const float* shift;
    // optional fused pointwise stage (matrix-core kernel only): y2 = fp16(t @ pw), t = the epilogue's fp16 output
    const half_t* pw;   // [C][cout]
    half_t* y2;         // [N][H][W][D][cout]
    float* amax_ws;     // one max|y2| per workgroup
    float* stats_ws;    // mode 3: per workgroup [2][slab channels] sums of y and y*y (y as stored, fp16)
    int H, W, D, C;
    int n_wt, n_dt, n_hc, n_slab, h_chunk;
    uint32_t nblocks;
    // balanced split (matrix-core kernel, modes 0 and 1): bal_group > 0 switches it on
    uint32_t bal_group, bal_q, bal_r;  // workgroups per group; bundles * H plane steps = groups * bal_q + bal_r
    uint32_t n_tiles;                  // tiles in the tensor
    uint32_t n_xcd;                    // accelerator dies of the device: the logical workgroup order follows them
    int stream_interior;               // host side only: selects the kernels built with the streaming hint (NTI)
};

// Packed weights of one thread: for every weight row kh and every channel j of the lane,
// the nine in-plane taps t = kw*3 + kd are held as four fp16 pairs (t = 0/1, 2/3, 4/5, 6/7)
// for the 2-way dot instruction plus the single tap t = 8.
template <int CL>
struct LaneWeights {
    half2_t pair[3][4][CL];
    half_t single[3][CL];
};

__device__ __forceinline__ half2_t pack_halves(uint32_t a, uint32_t b, int hi)
{
    // (half `hi` of a, half `hi` of b) as one dword: v_perm_b32 {b, a}
    const uint32_t r = hi ? __builtin_amdgcn_perm(b, a, 0x07060302u) : __builtin_amdgcn_perm(b, a, 0x05040100u);
    return __builtin_bit_cast(half2_t, r);
}

// Scatter one staged input plane into the three accumulator sets.  Per output piece and
// channel: 4 byte-permutes pair up the 9 in-plane neighbours once, then each of the three
// weight rows costs 4 two-way dots (fp16 x fp16 -> fp32) and 1 mixed-precision FMA:
// 19 instructions for 27 multiply-adds, all accumulation in fp32.
template <class Cfg, bool DO_F, bool DO_M, bool DO_S>
__device__ __forceinline__ void scatter_plane(const half_t* __restrict__ plane, const int (&lbase)[Cfg::P],
                                              const LaneWeights<Cfg::CL>& lw, float (&aF)[Cfg::P][Cfg::CL],
                                              float (&aM)[Cfg::P][Cfg::CL], float (&aS)[Cfg::P][Cfg::CL])
{
    constexpr int CL = Cfg::CL, ND = CL / 2;
    typedef uint32_t dv_t __attribute__((ext_vector_type(ND)));
#pragma unroll
    for (int k = 0; k < Cfg::P; ++k) {
        uint32_t v[9][ND];
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
#pragma unroll
            for (int kd = 0; kd < 3; ++kd) {
                if constexpr (ND == 1) {
                    v[kw * 3 + kd][0] =
                        *reinterpret_cast<const uint32_t*>(plane + lbase[k] + (kw * Cfg::PD + kd) * Cfg::SC);
                } else {
                    const dv_t q = *reinterpret_cast<const dv_t*>(plane + lbase[k] + (kw * Cfg::PD + kd) * Cfg::SC);
#pragma unroll
                    for (int e = 0; e < ND; ++e) v[kw * 3 + kd][e] = q[e];
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CL; ++c) {
            half2_t pr[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) pr[p] = pack_halves(v[2 * p][c / 2], v[2 * p + 1][c / 2], c & 1);
            const half2_t last = __builtin_bit_cast(half2_t, v[8][c / 2]);
            const float xs = (float)last[c & 1];
            if (DO_F) {
                float s = aF[k][c];
#pragma unroll
                for (int p = 0; p < 4; ++p) s = __builtin_amdgcn_fdot2(pr[p], lw.pair[2][p][c], s, false);
                aF[k][c] = __builtin_fmaf(xs, (float)lw.single[2][c], s);
            }
            if (DO_M) {
                float s = aM[k][c];
#pragma unroll
                for (int p = 0; p < 4; ++p) s = __builtin_amdgcn_fdot2(pr[p], lw.pair[1][p][c], s, false);
                aM[k][c] = __builtin_fmaf(xs, (float)lw.single[1][c], s);
            }
            if (DO_S) {
                // the row hp+1 starts here: the mixed-precision FMA takes the literal 0 as addend,
                // so no separate zeroing pass (and no register move) is needed
                float s = __builtin_fmaf(xs, (float)lw.single[0][c], 0.0f);
#pragma unroll
                for (int p = 0; p < 4; ++p) s = __builtin_amdgcn_fdot2(pr[p], lw.pair[0][p][c], s, false);
                aS[k][c] = s;
            }
        }
    }
}

// OUT_FULL: every output piece of the patch lies inside the volume (true for all patches
// but the last ones along W / D), so stores need no per-lane predicate.
template <class Cfg, bool OUT_FULL, bool EPI>
__device__ __forceinline__ void dwconv_fwd_body(const FwdArgs& a, half8_t (&lds)[2][Cfg::NCH + 1], int slab, int dt,
                                                int wt_i, int hc, int n)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, P = Cfg::P, NLD = Cfg::NLD, NCH = Cfg::NCH;
    constexpr int PD = Cfg::PD, CL = Cfg::CL, NCL = Cfg::NCL, SC = Cfg::SC;
    typedef typename HalfN<CL>::type hv_t;
    const int t = threadIdx.x;
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    const int w0 = wt_i * Cfg::TW, d0 = dt * TD;
    const int hs = hc * a.h_chunk;
    const int he = min(hs + a.h_chunk, H);
    const int cslab = slab * SC;
    const int64_t plane_stride = (int64_t)W * D * C;
    const half_t* xn = a.x + (int64_t)n * H * plane_stride;
    half_t* yn = a.y + (int64_t)n * H * plane_stride;

    // weights of this thread's lane group (CL channels), kept packed as fp16
    const int cl = t % NCL;
    LaneWeights<CL> lw;
    {
        hv_t wr[27];
#pragma unroll
        for (int tap = 0; tap < 27; ++tap)
            wr[tap] = *reinterpret_cast<const hv_t*>(a.wt + tap * C + cslab + cl * CL);
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int c = 0; c < CL; ++c) {
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    half2_t w2 = {wr[kh * 9 + 2 * p][c], wr[kh * 9 + 2 * p + 1][c]};
                    lw.pair[kh][p][c] = w2;
                }
                lw.single[kh][c] = wr[kh * 9 + 8][c];
            }
    }

    float esc[CL], esh[CL];
#pragma unroll
    for (int c = 0; c < CL; ++c) {
        esc[c] = EPI ? a.scale[cslab + cl * CL + c] : 1.0f;
        esh[c] = EPI ? a.shift[cslab + cl * CL + c] : 0.0f;
    }

    // staging assignment (fixed for the whole march)
    // Every lane issues every load and every LDS write unconditionally (straight-line code,
    // no per-lane branches around memory operations): a lane with nothing to stage loads the
    // first chunk of the plane and writes it to the dump slot.
    uint32_t goff[NLD];  // byte offset inside one (W, D, C) plane
    int ldst[NLD];       // destination chunk in the LDS plane buffer
    bool gval[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const int q = t + j * NT;
        const int wq = q / (PD * CG);
        const int r = q - wq * (PD * CG);
        const int dq = r / CG;
        const int cq = r - dq * CG;
        const int w = w0 - 1 + wq, d = d0 - 1 + dq;
        gval[j] = (q < NCH) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
        goff[j] = gval[j] ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
        ldst[j] = gval[j] ? q : NCH;
        // halo chunks outside the volume never change: zero them once in both buffers
        if (q < NCH && !gval[j]) {
            const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
            lds[0][q] = z;
            lds[1][q] = z;
        }
    }

    // output assignment
    int lbase[P];
    uint32_t ooff[P];  // byte offset inside one plane
    bool oval[P];
#pragma unroll
    for (int k = 0; k < P; ++k) {
        const int i = t + k * NT;
        const int dl = (i / NCL) % TD;
        const int wl = i / (NCL * TD);
        lbase[k] = (wl * PD + dl) * SC + cl * CL;  // in halves
        const int w = w0 + wl, d = d0 + dl;
        oval[k] = (w < W) && (d < D);
        ooff[k] = oval[k] ? (uint32_t)(((w * D + d) * C + cslab + cl * CL) * 2) : 0u;
    }

    float a0[P][CL], a1[P][CL], a2[P][CL];
#pragma unroll
    for (int k = 0; k < P; ++k)
#pragma unroll
        for (int c = 0; c < CL; ++c) a0[k][c] = a1[k][c] = a2[k][c] = 0.0f;

    if constexpr (Cfg::STRAIGHT) {
        // The march runs over the planes that exist, hp_lo..hp_hi; planes -1 and H are all zero and are
        // skipped (a volume border only changes which accumulator holds the last row, see the end).
        // Inside the loop every step does the same straight-line sequence, with no branch around a memory
        // operation: the compiler's wait-count bookkeeping is exact only on branch-free paths, and a
        // conservative wait would stall each step on the stores it has just issued.
        const int hp_lo = max(hs - 1, 0), hp_hi = min(he, H - 1);

        half8_t pre[NLD];
        auto prefetch = [&](int hp) {
            const char* xplane = reinterpret_cast<const char*>(xn + hp * plane_stride);  // wavefront-uniform
    #pragma unroll
            for (int j = 0; j < NLD; ++j) pre[j] = *reinterpret_cast<const half8_t*>(xplane + goff[j]);
        };

        // A finished row is rounded to fp16 at the end of its step but stored at the *start* of the next
        // step's arithmetic, ahead of the next prefetch: the vector-memory counter retires in issue order
        // and counts stores too, so a store issued right before the wait for the prefetched plane would
        // expose its full latency on every step.
        hv_t ostage[P];
        int pending_row = -1;
        auto round_row = [&](const float(&acc)[P][CL]) {
    #pragma unroll
            for (int k = 0; k < P; ++k) {
    #pragma unroll
                for (int c = 0; c < CL; ++c) {
                    float v = acc[k][c];
                    if (EPI) v = fmaxf(__builtin_fmaf(v, esc[c], esh[c]), 0.0f);
                    ostage[k][c] = (half_t)v;
                }
            }
        };
        auto flush_row = [&]() {
            if (pending_row >= 0) {
                char* yplane = reinterpret_cast<char*>(yn + pending_row * plane_stride);  // wavefront-uniform
    #pragma unroll
                for (int k = 0; k < P; ++k) {
                    if (OUT_FULL || oval[k]) {
                        // written once, never re-read: streaming hint keeps L2 for the halo rows
                        __builtin_nontemporal_store(ostage[k], reinterpret_cast<hv_t*>(yplane + ooff[k]));
                    }
                }
            }
        };

        int parity = 0;
        // aF: row hp-1 (finishing), aM: row hp, aS: row hp+1 (starting from zero)
        auto step = [&](int hp, float(&aF)[P][CL], float(&aM)[P][CL], float(&aS)[P][CL]) {
            half8_t* buf = lds[parity];
            parity ^= 1;
    #pragma unroll
            for (int j = 0; j < NLD; ++j) buf[ldst[j]] = pre[j];
            __syncthreads();
            flush_row();
            prefetch(min(hp + 1, hp_hi));  // the last one re-reads the current plane (cache hit) and is dropped
            // Scheduling fences: the loads stay ahead of the arithmetic that hides their latency, and the
            // arithmetic of one plane is scheduled on its own (one big region inflates register pressure).
            __builtin_amdgcn_sched_barrier(0);
            scatter_plane<Cfg, true, true, true>(reinterpret_cast<const half_t*>(buf), lbase, lw, aF, aM, aS);
            __builtin_amdgcn_sched_barrier(0);
            const int ho = hp - 1;
            pending_row = (ho >= hs) ? ho : -1;
            round_row(aF);
        };

        int hp = hp_lo, phase = 0;
        prefetch(hp);
        __syncthreads();  // the one-off zero fill of the halo chunks is visible before any plane is read
        for (;;) {
            step(hp, a0, a1, a2);
            phase = 1;
            if (++hp > hp_hi) break;
            step(hp, a1, a2, a0);
            phase = 2;
            if (++hp > hp_hi) break;
            step(hp, a2, a0, a1);
            phase = 0;
            if (++hp > hp_hi) break;
        }
        flush_row();
        if (he == H) {
            // bottom border of the volume: plane H does not exist, so row H-1 is complete after plane H-1,
            // where it was the middle row of the last step
            pending_row = H - 1;
            if (phase == 1) round_row(a1);
            else if (phase == 2) round_row(a2);
            else round_row(a0);
            flush_row();
        }
    } else {
        // Branching march: every step tests whether its plane exists. The branches keep the scheduling
        // regions (and with them the register pressure) small, at the price of conservative memory waits.
        half8_t pre[NLD];
        auto prefetch = [&](int hp) {
            if ((hp >= 0) && (hp < H)) {
                const char* xplane = reinterpret_cast<const char*>(xn + hp * plane_stride);  // wavefront-uniform
#pragma unroll
                for (int j = 0; j < NLD; ++j) pre[j] = *reinterpret_cast<const half8_t*>(xplane + goff[j]);
            }
        };

        int parity = 0;
        auto step = [&](int hp, float(&aF)[P][CL], float(&aM)[P][CL], float(&aS)[P][CL]) {
            const bool inb = (hp >= 0) && (hp < H);
            half8_t* buf = lds[parity];
            parity ^= 1;
            if (inb) {
#pragma unroll
                for (int j = 0; j < NLD; ++j) buf[ldst[j]] = pre[j];
            }
            __syncthreads();
            if (hp + 1 <= he) prefetch(hp + 1);
            if (inb) {
                scatter_plane<Cfg, true, true, true>(reinterpret_cast<const half_t*>(buf), lbase, lw, aF, aM, aS);
            } else {
#pragma unroll
                for (int k = 0; k < P; ++k)
#pragma unroll
                    for (int c = 0; c < CL; ++c) aS[k][c] = 0.0f;
            }
            const int ho = hp - 1;
            if (ho >= hs) {
                char* yplane = reinterpret_cast<char*>(yn + ho * plane_stride);  // wavefront-uniform
#pragma unroll
                for (int k = 0; k < P; ++k) {
                    if (OUT_FULL || oval[k]) {
                        hv_t o;
#pragma unroll
                        for (int c = 0; c < CL; ++c) {
                            float v = aF[k][c];
                            if (EPI) v = fmaxf(__builtin_fmaf(v, esc[c], esh[c]), 0.0f);
                            o[c] = (half_t)v;
                        }
                        // written once, never re-read: streaming hint keeps L2 for the halo rows
                        __builtin_nontemporal_store(o, reinterpret_cast<hv_t*>(yplane + ooff[k]));
                    }
                }
            }
        };

        int hp = hs - 1;
        prefetch(hp);
        __syncthreads();  // the one-off zero fill of the halo chunks is visible before any plane is read
        for (;;) {
            step(hp, a0, a1, a2);
            if (++hp > he) break;
            step(hp, a1, a2, a0);
            if (++hp > he) break;
            step(hp, a2, a0, a1);
            if (++hp > he) break;
        }
    }
}

template <class Cfg, bool EPI>
__global__ __launch_bounds__(Cfg::NT, Cfg::WPE) void dwconv_fwd_kernel(const FwdArgs a)
{
    __shared__ half8_t lds[2][Cfg::NCH + 1];  // +1: write-only dump slot for lanes with nothing to stage
    uint32_t L = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (L >= a.nblocks) return;
    // logical order, fastest first: slab, d-tile, w-tile, h-chunk, n
    const int slab = L % a.n_slab;
    L /= a.n_slab;
    const int dt = L % a.n_dt;
    L /= a.n_dt;
    const int wt_i = L % a.n_wt;
    L /= a.n_wt;
    const int hc = L % a.n_hc;
    const int n = L / a.n_hc;
    const bool out_full = ((wt_i + 1) * Cfg::TW <= a.W) && ((dt + 1) * Cfg::TD <= a.D);
    if (out_full) {
        dwconv_fwd_body<Cfg, true, EPI>(a, lds, slab, dt, wt_i, hc, n);
    } else {
        dwconv_fwd_body<Cfg, false, EPI>(a, lds, slab, dt, wt_i, hc, n);
    }
}

// ---------------------------------------------------------------------------------------------
// Matrix-core variant (lane_channels = 16).
//
// v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4 blocks, D_b[i][j] += sum_k A_b[i][k] * B_b[k][j];
// lane 4b+i holds row i of A_b as four fp16 (k = 0..3), lane 4b+j holds column j of B_b, and lane 4b+j
// receives column j of D_b in four fp32 registers (i = 0..3).  A depthwise convolution never mixes
// channels, so a block is one channel; the staged input plane hp is scattered, as in the vector
// kernel, into the output planes hp+1, hp, hp-1:
//
//   A_b[i][k] = wt[kh = i][kw][kd = k][c_b]            (weights; row 3 and column 3 are zero)
//   B_b[k][j] = x[hp][w][d0 + j + k - 1][c_b]           (lane j's window starts j-1 positions in)
//   D_b[i][j] += ... is the contribution of x row w to out[hp + 1 - i][w - kw + 1][d0 + j][c_b]
//
// One accumulator tile per output row w' therefore holds, in its registers i = 0, 1, 2, the partial
// sums of the output planes hp+1, hp, hp-1 for four D positions; the three x rows around w' add into
// it with the three kw operands.  After the plane, register 2 is complete (plane hp-1) and is stored;
// then the registers move up by one (a plane step renames 0 -> 1 -> 2, two moves and a zero).
// 576 of the 1024 multiply-adds of an instruction are useful; per x row, four positions and 16
// channels the cost is 3 matrix instructions, the operand comes from LDS as three dwords (two
// channels per lane and position) split into the even and the odd channel by byte permutes.
// The arithmetic is a fraction of the memory time; global loads run two planes ahead.
template <int CG_, int TW_, int TD_, int NT_>
struct FmCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_, NWAVE = NT_ / 64;
    static constexpr int SC = CG * 8;                      // channels in the slab
    static constexpr int PB = SC * 2;                      // bytes of one position
    static constexpr int NQ = SC >= 32 ? 16 : SC / 2;      // channel pairs per matrix instruction
    static constexpr int NSUB = 16 / NQ;                   // groups of 4 positions per instruction
    static constexpr int NHALF = SC / (2 * NQ);            // 32-channel halves of the slab
    static constexpr int NPART = NWAVE / NHALF;            // wavefronts that share a half split the patch
    static constexpr int GD = TD / (4 * NSUB);             // position groups along D, one per wavefront
    static constexpr int RSPLIT = NPART / GD;              // ... and row ranges along W
    static constexpr int RO = TW / RSPLIT;                 // output rows per wavefront (it reads RO + 2 x rows)
    static constexpr int R = TW + 2;                       // x rows incl. halo
    static constexpr int PDP = (TD + 3 + 3) / 4 * 4;       // x positions per row: halo + one over-read, padded to 4
    static constexpr int XSLOT = R * PDP * PB;
    static constexpr int DUMP = 2 * XSLOT;
    static constexpr int LDS_BYTES = DUMP + 16;
    static constexpr int NXCH = R * (TD + 2) * CG;
    static constexpr int NLDX = (NXCH + NT - 1) / NT;
    static_assert(TD % (4 * NSUB) == 0, "a row splits into whole position groups");
    static_assert(NPART % GD == 0 && NPART >= GD, "one position group per wavefront");
    static_assert(TW % RSPLIT == 0, "rows split evenly");
};

// MODE 0: y = conv; 3: the same plus per-channel sums of y and y*y over the workgroup's outputs (the statistics pass
// of a following batch norm, taken from the registers that hold the rounded outputs); 1: y = max(conv * scale +
// shift, 0); 2: that result (fp16) goes through an LDS tile into the
// pointwise GEMM [TW*TD positions][C] x [C][COUT] on the 32x32x16 matrix instruction (the product is computed
// transposed as in pointwise_kernel, a wavefront owns 32 positions x 32 output channels; pw^T sits in LDS), the
// [positions][COUT] result is bounced through LDS and stored as 16-byte chunks with the running max|y| fused in.
// One segment of a workgroup's work: the march over the rows [hs, he) of one tile (patch x slab x sample).
template <class Cfg, int MODE, int COUT, bool NTI>
__device__ __forceinline__ void dwconv_fwd_mfma_segment(const FwdArgs& a, unsigned char* smem, float* amax_red,
                                                        uint32_t wg_slot, uint32_t tile, int hs, int he,
                                                        float (&ssum)[2], float (&ssq)[2])
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RO = Cfg::RO, XSLOT = Cfg::XSLOT, NLDX = Cfg::NLDX;
    constexpr bool EPI = MODE == 1 || MODE == 2;
    constexpr bool STATS = MODE == 3;
    // fused pointwise stage: t tile [NPOS][SC + 8] fp16 and y tile [NPOS][COUT + 4] fp16 behind the staging buffers
    constexpr int NPOS = Cfg::TW * TD, RT = SC + 8, RY = COUT + 4;
    constexpr int KS = SC / 16, MT = COUT / 32, NPT = NPOS / 32;  // k = 16 per matrix instruction
    constexpr int T_OFF = Cfg::LDS_BYTES, Y_OFF = T_OFF + NPOS * RT * 2, A_OFF = Y_OFF + NPOS * RY * 2;
    // modes 0, 1 and 3: two output tiles [NPOS][PB] behind the staging buffers.  A finished plane is written to the
    // tile as dwords and leaves one step later, behind that step's barrier, as one 16-byte chunk per thread: whole
    // lines, one store instruction instead of RO.  With a 64-channel slab a wavefront owns 64-byte halves of the
    // 128-byte positions, which cost 10 % more HBM write traffic when written directly; narrower slabs would write
    // full lines either way, but the single store and the registers it frees (the RO store offsets; the 256-thread
    // shapes then hold four wavefronts per SIMD) are worth 3-20 % there.
    constexpr bool BOUNCE = MODE != 2;
    constexpr int OT_OFF = Cfg::LDS_BYTES, OT_BYTES = NPOS * PB;
    static_assert(!BOUNCE || NPOS * CG == NT, "one 16-byte output chunk per thread");
    constexpr int SMEM_BYTES = MODE == 2 ? A_OFF + MT * KS * 64 * 16 : (BOUNCE ? OT_OFF + 2 * OT_BYTES : Cfg::LDS_BYTES);
    constexpr bool SEGMENTS = MODE != 2;  // the fused pointwise mode always runs one segment (uniform chunks)
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    // The thread index is made opaque per segment: everything derived from it is then computed inside the segment
    // and dies with the prologue, instead of being hoisted out of the segment loop and held in registers across
    // the march.
    int t = threadIdx.x;
    if constexpr (SEGMENTS) asm volatile("" : "+v"(t));
    uint32_t L = tile;
    const int slab = L % a.n_slab;
    L /= a.n_slab;
    const int dt = L % a.n_dt;
    L /= a.n_dt;
    const int wt_i = L % a.n_wt;
    const int n = L / a.n_wt;
    const int w0 = wt_i * Cfg::TW, d0 = dt * TD;
    const int cslab = slab * SC;
    const int64_t plane_stride = (int64_t)W * D * C;
    const half_t* xn = a.x + (int64_t)n * H * plane_stride;
    half_t* yn = a.y + (int64_t)n * H * plane_stride;

    // positions that staging never writes (outside the volume, row padding) must read as zero
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int o = t * 16; o < Cfg::LDS_BYTES; o += NT * 16) *reinterpret_cast<half8_t*>(smem + o) = z8;

    // staging assignment, 16-byte chunks (8 channels of one position); lanes without a chunk inside the
    // volume load the plane's first chunk and write it to the dump slot
    uint32_t xgo[NLDX];
    int xls[NLDX];
    typedef HaloOrder<Cfg::TW, TD, CG> Order;  // shared chunks first, interior chunks last
#pragma unroll
    for (int j = 0; j < NLDX; ++j) {
        const int ch = t + j * NT;
        int wq, dq, cq;
        Order::decode(ch, wq, dq, cq);
        const int w = w0 - 1 + wq, d = d0 - 1 + dq;
        const bool ok = (ch < Cfg::NXCH) && (w >= 0) && (w < W) && (d >= 0) && (d < D);
        xgo[j] = ok ? (uint32_t)(((w * D + d) * C + cslab + cq * 8) * 2) : 0u;
        xls[j] = ok ? lds_swizzle<PB>(wq * PDP + dq, cq * 16) : -1;
    }

    // lane = (block b, index rr); block = (channel pair q, position group sub)
    const int lane = t % kWave, wave = t / kWave;
    const int half = wave % Cfg::NHALF, part = wave / Cfg::NHALF;
    const int gd = part % Cfg::GD, ra = (part / Cfg::GD) * RO;  // this wavefront: position group, first output row
    const int b = lane / 4, rr = lane % 4;
    const int q = b % NQ, sub = b / NQ;
    const int cb = half * 64 + q * 4;          // byte offset of the lane's channel pair inside a position
    const int c0 = cslab + half * 32 + 2 * q;  // its first channel
    const int pgrp = (gd * NSUB + sub) * 4;    // first output position of the lane's group inside the patch row

    // weight operands: (kd = 0, 1, 2, -) of tap row (kh, kw) for the even / odd channel, one kh per lane of a quad.
    // The four registers of an accumulator tile form a ring: output plane h lives in register (h - hs + 1) % 4 for
    // the three steps that add to it, so no register is moved between steps.  At step s (x plane hp = hs - 1 + s)
    // register i takes kh = (s + 1 - i) % 4 (3 = none: zero weights), i.e. every step each lane hands its weights
    // to the next lane of its quad (one DPP move per dword); a march of 4n steps leaves them where they started.
    half4_t wA[3][2];
    {
        const int r0 = (1 - rr) & 3;
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                half4_t v = {(half_t)0, (half_t)0, (half_t)0, (half_t)0};
                if (r0 < 3) {
#pragma unroll
                    for (int kd = 0; kd < 3; ++kd) v[kd] = a.wt[((r0 * 3 + kw) * 3 + kd) * C + c0 + e];
                }
                wA[kw][e] = v;
            }
    }
    float esc[2] = {1.0f, 1.0f}, esh[2] = {0.0f, 0.0f};
    if (EPI) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            esc[e] = a.scale[c0 + e];
            esh[e] = a.shift[c0 + e];
        }
    }

    // fused pointwise stage: this wavefront's 32 positions (pt) x 32 output channels (mt); A fragments =
    // rows of pw^T, k ordered as the 16-byte chunks the B fragments are read in (see pointwise_kernel)
    const int vl = lane % 32, hl = lane / 32;
    const int pt = wave % (NPT > 0 ? NPT : 1), mt = wave / (NPT > 0 ? NPT : 1);
    float amax = 0.0f;
    if constexpr (MODE == 2) {
        // pw^T fragments, pre-arranged so that lane l of block mt reads 16 contiguous bytes per k step:
        // [mt][s][l][8] = pw[16 s + 8 (l / 32) + 0..7][32 mt + l % 32]
        half_t* pa = reinterpret_cast<half_t*>(smem + A_OFF);
        for (int i = t; i < MT * KS * 64 * 8; i += NT) {
            const int jj = i % 8, l = (i / 8) % 64, s2 = (i / 512) % KS, m2 = i / (512 * KS);
            pa[i] = a.pw[(16 * s2 + 8 * (l / 32) + jj) * COUT + 32 * m2 + l % 32];
        }
    }
    half_t* yn2 = MODE == 2 ? a.y2 + (int64_t)n * H * W * D * COUT : nullptr;

    // x operand: lane rr = j reads the positions pgrp + j + k (patch column = position + 1 - 1), k = 0..2
    int boff[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) boff[k] = lds_swizzle<PB>(ra * PDP + pgrp + rr + k, cb);
    // output tile: LDS writes see 32 banks of 4 bytes (measured: 32 lanes of a dword write per clock), and half a
    // wavefront writes 8 dwords at each of four consecutive positions; the positions' bytes are rotated so that those
    // four runs fall into four different quarters of the 128 bytes of banks (no measurable change in time: the LDS
    // is a third busy in this kernel)
    auto ot_swz = [](int pos, int cbyte) {
        return PB == 128  ? pos * PB + ((cbyte + 32 * (pos & 3)) & 127)
               : PB == 64 ? pos * PB + ((cbyte + 32 * ((pos >> 1) & 1)) & 63)
                          : pos * PB + cbyte;
    };
    int owr[RO];  // the lane's dword (two channels) of position pgrp + rr in the output rows ra .. ra+RO-1
#pragma unroll
    for (int o = 0; o < RO; ++o) owr[o] = ot_swz((ra + o) * TD + pgrp + rr, cb);
    // the thread's 16-byte chunk of the tile: position t / CG, channels 8 (t % CG) ..
    const int opos = t / CG, ocq = t % CG;
    const int ord = ot_swz(opos, ocq * 16);
    const int ow = w0 + opos / TD, odd = d0 + opos % TD;
    const bool ovalid = (ow < W) && (odd < D);
    const uint32_t ogo = ovalid ? (uint32_t)(((ow * D + odd) * C + cslab + ocq * 8) * 2) : 0u;
    int pending_row = -1;
    auto flush_row = [&](int par) {  // stores the plane that the previous step left in output tile par
        if (BOUNCE && pending_row >= 0) {  // workgroup-uniform
            const half8_t o8 = *reinterpret_cast<const half8_t*>(smem + OT_OFF + par * OT_BYTES + ord);
            // written once, never re-read: streaming hint keeps L2 for the halo rows
            if (ovalid)
                __builtin_nontemporal_store(
                    o8, reinterpret_cast<half8_t*>(reinterpret_cast<char*>(yn + pending_row * plane_stride) + ogo));
        }
    };
    // mode 3: whether the lane's position pgrp + rr of the output rows ra .. ra+RO-1 lies inside the volume
    const int od = d0 + pgrp + rr;
    bool oval[RO];
#pragma unroll
    for (int o = 0; o < RO; ++o) oval[o] = (od < D) && (w0 + ra + o < W);

    float4_t T[RO][2];
#pragma unroll
    for (int o = 0; o < RO; ++o)
#pragma unroll
        for (int e = 0; e < 2; ++e) T[o][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // Global loads run two planes ahead of the arithmetic, into two register sets used alternately.
    // They are unconditional (plane indices are clamped; planes that do not exist are never used):
    // the compiler's wait-count bookkeeping is exact only on branch-free paths.
    // (the fused pointwise mode has no registers to spare for the second set and runs one plane ahead)
    // Planes in flight per workgroup: measured at (1,C,350,350,128), one plane ahead is faster with 8 and with 64
    // channels per slab (C = 8: 4 % for the plain kernel, 10 % with the statistics; C = 64, 128: 1 %), two planes
    // ahead with 16 and 32 (1-2 %), and three are slower everywhere: more planes in flight spread the workgroups
    // of a group further apart, and the halo lines they share leave the L2 before the neighbour asks for them.
    constexpr int AHEAD = MODE == 2 ? 1 : (SC == 8 || (SC == 64 && MODE != 3)) ? 1 : 2;
    half8_t xpre0[NLDX], xpre1[NLDX];
    auto prefetch = [&](int hp, half8_t(&xpre)[NLDX]) {
        const char* xplane = reinterpret_cast<const char*>(xn + min(max(hp, 0), H - 1) * plane_stride);
#pragma unroll
        for (int j = 0; j < NLDX; ++j) {
            // nobody else reads the interior chunks: with the hint they do not push shared lines out of the L2
            if (NTI && Order::interior_only(j * NT))
                xpre[j] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(xplane + xgo[j]));
            else
                xpre[j] = *reinterpret_cast<const half8_t*>(xplane + xgo[j]);
        }
    };

    int parity = 0;
    auto step = [&](auto ring, int hp, half8_t(&xpre)[NLDX], bool live) {
        constexpr int DONE = (decltype(ring)::value + 3) & 3;  // register of output plane hp-1, complete after this step
        const bool xin = live && (hp >= 0) && (hp < H);  // wavefront-uniform
        unsigned char* xbuf = smem + parity * XSLOT;
#pragma unroll
        for (int j = 0; j < NLDX; ++j) {
            unsigned char* dst = xls[j] >= 0 ? xbuf + xls[j] : smem + Cfg::DUMP;
            *reinterpret_cast<half8_t*>(dst) = xpre[j];
        }
        __syncthreads();
        // The loads of the next plane go out first and at raised wave priority, the stores of the finished plane
        // after them at the normal one: the memory instructions of the wavefronts of a compute unit share one issue
        // path, and loads queued behind other wavefronts' stores reach memory late (measured at C = 64: 0.703 ->
        // 0.694 ms; the same order without the priority, or the priority without the order, changes nothing).
        __builtin_amdgcn_s_setprio(3);
        prefetch(hp + AHEAD, xpre);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(0);
        flush_row(parity ^ 1);
        __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the arithmetic that hides their latency
        if (xin) {
#pragma unroll
            for (int xr = 0; xr < RO + 2; ++xr) {
                uint32_t r[3];
#pragma unroll
                for (int k = 0; k < 3; ++k)
                    r[k] = *reinterpret_cast<const uint32_t*>(xbuf + boff[k] + xr * PDP * PB);
                half4_t B[2];
                split_operands3(r, B[0], B[1]);
#pragma unroll
                for (int kw = 0; kw < 3; ++kw) {
                    // x patch row ra+xr (w = w0-1+ra+xr) adds to the output row ra+xr-kw at tap column kw
                    if (xr - kw >= 0 && xr - kw < RO) {
#pragma unroll
                        for (int e = 0; e < 2; ++e)
                            T[xr - kw][e] = __builtin_amdgcn_mfma_f32_4x4x4f16(wA[kw][e], B[e], T[xr - kw][e], 0, 0, 0);
                    }
                }
            }
        }
        // register DONE of every tile is the finished output plane hp-1
        const int ho = hp - 1;
        const bool finished = live && (ho >= hs);
        pending_row = finished ? ho : -1;
        if (finished) {  // workgroup-uniform
            unsigned char* otile = smem + OT_OFF + parity * OT_BYTES;
            half_t* tt = reinterpret_cast<half_t*>(smem + T_OFF);
            uint32_t vst[RO];  // mode 3: the rounded outputs of the lane's channel pair, row by row
#pragma unroll
            for (int o = 0; o < RO; ++o) {
                half2_t v;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    float f = T[o][e][DONE];
                    if (EPI) f = fmaxf(__builtin_fmaf(f, esc[e], esh[e]), 0.0f);
                    v[e] = (half_t)f;
                }
                if constexpr (STATS) {
                    // positions of the patch outside the volume hold values but are not outputs
                    vst[o] = oval[o] ? __builtin_bit_cast(uint32_t, v) : 0u;
                }
                if constexpr (MODE == 2) {
                    *reinterpret_cast<half2_t*>(tt + ((ra + o) * TD + pgrp + rr) * RT + half * 32 + 2 * q) = v;
                } else {
                    *reinterpret_cast<half2_t*>(otile + owr[o]) = v;
                }
            }
            if constexpr (STATS) {
                // the two channels of a row pair are regrouped into (row o, row o+1) pairs of one channel; the 2-way
                // fp16 dot product with fp32 accumulation then adds two outputs (against ones) or two squares (against
                // itself) per instruction: exact products, 16 instead of 28 vector instructions per plane
                static_assert(RO % 2 == 0, "rows are summed in pairs");
                const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
                for (int o = 0; o < RO; o += 2) {
                    const half2_t even = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(vst[o + 1], vst[o], 0x05040100u));
                    const half2_t odd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(vst[o + 1], vst[o], 0x07060302u));
                    ssum[0] = __builtin_amdgcn_fdot2(even, ones, ssum[0], false);
                    ssq[0] = __builtin_amdgcn_fdot2(even, even, ssq[0], false);
                    ssum[1] = __builtin_amdgcn_fdot2(odd, ones, ssum[1], false);
                    ssq[1] = __builtin_amdgcn_fdot2(odd, odd, ssq[1], false);
                }
            }
            if constexpr (MODE == 2) {
                typedef float float16_t __attribute__((ext_vector_type(16)));
                half_t* yt = reinterpret_cast<half_t*>(smem + Y_OFF);
                __syncthreads();
                if (mt < MT) {
                    const half_t* trow = tt + (32 * pt + vl) * RT;
                    const half8_t* pa = reinterpret_cast<const half8_t*>(smem + A_OFF) + mt * KS * 64 + lane;
                    float16_t pacc;
#pragma unroll
                    for (int i = 0; i < 16; ++i) pacc[i] = 0.0f;
#pragma unroll
                    for (int s2 = 0; s2 < KS; ++s2) {
                        // B fragment: channels 16 s + 8 hl + 0..7 of the lane's position = one 16-byte chunk
                        const half8_t bfrag = *reinterpret_cast<const half8_t*>(trow + 16 * s2 + 8 * hl);
                        pacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(pa[s2 * 64], bfrag, pacc, 0, 0, 0);
                    }
                    // pacc[i]: output channel 32*mt + 8*(i/4) + 4*hl + i%4 of position 32*pt + vl
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        half4_t o4;
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) o4[jj] = (half_t)pacc[4 * gq + jj];
                        *reinterpret_cast<half4_t*>(yt + (32 * pt + vl) * RY + 32 * mt + 8 * gq + 4 * hl) = o4;
                    }
                }
                __syncthreads();
                half_t* y2plane = yn2 + (int64_t)ho * W * D * COUT;
#pragma unroll
                for (int c = t; c < NPOS * (COUT / 8); c += NT) {
                    const int row = c / (COUT / 8), cc = c - row * (COUT / 8);
                    const int w = w0 + row / TD, d = d0 + row % TD;
                    if (w < W && d < D) {
                        const half4_t lo = *reinterpret_cast<const half4_t*>(yt + row * RY + cc * 8);
                        const half4_t hi = *reinterpret_cast<const half4_t*>(yt + row * RY + cc * 8 + 4);
                        const half8_t o8 = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
                        for (int jj = 0; jj < 8; ++jj) amax = fmaxf(amax, fabsf((float)o8[jj]));
                        store_c8_nt(y2plane + ((int64_t)w * D + d) * COUT + cc * 8, o8);
                    }
                }
            }
        }
        // the finished register rests for one step (its lane has zero weights then) and starts its next plane
        // from zero; the weights move on by one lane
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

    prefetch(hs - 1, xpre0);
    if (AHEAD >= 2) prefetch(hs, xpre1);
    __syncthreads();  // the one-off zero fill is complete before staging writes anything
    // The steps hp = hs-1 .. he run in groups of four (the period of the accumulator ring; the register sets
    // alternate inside a group), in a loop whose only exit is at its end: an exit between two steps would give the
    // loop a second way into its first step, on which the newest set is the oldest, and the compiler's wait before
    // that step's staging writes would cover every load in flight.  A count that does not divide ends with steps
    // that stage planes nobody reads, compute and store nothing.
    using std::integral_constant;
    if constexpr (AHEAD == 1) {
        for (int hp = hs - 1; hp <= he; hp += 4) {
            step(integral_constant<int, 0>{}, hp, xpre0, true);
            step(integral_constant<int, 1>{}, hp + 1, xpre0, hp + 1 <= he);
            step(integral_constant<int, 2>{}, hp + 2, xpre0, hp + 2 <= he);
            step(integral_constant<int, 3>{}, hp + 3, xpre0, hp + 3 <= he);
        }
    } else {
        for (int hp = hs - 1; hp <= he; hp += 4) {
            step(integral_constant<int, 0>{}, hp, xpre0, true);
            step(integral_constant<int, 1>{}, hp + 1, xpre1, hp + 1 <= he);
            step(integral_constant<int, 2>{}, hp + 2, xpre0, hp + 2 <= he);
            step(integral_constant<int, 3>{}, hp + 3, xpre1, hp + 3 <= he);
        }
    }
    if constexpr (BOUNCE) {
        __syncthreads();
        flush_row(parity ^ 1);
    } else if constexpr (SEGMENTS) {
        __syncthreads();  // the staging buffers are free before the next segment refills them
    }
    if constexpr (MODE == 2) {
        amax = wave_max(amax);
        if (lane == 0) amax_red[wave] = amax;
        __syncthreads();
        if (t == 0) {
            float m = amax_red[0];
#pragma unroll
            for (int wv = 1; wv < Cfg::NWAVE; ++wv) m = fmaxf(m, amax_red[wv]);
            a.amax_ws[wg_slot] = m;
        }
    }
}

// NTI: loads of chunks no other workgroup reads carry the streaming hint (a compile-time choice: a run-time branch
// next to the loads would make the compiler wait for every load in flight)
template <class Cfg, int MODE, int COUT = 0, bool NTI = false>
__global__ __launch_bounds__(Cfg::NT, Cfg::NT >= 512 ? 4 : 3) void dwconv_fwd_mfma_kernel(const FwdArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, SC = Cfg::SC, PB = Cfg::PB, PDP = Cfg::PDP;
    constexpr int NQ = Cfg::NQ, NSUB = Cfg::NSUB, RO = Cfg::RO, XSLOT = Cfg::XSLOT, NLDX = Cfg::NLDX;
    constexpr bool EPI = MODE == 1 || MODE == 2;
    constexpr bool STATS = MODE == 3;
    // fused pointwise stage: t tile [NPOS][SC + 8] fp16 and y tile [NPOS][COUT + 4] fp16 behind the staging buffers
    constexpr int NPOS = Cfg::TW * TD, RT = SC + 8, RY = COUT + 4;
    constexpr int KS = SC / 16, MT = COUT / 32, NPT = NPOS / 32;  // k = 16 per matrix instruction
    constexpr int T_OFF = Cfg::LDS_BYTES, Y_OFF = T_OFF + NPOS * RT * 2, A_OFF = Y_OFF + NPOS * RY * 2;
    // modes 0, 1 and 3: two output tiles [NPOS][PB] behind the staging buffers.  A finished plane is written to the
    // tile as dwords and leaves one step later, behind that step's barrier, as one 16-byte chunk per thread: whole
    // lines, one store instruction instead of RO.  With a 64-channel slab a wavefront owns 64-byte halves of the
    // 128-byte positions, which cost 10 % more HBM write traffic when written directly; narrower slabs would write
    // full lines either way, but the single store and the registers it frees (the RO store offsets; the 256-thread
    // shapes then hold four wavefronts per SIMD) are worth 3-20 % there.
    constexpr bool BOUNCE = MODE != 2;
    constexpr int OT_OFF = Cfg::LDS_BYTES, OT_BYTES = NPOS * PB;
    static_assert(!BOUNCE || NPOS * CG == NT, "one 16-byte output chunk per thread");
    constexpr int SMEM_BYTES = MODE == 2 ? A_OFF + MT * KS * 64 * 16 : (BOUNCE ? OT_OFF + 2 * OT_BYTES : Cfg::LDS_BYTES);
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    __shared__ float amax_red[Cfg::NWAVE];

    const uint32_t wg_slot = remap_xcd(blockIdx.x, a.nblocks, a.n_xcd);
    if (wg_slot >= a.nblocks) return;
    // mode 3: sums over the lane's channel pair, carried over every segment (all tiles of a workgroup belong to
    // the same slab: the group size of the balanced split is a multiple of the slab count)
    float ssum[2] = {0.0f, 0.0f}, ssq[2] = {0.0f, 0.0f};
    constexpr bool SEGMENTS = MODE != 2;  // the fused pointwise mode always runs one segment (uniform chunks)
    SegmentWalk walk = segment_walk_begin(wg_slot, SEGMENTS ? a.bal_group : 0u, a.bal_q, a.bal_r);
    uint32_t ws_row = wg_slot;  // mode 3: the workgroup's row of partial sums; row % slabs is its slab
    if constexpr (SEGMENTS) {
        // Two slabs (128 channels): the first half of a group's members takes slab 0 of the bundle's patches, the
        // second half slab 1, instead of alternating.  Each half (32 workgroups of the XCD's 64) then holds whole
        // patch rows of one slab, which share their halo voxels in the L2 (1.56 -> 1.52 ms at (1,128,350,350,128)).
        if (a.n_slab == 2 && walk.group > 0 && walk.group % 2 == 0) {
            const uint32_t halfg = walk.group / 2, m = walk.member;
            walk.member = (m % halfg) * 2 + m / halfg;
            ws_row = wg_slot - m + walk.member;
        }
    }
    uint32_t tile;
    int hs, he;
    const uint32_t per_sample = (uint32_t)(a.n_slab * a.n_dt * a.n_wt);
    if constexpr (SEGMENTS) {
        while (segment_walk_next(walk, wg_slot, a.H, a.n_tiles, per_sample, a.n_hc, a.h_chunk, tile, hs, he))
            dwconv_fwd_mfma_segment<Cfg, MODE, COUT, NTI>(a, smem, amax_red, wg_slot, tile, hs, he, ssum, ssq);
    } else {
        segment_walk_next(walk, wg_slot, a.H, a.n_tiles, per_sample, a.n_hc, a.h_chunk, tile, hs, he);
        dwconv_fwd_mfma_segment<Cfg, MODE, COUT, NTI>(a, smem, amax_red, wg_slot, tile, hs, he, ssum, ssq);
    }
    if constexpr (STATS) {
        const int t = threadIdx.x;
        const int lane = t % kWave, wave = t / kWave;
        const int b = lane / 4, rr = lane % 4;
        const int q = b % NQ, sub = b / NQ;
        // lanes of a wavefront that share the channel pair differ in rr (lane bits 0-1) and sub (the bits above q)
        float v4[4] = {ssum[0], ssum[1], ssq[0], ssq[1]};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v4[i] += __shfl_xor(v4[i], 1);
            v4[i] += __shfl_xor(v4[i], 2);
#pragma unroll
            for (int m = 4 * NQ; m < kWave; m <<= 1) v4[i] += __shfl_xor(v4[i], m);
        }
        __syncthreads();  // the staging buffers are free now
        float* sred = reinterpret_cast<float*>(smem);  // [wavefront][2 NQ channels][sum, sum of squares]
        if (rr == 0 && sub == 0) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                sred[(wave * 2 * NQ + 2 * q + e) * 2 + 0] = v4[e];
                sred[(wave * 2 * NQ + 2 * q + e) * 2 + 1] = v4[2 + e];
            }
        }
        __syncthreads();
        if (t < 2 * SC) {  // wavefronts that share a half of the slab, in a fixed order
            const int st = t / SC, ch = t % SC;
            const int hf = ch / (2 * NQ), cl = ch % (2 * NQ);
            float acc = 0.0f;
#pragma unroll
            for (int pp = 0; pp < Cfg::NPART; ++pp) acc += sred[((pp * Cfg::NHALF + hf) * 2 * NQ + cl) * 2 + st];
            a.stats_ws[(int64_t)ws_row * 2 * SC + st * SC + ch] = acc;
        }
    }
}

// grid of the matrix-core kernels: fills the n_* fields and nblocks of `a`
template <int CG, int TW, int TD, int NT>
static int plan_fwd_mfma(FwdArgs& a, int N, int h_chunk, bool balanced_ok = false, bool per_slab_state = false)
{
    a.n_slab = a.C / (CG * 8);
    a.n_wt = ceil_div(a.W, TW);
    a.n_dt = ceil_div(a.D, TD);
    a.bal_group = 0;
    const DeviceGeometry geo = device_geometry();
    a.n_xcd = (uint32_t)geo.xcds;
    const int slots = geo.resident_workgroups(NT);  // 2 workgroups of 512 threads or 4 of 256 per compute unit
    // h_chunk 0: balanced split with the group size of the cost model (-g: groups of g workgroups) for the kernels
    // that support it; > 0: uniform chunks of that many rows
    if (h_chunk < 0 || (h_chunk == 0 && balanced_ok)) {
        const int64_t tiles = (int64_t)N * a.n_wt * a.n_dt * a.n_slab;
        const BalancedSplit b = h_chunk < 0 ? make_balanced(a.H, tiles, slots, -h_chunk)
                                            : pick_balanced(a.H, tiles, a.n_dt * a.n_slab, slots, 6,
                                                            per_slab_state ? a.n_slab : 1, geo.xcds);
        const bool fits = b.units < (1LL << 31) && tiles + b.group < (1LL << 31);  // 32-bit counters in the kernel
        if (!fits && h_chunk < 0) {
            set_error("dwconv_fwd: too many plane steps for the balanced split");
            return KEROPS_E_BADARG;
        }
        if (fits) {
            a.bal_group = b.group;
            a.bal_q = (uint32_t)(b.units / b.ngroups);
            a.bal_r = (uint32_t)(b.units % b.ngroups);
            a.n_tiles = (uint32_t)tiles;
            a.h_chunk = a.H;
            a.n_hc = 1;
            a.nblocks = b.group * b.ngroups;
            return KEROPS_OK;
        }
    }
    if (h_chunk <= 0) {
        const int64_t per_plane = (int64_t)N * a.n_wt * a.n_dt * a.n_slab;
        h_chunk = pick_h_chunk(a.H, per_plane, slots, 6);
    }
    h_chunk = std::min(h_chunk, a.H);
    a.h_chunk = h_chunk;
    a.n_hc = ceil_div(a.H, h_chunk);
    const int64_t nb = (int64_t)N * a.n_hc * a.n_wt * a.n_dt * a.n_slab;
    if (nb > 0x7fffff00LL) {
        set_error("dwconv_fwd: too many workgroups (%lld)", (long long)nb);
        return KEROPS_E_BADARG;
    }
    a.nblocks = (uint32_t)nb;
    return KEROPS_OK;
}

template <int CG, int TW, int TD, int NT>
static int launch_fwd_mfma(const FwdArgs& base, int N, int h_chunk, hipStream_t stream)
{
    using Cfg = FmCfg<CG, TW, TD, NT>;
    FwdArgs a = base;
    int rc = plan_fwd_mfma<CG, TW, TD, NT>(a, N, h_chunk, true);
    if (rc != KEROPS_OK) return rc;
    if (a.scale) {
        hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 1>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, stream,
                           a);
    } else if (a.stream_interior) {
        hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 0, 0, true>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0,
                           stream, a);
    } else {
        hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 0>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, stream,
                           a);
    }
    return check_launch("dwconv_fwd");
}

// Adds the per-workgroup sums of one channel in a fixed order (fp64) and divides by the number of voxels:
// one workgroup per (statistic, channel); row r of the workspace belongs to slab r % n_slab.
__global__ __launch_bounds__(256) void dwconv_stats_reduce_kernel(const float* __restrict__ ws, uint32_t nblocks,
                                                                  int n_slab, int SC, double inv_count,
                                                                  float* __restrict__ mean, float* __restrict__ sqmean)
{
    __shared__ double part[256];
    const int C = n_slab * SC;
    const int st = blockIdx.x / C, c = blockIdx.x % C;
    const int slab = c / SC, ch = c % SC;
    double s = 0.0;
    for (uint32_t r = slab + (uint32_t)n_slab * threadIdx.x; r < nblocks; r += (uint32_t)n_slab * 256)
        s += (double)ws[(int64_t)r * 2 * SC + st * SC + ch];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) (st == 0 ? mean : sqmean)[c] = (float)(part[0] * inv_count);
}

// launch shape of the convolution + statistics kernel for a channel count (the default shapes of dwconv_fwd_run)
template <class F>
static int with_stats_shape(int C, F&& f)
{
    switch (C >= 64 ? 8 : C / 8) {
        case 1: return f(std::integral_constant<int, 1>{}, std::integral_constant<int, 8>{},
                         std::integral_constant<int, 32>{}, std::integral_constant<int, 256>{});
        case 2: return f(std::integral_constant<int, 2>{}, std::integral_constant<int, 8>{},
                         std::integral_constant<int, 32>{}, std::integral_constant<int, 512>{});
        case 4: return f(std::integral_constant<int, 4>{}, std::integral_constant<int, 8>{},
                         std::integral_constant<int, 16>{}, std::integral_constant<int, 512>{});
        default: return f(std::integral_constant<int, 8>{}, std::integral_constant<int, 8>{},
                          std::integral_constant<int, 8>{}, std::integral_constant<int, 512>{});
    }
}

template <int CG, int TW, int TD, int CL, int WPE, int NT = 256>
static int launch_fwd(const FwdArgs& base, int N, int h_chunk, hipStream_t stream)
{
    using Cfg = FwdCfg<CG, TW, TD, CL, NT, WPE>;
    FwdArgs a = base;
    a.n_slab = a.C / (CG * 8);
    a.n_wt = ceil_div(a.W, TW);
    a.n_dt = ceil_div(a.D, TD);
    const DeviceGeometry geo = device_geometry();
    a.n_xcd = (uint32_t)geo.xcds;
    if (h_chunk <= 0) {
        // enough workgroups to fill the compute units several times over (11 each), but rows per chunk
        // large enough that the two halo planes of a chunk stay a small overhead
        const int64_t per_plane = (int64_t)N * a.n_wt * a.n_dt * a.n_slab;
        const int want_chunks = (int)std::max<int64_t>(1, ceil_div64(11 * geo.cus, per_plane));
        h_chunk = std::max(ceil_div(a.H, want_chunks), std::min(a.H, 24));
    }
    h_chunk = std::min(h_chunk, a.H);
    a.h_chunk = h_chunk;
    a.n_hc = ceil_div(a.H, h_chunk);
    const int64_t nb = (int64_t)N * a.n_hc * a.n_wt * a.n_dt * a.n_slab;
    if (nb > 0x7fffff00LL) {
        set_error("dwconv_fwd: too many workgroups (%lld)", (long long)nb);
        return KEROPS_E_BADARG;
    }
    a.nblocks = (uint32_t)nb;
    if (a.scale) {
        if constexpr (CG == 8 && TW == 8 && TD == 8 && CL == 2 && NT == 512) {
            hipLaunchKernelGGL((dwconv_fwd_kernel<Cfg, true>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0,
                               stream, a);
        } else {
            set_error("dwconv_fwd: the fused affine+ReLU epilogue is built for the 64-channel 8x8 patch only");
            return KEROPS_E_BADARG;
        }
    } else {
        hipLaunchKernelGGL((dwconv_fwd_kernel<Cfg, false>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, stream,
                           a);
    }
    return check_launch("dwconv_fwd");
}

}  // namespace kerops

using namespace kerops;

namespace kerops {
int dwconv_fwd_run(const void* x, const void* wt, void* y, const float* scale, const float* shift, int32_t N,
                   int32_t H, int32_t W, int32_t D, int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                   int32_t lane_channels, void* stream)
{
    if (!x || !wt || !y || !aligned16(x) || !aligned16(wt) || !aligned16(y)) {
        set_error("dwconv_fwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwconv_fwd: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if (plane_exceeds_i32(W, D, C)) {
        set_error("dwconv_fwd: one (W,D,C) plane must stay below 2^31 elements");
        return KEROPS_E_BADARG;
    }
    if (!(C == 8 || C == 16 || C == 32 || C == 64 || C == 128)) {
        set_error("dwconv_fwd: unsupported channel count %d", C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    FwdArgs a{};
    a.x = (const half_t*)x;
    a.wt = (const half_t*)wt;
    a.y = (half_t*)y;
    a.scale = scale;
    a.shift = shift;
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    a.stream_interior = (int64_t)N * H * W * D * C * 2 >= kStreamInteriorMinBytes;
    hipStream_t s = (hipStream_t)stream;
    const int cg = C >= 64 ? 8 : C / 8;
    if (tile_w == 0 && tile_d == 0 && lane_channels == 0) {
        // measured best on MI355X at (1, C, 350, 350, 128)
        // (the matrix-core kernels)
        switch (cg) {
            case 1: tile_w = 8; tile_d = D > 32 ? 64 : 32; break;
            case 2: tile_w = 8; tile_d = 32; break;
            case 4: tile_w = 8; tile_d = 16; break;
            default: tile_w = 8; tile_d = 8; break;
        }
        lane_channels = 16;
    }
    // (channel groups of 8, patch W, patch D, channels per lane, wavefronts per SIMD, threads)
#define KEROPS_FWD_CASE(CGv, TWv, TDv, CLv, WPEv, NTv)                             \
    if (cg == CGv && tile_w == TWv && tile_d == TDv && lane_channels == CLv) \
        return launch_fwd<CGv, TWv, TDv, CLv, WPEv, NTv>(a, N, h_chunk, s);
    KEROPS_FWD_CASE(1, 16, 32, 4, 3, 256)
    KEROPS_FWD_CASE(1, 16, 32, 2, 3, 256)
    KEROPS_FWD_CASE(2, 8, 32, 4, 3, 256)
    KEROPS_FWD_CASE(2, 8, 32, 2, 3, 256)
    KEROPS_FWD_CASE(4, 8, 16, 4, 3, 256)
    KEROPS_FWD_CASE(4, 8, 16, 2, 3, 256)
    KEROPS_FWD_CASE(8, 4, 8, 4, 3, 256)
    KEROPS_FWD_CASE(8, 4, 8, 2, 4, 256)
    KEROPS_FWD_CASE(8, 4, 16, 2, 3, 256)
    KEROPS_FWD_CASE(8, 8, 8, 2, 4, 512)
#undef KEROPS_FWD_CASE
    // matrix-core kernels: (channel groups of 8, patch W, patch D, threads)
#define KEROPS_FM_CASE(CGv, TWv, TDv, NTv)                                  \
    if (cg == CGv && tile_w == TWv && tile_d == TDv && lane_channels == 16) \
        return launch_fwd_mfma<CGv, TWv, TDv, NTv>(a, N, h_chunk, s);
    KEROPS_FM_CASE(1, 8, 32, 256)
    KEROPS_FM_CASE(2, 8, 16, 256)
    KEROPS_FM_CASE(4, 4, 16, 256)
    KEROPS_FM_CASE(1, 8, 64, 512)
    KEROPS_FM_CASE(2, 8, 32, 512)
    KEROPS_FM_CASE(4, 8, 16, 512)
    KEROPS_FM_CASE(8, 4, 8, 256)
    KEROPS_FM_CASE(8, 8, 8, 512)
    KEROPS_FM_CASE(8, 4, 16, 512)
#undef KEROPS_FM_CASE
    set_error("dwconv_fwd: no kernel built for C=%d tile_w=%d tile_d=%d lane_channels=%d", C, tile_w, tile_d,
              lane_channels);
    return KEROPS_E_BADARG;
}
}  // namespace kerops

namespace kerops {
// Fused depthwise -> affine -> ReLU -> pointwise block for 64 input channels (8x8 patch, 512 threads).
int dwsep_fused_blocks(int32_t N, int32_t H, int32_t W, int32_t D)
{
    FwdArgs a{};
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = 64;
    if (plan_fwd_mfma<8, 8, 8, 512>(a, N, 0) != KEROPS_OK) return -1;
    return (int)a.nblocks;
}

int dwsep_fused_run(const void* x, const void* wt, const float* scale, const float* shift, const void* pw, void* y2,
                    float* amax_ws, int32_t N, int32_t H, int32_t W, int32_t D, int32_t Cout, void* stream)
{
    using Cfg = FmCfg<8, 8, 8, 512>;
    FwdArgs a{};
    a.x = (const half_t*)x;
    a.wt = (const half_t*)wt;
    a.scale = scale;
    a.shift = shift;
    a.pw = (const half_t*)pw;
    a.y2 = (half_t*)y2;
    a.amax_ws = amax_ws;
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = 64;
    a.stream_interior = (int64_t)N * H * W * D * 64 * 2 >= kStreamInteriorMinBytes;
    int rc = plan_fwd_mfma<8, 8, 8, 512>(a, N, 0);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (Cout == 128) {
        hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 2, 128>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, s, a);
    } else if (Cout == 64) {
        hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 2, 64>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, s, a);
    } else {
        set_error("dwsep_block: the fused kernel is built for Cout in {64,128}");
        return KEROPS_E_UNSUPPORTED_C;
    }
    return check_launch("dwsep_block");
}
}  // namespace kerops

static int dwconv_stats_check(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C)
{
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwconv_stats: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if (plane_exceeds_i32(W, D, C)) {
        set_error("dwconv_stats: one (W,D,C) plane must stay below 2^31 elements");
        return KEROPS_E_BADARG;
    }
    if (!(C == 8 || C == 16 || C == 32 || C == 64 || C == 128)) {
        set_error("dwconv_stats: unsupported channel count %d", C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    return KEROPS_OK;
}

extern "C" int64_t kerops_dwconv_stats_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C)
{
    int rc = dwconv_stats_check(N, H, W, D, C);
    if (rc != KEROPS_OK) return rc;
    FwdArgs a{};
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    rc = with_stats_shape(C, [&](auto cg, auto tw, auto td, auto nt) {
        return plan_fwd_mfma<cg(), tw(), td(), nt()>(a, N, 0, true, true);
    });
    if (rc != KEROPS_OK) return rc;
    return (int64_t)a.nblocks * 2 * std::min(C, 64) * (int64_t)sizeof(float);
}

extern "C" int kerops_dwconv_stats_f16(const void* x, const void* wt, void* y, float* mean, float* sqmean,
                                       void* workspace, int64_t workspace_bytes, int32_t N, int32_t H, int32_t W,
                                       int32_t D, int32_t C, void* stream)
{
    const int64_t need = kerops_dwconv_stats_workspace_bytes(N, H, W, D, C);
    if (need < 0) return (int)need;
    if (!x || !wt || !y || !mean || !sqmean || !aligned16(x) || !aligned16(wt) || !aligned16(y)) {
        set_error("dwconv_stats: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("dwconv_stats: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    FwdArgs a{};
    a.x = (const half_t*)x;
    a.wt = (const half_t*)wt;
    a.y = (half_t*)y;
    a.stats_ws = (float*)workspace;
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    a.stream_interior = (int64_t)N * H * W * D * C * 2 >= kStreamInteriorMinBytes;
    hipStream_t s = (hipStream_t)stream;
    int rc = with_stats_shape(C, [&](auto cg, auto tw, auto td, auto nt) {
        using Cfg = FmCfg<cg(), tw(), td(), nt()>;
        int r = plan_fwd_mfma<cg(), tw(), td(), nt()>(a, N, 0, true, true);
        if (r != KEROPS_OK) return r;
        if (a.stream_interior)
            hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 3, 0, true>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0,
                               s, a);
        else
            hipLaunchKernelGGL((dwconv_fwd_mfma_kernel<Cfg, 3>), dim3(xcd_padded_grid(a.nblocks, a.n_xcd)), dim3(Cfg::NT), 0, s, a);
        return check_launch("dwconv_stats");
    });
    if (rc != KEROPS_OK) return rc;
    const double inv_count = 1.0 / ((double)N * H * W * D);
    hipLaunchKernelGGL(dwconv_stats_reduce_kernel, dim3(2 * C), dim3(256), 0, s, (const float*)workspace, a.nblocks,
                       a.n_slab, std::min(C, 64), inv_count, mean, sqmean);
    return check_launch("dwconv_stats_reduce");
}

extern "C" int kerops_dwconv_fwd_f16(const void* x, const void* wt, void* y, int32_t N, int32_t H, int32_t W,
                                     int32_t D, int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                                     int32_t lane_channels, void* stream)
{
    return kerops::dwconv_fwd_run(x, wt, y, nullptr, nullptr, N, H, W, D, C, tile_w, tile_d, h_chunk, lane_channels,
                                  stream);
}
