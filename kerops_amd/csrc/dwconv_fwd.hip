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
// reads are consecutive 16-byte words (conflict free).  The 27 weight chunks of the
// thread's channel group stay packed as fp16 in registers; products are formed by
// mixed-precision FMA (fp16 x fp16 + fp32 -> fp32).
#include "common.hpp"

namespace kerops {

template <int CG_, int TW_, int TD_, int NT_>
struct FwdCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, NT = NT_;
    static constexpr int PW = TW + 2, PD = TD + 2;
    static constexpr int NPOS = TW * TD * CG;  // output chunks per plane
    static constexpr int P = NPOS / NT;        // output chunks per thread per plane
    static constexpr int NCH = PW * PD * CG;   // staged chunks per plane
    static constexpr int NLD = (NCH + NT - 1) / NT;
    static_assert(NPOS % NT == 0, "patch must divide evenly over the threads");
    static_assert(NT % CG == 0, "a thread keeps one channel group");
    static_assert((TD & (TD - 1)) == 0, "TD power of two");
};

struct FwdArgs {
    const half_t* x;
    const half_t* wt;
    half_t* y;
    int H, W, D, C;
    int n_wt, n_dt, n_hc, n_slab, h_chunk;
    uint32_t nblocks;
};

template <class Cfg, bool DO_F, bool DO_M, bool DO_S>
__device__ __forceinline__ void scatter_plane(const half8_t* __restrict__ plane, const int (&lbase)[Cfg::P],
                                              const half8_t (&wr)[27], float (&aF)[Cfg::P][8],
                                              float (&aM)[Cfg::P][8], float (&aS)[Cfg::P][8])
{
#pragma unroll
    for (int k = 0; k < Cfg::P; ++k) {
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
#pragma unroll
            for (int kd = 0; kd < 3; ++kd) {
                const half8_t v = plane[lbase[k] + (kw * Cfg::PD + kd) * Cfg::CG];
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const float xv = (float)v[c];
                    if (DO_F) aF[k][c] = __builtin_fmaf(xv, (float)wr[(2 * 3 + kw) * 3 + kd][c], aF[k][c]);
                    if (DO_M) aM[k][c] = __builtin_fmaf(xv, (float)wr[(1 * 3 + kw) * 3 + kd][c], aM[k][c]);
                    if (DO_S) aS[k][c] = __builtin_fmaf(xv, (float)wr[(0 * 3 + kw) * 3 + kd][c], aS[k][c]);
                }
            }
        }
    }
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 2) void dwconv_fwd_kernel(const FwdArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, P = Cfg::P, NLD = Cfg::NLD, NCH = Cfg::NCH;
    constexpr int PD = Cfg::PD;
    __shared__ half8_t lds[2][NCH];

    uint32_t L = remap_xcd(blockIdx.x, a.nblocks);
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

    const int t = threadIdx.x;
    const int H = a.H, W = a.W, D = a.D, C = a.C;
    const int w0 = wt_i * Cfg::TW, d0 = dt * TD;
    const int hs = hc * a.h_chunk;
    const int he = min(hs + a.h_chunk, H);
    const int cslab = slab * CG * 8;
    const int64_t plane_stride = (int64_t)W * D * C;
    const half_t* xn = a.x + (int64_t)n * H * plane_stride;
    half_t* yn = a.y + (int64_t)n * H * plane_stride;

    // weights of this thread's channel group
    const int cg = t % CG;
    half8_t wr[27];
#pragma unroll
    for (int tap = 0; tap < 27; ++tap) wr[tap] = load_c8(a.wt + tap * C + cslab + cg * 8);

    // staging assignment (fixed for the whole march)
    int goff[NLD];
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
        goff[j] = (w * D + d) * C + cslab + cq * 8;
    }

    // output assignment
    int lbase[P], ooff[P];
    bool oval[P];
#pragma unroll
    for (int k = 0; k < P; ++k) {
        const int i = t + k * NT;
        const int dl = (i / CG) % TD;
        const int wl = i / (CG * TD);
        lbase[k] = (wl * PD + dl) * CG + cg;
        const int w = w0 + wl, d = d0 + dl;
        oval[k] = (w < W) && (d < D);
        ooff[k] = (w * D + d) * C + cslab + cg * 8;
    }

    float a0[P][8], a1[P][8], a2[P][8];
#pragma unroll
    for (int k = 0; k < P; ++k)
#pragma unroll
        for (int c = 0; c < 8; ++c) a0[k][c] = a1[k][c] = a2[k][c] = 0.0f;

    half8_t pre[NLD];
    auto prefetch = [&](int hp) {
        const bool inb = (hp >= 0) && (hp < H);
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (inb && gval[j]) v = load_c8(xn + hp * plane_stride + goff[j]);
            pre[j] = v;
        }
    };

    int parity = 0;
    auto step = [&](int hp, float(&aF)[P][8], float(&aM)[P][8], float(&aS)[P][8]) {
        const bool inb = (hp >= 0) && (hp < H);
        half8_t* buf = lds[parity];
        parity ^= 1;
        if (inb) {
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int q = t + j * NT;
                if (q < NCH) buf[q] = pre[j];
            }
        }
        __syncthreads();
        if (hp + 1 <= he) prefetch(hp + 1);
        // Keep the weights packed as fp16: without this the compiler hoists the 216
        // fp16->fp32 conversions out of the march and holds them in 216 registers.
#pragma unroll
        for (int tap = 0; tap < 27; ++tap) asm("" : "+v"(wr[tap]));
#pragma unroll
        for (int k = 0; k < P; ++k)
#pragma unroll
            for (int c = 0; c < 8; ++c) aS[k][c] = 0.0f;
        if (inb) scatter_plane<Cfg, true, true, true>(buf, lbase, wr, aF, aM, aS);
        const int ho = hp - 1;
        if (ho >= hs) {
#pragma unroll
            for (int k = 0; k < P; ++k) {
                if (oval[k]) {
                    half8_t o;
#pragma unroll
                    for (int c = 0; c < 8; ++c) o[c] = (half_t)aF[k][c];
                    store_c8(yn + ho * plane_stride + ooff[k], o);
                }
            }
        }
    };

    int hp = hs - 1;
    prefetch(hp);
    for (;;) {
        step(hp, a0, a1, a2);
        if (++hp > he) break;
        step(hp, a1, a2, a0);
        if (++hp > he) break;
        step(hp, a2, a0, a1);
        if (++hp > he) break;
    }
}

template <int CG, int TW, int TD>
static int launch_fwd(const FwdArgs& base, int N, int h_chunk, hipStream_t stream)
{
    using Cfg = FwdCfg<CG, TW, TD, 256>;
    FwdArgs a = base;
    a.n_slab = a.C / (CG * 8);
    a.n_wt = ceil_div(a.W, TW);
    a.n_dt = ceil_div(a.D, TD);
    if (h_chunk <= 0) {
        // enough workgroups to fill 256 CUs several times over, but rows per chunk
        // large enough that the two halo planes of a chunk stay a small overhead
        const int64_t per_plane = (int64_t)N * a.n_wt * a.n_dt * a.n_slab;
        const int want_chunks = (int)std::max<int64_t>(1, ceil_div64(4096, per_plane));
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
    hipLaunchKernelGGL(dwconv_fwd_kernel<Cfg>, dim3(xcd_padded_grid(a.nblocks)), dim3(Cfg::NT), 0, stream, a);
    return check_launch("dwconv_fwd");
}

}  // namespace kerops

using namespace kerops;

extern "C" int kerops_dwconv_fwd_f16(const void* x, const void* wt, void* y, int32_t N, int32_t H, int32_t W,
                                     int32_t D, int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                                     void* stream)
{
    if (!x || !wt || !y || !aligned16(x) || !aligned16(wt) || !aligned16(y)) {
        set_error("dwconv_fwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwconv_fwd: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if ((int64_t)W * D * C >= (1LL << 31)) {
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
    a.H = H;
    a.W = W;
    a.D = D;
    a.C = C;
    hipStream_t s = (hipStream_t)stream;
    const int cg = C >= 64 ? 8 : C / 8;
    if (tile_w == 0 && tile_d == 0) {
        switch (cg) {
            case 1: tile_w = 8; tile_d = 32; break;
            case 2: tile_w = 8; tile_d = 16; break;
            case 4: tile_w = 4; tile_d = 16; break;
            default: tile_w = 4; tile_d = 16; break;
        }
    }
#define KEROPS_FWD_CASE(CGv, TWv, TDv) \
    if (cg == CGv && tile_w == TWv && tile_d == TDv) return launch_fwd<CGv, TWv, TDv>(a, N, h_chunk, s);
    KEROPS_FWD_CASE(1, 8, 32)
    KEROPS_FWD_CASE(1, 16, 32)
    KEROPS_FWD_CASE(2, 8, 16)
    KEROPS_FWD_CASE(2, 8, 32)
    KEROPS_FWD_CASE(4, 4, 16)
    KEROPS_FWD_CASE(4, 8, 16)
    KEROPS_FWD_CASE(8, 4, 8)
    KEROPS_FWD_CASE(8, 4, 16)
    KEROPS_FWD_CASE(8, 8, 8)
#undef KEROPS_FWD_CASE
    set_error("dwconv_fwd: no kernel built for C=%d tile_w=%d tile_d=%d", C, tile_w, tile_d);
    return KEROPS_E_BADARG;
}
