// Depthwise 3x3x3 weight gradient for [N][H][W][D][C] fp16 (gfx950), fp32 end to end.
//
//   gw[kh,kw,kd,c] = sum_{n,h,w,d} g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]
//
// Same march as the forward kernel: a workgroup owns a (TW x TD) patch of the (W, D)
// plane for a slab of CG*8 channels and walks a chunk of rows along H.  Each x plane
// hp (with its halo) is staged through LDS once; a thread owns CL channels of a few
// patch positions, reads the 9 in-plane neighbours of x from LDS and multiplies them
// with the three rows of g that see this plane (g[hp+1] for kh=0, g[hp] for kh=1,
// g[hp-1] for kh=2).  g needs no halo: it is read straight from global memory, one
// row ahead, and kept in registers for three steps.  The 27*CL fp32 accumulators of a
// thread live for the whole march; at the end lanes that own the same channels are
// combined with wavefront shuffles, wavefronts through LDS, and the workgroup writes
// one partial [27][slab] to the workspace.  A second kernel adds the partials in a
// fixed order, so the result is deterministic (no atomics).
#include "common.hpp"

namespace kerops {

template <int CG_, int TW_, int TD_, int CL_, int NT_>
struct WgCfg {
    static constexpr int CG = CG_, TW = TW_, TD = TD_, CL = CL_, NT = NT_;
    static constexpr int SC = CG * 8;          // channels in the slab
    static constexpr int NCL = SC / CL;        // lane groups per voxel
    static constexpr int PW = TW + 2, PD = TD + 2;
    static constexpr int NPOS = TW * TD * NCL;
    static constexpr int P = NPOS / NT;
    static constexpr int NCH = PW * PD * CG;   // staged c8 chunks per plane
    static constexpr int NLD = (NCH + NT - 1) / NT;
    static constexpr int NWAVE = NT / kWave;
    static constexpr int STAGE_BYTES = 2 * NCH * 16;
    static constexpr int RED_BYTES = NWAVE * 27 * SC * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
    static_assert(NPOS % NT == 0, "patch must divide evenly over the threads");
    static_assert(NT % NCL == 0 && (kWave % NCL == 0 || NCL % kWave == 0), "lane groups tile a wavefront");
    static_assert(NCL <= kWave, "a wavefront holds every lane group of a voxel");
    static_assert((TD & (TD - 1)) == 0, "TD power of two");
    static_assert(CL == 2 || CL == 4, "2 or 4 channels per lane");
};

struct WgArgs {
    const half_t* x;
    const half_t* g;
    float* ws;
    int H, W, D, C;
    int n_wt, n_dt, n_hc, n_slab, h_chunk;
    uint32_t nblocks;
};

template <int CL>
struct HalfVec;
template <>
struct HalfVec<2> {
    typedef half2_t type;
};
template <>
struct HalfVec<4> {
    typedef half4_t type;
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 2) void dwconv_wgrad_kernel(const WgArgs a)
{
    constexpr int CG = Cfg::CG, TD = Cfg::TD, NT = Cfg::NT, P = Cfg::P, NLD = Cfg::NLD, NCH = Cfg::NCH;
    constexpr int PD = Cfg::PD, CL = Cfg::CL, NCL = Cfg::NCL, SC = Cfg::SC;
    typedef typename HalfVec<CL>::type hv_t;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half8_t* stage = reinterpret_cast<half8_t*>(smem);

    uint32_t L = remap_xcd(blockIdx.x, a.nblocks);
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

    // staging assignment (c8 chunks of the halo patch)
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

    // positions of this thread
    const int cl = t % NCL;
    int lbase[P], poff[P];
    bool pval[P];
#pragma unroll
    for (int k = 0; k < P; ++k) {
        const int i = t + k * NT;
        const int dl = (i / NCL) % TD;
        const int wl = i / (NCL * TD);
        lbase[k] = ((wl * PD + dl) * CG) * 8 + cl * CL;  // in halves
        const int w = w0 + wl, d = d0 + dl;
        pval[k] = (w < W) && (d < D);
        poff[k] = (w * D + d) * C + cslab + cl * CL;
    }

    float acc[27][CL];
#pragma unroll
    for (int tap = 0; tap < 27; ++tap)
#pragma unroll
        for (int c = 0; c < CL; ++c) acc[tap][c] = 0.0f;

    half8_t pre[NLD];
    auto prefetch_x = [&](int hp) {
        const bool inb = (hp >= 0) && (hp < H);
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (inb && gval[j]) v = load_c8(xn + hp * plane_stride + goff[j]);
            pre[j] = v;
        }
    };
    auto load_g = [&](int h, hv_t(&dst)[P]) {
        const bool inb = (h >= hs) && (h < he);
#pragma unroll
        for (int k = 0; k < P; ++k) {
            hv_t v;
#pragma unroll
            for (int c = 0; c < CL; ++c) v[c] = (half_t)0;
            if (inb && pval[k]) v = *reinterpret_cast<const hv_t*>(gn_ptr + h * plane_stride + poff[k]);
            dst[k] = v;
        }
    };

    hv_t gm[P], gc[P], gnx[P], gpre[P];
#pragma unroll
    for (int k = 0; k < P; ++k)
#pragma unroll
        for (int c = 0; c < CL; ++c) gm[k][c] = gc[k][c] = (half_t)0;
    load_g(hs, gnx);

    int parity = 0;
    prefetch_x(hs - 1);
    for (int hp = hs - 1; hp <= he; ++hp) {
        const bool inb = (hp >= 0) && (hp < H);
        half8_t* buf = stage + parity * NCH;
        parity ^= 1;
        if (inb) {
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int q = t + j * NT;
                if (q < NCH) buf[q] = pre[j];
            }
        }
        __syncthreads();
        if (hp + 1 <= he) prefetch_x(hp + 1);
        load_g(hp + 2, gpre);
        if (inb) {
            const half_t* plane = reinterpret_cast<const half_t*>(buf);
#pragma unroll
            for (int k = 0; k < P; ++k) {
#pragma unroll
                for (int kw = 0; kw < 3; ++kw) {
#pragma unroll
                    for (int kd = 0; kd < 3; ++kd) {
                        const hv_t xv =
                            *reinterpret_cast<const hv_t*>(plane + lbase[k] + ((kw * PD + kd) * CG) * 8);
#pragma unroll
                        for (int c = 0; c < CL; ++c) {
                            const float xf = (float)xv[c];
                            acc[(0 * 3 + kw) * 3 + kd][c] =
                                __builtin_fmaf((float)gnx[k][c], xf, acc[(0 * 3 + kw) * 3 + kd][c]);
                            acc[(1 * 3 + kw) * 3 + kd][c] =
                                __builtin_fmaf((float)gc[k][c], xf, acc[(1 * 3 + kw) * 3 + kd][c]);
                            acc[(2 * 3 + kw) * 3 + kd][c] =
                                __builtin_fmaf((float)gm[k][c], xf, acc[(2 * 3 + kw) * 3 + kd][c]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < P; ++k) {
            gm[k] = gc[k];
            gc[k] = gnx[k];
            gnx[k] = gpre[k];
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

// out[tap][slab*SC + cs] = sum over the partial slots that belong to `slab`, added in
// slot order by 16 interleaved running sums that are then combined as a fixed tree.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ ws, float* __restrict__ gw,
                                                           int n_rest, int n_slab, int SC, int C)
{
    __shared__ float part[16][17];
    const int lo = threadIdx.x % 16;   // output within the group of 16
    const int sl = threadIdx.x / 16;   // slice of the slot range
    const int o = blockIdx.x * 16 + lo;  // index into [27][C]
    float s = 0.0f;
    if (o < 27 * C) {
        const int tap = o / C, c = o % C;
        const int slab = c / SC, cs = c % SC;
        for (int r = sl; r < n_rest; r += 16) {
            s += ws[((int64_t)(r * n_slab + slab) * 27 + tap) * SC + cs];
        }
    }
    part[sl][lo] = s;
    __syncthreads();
    if (sl == 0 && o < 27 * C) {
        float v = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) v += part[i][lo];
        gw[o] = v;
    }
}

struct WgPlan {
    int cg, tile_w, tile_d, cl, h_chunk, n_wt, n_dt, n_hc, n_slab;
    int64_t nblocks;
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
    if ((int64_t)W * D * C >= (1LL << 31)) {
        set_error("dwconv_wgrad: one (W,D,C) plane must stay below 2^31 elements");
        return KEROPS_E_BADARG;
    }
    p->cg = C >= 64 ? 8 : C / 8;
    if (tile_w == 0 && tile_d == 0 && lane_channels == 0) {
        // measured best on MI355X at (1, C, 350, 350, 128)
        switch (p->cg) {
            case 1: tile_w = 16; tile_d = 32; break;
            case 2: tile_w = 8; tile_d = 32; break;
            case 4: tile_w = 8; tile_d = 16; break;
            default: tile_w = 8; tile_d = 8; break;
        }
        lane_channels = 2;
    }
    p->cl = lane_channels;
    p->tile_w = tile_w;
    p->tile_d = tile_d;
    p->n_slab = C / (p->cg * 8);
    p->n_wt = ceil_div(W, tile_w);
    p->n_dt = ceil_div(D, tile_d);
    if (h_chunk <= 0) {
        // every workgroup leaves one partial, so aim at a few workgroups per CU only
        const int64_t per_plane = (int64_t)N * p->n_wt * p->n_dt * p->n_slab;
        const int want_chunks = (int)std::max<int64_t>(1, ceil_div64(2048, per_plane));
        h_chunk = std::max(ceil_div(H, want_chunks), std::min(H, 32));
    }
    p->h_chunk = std::min(h_chunk, H);
    p->n_hc = ceil_div(H, p->h_chunk);
    p->nblocks = (int64_t)N * p->n_hc * p->n_wt * p->n_dt * p->n_slab;
    if (p->nblocks > 0x7fffff00LL) {
        set_error("dwconv_wgrad: too many workgroups (%lld)", (long long)p->nblocks);
        return KEROPS_E_BADARG;
    }
    return KEROPS_OK;
}

template <int CG, int TW, int TD, int CL>
static int launch_wgrad(const WgArgs& base, const WgPlan& p, float* gw, hipStream_t stream)
{
    using Cfg = WgCfg<CG, TW, TD, CL, 256>;
    WgArgs a = base;
    a.n_wt = p.n_wt;
    a.n_dt = p.n_dt;
    a.n_hc = p.n_hc;
    a.n_slab = p.n_slab;
    a.h_chunk = p.h_chunk;
    a.nblocks = (uint32_t)p.nblocks;
    hipLaunchKernelGGL(dwconv_wgrad_kernel<Cfg>, dim3(xcd_padded_grid(a.nblocks)), dim3(Cfg::NT), 0, stream, a);
    int rc = check_launch("dwconv_wgrad");
    if (rc != KEROPS_OK) return rc;
    const int n_rest = (int)(p.nblocks / p.n_slab);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(ceil_div(27 * a.C, 16)), dim3(256), 0, stream, a.ws, gw, n_rest,
                       p.n_slab, Cfg::SC, a.C);
    return check_launch("dwconv_wgrad_reduce");
}

}  // namespace kerops

using namespace kerops;

extern "C" int64_t kerops_dwconv_wgrad_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                                       int32_t tile_w, int32_t tile_d, int32_t h_chunk,
                                                       int32_t lane_channels)
{
    WgPlan p;
    int rc = plan_wgrad(N, H, W, D, C, tile_w, tile_d, h_chunk, lane_channels, &p);
    if (rc != KEROPS_OK) return rc;
    return p.nblocks * 27 * (p.cg * 8) * (int64_t)sizeof(float);
}

extern "C" int kerops_dwconv_wgrad_f16(const void* x, const void* g, float* gw, void* workspace,
                                       int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                       int32_t tile_w, int32_t tile_d, int32_t h_chunk, int32_t lane_channels,
                                       void* stream)
{
    if (!x || !g || !gw || !aligned16(x) || !aligned16(g) || !aligned16(gw)) {
        set_error("dwconv_wgrad: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    WgPlan p;
    int rc = plan_wgrad(N, H, W, D, C, tile_w, tile_d, h_chunk, lane_channels, &p);
    if (rc != KEROPS_OK) return rc;
    const int64_t need = p.nblocks * 27 * (p.cg * 8) * (int64_t)sizeof(float);
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
    hipStream_t s = (hipStream_t)stream;
#define KEROPS_WG_CASE(CGv, TWv, TDv, CLv) \
    if (p.cg == CGv && p.tile_w == TWv && p.tile_d == TDv && p.cl == CLv) \
        return launch_wgrad<CGv, TWv, TDv, CLv>(a, p, gw, s);
    KEROPS_WG_CASE(1, 16, 32, 2)
    KEROPS_WG_CASE(1, 16, 32, 4)
    KEROPS_WG_CASE(2, 8, 32, 2)
    KEROPS_WG_CASE(2, 8, 32, 4)
    KEROPS_WG_CASE(4, 8, 16, 2)
    KEROPS_WG_CASE(4, 8, 16, 4)
    KEROPS_WG_CASE(8, 8, 8, 2)
    KEROPS_WG_CASE(8, 4, 16, 2)
    KEROPS_WG_CASE(8, 4, 16, 4)
#undef KEROPS_WG_CASE
    set_error("dwconv_wgrad: no kernel built for C=%d tile_w=%d tile_d=%d lane_channels=%d", C, p.tile_w, p.tile_d,
              p.cl);
    return KEROPS_E_BADARG;
}
