// Backward of the pointwise (1x1x1) ReLU-linear op on the matrix cores (gfx950), one pass over x and grad:
//
//   dx[v, ci] = (x[v, ci] > 0) ? fp16( sum_co g[v, co] * Wm[ci, co] ) : 0
//   dW[ci, co] = sum_v relu(x[v, ci]) * g[v, co]                          (fp32 end to end)
//
// x is [V][CIN] fp16, g is [V][COUT] fp16 (the memory of channels_last_3d tensors), Wm is [CIN][COUT] fp16.
// The op moves 2*V*(2*CIN + COUT) bytes: it is HBM-bound; both products run on v_mfma_f32_32x32x16_f16 so
// that the arithmetic stays a fraction of the memory time.
//
// A workgroup of four wavefronts loops over tiles of 64 voxels.  The tile of x and of g is staged through LDS
// (global -> registers one tile ahead -> LDS, rows of 16-byte chunks).
//  * dx is computed transposed, dx^T[ci, v] = Wm[ci, :] . g^T[:, v]: the A operand is a 32-row block of Wm
//    (16-byte fragments pre-arranged in LDS), the B operand is one 16-byte chunk of a voxel's g row.  One
//    (32 voxels x 32 input channels) block per wavefront; the fp32 result is rounded to fp16, bounced through
//    an LDS tile and written back as 16-byte chunks with the (x > 0) mask applied from the staged x tile.
//  * dW[ci, co] reduces over voxels, which is the slow axis of both operands in memory: the fragments
//    "8 consecutive voxels of one channel" are gathered from the LDS tiles with transposing reads (two
//    ds_read_b64_tr_b16 per fragment, see SwizzledRows in common.hpp; the ReLU is
//    applied to the x fragment in registers).  The (32 x 32) output blocks are distributed over the
//    wavefronts (with fewer than four blocks the wavefronts split the voxels instead) and accumulated in
//    fp32 registers over all tiles of the workgroup; at the end every workgroup writes its partial
//    [CIN][COUT] matrices to the workspace and a second kernel adds them in a fixed order (deterministic).
#include "common.hpp"

namespace kerops {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kLbThreads = 256;
constexpr int kLbWaves = kLbThreads / kWave;
constexpr int kLbTile = 64;  // voxels per tile

template <int CIN, int COUT>
struct LbCfg {
    static constexpr int MTI = (CIN + 31) / 32, MTO = (COUT + 31) / 32;  // 32-channel blocks
    static constexpr int KSO = COUT / 16;                                 // k steps of the dx product
    static constexpr int KSV = kLbTile / 16;                              // k steps (voxels) of the dW product
    static constexpr int XP = CIN, GP = COUT, DP = CIN;  // dense rows (halves); swizzled: SwizzledRows / BounceTile in common.hpp
    static constexpr int NBD = 2 * MTI;                                   // dx blocks (32 voxels x 32 channels) per tile
    static constexpr int NBW = MTI * MTO;                                 // dW blocks
    static constexpr int KSPL = NBW >= kLbWaves ? 1 : kLbWaves / NBW;     // voxel split when blocks are few
    static constexpr int BPW = NBW >= kLbWaves ? NBW / kLbWaves : 1;      // dW blocks per wavefront
    static constexpr int NXC = kLbTile * CIN / 8, NGC = kLbTile * COUT / 8;  // 16-byte chunks per tile
    static constexpr int NLX = (NXC + kLbThreads - 1) / kLbThreads, NLG = (NGC + kLbThreads - 1) / kLbThreads;
    static constexpr int XS_OFF = 0;
    static constexpr int GS_OFF = XS_OFF + kLbTile * XP * 2;
    static constexpr int DS_OFF = GS_OFF + kLbTile * GP * 2;
    static constexpr int WL_OFF = (DS_OFF + kLbTile * DP * 2 + 15) / 16 * 16;
    static constexpr int LDS_BYTES = WL_OFF + MTI * KSO * 64 * 16;
    static_assert(CIN % 16 == 0 && CIN <= 128 && COUT % 16 == 0 && COUT <= 128, "channels in {16,32,64,128}");
    static_assert(NBW % kLbWaves == 0 || kLbWaves % NBW == 0, "blocks divide over the wavefronts");
    static_assert(KSV % KSPL == 0, "voxel steps divide over the split");
};

template <int CIN, int COUT>
__global__ __launch_bounds__(kLbThreads) void relu_linear_bwd_kernel(const half_t* __restrict__ x,
                                                                     const half_t* __restrict__ g,
                                                                     const half_t* __restrict__ Wm,
                                                                     half_t* __restrict__ dx, float* __restrict__ ws,
                                                                     int64_t V)
{
    using Cfg = LbCfg<CIN, COUT>;
    constexpr int XP = Cfg::XP, GP = Cfg::GP, DP = Cfg::DP, KSO = Cfg::KSO, KSV = Cfg::KSV;
    constexpr int NLX = Cfg::NLX, NLG = Cfg::NLG, BPW = Cfg::BPW, KSPL = Cfg::KSPL;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    unsigned char* xs = smem + Cfg::XS_OFF;
    unsigned char* gs = smem + Cfg::GS_OFF;
    using XT = SwizzledRows<CIN>;
    using GT = SwizzledRows<COUT>;
    half_t* ds = reinterpret_cast<half_t*>(smem + Cfg::DS_OFF);
    half8_t* wl = reinterpret_cast<half8_t*>(smem + Cfg::WL_OFF);

    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int il = lane % 32, hl = lane / 32;
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // A fragments of the dx product: wl[(mt*KSO + s)*64 + lane] = Wm[32 mt + il][16 s + 8 hl + 0..7]
    for (int i = t; i < Cfg::MTI * KSO * 64; i += kLbThreads) {
        const int l = i % 64, s = (i / 64) % KSO, mt = i / (64 * KSO);
        const int ci = 32 * mt + l % 32;
        wl[i] = ci < CIN ? load_c8(Wm + ci * COUT + 16 * s + 8 * (l / 32)) : z8;
    }

    // this wavefront's dW blocks (mi, ni) and its share of the voxel steps
    const int wb0 = Cfg::NBW >= kLbWaves ? wave : wave % Cfg::NBW;
    const int kpart = Cfg::NBW >= kLbWaves ? 0 : wave / Cfg::NBW;
    float16_t wacc[BPW];
#pragma unroll
    for (int bb = 0; bb < BPW; ++bb)
#pragma unroll
        for (int i = 0; i < 16; ++i) wacc[bb][i] = 0.0f;

    const int64_t ntiles = (V + kLbTile - 1) / kLbTile;
    half8_t xpre[NLX], gpre[NLG];
    auto prefetch = [&](int64_t tile) {
        const int64_t v0 = tile * kLbTile;
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kLbThreads;
            const int64_t v = v0 + c / (CIN / 8);
            xpre[j] = (c < Cfg::NXC && v < V) ? load_c8_nt(x + v * CIN + (c % (CIN / 8)) * 8) : z8;
        }
#pragma unroll
        for (int j = 0; j < NLG; ++j) {
            const int c = t + j * kLbThreads;
            const int64_t v = v0 + c / (COUT / 8);
            gpre[j] = (c < Cfg::NGC && v < V) ? load_c8_nt(g + v * COUT + (c % (COUT / 8)) * 8) : z8;
        }
    };

    int64_t tile = blockIdx.x;
    if (tile < ntiles) prefetch(tile);
    for (; tile < ntiles; tile += gridDim.x) {
        const int64_t v0 = tile * kLbTile;
        // ---- stage the tile (rows past V are zero: they add nothing to dW) ----
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kLbThreads;
            if (c < Cfg::NXC) *reinterpret_cast<half8_t*>(xs + XT::chunk16(c / (CIN / 8), c % (CIN / 8))) = xpre[j];
        }
#pragma unroll
        for (int j = 0; j < NLG; ++j) {
            const int c = t + j * kLbThreads;
            if (c < Cfg::NGC) *reinterpret_cast<half8_t*>(gs + GT::chunk16(c / (COUT / 8), c % (COUT / 8))) = gpre[j];
        }
        __syncthreads();
        if (tile + gridDim.x < ntiles) prefetch(tile + gridDim.x);

        // ---- dx^T blocks: (vt, mt) = 32 voxels x 32 input channels ----
#pragma unroll
        for (int bd = 0; bd < (Cfg::NBD + kLbWaves - 1) / kLbWaves; ++bd) {
            const int blk = wave + bd * kLbWaves;
            if (blk < Cfg::NBD) {  // wavefront-uniform
                const int vt = blk % 2, mt = blk / 2;
                // chunk 2 s + hl of the lane's voxel row: the swizzle is an XOR, so step s is the offset of step 0 ^ 32 s
                const int grow = GT::chunk16(32 * vt + il, hl);
                float16_t acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
                for (int s = 0; s < KSO; ++s) {
                    const half8_t bfrag = *reinterpret_cast<const half8_t*>(gs + (grow ^ (32 * s)));
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(wl[(mt * KSO + s) * 64 + lane], bfrag, acc, 0, 0, 0);
                }
                // acc[i]: input channel 32 mt + 8 (i/4) + 4 hl + i%4 of voxel 32 vt + il
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int ci = 32 * mt + 8 * gq + 4 * hl;
                    if (ci < CIN) {
                        half4_t o;
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) o[jj] = (half_t)acc[4 * gq + jj];
                        *reinterpret_cast<half4_t*>(reinterpret_cast<unsigned char*>(ds) + BounceTile<CIN>::piece(32 * vt + il, 4 * mt + gq, hl)) = o;
                    }
                }
            }
        }

        // ---- dW blocks: A = relu(x)^T (channel il of 8 consecutive voxels), B = g likewise ----
#pragma unroll
        for (int bb = 0; bb < BPW; ++bb) {
            const int blk = wb0 + bb * kLbWaves;
            const int mi = blk / Cfg::MTO, ni = blk % Cfg::MTO;
            int xoff[2], goff[2];  // transposing reads: lane = channel 32 mi + il / 32 ni + il, registers = 8 voxels
            XT::tr_offsets(lane, mi, xoff);
            GT::tr_offsets(lane, ni, goff);
#pragma unroll
            for (int sp = 0; sp < KSV / KSPL; ++sp) {
                const int s = kpart + sp * KSPL;
                const half8_t af = __builtin_elementwise_max(XT::read_tr(xs, xoff, s), z8);  // relu(x), packed
                const half8_t bf = GT::read_tr(gs, goff, s);
                wacc[bb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, wacc[bb], 0, 0, 0);
            }
        }
        __syncthreads();

        // ---- dx write-back: 16-byte chunks, masked by x > 0 ----
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kLbThreads;
            const int row = c / (CIN / 8), cc = c % (CIN / 8);
            if (c < Cfg::NXC && v0 + row < V) {
                const half8_t xv = *reinterpret_cast<const half8_t*>(xs + XT::chunk16(row, cc));
                half8_t o = BounceTile<CIN>::read(reinterpret_cast<const unsigned char*>(ds), row, cc);
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) o[jj] = xv[jj] > (half_t)0 ? o[jj] : (half_t)0;
                store_c8_nt(dx + (v0 + row) * CIN + cc * 8, o);
            }
        }
        __syncthreads();
    }

    // ---- partial dW of this workgroup: row (blockIdx, kpart) of the workspace, [CIN][COUT] fp32 ----
    float* out = ws + ((int64_t)blockIdx.x * KSPL + kpart) * (CIN * COUT);
#pragma unroll
    for (int bb = 0; bb < BPW; ++bb) {
        const int blk = wb0 + bb * kLbWaves;
        const int mi = blk / Cfg::MTO, ni = blk % Cfg::MTO;
        const int co = 32 * ni + il;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int ci = 32 * mi + 8 * (i / 4) + 4 * hl + i % 4;
            if (ci < CIN && co < COUT) out[ci * COUT + co] = wacc[bb][i];
        }
    }
}

static int lb_blocks(int64_t V)
{
    const int64_t ntiles = (V + kLbTile - 1) / kLbTile;
    return (int)std::max<int64_t>(1, std::min<int64_t>(ntiles, 768));  // three workgroups per CU
}

template <int CIN, int COUT>
static int launch_lb(const half_t* x, const half_t* g, const half_t* Wm, half_t* dx, void* dW, int dw_dtype, float* ws,
                     int64_t V, hipStream_t s)
{
    using Cfg = LbCfg<CIN, COUT>;
    const int blocks = lb_blocks(V);
    hipLaunchKernelGGL((relu_linear_bwd_kernel<CIN, COUT>), dim3(blocks), dim3(kLbThreads), 0, s, x, g, Wm, dx, ws, V);
    int rc = check_launch("relu_linear_bwd");
    if (rc != KEROPS_OK) return rc;
    if (dw_dtype == KEROPS_DTYPE_F16)
        launch_reduce_rows_f16(ws, blocks * Cfg::KSPL, CIN * COUT, (half_t*)dW, (half_t*)dW, CIN * COUT, 1.0, s);
    else
        launch_reduce_rows(ws, blocks * Cfg::KSPL, CIN * COUT, (float*)dW, (float*)dW, CIN * COUT, 1.0, s);
    return check_launch("relu_linear_bwd_reduce");
}

static int lb_kspl(int Cin, int Cout)
{
    const int nbw = ((Cin + 31) / 32) * ((Cout + 31) / 32);
    return nbw >= kLbWaves ? 1 : kLbWaves / nbw;
}

}  // namespace kerops

using namespace kerops;

static bool lb_channels_ok(int c) { return c == 16 || c == 32 || c == 64 || c == 128; }

extern "C" int64_t kerops_relu_linear_bwd_workspace_bytes(int64_t V, int32_t Cin, int32_t Cout)
{
    if (V <= 0) {
        set_error("relu_linear_bwd: non-positive size");
        return KEROPS_E_BADARG;
    }
    if (!lb_channels_ok(Cin) || !lb_channels_ok(Cout)) {
        set_error("relu_linear_bwd: built for Cin, Cout in {16,32,64,128} (got %d -> %d)", Cin, Cout);
        return KEROPS_E_UNSUPPORTED_C;
    }
    return (int64_t)lb_blocks(V) * lb_kspl(Cin, Cout) * Cin * Cout * (int64_t)sizeof(float);
}

extern "C" int kerops_relu_linear_bwd_f16(const void* x, const void* g, const void* Wm, void* dx, float* dW,
                                          void* workspace, int64_t workspace_bytes, int64_t V, int32_t Cin,
                                          int32_t Cout, void* stream)
{
    return kerops_relu_linear_bwd_f16_out(x, g, Wm, dx, dW, KEROPS_DTYPE_F32, workspace, workspace_bytes, V, Cin, Cout,
                                          stream);
}

extern "C" int kerops_relu_linear_bwd_f16_out(const void* x, const void* g, const void* Wm, void* dx, void* dW,
                                              int32_t dw_dtype, void* workspace, int64_t workspace_bytes, int64_t V,
                                              int32_t Cin, int32_t Cout, void* stream)
{
    if (!grad_dtype_ok(dw_dtype)) {
        set_error("relu_linear_bwd: dw_dtype must be KEROPS_DTYPE_F32 or KEROPS_DTYPE_F16");
        return KEROPS_E_BADARG;
    }
    const int64_t need = kerops_relu_linear_bwd_workspace_bytes(V, Cin, Cout);
    if (need < 0) return (int)need;
    if (!x || !g || !Wm || !dx || !dW || !aligned16(x) || !aligned16(g) || !aligned16(Wm) || !aligned16(dx)) {
        set_error("relu_linear_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("relu_linear_bwd: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    const half_t* xh = (const half_t*)x;
    const half_t* gh = (const half_t*)g;
    const half_t* wh = (const half_t*)Wm;
    hipStream_t s = (hipStream_t)stream;
#define KEROPS_LB_CASE(CI, CO) \
    if (Cin == CI && Cout == CO) return launch_lb<CI, CO>(xh, gh, wh, (half_t*)dx, dW, dw_dtype, (float*)workspace, V, s);
    KEROPS_LB_CASE(16, 16)
    KEROPS_LB_CASE(16, 32)
    KEROPS_LB_CASE(16, 64)
    KEROPS_LB_CASE(16, 128)
    KEROPS_LB_CASE(32, 16)
    KEROPS_LB_CASE(32, 32)
    KEROPS_LB_CASE(32, 64)
    KEROPS_LB_CASE(32, 128)
    KEROPS_LB_CASE(64, 16)
    KEROPS_LB_CASE(64, 32)
    KEROPS_LB_CASE(64, 64)
    KEROPS_LB_CASE(64, 128)
    KEROPS_LB_CASE(128, 16)
    KEROPS_LB_CASE(128, 32)
    KEROPS_LB_CASE(128, 64)
    KEROPS_LB_CASE(128, 128)
#undef KEROPS_LB_CASE
    set_error("relu_linear_bwd: no kernel for %d -> %d", Cin, Cout);
    return KEROPS_E_UNSUPPORTED_C;
}
