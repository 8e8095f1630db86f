// Inverted-bottleneck pointwise block on the matrix cores (gfx950):
//
//   hid[v, :] = relu( fp16(x[v, :] @ Wup) + bias )      (fp16 add, C -> 2C channels)
//   out[v, :] = fp16( hid[v, :] @ Wdown ) + add[v, :]   (fp16 add, 2C -> C channels)
//
// x, add, out are [V][C] fp16 (the memory of channels_last_3d tensors), Wup [C][2C], Wdown [2C][C], bias [2C].
// The op moves 6*V*C bytes; the hidden activation never leaves the registers.
//
// Each wavefront owns tiles of 32 voxels and computes both products transposed on v_mfma_f32_32x32x16_f16
// (A = rows of W^T, pre-arranged 16-byte fragments in LDS; B = the voxel's channel vector).  The first
// product leaves lane (v, h) with the hidden channels 32 mt + 8 gq + 4 h + 0..3 of voxel v; since the
// reduction index of the second product may be enumerated in any order as long as both operands agree, its
// k step (mt, gp) takes exactly the 8 values the lane already holds for gq = 2 gp, 2 gp + 1, and the
// fragments of Wdown^T are arranged in the same order.  The result is bounced through a wavefront-private
// LDS tile and written back as 16-byte chunks with the fp16 residual add fused in.
#include "common.hpp"

namespace kerops {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kMlpThreads = 256;
constexpr int kMlpWaves = kMlpThreads / kWave;

template <int C>
struct MlpCfg {
    static constexpr int HID = 2 * C;
    static constexpr int MT1 = HID / 32;        // 32-row blocks of hidden channels
    static constexpr int KS1 = C / 16;          // k steps of the first product
    static constexpr int MO = (C + 31) / 32;    // 32-row blocks of output channels
    static constexpr int KS2 = HID / 16;        // k steps of the second product: (mt, gp)
    static constexpr int RH = C;                // output tile: dense rows, swizzled (BounceTile in common.hpp)
    static constexpr int A1_OFF = 0;
    static constexpr int A2_OFF = A1_OFF + MT1 * KS1 * 64 * 16;
    static constexpr int B_OFF = A2_OFF + MO * KS2 * 64 * 16;
    static constexpr int T_OFF = (B_OFF + HID * 2 + 15) / 16 * 16;
    static constexpr int LDS_BYTES = T_OFF + kMlpWaves * 32 * RH * 2;
    static_assert(C == 16 || C == 32 || C == 64, "C in {16,32,64}");
};

template <int C>
__global__ __launch_bounds__(kMlpThreads) void lin_brelu_lin_add_kernel(const half_t* __restrict__ x,
                                                                        const half_t* __restrict__ Wup,
                                                                        const half_t* __restrict__ Wdown,
                                                                        const half_t* __restrict__ bias,
                                                                        const half_t* __restrict__ add,
                                                                        half_t* __restrict__ out, int64_t V)
{
    using Cfg = MlpCfg<C>;
    constexpr int HID = Cfg::HID, MT1 = Cfg::MT1, KS1 = Cfg::KS1, MO = Cfg::MO, KS2 = Cfg::KS2, RH = Cfg::RH;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half_t* a1 = reinterpret_cast<half_t*>(smem + Cfg::A1_OFF);
    half_t* a2 = reinterpret_cast<half_t*>(smem + Cfg::A2_OFF);
    half_t* bs = reinterpret_cast<half_t*>(smem + Cfg::B_OFF);

    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int vl = lane % 32, hl = lane / 32;

    // a1[((mt*KS1 + s)*64 + l)*8 + j] = Wup[16 s + 8 (l/32) + j][32 mt + l%32]
    for (int i = t; i < MT1 * KS1 * 64 * 8; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KS1, mt = i / (512 * KS1);
        a1[i] = Wup[(16 * s + 8 * (l / 32) + j) * HID + 32 * mt + l % 32];
    }
    // a2[((mo*KS2 + s)*64 + l)*8 + j] = Wdown[hidden channel of (s = 2 mt + gp, l/32, j)][32 mo + l%32]
    for (int i = t; i < MO * KS2 * 64 * 8; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KS2, mo = i / (512 * KS2);
        const int mt = s / 2, gp = s % 2;
        const int ch = 32 * mt + 8 * (2 * gp + j / 4) + 4 * (l / 32) + j % 4;
        const int co = 32 * mo + l % 32;
        a2[i] = co < C ? Wdown[ch * C + co] : (half_t)0;
    }
    for (int i = t; i < HID; i += kMlpThreads) bs[i] = bias[i];
    __syncthreads();

    const half8_t* a1f = reinterpret_cast<const half8_t*>(a1) + lane;
    const half8_t* a2f = reinterpret_cast<const half8_t*>(a2) + lane;
    unsigned char* my = smem + Cfg::T_OFF + wave * 32 * RH * 2;
    using Tile = BounceTile<C>;

    const int64_t ntiles = (V + 31) / 32;
    const int64_t tiles_per_round = (int64_t)gridDim.x * kMlpWaves;
    const int64_t nrounds = (ntiles + tiles_per_round - 1) / tiles_per_round;
    for (int64_t r = 0; r < nrounds; ++r) {
        const int64_t tidx = (r * gridDim.x + blockIdx.x) * kMlpWaves + wave;
        const bool live = tidx < ntiles;  // wavefront-uniform
        const int64_t v0 = tidx * 32;
        if (live) {
            int64_t v = v0 + vl;
            if (v >= V) v = V - 1;  // ragged last tile: clamp the read, the write is masked
            half8_t xb[KS1];
#pragma unroll
            for (int s = 0; s < KS1; ++s) {
                // rows of 128 bytes need the cache to hold the line until the row's other loads arrive
                if constexpr (C <= 32) xb[s] = load_c8_nt(x + v * C + 16 * s + 8 * hl);
                else xb[s] = load_c8(x + v * C + 16 * s + 8 * hl);
            }
            // ---- first product, bias, ReLU: the B fragments of the second product ----
            half8_t hb[KS2];
#pragma unroll
            for (int mt = 0; mt < MT1; ++mt) {
                float16_t acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
                for (int s = 0; s < KS1; ++s)
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1f[(mt * KS1 + s) * 64], xb[s], acc, 0, 0, 0);
                // acc[i]: hidden channel 32 mt + 8 (i/4) + 4 hl + i%4 of voxel vl
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const half4_t b4 = *reinterpret_cast<const half4_t*>(bs + 32 * mt + 8 * gq + 4 * hl);
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const half_t hsum = (half_t)((float)(half_t)acc[4 * gq + jj] + (float)b4[jj]);  // fp16 add, RNE
                        hb[2 * mt + gq / 2][4 * (gq % 2) + jj] = hsum > (half_t)0 ? hsum : (half_t)0;
                    }
                }
            }
            // ---- second product ----
#pragma unroll
            for (int mo = 0; mo < MO; ++mo) {
                float16_t acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
                for (int s = 0; s < KS2; ++s)
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2f[(mo * KS2 + s) * 64], hb[s], acc, 0, 0, 0);
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int co = 32 * mo + 8 * gq + 4 * hl;
                    if (co < C) {
                        half4_t o;
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) o[jj] = (half_t)acc[4 * gq + jj];
                        *reinterpret_cast<half4_t*>(my + Tile::piece(vl, 4 * mo + gq, hl)) = o;
                    }
                }
            }
            // ---- write-back of the wavefront's own tile: no other wavefront touches it, and the LDS
            // operations of one wavefront complete in issue order, so no workgroup barrier is needed ----
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int c0 = 0; c0 < 32 * C / 8; c0 += kWave) {
                const int c = c0 + lane;
                const int row = c / (C / 8), cc = c % (C / 8);
                if (c < 32 * C / 8 && v0 + row < V) {
                    half8_t o = Tile::read(my, row, cc);
                    const int64_t off = (v0 + row) * C + cc * 8;
                    const half8_t a8 = load_c8_nt(add + off);
#pragma unroll
                    for (int jj = 0; jj < 8; ++jj) o[jj] = (half_t)((float)o[jj] + (float)a8[jj]);  // fp16 add, RNE
                    store_c8_nt(out + off, o);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

static int mlp_blocks(int64_t V)
{
    const int64_t ntiles = (V + 31) / 32;
    int64_t b = (ntiles + kMlpWaves - 1) / kMlpWaves;
    if (b > 1024) b = 1024;
    return (int)std::max<int64_t>(b, 1);
}

}  // namespace kerops

using namespace kerops;

extern "C" int kerops_lin_brelu_lin_add_f16(const void* x, const void* Wup, const void* Wdown, const void* bias,
                                            const void* add, void* out, int64_t V, int32_t C, void* stream)
{
    if (!x || !Wup || !Wdown || !bias || !add || !out || !aligned16(x) || !aligned16(add) || !aligned16(out)) {
        set_error("lin_brelu_lin_add: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (V <= 0) {
        set_error("lin_brelu_lin_add: non-positive size");
        return KEROPS_E_BADARG;
    }
    const int blocks = mlp_blocks(V);
    hipStream_t s = (hipStream_t)stream;
#define KEROPS_MLP_CASE(CV)                                                                                      \
    if (C == CV) {                                                                                               \
        hipLaunchKernelGGL((lin_brelu_lin_add_kernel<CV>), dim3(blocks), dim3(kMlpThreads), 0, s,               \
                           (const half_t*)x, (const half_t*)Wup, (const half_t*)Wdown, (const half_t*)bias,     \
                           (const half_t*)add, (half_t*)out, V);                                                \
        return check_launch("lin_brelu_lin_add");                                                                \
    }
    KEROPS_MLP_CASE(16)
    KEROPS_MLP_CASE(32)
    KEROPS_MLP_CASE(64)
#undef KEROPS_MLP_CASE
    set_error("lin_brelu_lin_add: built for C in {16,32,64} (got %d)", C);
    return KEROPS_E_UNSUPPORTED_C;
}

// =============================================================================================
// Backward of the block above, one pass over x and grad:
//
//   linup = fp16(x @ Wup) + bias (fp16 add);  hid = relu(linup)
//   dWdown[h, c] = sum_v hid[v, h] * g[v, c]
//   lg[v, h]     = linup[v, h] > 0 ? fp16(sum_c Wdown[h, c] * g[v, c]) : 0
//   dWup[c, h]   = sum_v x[v, c] * lg[v, h];   dbias[h] = sum_v lg[v, h]
//   dx[v, c]     = fp16(sum_h Wup[c, h] * lg[v, h])
//
// Two kernels: C <= 32 (one block of in / out channels) runs lin_brelu_lin_bwd_wave_kernel further down,
// where a wavefront needs no LDS tiles and no workgroup barrier per tile; C = 64 runs the kernel below.
//
// A workgroup of four wavefronts loops over tiles of 64 voxels; x and g tiles are staged through LDS.
// Phase A: per (32 voxels, 32 hidden channels) block a wavefront computes linup^T and (Wdown g^T) with the
// same output layout, applies bias / ReLU / mask in registers and writes the hid and lg tiles to LDS.
// Phase B: dx^T = Wup lg^T from the lg tile (bounced through LDS for 16-byte stores), and the three
// reductions over voxels: the 32x32 blocks of dWdown = hid^T g and dWup = x^T lg take their fragments
// (8 consecutive voxels of one channel) from the LDS tiles with 2-byte reads and stay in fp32 registers
// for all tiles of the workgroup; dbias is a per-thread column sum of the lg tile.  Partials go to the
// workspace, a second kernel adds them in a fixed order (fp64): deterministic, no atomics.
namespace kerops {

constexpr int kMbTile = 64;

template <int C>
struct MbCfg {
    static constexpr int H = 2 * C;
    static constexpr int MH = H / 32, MO = (C + 31) / 32;  // 32-channel blocks of hidden / in-out channels
    static constexpr int KC = C / 16, KH = H / 16;         // k steps over C / over H
    static constexpr int KV = kMbTile / 16;                // k steps over the voxels of a tile
    static constexpr int XP = C + 8, HP = H + 8, DP = C;      // LDS row pitches in halves (the dx tile: dense rows, BounceTile)
    static constexpr int NBA = 2 * MH;                     // phase A blocks (vt, mh)
    static constexpr int NB6 = 2 * MO;                     // dx blocks (vt, mo)
    static constexpr int NU = 2 * MH * MO;                 // reduction blocks: (type, mh, mc)
    static constexpr int KSPL = NU >= kMlpWaves ? 1 : kMlpWaves / NU;
    static constexpr int UPW = NU >= kMlpWaves ? NU / kMlpWaves : 1;
    static constexpr int NXC = kMbTile * C / 8;            // 16-byte chunks of an x / g / dx tile
    static constexpr int NLX = (NXC + kMlpThreads - 1) / kMlpThreads;
    static constexpr int BPARTS = kMlpThreads / H;         // threads per hidden channel in the bias sum
    static constexpr int RW = 2 * C * H + H;               // floats of one partial: dWup, dWdown, dbias
    static constexpr int XS_OFF = 0;
    static constexpr int GS_OFF = XS_OFF + kMbTile * XP * 2;
    static constexpr int HS_OFF = GS_OFF + kMbTile * XP * 2;
    static constexpr int LS_OFF = HS_OFF + kMbTile * HP * 2;
    static constexpr int DS_OFF = LS_OFF + kMbTile * HP * 2;
    static constexpr int A1_OFF = (DS_OFF + kMbTile * DP * 2 + 15) / 16 * 16;
    static constexpr int A3_OFF = A1_OFF + MH * KC * 64 * 16;
    static constexpr int A6_OFF = A3_OFF + MH * KC * 64 * 16;
    static constexpr int BS_OFF = A6_OFF + MO * KH * 64 * 16;
    static constexpr int BH_OFF = BS_OFF + kMlpThreads * 4;  // fp16 copy of the bias
    static constexpr int LDS_BYTES = BH_OFF + H * 2;
    static_assert(C == 16 || C == 32 || C == 64, "C in {16,32,64}");
    static_assert(KV % KSPL == 0 && kMbTile % BPARTS == 0, "even splits");
};

template <int C>
__global__ __launch_bounds__(kMlpThreads) void lin_brelu_lin_bwd_kernel(const half_t* __restrict__ x,
                                                                        const half_t* __restrict__ g,
                                                                        const half_t* __restrict__ Wup,
                                                                        const half_t* __restrict__ Wdown,
                                                                        const half_t* __restrict__ bias,
                                                                        half_t* __restrict__ dx, float* __restrict__ ws,
                                                                        int64_t V)
{
    using Cfg = MbCfg<C>;
    constexpr int H = Cfg::H, MH = Cfg::MH, MO = Cfg::MO, KC = Cfg::KC, KH = Cfg::KH, KV = Cfg::KV;
    constexpr int XP = Cfg::XP, HP = Cfg::HP, DP = Cfg::DP, NLX = Cfg::NLX, KSPL = Cfg::KSPL, UPW = Cfg::UPW;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half_t* xs = reinterpret_cast<half_t*>(smem + Cfg::XS_OFF);
    half_t* gs = reinterpret_cast<half_t*>(smem + Cfg::GS_OFF);
    half_t* hs = reinterpret_cast<half_t*>(smem + Cfg::HS_OFF);
    half_t* ls = reinterpret_cast<half_t*>(smem + Cfg::LS_OFF);
    half_t* ds = reinterpret_cast<half_t*>(smem + Cfg::DS_OFF);
    half_t* a1 = reinterpret_cast<half_t*>(smem + Cfg::A1_OFF);
    half8_t* a3 = reinterpret_cast<half8_t*>(smem + Cfg::A3_OFF);
    half8_t* a6 = reinterpret_cast<half8_t*>(smem + Cfg::A6_OFF);
    float* bred = reinterpret_cast<float*>(smem + Cfg::BS_OFF);
    half_t* bsh = reinterpret_cast<half_t*>(smem + Cfg::BH_OFF);

    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int il = lane % 32, hl = lane / 32;
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // fragments of the three per-voxel products (lane l: row l%32 of the block, k = 16 s + 8 (l/32) + 0..7)
    // a1: linup^T = Wup^T x^T     -> Wup[k][32 mh + l%32]
    for (int i = t; i < MH * KC * 64 * 8; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KC, mh = i / (512 * KC);
        a1[i] = Wup[(16 * s + 8 * (l / 32) + j) * H + 32 * mh + l % 32];
    }
    // a3: (Wdown g^T)             -> Wdown[32 mh + l%32][k .. k+7]
    for (int i = t; i < MH * KC * 64; i += kMlpThreads) {
        const int l = i % 64, s = (i / 64) % KC, mh = i / (64 * KC);
        a3[i] = load_c8(Wdown + (32 * mh + l % 32) * C + 16 * s + 8 * (l / 32));
    }
    // a6: dx^T = Wup lg^T         -> Wup[32 mo + l%32][k .. k+7]
    for (int i = t; i < MO * KH * 64; i += kMlpThreads) {
        const int l = i % 64, s = (i / 64) % KH, mo = i / (64 * KH);
        const int c = 32 * mo + l % 32;
        a6[i] = c < C ? load_c8(Wup + c * H + 16 * s + 8 * (l / 32)) : z8;
    }
    for (int i = t; i < H; i += kMlpThreads) bsh[i] = bias[i];
    const half8_t* a1f = reinterpret_cast<const half8_t*>(a1);

    // reduction blocks of this wavefront: unit u = (type = u % 2, mh = (u / 2) % MH, mc = u / (2 MH));
    // type 0: dWdown[h, c] = hid^T g, type 1: dWup[c, h] = x^T lg
    const int u0 = Cfg::NU >= kMlpWaves ? wave : wave % Cfg::NU;
    const int kpart = Cfg::NU >= kMlpWaves ? 0 : wave / Cfg::NU;
    float16_t wacc[UPW];
#pragma unroll
    for (int uu = 0; uu < UPW; ++uu)
#pragma unroll
        for (int i = 0; i < 16; ++i) wacc[uu][i] = 0.0f;
    float bacc = 0.0f;  // dbias: hidden channel t % H, voxels t / H + BPARTS * n
    const int bh = t % H, bp = t / H;

    const int64_t ntiles = (V + kMbTile - 1) / kMbTile;
    half8_t xpre[NLX], gpre[NLX];
    auto prefetch = [&](int64_t tile) {
        const int64_t v0 = tile * kMbTile;
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kMlpThreads;
            const int64_t v = v0 + c / (C / 8);
            const bool ok = (c < Cfg::NXC) && (v < V);
            xpre[j] = ok ? load_c8_nt(x + v * C + (c % (C / 8)) * 8) : z8;
            gpre[j] = ok ? load_c8_nt(g + v * C + (c % (C / 8)) * 8) : z8;
        }
    };

    int64_t tile = blockIdx.x;
    if (tile < ntiles) prefetch(tile);
    for (; tile < ntiles; tile += gridDim.x) {
        const int64_t v0 = tile * kMbTile;
        // ---- stage the tile (rows past V are zero: they add nothing to the reductions) ----
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kMlpThreads;
            if (c < Cfg::NXC) {
                *reinterpret_cast<half8_t*>(xs + (c / (C / 8)) * XP + (c % (C / 8)) * 8) = xpre[j];
                *reinterpret_cast<half8_t*>(gs + (c / (C / 8)) * XP + (c % (C / 8)) * 8) = gpre[j];
            }
        }
        __syncthreads();
        if (tile + gridDim.x < ntiles) prefetch(tile + gridDim.x);

        // ---- phase A: hid and lg tiles, blocks (vt, mh) of 32 voxels x 32 hidden channels ----
#pragma unroll
        for (int ba = 0; ba < (Cfg::NBA + kMlpWaves - 1) / kMlpWaves; ++ba) {
            const int blk = wave + ba * kMlpWaves;
            if (blk < Cfg::NBA) {  // wavefront-uniform
                const int vt = blk % 2, mh = blk / 2;
                const int row = 32 * vt + il;
                float16_t up, dn;
#pragma unroll
                for (int i = 0; i < 16; ++i) up[i] = dn[i] = 0.0f;
#pragma unroll
                for (int s = 0; s < KC; ++s) {
                    const half8_t xb = *reinterpret_cast<const half8_t*>(xs + row * XP + 16 * s + 8 * hl);
                    const half8_t gb = *reinterpret_cast<const half8_t*>(gs + row * XP + 16 * s + 8 * hl);
                    up = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1f[(mh * KC + s) * 64 + lane], xb, up, 0, 0, 0);
                    dn = __builtin_amdgcn_mfma_f32_32x32x16_f16(a3[(mh * KC + s) * 64 + lane], gb, dn, 0, 0, 0);
                }
                // up[i], dn[i]: hidden channel 32 mh + 8 (i/4) + 4 hl + i%4 of voxel row
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int hc = 32 * mh + 8 * gq + 4 * hl;
                    const half4_t b4 = *reinterpret_cast<const half4_t*>(bsh + hc);
                    half4_t hv, lv;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const half_t lin = (half_t)((float)(half_t)up[4 * gq + jj] + (float)b4[jj]);  // fp16 add
                        const bool pos = lin > (half_t)0;
                        hv[jj] = pos ? lin : (half_t)0;
                        lv[jj] = pos ? (half_t)dn[4 * gq + jj] : (half_t)0;
                    }
                    // rows past V hold x = g = 0: hid = relu(bias) there, which must not reach dWdown ... but
                    // it is multiplied by g = 0; lg = fp16(0) = 0, so dWup and dbias are unaffected as well
                    *reinterpret_cast<half4_t*>(hs + row * HP + hc) = hv;
                    *reinterpret_cast<half4_t*>(ls + row * HP + hc) = lv;
                }
            }
        }
        __syncthreads();

        // ---- phase B1: dx^T blocks (vt, mo) from the lg tile ----
#pragma unroll
        for (int b6 = 0; b6 < (Cfg::NB6 + kMlpWaves - 1) / kMlpWaves; ++b6) {
            const int blk = wave + b6 * kMlpWaves;
            if (blk < Cfg::NB6) {  // wavefront-uniform
                const int vt = blk % 2, mo = blk / 2;
                const int row = 32 * vt + il;
                float16_t acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
                for (int s = 0; s < KH; ++s) {
                    const half8_t lb = *reinterpret_cast<const half8_t*>(ls + row * HP + 16 * s + 8 * hl);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a6[(mo * KH + s) * 64 + lane], lb, acc, 0, 0, 0);
                }
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int c = 32 * mo + 8 * gq + 4 * hl;
                    if (c < C) {
                        half4_t o;
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) o[jj] = (half_t)acc[4 * gq + jj];
                        *reinterpret_cast<half4_t*>(reinterpret_cast<unsigned char*>(ds) + BounceTile<C>::piece(row, 4 * mo + gq, hl)) = o;
                    }
                }
            }
        }
        // ---- phase B2: the reductions over the voxels of the tile ----
#pragma unroll
        for (int uu = 0; uu < UPW; ++uu) {
            const int u = u0 + uu * kMlpWaves;
            const int type = u % 2, mh = (u / 2) % MH, mc = u / (2 * MH);
            const int cc = min(32 * mc + il, C - 1), hh = 32 * mh + il;
            // A rows / B columns: type 0: (hid[:, hh], g[:, cc]); type 1: (x[:, cc], lg[:, hh])
            const half_t* ap = type == 0 ? hs + hh : xs + cc;
            const half_t* bp2 = type == 0 ? gs + cc : ls + hh;
            const int apitch = type == 0 ? HP : XP, bpitch = type == 0 ? XP : HP;
#pragma unroll
            for (int sp = 0; sp < KV / KSPL; ++sp) {
                const int s = kpart + sp * KSPL;
                half8_t af, bf;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    af[jj] = ap[(16 * s + 8 * hl + jj) * apitch];
                    bf[jj] = bp2[(16 * s + 8 * hl + jj) * bpitch];
                }
                wacc[uu] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, wacc[uu], 0, 0, 0);
            }
        }
        // dbias: column sums of the lg tile
#pragma unroll
        for (int n = 0; n < kMbTile / Cfg::BPARTS; ++n) bacc += (float)ls[(bp + Cfg::BPARTS * n) * HP + bh];
        __syncthreads();

        // ---- phase C: dx write-back, 16-byte chunks ----
#pragma unroll
        for (int j = 0; j < NLX; ++j) {
            const int c = t + j * kMlpThreads;
            const int row = c / (C / 8), cc = c % (C / 8);
            if (c < Cfg::NXC && v0 + row < V) {
                const half8_t o = BounceTile<C>::read(reinterpret_cast<const unsigned char*>(ds), row, cc);
                store_c8_nt(dx + (v0 + row) * C + cc * 8, o);
            }
        }
        __syncthreads();
    }

    // ---- partials of this workgroup: row (blockIdx, kpart) = [dWup C*H][dWdown H*C][dbias H] ----
    float* out = ws + ((int64_t)blockIdx.x * KSPL + kpart) * Cfg::RW;
#pragma unroll
    for (int uu = 0; uu < UPW; ++uu) {
        const int u = u0 + uu * kMlpWaves;
        const int type = u % 2, mh = (u / 2) % MH, mc = u / (2 * MH);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int ri = 8 * (i / 4) + 4 * hl + i % 4;  // row of the block held in register i
            if (type == 0) {  // D[i = h][j = c]
                const int h = 32 * mh + ri, c = 32 * mc + il;
                if (c < C) out[C * H + h * C + c] = wacc[uu][i];
            } else {  // D[i = c][j = h]
                const int c = 32 * mc + ri, h = 32 * mh + il;
                if (c < C) out[c * H + h] = wacc[uu][i];
            }
        }
    }
    bred[t] = bacc;
    __syncthreads();
    if (t < H) {
        float s = 0.0f;
#pragma unroll
        for (int p = 0; p < Cfg::BPARTS; ++p) s += bred[p * H + t];
        ws[((int64_t)blockIdx.x * KSPL) * Cfg::RW + 2 * C * H + t] = s;
        for (int kp = 1; kp < KSPL; ++kp) ws[((int64_t)blockIdx.x * KSPL + kp) * Cfg::RW + 2 * C * H + t] = 0.0f;
    }
}

// ---------------------------------------------------------------------------------------------
// C <= 32: every wavefront works alone on tiles of 32 voxels, no workgroup barrier inside the loop.
//
// The per-voxel products want "voxel per lane" results (lane = voxel, registers = channels: the B operand
// of the next per-voxel product), the reductions over voxels want "channel per lane" operands (lane =
// channel, registers = 8 voxels).  A 32x32 matrix-core block D = A B holds column j in lane j%32, so the
// second form of a tile M[v][c] is the product M I with an identity B fragment: exact, since every sum has
// one non-zero term.  Fragments of x and g come straight from global memory (16-byte chunk 2 s + l/32 of
// voxel l%32: the same registers serve as A operand of the transposing product and B operand of the
// per-voxel products); hid and lg are transposed from their packed fp16 registers, whose reduction index
// runs over the hidden channels in the order the accumulator leaves them, with a matching permuted
// identity.  Weight and identity fragments sit in LDS (one 16-byte read per lane and use).  The
// accumulators of dWup, dWdown and dbias stay in registers for all tiles of the wavefront; at the end the
// four wavefronts add theirs in LDS in a fixed order and the workgroup writes one partial row.
template <int C>
struct MtCfg {
    static constexpr int H = 2 * C;
    static constexpr int MH = H / 32;   // 32-channel blocks of the hidden channels
    static constexpr int KC = C / 16;   // k steps over the in / out channels
    static constexpr int DP = C;        // row pitch of the dx tile (halves): dense rows, BounceTile in common.hpp
    static constexpr int RW = 2 * C * H + H;
    static constexpr int F1_OFF = 0;                              // Wup^T rows   [mh][s]
    static constexpr int F2_OFF = F1_OFF + MH * KC * 1024;        // Wdown rows   [mh][s]
    static constexpr int F3_OFF = F2_OFF + MH * KC * 1024;        // Wup rows, hidden order of the accumulator
    static constexpr int IP_OFF = F3_OFF + 2 * MH * 1024;         // identity in that order [half]
    static constexpr int ID_OFF = IP_OFF + 2 * 1024;              // identity [s]
    static constexpr int BH_OFF = ID_OFF + KC * 1024;             // bias
    static constexpr int DS_OFF = (BH_OFF + H * 2 + 15) / 16 * 16;
    static constexpr int LOOP_BYTES = DS_OFF + kMlpWaves * 32 * DP * 2;
    static constexpr int LDS_BYTES = LOOP_BYTES > RW * 4 ? LOOP_BYTES : RW * 4;
    static_assert(C == 16 || C == 32, "one 32-channel block of in / out channels");
};

// fp32 accumulator -> the two packed fp16 operands (registers 0..7 and 8..15)
__device__ __forceinline__ void pack_acc(const float16_t& a, half8_t& lo, half8_t& hi)
{
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        lo[i] = (half_t)a[i];
        hi[i] = (half_t)a[8 + i];
    }
}

typedef short i16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

// Two neighbouring accumulator registers of both products -> packed (hid, lg), 16-bit packed operations only:
// lin = fp16(up) + bias (fp16 add);  hid = relu(lin) as the signed integer maximum of the bit pattern with 0
// (negative values and -0 have the sign bit set, positive ones compare like integers);  lg = fp16(dn) where
// hid has a non-zero bit pattern, i.e. where lin > 0.
__device__ __forceinline__ void hid_lg_pair(float u0, float u1, float d0, float d1, half2_t b, half2_t& hid,
                                            half2_t& lg)
{
    const half2_t up2 = {(half_t)u0, (half_t)u1};
    const half2_t dn2 = {(half_t)d0, (half_t)d1};
    const half2_t lin = up2 + b;
    const i16x2_t hb = __builtin_elementwise_max(__builtin_bit_cast(i16x2_t, lin), i16x2_t{0, 0});
    hid = __builtin_bit_cast(half2_t, hb);
    const u16x2_t one = {1, 1}, zero = {0, 0};
    uint32_t nz;  // written out: the compiler would turn the minimum into two compares and selects
    asm("v_pk_min_u16 %0, %1, %2" : "=v"(nz) : "v"(__builtin_bit_cast(uint32_t, hb)), "v"(__builtin_bit_cast(uint32_t, one)));
    const u16x2_t m = zero - __builtin_bit_cast(u16x2_t, nz);  // 0 or 0xffff per half
    lg = __builtin_bit_cast(half2_t, __builtin_bit_cast(uint32_t, dn2) & __builtin_bit_cast(uint32_t, m));
}

template <int C>
__global__ __launch_bounds__(kMlpThreads, 2) void lin_brelu_lin_bwd_wave_kernel(
    const half_t* __restrict__ x, const half_t* __restrict__ g, const half_t* __restrict__ Wup,
    const half_t* __restrict__ Wdown, const half_t* __restrict__ bias, half_t* __restrict__ dx,
    float* __restrict__ ws, int64_t V)
{
    using Cfg = MtCfg<C>;
    constexpr int H = Cfg::H, MH = Cfg::MH, KC = Cfg::KC, DP = Cfg::DP;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half_t* f1w = reinterpret_cast<half_t*>(smem + Cfg::F1_OFF);
    half_t* f3w = reinterpret_cast<half_t*>(smem + Cfg::F3_OFF);
    half_t* ipw = reinterpret_cast<half_t*>(smem + Cfg::IP_OFF);
    half_t* idw = reinterpret_cast<half_t*>(smem + Cfg::ID_OFF);
    half_t* bsh = reinterpret_cast<half_t*>(smem + Cfg::BH_OFF);

    const int t = threadIdx.x, lane = t % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(t / kWave);  // scalar: tile indices stay wavefront-uniform
    const int il = lane % 32, hl = lane / 32;
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // hidden channel (within a block of 32) that element j of reduction group `half` of lane half hl holds
    auto hperm = [](int half, int hl_, int j) { return 16 * half + 8 * (j / 4) + 4 * hl_ + j % 4; };

    for (int i = t; i < MH * KC * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KC, mh = i / (512 * KC);
        f1w[i] = Wup[(16 * s + 8 * (l / 32) + j) * H + 32 * mh + l % 32];
    }
    for (int i = t; i < MH * KC * 64; i += kMlpThreads) {
        const int l = i % 64, s = (i / 64) % KC, mh = i / (64 * KC);
        reinterpret_cast<half8_t*>(smem + Cfg::F2_OFF)[i] = load_c8(Wdown + (32 * mh + l % 32) * C + 16 * s + 8 * (l / 32));
    }
    for (int i = t; i < 2 * MH * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, f = i / 512;
        const int c = l % 32, h = 32 * (f / 2) + hperm(f % 2, l / 32, j);
        f3w[i] = c < C ? Wup[c * H + h] : (half_t)0;
    }
    for (int i = t; i < 2 * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, half = i / 512;
        ipw[i] = hperm(half, l / 32, j) == l % 32 ? (half_t)1 : (half_t)0;
    }
    for (int i = t; i < KC * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = i / 512;
        idw[i] = 16 * s + 8 * (l / 32) + j == l % 32 ? (half_t)1 : (half_t)0;
    }
    for (int i = t; i < H; i += kMlpThreads) bsh[i] = bias[i];
    __syncthreads();

    const half8_t* f1 = reinterpret_cast<const half8_t*>(smem + Cfg::F1_OFF) + lane;
    const half8_t* f2 = reinterpret_cast<const half8_t*>(smem + Cfg::F2_OFF) + lane;
    const half8_t* f3 = reinterpret_cast<const half8_t*>(smem + Cfg::F3_OFF) + lane;
    const half8_t* ip = reinterpret_cast<const half8_t*>(smem + Cfg::IP_OFF) + lane;
    const half8_t* id = reinterpret_cast<const half8_t*>(smem + Cfg::ID_OFF) + lane;
    unsigned char* my = smem + Cfg::DS_OFF + wave * 32 * DP * 2;
    using Tile = BounceTile<C>;

    float16_t wdn[MH], wup[MH];  // dWdown block: D[h][c];  dWup block: D[c][h]
    float bacc[MH];
#pragma unroll
    for (int mh = 0; mh < MH; ++mh) {
#pragma unroll
        for (int i = 0; i < 16; ++i) wdn[mh][i] = wup[mh][i] = 0.0f;
        bacc[mh] = 0.0f;
    }

    const int64_t ntiles = (V + 31) / 32;
    const int64_t stride = (int64_t)gridDim.x * kMlpWaves;
    half8_t xn[KC], gn[KC];
    auto fetch = [&](int64_t tile) {  // rows past V read the last voxel and are zeroed before use
        int64_t v = tile * 32 + il;
        v = v < V ? v : V - 1;
#pragma unroll
        for (int s = 0; s < KC; ++s) {
            xn[s] = load_c8_nt(x + v * C + 16 * s + 8 * hl);
            gn[s] = load_c8_nt(g + v * C + 16 * s + 8 * hl);
        }
    };

    // dx leaves one tile late: the wait for the operands of a tile then only covers stores issued a whole
    // tile earlier (the memory counter retires loads and stores in issue order)
    auto flush = [&](int64_t pv0, bool ragged) {
#pragma unroll
        for (int c0 = 0; c0 < 32 * C / 8; c0 += kWave) {
            const int c = c0 + lane;
            const int row = c / (C / 8), cc = c % (C / 8);
            if (!ragged || pv0 + row < V) {
                store_c8_nt(dx + (pv0 + row) * C + cc * 8, Tile::read(my, row, cc));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    const int64_t first = (int64_t)blockIdx.x * kMlpWaves + wave;
    int64_t tile = first;
    if (tile < ntiles) fetch(tile);
    for (; tile < ntiles; tile += stride) {
        const int64_t v0 = tile * 32;
        half8_t xc[KC], gc[KC];
#pragma unroll
        for (int s = 0; s < KC; ++s) {
            xc[s] = xn[s];
            gc[s] = gn[s];
        }
        if (v0 + 32 > V) {  // ragged last tile (wavefront-uniform)
            const bool ok = v0 + il < V;
#pragma unroll
            for (int s = 0; s < KC; ++s) {
                xc[s] = ok ? xc[s] : z8;
                gc[s] = ok ? gc[s] : z8;
            }
        }
        if (tile != first) flush(v0 - stride * 32, false);  // an earlier tile of this wavefront is never ragged
        {
            const int64_t nt = tile + stride;
            fetch(nt < ntiles ? nt : tile);
        }
        __builtin_amdgcn_sched_barrier(0);

        // x^T, g^T: lane = channel, registers = voxels 8 (i/4) + 4 hl + i%4
        half8_t xT[2], gT[2];
        {
            float16_t tx, tg;
#pragma unroll
            for (int i = 0; i < 16; ++i) tx[i] = tg[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < KC; ++s) {
                const half8_t e = id[s * 64];
                tx = __builtin_amdgcn_mfma_f32_32x32x16_f16(xc[s], e, tx, 0, 0, 0);
                tg = __builtin_amdgcn_mfma_f32_32x32x16_f16(gc[s], e, tg, 0, 0, 0);
            }
            pack_acc(tx, xT[0], xT[1]);
            pack_acc(tg, gT[0], gT[1]);
        }

        float16_t dacc;  // dx^T: D[c][v]
#pragma unroll
        for (int i = 0; i < 16; ++i) dacc[i] = 0.0f;

#pragma unroll
        for (int mh = 0; mh < MH; ++mh) {
            float16_t up, dn;
#pragma unroll
            for (int i = 0; i < 16; ++i) up[i] = dn[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < KC; ++s) {
                up = __builtin_amdgcn_mfma_f32_32x32x16_f16(f1[(mh * KC + s) * 64], xc[s], up, 0, 0, 0);
                dn = __builtin_amdgcn_mfma_f32_32x32x16_f16(f2[(mh * KC + s) * 64], gc[s], dn, 0, 0, 0);
            }
            // up[i], dn[i]: hidden channel 32 mh + 8 (i/4) + 4 hl + i%4 of voxel il
            half8_t hv[2], lv[2];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const half4_t b4 = *reinterpret_cast<const half4_t*>(bsh + 32 * mh + 8 * gq + 4 * hl);
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    const int i = 4 * gq + 2 * jp, e = 4 * (gq % 2) + 2 * jp;
                    half2_t hid, lg;
                    hid_lg_pair(up[i], up[i + 1], dn[i], dn[i + 1], half2_t{b4[2 * jp], b4[2 * jp + 1]}, hid, lg);
                    hv[gq / 2][e] = hid[0];
                    hv[gq / 2][e + 1] = hid[1];
                    lv[gq / 2][e] = lg[0];
                    lv[gq / 2][e + 1] = lg[1];
                }
            }
            // rows past V hold x = g = 0: hid = relu(bias) there meets g = 0 in dWdown, lg = 0 everywhere else
            dacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(f3[(2 * mh) * 64], lv[0], dacc, 0, 0, 0);
            dacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(f3[(2 * mh + 1) * 64], lv[1], dacc, 0, 0, 0);

            // hid^T, lg^T: lane = hidden channel 32 mh + il, registers = voxels
            half8_t hT[2], lT[2];
            {
                float16_t th, tl;
#pragma unroll
                for (int i = 0; i < 16; ++i) th[i] = tl[i] = 0.0f;
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const half8_t e = ip[hf * 64];
                    th = __builtin_amdgcn_mfma_f32_32x32x16_f16(hv[hf], e, th, 0, 0, 0);
                    tl = __builtin_amdgcn_mfma_f32_32x32x16_f16(lv[hf], e, tl, 0, 0, 0);
                }
                pack_acc(th, hT[0], hT[1]);
#pragma unroll
                for (int i = 0; i < 16; ++i) bacc[mh] += tl[i];
                pack_acc(tl, lT[0], lT[1]);
            }
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                wdn[mh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hT[hf], gT[hf], wdn[mh], 0, 0, 0);
                wup[mh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xT[hf], lT[hf], wup[mh], 0, 0, 0);
            }
        }

        // ---- dx: into the wavefront's own LDS tile; the LDS operations of one wavefront complete in issue
        // order, so no workgroup barrier is needed ----
#pragma unroll
        for (int gq = 0; gq < C / 8; ++gq) {
            half4_t o;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) o[jj] = (half_t)dacc[4 * gq + jj];
            *reinterpret_cast<half4_t*>(my + Tile::piece(il, gq, hl)) = o;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (first < ntiles) flush((tile - stride) * 32, true);

    // ---- the four wavefronts add their partials in LDS, wavefront 0 first: [dWup C*H][dWdown H*C][dbias H] ----
    float* red = reinterpret_cast<float*>(smem);
    __syncthreads();  // every wavefront is done with the fragments
#pragma unroll 1
    for (int w = 0; w < kMlpWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int mh = 0; mh < MH; ++mh) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int ri = 8 * (i / 4) + 4 * hl + i % 4;  // row of the block held in register i
                    if (il < C) {  // dWdown[h = 32 mh + ri][c = il]
                        float* p = red + C * H + (32 * mh + ri) * C + il;
                        *p = w == 0 ? wdn[mh][i] : *p + wdn[mh][i];
                    }
                    if (ri < C) {  // dWup[c = ri][h = 32 mh + il]
                        float* p = red + ri * H + 32 * mh + il;
                        *p = w == 0 ? wup[mh][i] : *p + wup[mh][i];
                    }
                }
                const float b = bacc[mh] + __shfl_xor(bacc[mh], 32);  // both lane halves hold 16 voxels each
                if (hl == 0) {
                    float* p = red + 2 * C * H + 32 * mh + il;
                    *p = w == 0 ? b : *p + b;
                }
            }
        }
        __syncthreads();
    }
    float* out = ws + (int64_t)blockIdx.x * Cfg::RW;
    for (int i = t; i < Cfg::RW; i += kMlpThreads) out[i] = red[i];
}

// ---------------------------------------------------------------------------------------------
// C = 32 with transposing LDS reads.
//
// Same tiles, products and accumulators as lin_brelu_lin_bwd_wave_kernel; what differs is how the "channel per
// lane" operands of the two weight-gradient products are made.  gfx950 reads LDS transposed: ds_read_b64_tr_b16
// takes, in every block of 16 lanes, the 16 x 4 matrix M of 16-bit values that the lanes address (lane s supplies
// the address of four consecutive values M[s][0..3]) and returns to lane i the values M[4 j + i/4][i%4], j = 0..3.
// With lane s pointing at row s/4, columns 4 (s%4) .. 4 (s%4) + 3 of a row-major [voxel][channel] tile, lane i
// receives channel i of four consecutive voxels: one instruction transposes a 4 x 16 patch, two of them make the
// eight reduction values of a 32x32x16 operand.  So the x, g, hid and lg tiles of a wavefront are written to its own
// LDS area as they sit in the registers (one 64-byte row per voxel) and read back transposed, instead of being
// multiplied with an identity on the matrix cores and converted back to fp16: 12 of 32 matrix instructions and the
// conversions of their results go.
// LDS layout: measured on gfx950, reads see 64 banks of 4 bytes (32 lanes of an 8-byte read or 16 lanes of a 16-byte
// read per clock), writes see 32 (16 lanes of an 8-byte write, 8 lanes of a 16-byte write per clock).  Chunk c of
// row r sits in chunk slot c ^ tr_slot(r) = c ^ ((r / 2) % 4) ^ ((r / 8) % 2): the eight rows of a write phase then
// cover the 128 bytes of write banks once, the sixteen rows of a 16-byte read phase (the same chunk of each) the 256
// of read banks once, and a transposing read phase takes four whole rows.
// x and g are fetched as whole rows (one instruction = 16 voxels x 64 bytes = 1 KB of consecutive memory) into the
// tiles; the lane's own row comes back from there as the operand of the per-voxel products.
// The hidden channels of a tile row are stored in the order the accumulator leaves them (position p of the row is
// hidden channel tr_hidden(p) of the 32-block), which only permutes the rows / columns of the gradient blocks.
// The bias gradient is a product of its own on the 16x16x32 instruction: an operand of ones in row 0 for the even
// 16-lane groups and in row 1 for the odd ones adds the lg values of hidden positions 0..15 and 16..31.
struct MrCfg {
    static constexpr int C = 32, H = 64, MH = 2, KC = 2;
    static constexpr int RW = 2 * C * H + H;
    static constexpr int F1_OFF = 0;                              // Wup^T rows   [mh][s]
    static constexpr int F2_OFF = F1_OFF + MH * KC * 1024;        // Wdown rows   [mh][s]
    static constexpr int F3_OFF = F2_OFF + MH * KC * 1024;        // Wup rows, hidden order of the accumulator
    static constexpr int BH_OFF = F3_OFF + 2 * MH * 1024;         // bias
    static constexpr int WV_OFF = (BH_OFF + H * 2 + 15) / 16 * 16;
    static constexpr int TILE = 32 * 64;                          // one [32 voxels][32 values] fp16 tile
    static constexpr int WV_BYTES = 5 * TILE;                     // per wavefront: x, g, hid, lg, dx
    static constexpr int LOOP_BYTES = WV_OFF + kMlpWaves * WV_BYTES;
    static constexpr int LDS_BYTES = LOOP_BYTES > RW * 4 ? LOOP_BYTES : RW * 4;
};

// chunk-slot swizzle of tile row r (unchanged by r + 16)
__host__ __device__ constexpr int tr_slot(int r) { return ((r >> 1) & 3) ^ ((r >> 3) & 1); }
// hidden channel (inside its block of 32) stored at position p of a tile row
__host__ __device__ constexpr int tr_hidden(int p) { return 16 * (p / 16) + 8 * ((p % 8) / 4) + 4 * ((p / 8) % 2) + p % 4; }


__global__ __launch_bounds__(kMlpThreads, 2) void lin_brelu_lin_bwd_tr_kernel(
    const half_t* __restrict__ x, const half_t* __restrict__ g, const half_t* __restrict__ Wup,
    const half_t* __restrict__ Wdown, const half_t* __restrict__ bias, half_t* __restrict__ dx,
    float* __restrict__ ws, int64_t V)
{
    using Cfg = MrCfg;
    constexpr int C = Cfg::C, H = Cfg::H, MH = Cfg::MH, KC = Cfg::KC, TILE = Cfg::TILE;
    __shared__ __attribute__((aligned(16))) unsigned char smem[Cfg::LDS_BYTES];
    half_t* f1w = reinterpret_cast<half_t*>(smem + Cfg::F1_OFF);
    half_t* f3w = reinterpret_cast<half_t*>(smem + Cfg::F3_OFF);
    half_t* bsh = reinterpret_cast<half_t*>(smem + Cfg::BH_OFF);

    const int t = threadIdx.x, lane = t % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(t / kWave);  // scalar: tile indices stay wavefront-uniform
    const int il = lane % 32, hl = lane / 32;
    const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // hidden channel (within a block of 32) that element j of reduction group `half` of lane half hl holds
    auto hperm = [](int half, int hl_, int j) { return 16 * half + 8 * (j / 4) + 4 * hl_ + j % 4; };

    for (int i = t; i < MH * KC * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KC, mh = i / (512 * KC);
        f1w[i] = Wup[(16 * s + 8 * (l / 32) + j) * H + 32 * mh + l % 32];
    }
    for (int i = t; i < MH * KC * 64; i += kMlpThreads) {
        const int l = i % 64, s = (i / 64) % KC, mh = i / (64 * KC);
        reinterpret_cast<half8_t*>(smem + Cfg::F2_OFF)[i] = load_c8(Wdown + (32 * mh + l % 32) * C + 16 * s + 8 * (l / 32));
    }
    for (int i = t; i < 2 * MH * 512; i += kMlpThreads) {
        const int j = i % 8, l = (i / 8) % 64, f = i / 512;
        f3w[i] = Wup[(l % 32) * H + 32 * (f / 2) + hperm(f % 2, l / 32, j)];
    }
    for (int i = t; i < H; i += kMlpThreads) bsh[i] = bias[i];
    __syncthreads();

    const half8_t* f1 = reinterpret_cast<const half8_t*>(smem + Cfg::F1_OFF) + lane;
    const half8_t* f2 = reinterpret_cast<const half8_t*>(smem + Cfg::F2_OFF) + lane;
    const half8_t* f3 = reinterpret_cast<const half8_t*>(smem + Cfg::F3_OFF) + lane;
    unsigned char* mine = smem + Cfg::WV_OFF + wave * Cfg::WV_BYTES;
    unsigned char* xt = mine;             // [32 voxels][32 channels]
    unsigned char* gt = mine + TILE;
    unsigned char* ht = mine + 2 * TILE;  // [32 voxels][32 hidden positions] of the current block
    unsigned char* lt = mine + 3 * TILE;
    unsigned char* dt = mine + 4 * TILE;  // [32 voxels][32 channels] of dx

    // the lane's row: 16-byte chunks hl and 2 + hl
    const int wsw = tr_slot(il);
    const int woff0 = il * 64 + ((hl ^ wsw) * 16), woff1 = il * 64 + (((2 + hl) ^ wsw) * 16);
    // the fetched chunk: row lane / 4 (+ 16 for the second instruction: the same swizzle term), chunk lane % 4
    const int foff = (lane / 4) * 64 + (((lane % 4) ^ tr_slot(lane / 4)) * 16);
    // transposing read of reduction half hf: lane (il, hl) receives position il of the voxels 16 hf + 8 hl + 0..7;
    // inside its block of 16 lanes, lane s addresses row 8 hl + 4 r + s/4, positions 16 (block % 2) + 4 (s%4) ..
    // (rows 16 hf + ...: the swizzle term does not depend on hf)
    int toff[2];
    {
        const int s = lane % 16, blk = lane / 16;
        const int pos = 16 * (blk % 2) + 4 * (s % 4);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int row = 8 * (blk / 2) + 4 * r + s / 4;
            toff[r] = row * 64 + (((pos / 8) ^ tr_slot(row)) * 16) + (pos % 8) * 2;
        }
    }
    auto read_T = [&](const unsigned char* tile, int hf) {
        const half4_t a = lds_read_tr16(tile + hf * 1024 + toff[0]);
        const half4_t b = lds_read_tr16(tile + hf * 1024 + toff[1]);
        return half8_t{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    };
    auto wave_sync = [] {  // LDS operations of one wavefront complete in issue order: only the compiler must not reorder
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // bias gradient: ones in row 0 for the even 16-lane groups, in row 1 for the odd ones
    const half_t one_h = (lane % 16) == ((lane / 16) % 2) ? (half_t)1 : (half_t)0;
    const half8_t ones = {one_h, one_h, one_h, one_h, one_h, one_h, one_h, one_h};

    float16_t wdn[MH], wup[MH];  // dWdown block: D[h][c];  dWup block: D[c][h]
    float4_t bacc[MH];
#pragma unroll
    for (int mh = 0; mh < MH; ++mh) {
#pragma unroll
        for (int i = 0; i < 16; ++i) wdn[mh][i] = wup[mh][i] = 0.0f;
        bacc[mh] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    const int64_t ntiles = (V + 31) / 32;
    const int64_t stride = (int64_t)gridDim.x * kMlpWaves;
    half8_t xn[KC], gn[KC];
    // one instruction fetches 16 whole rows (1 KB): lane -> 16-byte chunk lane % 4 of voxel 16 s + lane / 4
    // (rows past V read the last voxel and are zeroed before use)
    auto fetch = [&](int64_t tile) {
#pragma unroll
        for (int s = 0; s < KC; ++s) {
            int64_t v = tile * 32 + 16 * s + lane / 4;
            v = v < V ? v : V - 1;
            xn[s] = load_c8_nt(x + v * C + (lane % 4) * 8);
            gn[s] = load_c8_nt(g + v * C + (lane % 4) * 8);
        }
    };

    // dx leaves one tile late: the wait for the operands of a tile then only covers stores issued a whole
    // tile earlier (the memory counter retires loads and stores in issue order)
    auto flush = [&](int64_t pv0, bool ragged) {
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {  // lane -> 16-byte chunk lane % 4 of row 16 pass + lane / 4
            const int row = 16 * pass + lane / 4, cc = lane % 4;
            if (!ragged || pv0 + row < V) {
                const half8_t o = *reinterpret_cast<const half8_t*>(dt + row * 64 + ((cc ^ tr_slot(row)) * 16));
                // rows 8..15 and 24..31 hold the two 8-byte halves of a chunk swapped
                const bool sw = (row >> 3) & 1;
                const half8_t w = {sw ? o[4] : o[0], sw ? o[5] : o[1], sw ? o[6] : o[2], sw ? o[7] : o[3],
                                   sw ? o[0] : o[4], sw ? o[1] : o[5], sw ? o[2] : o[6], sw ? o[3] : o[7]};
                store_c8_nt(dx + (pv0 + row) * C + cc * 8, w);
            }
        }
        wave_sync();
    };

    const int64_t first = (int64_t)blockIdx.x * kMlpWaves + wave;
    int64_t tile = first;
    if (tile < ntiles) fetch(tile);
    for (; tile < ntiles; tile += stride) {
        const int64_t v0 = tile * 32;
        half8_t xc[KC], gc[KC];
#pragma unroll
        for (int s = 0; s < KC; ++s) {
            xc[s] = xn[s];
            gc[s] = gn[s];
        }
        if (v0 + 32 > V) {  // ragged last tile (wavefront-uniform)
#pragma unroll
            for (int s = 0; s < KC; ++s) {
                const bool ok = v0 + 16 * s + lane / 4 < V;
                xc[s] = ok ? xc[s] : z8;
                gc[s] = ok ? gc[s] : z8;
            }
        }
        if (tile != first) flush(v0 - stride * 32, false);  // an earlier tile of this wavefront is never ragged
        {
            const int64_t nt = tile + stride;
            fetch(nt < ntiles ? nt : tile);
        }
        __builtin_amdgcn_sched_barrier(0);

        // x and g into the tiles as fetched; back as the lane's own row (chunks hl and 2 + hl: the operands of the
        // per-voxel products) and transposed
        *reinterpret_cast<half8_t*>(xt + foff) = xc[0];
        *reinterpret_cast<half8_t*>(xt + 1024 + foff) = xc[1];
        *reinterpret_cast<half8_t*>(gt + foff) = gc[0];
        *reinterpret_cast<half8_t*>(gt + 1024 + foff) = gc[1];
        wave_sync();
        xc[0] = *reinterpret_cast<const half8_t*>(xt + woff0);
        xc[1] = *reinterpret_cast<const half8_t*>(xt + woff1);
        gc[0] = *reinterpret_cast<const half8_t*>(gt + woff0);
        gc[1] = *reinterpret_cast<const half8_t*>(gt + woff1);
        half8_t xT[2], gT[2];  // lane = channel, registers = voxels 16 hf + 8 hl + 0..7
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            xT[hf] = read_T(xt, hf);
            gT[hf] = read_T(gt, hf);
        }

        float16_t dacc;  // dx^T: D[c][v]
#pragma unroll
        for (int i = 0; i < 16; ++i) dacc[i] = 0.0f;

            // (measurement switch: -DKEROPS_MLP_MH=0 builds the kernel without its arithmetic, i.e. the time of its
            // memory traffic alone: 0.56 ms at (1,32,350,350,128) against 0.61 ms with the arithmetic; two more tiles
            // in flight per wavefront change neither, half as many wavefronts per compute unit bring the traffic
            // alone to 0.52 ms and the whole kernel to 0.69 ms)
#ifndef KEROPS_MLP_MH
#define KEROPS_MLP_MH MH
#endif
#pragma unroll
        for (int mh = 0; mh < KEROPS_MLP_MH; ++mh) {
            float16_t up, dn;
#pragma unroll
            for (int i = 0; i < 16; ++i) up[i] = dn[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < KC; ++s) {
                up = __builtin_amdgcn_mfma_f32_32x32x16_f16(f1[(mh * KC + s) * 64], xc[s], up, 0, 0, 0);
                dn = __builtin_amdgcn_mfma_f32_32x32x16_f16(f2[(mh * KC + s) * 64], gc[s], dn, 0, 0, 0);
            }
            // up[i], dn[i]: hidden channel 32 mh + 8 (i/4) + 4 hl + i%4 of voxel il
            half8_t hv[2], lv[2];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const half4_t b4 = *reinterpret_cast<const half4_t*>(bsh + 32 * mh + 8 * gq + 4 * hl);
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    const int i = 4 * gq + 2 * jp, e = 4 * (gq % 2) + 2 * jp;
                    half2_t hid, lg;
                    hid_lg_pair(up[i], up[i + 1], dn[i], dn[i + 1], half2_t{b4[2 * jp], b4[2 * jp + 1]}, hid, lg);
                    hv[gq / 2][e] = hid[0];
                    hv[gq / 2][e + 1] = hid[1];
                    lv[gq / 2][e] = lg[0];
                    lv[gq / 2][e + 1] = lg[1];
                }
            }
            // rows past V hold x = g = 0: hid = relu(bias) there meets g = 0 in dWdown, lg = 0 everywhere else
            dacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(f3[(2 * mh) * 64], lv[0], dacc, 0, 0, 0);
            dacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(f3[(2 * mh + 1) * 64], lv[1], dacc, 0, 0, 0);

            // hid and lg rows of the voxel (positions 8 (2 f + hl) + e) into the tiles, back transposed
            wave_sync();  // (the reads of the previous block are issued)
            *reinterpret_cast<half8_t*>(ht + woff0) = hv[0];
            *reinterpret_cast<half8_t*>(ht + woff1) = hv[1];
            *reinterpret_cast<half8_t*>(lt + woff0) = lv[0];
            *reinterpret_cast<half8_t*>(lt + woff1) = lv[1];
            wave_sync();
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const half8_t hT = read_T(ht, hf), lT = read_T(lt, hf);  // lane = hidden position il
                wdn[mh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hT, gT[hf], wdn[mh], 0, 0, 0);
                wup[mh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xT[hf], lT, wup[mh], 0, 0, 0);
                bacc[mh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, lT, bacc[mh], 0, 0, 0);
            }
        }

        // ---- dx: row il of the wavefront's tile, 8 bytes (channels 8 gq + 4 hl + 0..3) at a time; the two halves
        // of a chunk are swapped in every second group of eight rows so that the 16 lanes of a write phase hit 16
        // different pairs of the 32 write banks ----
#pragma unroll
        for (int gq = 0; gq < C / 8; ++gq) {
            half4_t o;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) o[jj] = (half_t)dacc[4 * gq + jj];
            *reinterpret_cast<half4_t*>(dt + il * 64 + ((gq ^ wsw) * 16) + ((hl ^ ((il >> 3) & 1)) * 8)) = o;
        }
        wave_sync();
    }
    if (first < ntiles) flush((tile - stride) * 32, true);

    // ---- the four wavefronts add their partials in LDS, wavefront 0 first: [dWup C*H][dWdown H*C][dbias H] ----
    float* red = reinterpret_cast<float*>(smem);
    __syncthreads();  // every wavefront is done with the fragments
#pragma unroll 1
    for (int w = 0; w < kMlpWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int mh = 0; mh < MH; ++mh) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int ri = 8 * (i / 4) + 4 * hl + i % 4;  // row of the block held in register i
                    {  // dWdown[h = 32 mh + hidden of position ri][c = il]
                        float* p = red + C * H + (32 * mh + tr_hidden(ri)) * C + il;
                        *p = w == 0 ? wdn[mh][i] : *p + wdn[mh][i];
                    }
                    {  // dWup[c = ri][h = 32 mh + hidden of position il]
                        float* p = red + ri * H + 32 * mh + tr_hidden(il);
                        *p = w == 0 ? wup[mh][i] : *p + wup[mh][i];
                    }
                }
                if (lane < 16) {  // rows 0 and 1 of the 16x16 block: hidden positions lane and 16 + lane
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        float* p = red + 2 * C * H + 32 * mh + tr_hidden(16 * r + lane);
                        *p = w == 0 ? bacc[mh][r] : *p + bacc[mh][r];
                    }
                }
            }
        }
        __syncthreads();
    }
    float* out = ws + (int64_t)blockIdx.x * Cfg::RW;
    for (int i = t; i < Cfg::RW; i += kMlpThreads) out[i] = red[i];
}

// sums the rows of the partial buffer in a fixed order (16 columns per workgroup, 64 interleaved row slices with four
// loads in flight, fixed tree in LDS; fp64) and scatters the three results
// (OutT: fp32, or fp16 = the fp32 results rounded once)
template <class OutT>
__global__ __launch_bounds__(1024) void mlp_reduce_kernel(const float* __restrict__ ws, int nrows, int RW, int n_up,
                                                          int n_down, OutT* __restrict__ d_up,
                                                          OutT* __restrict__ d_down, OutT* __restrict__ d_bias)
{
    __shared__ double part[64][17];
    const int lo = threadIdx.x % 16, sl = threadIdx.x / 16;
    const int j = blockIdx.x * 16 + lo;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    if (j < RW) {
        int r = sl;
        for (; r + 192 < nrows; r += 256) {
            const float a = ws[(int64_t)r * RW + j], b = ws[(int64_t)(r + 64) * RW + j];
            const float c = ws[(int64_t)(r + 128) * RW + j], d = ws[(int64_t)(r + 192) * RW + j];
            s0 += (double)a;
            s1 += (double)b;
            s2 += (double)c;
            s3 += (double)d;
        }
        for (; r < nrows; r += 64) s0 += (double)ws[(int64_t)r * RW + j];
    }
    part[sl][lo] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int w = 32; w > 0; w >>= 1) {
        if (sl < w) part[sl][lo] += part[sl + w][lo];
        __syncthreads();
    }
    if (sl == 0 && j < RW) {
        const double v = part[0][lo];
        if (j < n_up) d_up[j] = (OutT)(float)v;
        else if (j < n_up + n_down) d_down[j - n_up] = (OutT)(float)v;
        else d_bias[j - n_up - n_down] = (OutT)(float)v;
    }
}

static void launch_mlp_reduce(const float* ws, int nrows, int RW, int n_up, int n_down, void* d_up, void* d_down,
                              void* d_bias, int dtype, hipStream_t s)
{
    if (dtype == KEROPS_DTYPE_F16)
        hipLaunchKernelGGL(mlp_reduce_kernel<half_t>, dim3(ceil_div(RW, 16)), dim3(1024), 0, s, ws, nrows, RW, n_up,
                           n_down, (half_t*)d_up, (half_t*)d_down, (half_t*)d_bias);
    else
        hipLaunchKernelGGL(mlp_reduce_kernel<float>, dim3(ceil_div(RW, 16)), dim3(1024), 0, s, ws, nrows, RW, n_up,
                           n_down, (float*)d_up, (float*)d_down, (float*)d_bias);
}

// workgroups and partial rows per workgroup
static int mb_blocks(int64_t V, int C)
{
    if (C <= 32) {  // wavefront-per-tile kernel: as many workgroups per compute unit as its registers allow
        const int64_t ntiles = (V + 31) / 32;
        return (int)std::max<int64_t>(1, std::min<int64_t>((ntiles + kMlpWaves - 1) / kMlpWaves, C == 16 ? 768 : 512));
    }
    const int64_t ntiles = (V + kMbTile - 1) / kMbTile;
    return (int)std::max<int64_t>(1, std::min<int64_t>(ntiles, 512));
}

static int mb_kspl(int C)
{
    if (C <= 32) return 1;
    const int nu = 2 * (2 * C / 32) * ((C + 31) / 32);
    return nu >= kMlpWaves ? 1 : kMlpWaves / nu;
}

}  // namespace kerops

extern "C" int64_t kerops_lin_brelu_lin_bwd_workspace_bytes(int64_t V, int32_t C)
{
    if (V <= 0) {
        set_error("lin_brelu_lin_bwd: non-positive size");
        return KEROPS_E_BADARG;
    }
    if (!(C == 16 || C == 32 || C == 64)) {
        set_error("lin_brelu_lin_bwd: built for C in {16,32,64} (got %d)", C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    return (int64_t)mb_blocks(V, C) * mb_kspl(C) * (4 * C * C + 2 * C) * (int64_t)sizeof(float);
}

extern "C" int kerops_lin_brelu_lin_bwd_f16(const void* x, const void* g, const void* Wup, const void* Wdown,
                                            const void* bias, void* dx, float* dWup, float* dWdown, float* dbias,
                                            void* workspace, int64_t workspace_bytes, int64_t V, int32_t C,
                                            void* stream)
{
    return kerops_lin_brelu_lin_bwd_f16_out(x, g, Wup, Wdown, bias, dx, dWup, dWdown, dbias, KEROPS_DTYPE_F32, workspace,
                                            workspace_bytes, V, C, stream);
}

extern "C" int kerops_lin_brelu_lin_bwd_f16_out(const void* x, const void* g, const void* Wup, const void* Wdown,
                                                const void* bias, void* dx, void* dWup, void* dWdown, void* dbias,
                                                int32_t grad_dtype, void* workspace, int64_t workspace_bytes, int64_t V,
                                                int32_t C, void* stream)
{
    if (!grad_dtype_ok(grad_dtype)) {
        set_error("lin_brelu_lin_bwd: grad_dtype must be KEROPS_DTYPE_F32 or KEROPS_DTYPE_F16");
        return KEROPS_E_BADARG;
    }
    const int64_t need = kerops_lin_brelu_lin_bwd_workspace_bytes(V, C);
    if (need < 0) return (int)need;
    if (!x || !g || !Wup || !Wdown || !bias || !dx || !dWup || !dWdown || !dbias || !aligned16(x) || !aligned16(g) ||
        !aligned16(Wup) || !aligned16(Wdown) || !aligned16(dx)) {
        set_error("lin_brelu_lin_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("lin_brelu_lin_bwd: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    const int blocks = mb_blocks(V, C);
    hipStream_t s = (hipStream_t)stream;
    float* ws = (float*)workspace;
#define KEROPS_MT_CASE(CV)                                                                                        \
    if (C == CV) {                                                                                                \
        hipLaunchKernelGGL((lin_brelu_lin_bwd_wave_kernel<CV>), dim3(blocks), dim3(kMlpThreads), 0, s,           \
                           (const half_t*)x, (const half_t*)g, (const half_t*)Wup, (const half_t*)Wdown,         \
                           (const half_t*)bias, (half_t*)dx, ws, V);                                             \
        int rc = check_launch("lin_brelu_lin_bwd");                                                               \
        if (rc != KEROPS_OK) return rc;                                                                           \
        const int RW = MtCfg<CV>::RW;                                                                             \
        launch_mlp_reduce(ws, blocks, RW, 2 * CV * CV, 2 * CV * CV, dWup, dWdown, dbias, grad_dtype, s);          \
        return check_launch("lin_brelu_lin_bwd_reduce");                                                          \
    }
    KEROPS_MT_CASE(16)
#ifdef KEROPS_MLP_BWD32_IDENTITY  // (comparison build: the identity-product transposes at C = 32 as well)
    KEROPS_MT_CASE(32)
#endif
#undef KEROPS_MT_CASE
    if (C == 32) {
        hipLaunchKernelGGL(lin_brelu_lin_bwd_tr_kernel, dim3(blocks), dim3(kMlpThreads), 0, s, (const half_t*)x,
                           (const half_t*)g, (const half_t*)Wup, (const half_t*)Wdown, (const half_t*)bias, (half_t*)dx,
                           ws, V);
        int rc = check_launch("lin_brelu_lin_bwd");
        if (rc != KEROPS_OK) return rc;
        const int RW = MrCfg::RW;
        launch_mlp_reduce(ws, blocks, RW, 2 * 32 * 32, 2 * 32 * 32, dWup, dWdown, dbias, grad_dtype, s);
        return check_launch("lin_brelu_lin_bwd_reduce");
    }
#define KEROPS_MB_CASE(CV)                                                                                        \
    if (C == CV) {                                                                                                \
        hipLaunchKernelGGL((lin_brelu_lin_bwd_kernel<CV>), dim3(blocks), dim3(kMlpThreads), 0, s,                \
                           (const half_t*)x, (const half_t*)g, (const half_t*)Wup, (const half_t*)Wdown,         \
                           (const half_t*)bias, (half_t*)dx, ws, V);                                             \
        int rc = check_launch("lin_brelu_lin_bwd");                                                               \
        if (rc != KEROPS_OK) return rc;                                                                           \
        const int RW = MbCfg<CV>::RW;                                                                             \
        launch_mlp_reduce(ws, blocks * MbCfg<CV>::KSPL, RW, 2 * CV * CV, 2 * CV * CV, dWup, dWdown, dbias,        \
                          grad_dtype, s);                                                                         \
        return check_launch("lin_brelu_lin_bwd_reduce");                                                          \
    }
    KEROPS_MB_CASE(64)
#undef KEROPS_MB_CASE
    set_error("lin_brelu_lin_bwd: built for C in {16,32,64} (got %d)", C);
    return KEROPS_E_UNSUPPORTED_C;
}
