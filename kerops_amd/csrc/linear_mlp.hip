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
    static constexpr int RH = C + 4;            // LDS row pitch of the output tile (halves)
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
    half_t* my = reinterpret_cast<half_t*>(smem + Cfg::T_OFF) + wave * 32 * RH;

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
            for (int s = 0; s < KS1; ++s) xb[s] = load_c8_nt(x + v * C + 16 * s + 8 * hl);
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
                        *reinterpret_cast<half4_t*>(my + vl * RH + co) = o;
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
                    const half4_t lo = *reinterpret_cast<const half4_t*>(my + row * RH + cc * 8);
                    const half4_t hi = *reinterpret_cast<const half4_t*>(my + row * RH + cc * 8 + 4);
                    half8_t o = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
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
