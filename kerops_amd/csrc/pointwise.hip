// Pointwise (1x1x1) channel mixing on the matrix cores (gfx950):
//
//   out[v, co] = fp16( sum_ci act(x[v, ci]) * Wm[ci, co] )  (+ add[v, co] in fp16)
//
// x is [V][CIN] fp16 (the memory of a channels_last_3d activation), Wm is [CIN][COUT] fp16.
// The op moves 2*V*(CIN + COUT) bytes and does only 2*V*CIN*COUT flops: it is HBM-bound, the
// matrix cores are used so that the arithmetic never shows up next to the memory stream.
//
// Each wavefront owns tiles of 32 voxels.  The product is computed transposed,
// out^T[co, v] = Wm^T[co, :] . x^T[:, v], with v_mfma_f32_32x32x16_f16: the A operand is a
// 32-row block of Wm^T (16-byte fragments pre-arranged in LDS, one ds_read_b128 per instruction), the
// B operand is x^T, whose per-lane fragment "8 consecutive k of voxel lane%32" is simply one 16-byte
// chunk of the voxel's channel vector: lane half h = lane/32 takes chunk 2s+h in step s.
// The fp32 result fragment of a lane is 4 consecutive output channels
// of one voxel (x 4 row groups x COUT/32 blocks); it is rounded to fp16, bounced through a
// wavefront-private LDS tile [32][COUT] and written back as 16-byte chunks, coalesced, with
// the optional fp16 residual add and the optional running max|out| fused into that pass.
#include "common.hpp"

namespace kerops {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kPwThreads = 256;
constexpr int kPwWaves = kPwThreads / kWave;

template <int CIN, int COUT>
struct PwCfg {
    static constexpr int MT = (COUT + 31) / 32;      // 32-row blocks of output channels
    static constexpr int KS = CIN / 16;              // MFMA steps (k = 16 each) = 16-byte chunks a lane loads per voxel
    static constexpr int TILE_HALVES = 32 * COUT;    // dense rows, swizzled: BounceTile in common.hpp
    static constexpr int OUT_CHUNKS = 32 * COUT / 8; // 16-byte chunks of one output tile
    static_assert(CIN % 16 == 0 && CIN <= 128, "CIN in {16,32,64,128}");
    static_assert(COUT % 8 == 0 && COUT <= 128, "COUT in {16,32,64,128}");
};

// AFFINE: x is first mapped to fp16(max(fma(x, scale[c], shift[c]), 0)), the arithmetic of the batch-norm + ReLU
// stream op, so that op and the product run as one pass and its result never reaches memory.
template <int CIN, int COUT, bool RELU_IN, bool HAS_ADD, bool ABSMAX, bool AFFINE = false>
__global__ __launch_bounds__(kPwThreads) void pointwise_kernel(const half_t* __restrict__ x,
                                                               const half_t* __restrict__ Wm,
                                                               const half_t* __restrict__ add,
                                                               half_t* __restrict__ out, float* __restrict__ amax_ws,
                                                               int64_t V, const float* __restrict__ scale = nullptr,
                                                               const float* __restrict__ shift = nullptr)
{
    using Cfg = PwCfg<CIN, COUT>;
    constexpr int MT = Cfg::MT, KS = Cfg::KS;
    using Tile = BounceTile<COUT>;
    __shared__ __attribute__((aligned(16))) half_t tile[kPwWaves][Cfg::TILE_HALVES];
    __shared__ __attribute__((aligned(16))) half_t wfrag[MT * KS * 64 * 8];
    __shared__ float red[kPwWaves];
    __shared__ __attribute__((aligned(16))) float aff[AFFINE ? 2 * CIN : 4];  // [scale | shift]

    const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
    const int vl = lane % 32, hl = lane / 32;

    // A fragments: wfrag[((mt*KS + s)*64 + l)*8 + j] = Wm[16 s + 8 (l/32) + j][32 mt + l%32]
    for (int i = t; i < MT * KS * 64 * 8; i += kPwThreads) {
        const int j = i % 8, l = (i / 8) % 64, s = (i / 512) % KS, mt = i / (512 * KS);
        const int co = 32 * mt + l % 32;
        wfrag[i] = (co < COUT) ? Wm[(16 * s + 8 * (l / 32) + j) * COUT + co] : (half_t)0;
    }
    if constexpr (AFFINE) {
        for (int i = t; i < CIN; i += kPwThreads) {
            aff[i] = scale[i];
            aff[CIN + i] = shift[i];
        }
    }
    __syncthreads();
    const half8_t* wa = reinterpret_cast<const half8_t*>(wfrag) + lane;

    float amax = 0.0f;
    const int64_t ntiles = (V + 31) / 32;
    const int64_t tiles_per_round = (int64_t)gridDim.x * kPwWaves;
    const int64_t nrounds = (ntiles + tiles_per_round - 1) / tiles_per_round;
    unsigned char* my = reinterpret_cast<unsigned char*>(tile[wave]);

    // B fragments of a tile: this lane's voxel, chunks 2q+hl.  A tile index past the end reads the last voxel (the
    // loads are unconditional, the tile is then never used).
    auto load_x = [&](int64_t tidx, half8_t(&xb)[KS]) {
        int64_t v = tidx * 32 + vl;
        if (v >= V) v = V - 1;  // ragged last tile: clamp the read, the write is masked
#pragma unroll
        for (int q = 0; q < KS; ++q) {
            // a load instruction touches 32 bytes of every voxel row: rows of 128 bytes and more need the
            // cache to hold the line until the row's other loads arrive, so only narrow rows stream
            if constexpr (CIN <= 32) xb[q] = load_c8_nt(x + v * CIN + 8 * (2 * q + hl));
            else xb[q] = load_c8(x + v * CIN + 8 * (2 * q + hl));
        }
    };
    // Without a residual the loads of the next tile are issued before this tile's arithmetic and stores: the wait
    // for them at the top of the next round then leaves the stores in flight, and the memory pipe never drains
    // between tiles (7 % faster at 32 -> 32 channels, 3 % at 64 -> 128).  With the residual as a third stream the
    // same prefetch is 2-4 % slower than loading each tile where it is used, so those variants do that.
    constexpr bool PIPE = !HAS_ADD;
    half8_t xb[KS];
    if constexpr (PIPE) load_x((int64_t)blockIdx.x * kPwWaves + wave, xb);
    for (int64_t r = 0; r < nrounds; ++r) {
        const int64_t tidx = (r * gridDim.x + blockIdx.x) * kPwWaves + wave;
        const bool live = tidx < ntiles;
        const int64_t v0 = tidx * 32;
        half8_t xn[KS];
        if constexpr (PIPE) load_x(tidx + tiles_per_round, xn);
        if (live) {
            if constexpr (!PIPE) {
                int64_t v = v0 + vl;
                if (v >= V) v = V - 1;
#pragma unroll
                for (int q = 0; q < KS; ++q) {
                    if constexpr (CIN <= 32) xb[q] = load_c8_nt(x + v * CIN + 8 * (2 * q + hl));
                    else xb[q] = load_c8(x + v * CIN + 8 * (2 * q + hl));
                }
            }
            if constexpr (AFFINE) {
#pragma unroll
                for (int q = 0; q < KS; ++q) {
                    const int c0 = 8 * (2 * q + hl);  // the chunk's first channel: two addresses per wavefront
                    const float4_t s0 = *reinterpret_cast<const float4_t*>(aff + c0);
                    const float4_t s1 = *reinterpret_cast<const float4_t*>(aff + c0 + 4);
                    const float4_t b0 = *reinterpret_cast<const float4_t*>(aff + CIN + c0);
                    const float4_t b1 = *reinterpret_cast<const float4_t*>(aff + CIN + c0 + 4);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        xb[q][j] = (half_t)fmaxf(__builtin_fmaf((float)xb[q][j], s0[j], b0[j]), 0.0f);
                        xb[q][4 + j] = (half_t)fmaxf(__builtin_fmaf((float)xb[q][4 + j], s1[j], b1[j]), 0.0f);
                    }
                }
            }
            if (RELU_IN) {
                const half8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int q = 0; q < KS; ++q) xb[q] = __builtin_elementwise_max(xb[q], z8);  // packed maximum
            }
            float16_t acc[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[mt][i] = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa[(mt * KS + s) * 64], xb[s], acc[mt], 0, 0, 0);
            }
            // acc[mt][i]: output channel 32*mt + 8*(i/4) + 4*hl + i%4 of voxel vl
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int co = 32 * mt + 8 * gq + 4 * hl;
                    if (co < COUT) {
                        half4_t o;
#pragma unroll
                        for (int j = 0; j < 4; ++j) o[j] = (half_t)acc[mt][4 * gq + j];
                        *reinterpret_cast<half4_t*>(my + Tile::piece(vl, 4 * mt + gq, hl)) = o;
                    }
                }
        }
        // the tile is private to the wavefront and its LDS operations complete in issue order: no workgroup
        // barrier, the wavefronts of a workgroup run independently
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (live) {
#pragma unroll
            for (int c0 = 0; c0 < Cfg::OUT_CHUNKS; c0 += kWave) {
                const int c = c0 + lane;
                const int row = c / (COUT / 8), cc = c % (COUT / 8);
                if (c < Cfg::OUT_CHUNKS && v0 + row < V) {
                    half8_t o = Tile::read(my, row, cc);
                    const int64_t off = (v0 + row) * COUT + cc * 8;
                    if (HAS_ADD) {
                        const half8_t a8 = load_c8_nt(add + off);
#pragma unroll
                        for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)o[j] + (float)a8[j]);  // fp16 add, RNE
                    }
                    if (ABSMAX) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf((float)o[j]));
                    }
                    store_c8_nt(out + off, o);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if constexpr (PIPE) {
#pragma unroll
            for (int q = 0; q < KS; ++q) xb[q] = xn[q];
        }
    }
    if (ABSMAX) {
        amax = wave_max(amax);
        if (lane == 0) red[wave] = amax;
        __syncthreads();
        if (t == 0) {
            float m = red[0];
#pragma unroll
            for (int wv = 1; wv < kPwWaves; ++wv) m = fmaxf(m, red[wv]);
            amax_ws[blockIdx.x] = m;
        }
    }
}

__global__ __launch_bounds__(256) void pw_absmax_final_kernel(const float* __restrict__ ws, int n,
                                                              float* __restrict__ out)
{
    __shared__ float red[4];
    float m = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) m = fmaxf(m, ws[i]);
    m = wave_max(m);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) out[0] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

static int pw_blocks(int64_t V)
{
    const int64_t ntiles = (V + 31) / 32;
    int64_t b = (ntiles + kPwWaves - 1) / kPwWaves;
    if (b > 1024) b = 1024;  // 4 workgroups of 4 wavefronts per CU, each looping over tiles
    return (int)std::max<int64_t>(b, 1);
}

template <int CIN, int COUT>
static int launch_pw(const half_t* x, const half_t* Wm, const half_t* add, half_t* out, float* amax_ws, int64_t V,
                     bool relu_in, bool absmax, int blocks, hipStream_t s, const float* scale = nullptr,
                     const float* shift = nullptr)
{
    if (absmax && (add || scale)) {  // no instantiation keeps the running max next to a residual or the affine map
        set_error("pointwise: the running max is built without residual add and without the affine map");
        return KEROPS_E_BADARG;
    }
    if (scale) {  // the affine map ends in a ReLU of its own
        if (add) {
            hipLaunchKernelGGL((pointwise_kernel<CIN, COUT, false, true, false, true>), dim3(blocks), dim3(kPwThreads), 0,
                               s, x, Wm, add, out, amax_ws, V, scale, shift);
        } else {
            hipLaunchKernelGGL((pointwise_kernel<CIN, COUT, false, false, false, true>), dim3(blocks), dim3(kPwThreads),
                               0, s, x, Wm, add, out, amax_ws, V, scale, shift);
        }
        return check_launch("bnrelu_pointwise");
    }
#define KEROPS_PW_GO(R, A, M)                                                                                    \
    hipLaunchKernelGGL((pointwise_kernel<CIN, COUT, R, A, M>), dim3(blocks), dim3(kPwThreads), 0, s, x, Wm, add, \
                       out, amax_ws, V, nullptr, nullptr)
    if (absmax) {
        if (relu_in) KEROPS_PW_GO(true, false, true);
        else KEROPS_PW_GO(false, false, true);
    } else if (add) {
        if (relu_in) KEROPS_PW_GO(true, true, false);
        else KEROPS_PW_GO(false, true, false);
    } else {
        if (relu_in) KEROPS_PW_GO(true, false, false);
        else KEROPS_PW_GO(false, false, false);
    }
#undef KEROPS_PW_GO
    return check_launch("pointwise");
}

int pointwise_dispatch(const half_t* x, const half_t* Wm, const half_t* add, half_t* out, float* amax_ws, int64_t V,
                       int Cin, int Cout, bool relu_in, bool absmax, int blocks, hipStream_t s, const float* scale,
                       const float* shift)
{
#define KEROPS_PW_CASE(CI, CO)      \
    if (Cin == CI && Cout == CO)    \
        return launch_pw<CI, CO>(x, Wm, add, out, amax_ws, V, relu_in, absmax, blocks, s, scale, shift);
    KEROPS_PW_CASE(16, 16)
    KEROPS_PW_CASE(16, 32)
    KEROPS_PW_CASE(32, 16)
    KEROPS_PW_CASE(32, 32)
    KEROPS_PW_CASE(64, 16)
    KEROPS_PW_CASE(64, 32)
    KEROPS_PW_CASE(64, 64)
    KEROPS_PW_CASE(64, 128)
    KEROPS_PW_CASE(128, 16)
    KEROPS_PW_CASE(128, 32)
    KEROPS_PW_CASE(128, 64)
    KEROPS_PW_CASE(128, 128)
    KEROPS_PW_CASE(16, 64)
    KEROPS_PW_CASE(32, 64)
    KEROPS_PW_CASE(16, 128)
    KEROPS_PW_CASE(32, 128)
#undef KEROPS_PW_CASE
    set_error("pointwise: no kernel built for Cin=%d Cout=%d (both in {16,32,64,128})", Cin, Cout);
    return KEROPS_E_UNSUPPORTED_C;
}

int pointwise_blocks(int64_t V) { return pw_blocks(V); }

void launch_pw_absmax_final(const float* ws, int n, float* out, hipStream_t s)
{
    hipLaunchKernelGGL(pw_absmax_final_kernel, dim3(1), dim3(256), 0, s, ws, n, out);
}

}  // namespace kerops

using namespace kerops;

extern "C" int kerops_pointwise_f16(const void* x, const void* Wm, const void* add, void* out, int64_t V, int32_t Cin,
                                    int32_t Cout, int32_t relu_in, void* stream)
{
    if (!x || !Wm || !out || !aligned16(x) || !aligned16(Wm) || !aligned16(out) || (add && !aligned16(add))) {
        set_error("pointwise: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (V <= 0) {
        set_error("pointwise: V must be positive");
        return KEROPS_E_BADARG;
    }
    return pointwise_dispatch((const half_t*)x, (const half_t*)Wm, (const half_t*)add, (half_t*)out, nullptr, V, Cin,
                              Cout, relu_in != 0, false, pw_blocks(V), (hipStream_t)stream);
}

extern "C" int kerops_bnrelu_pointwise_f16(const void* x, const float* scale, const float* shift, const void* Wm,
                                           const void* add, void* out, int64_t V, int32_t Cin, int32_t Cout,
                                           void* stream)
{
    if (!x || !scale || !shift || !Wm || !out || !aligned16(x) || !aligned16(Wm) || !aligned16(out) ||
        (add && !aligned16(add))) {
        set_error("bnrelu_pointwise: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (V <= 0) {
        set_error("bnrelu_pointwise: V must be positive");
        return KEROPS_E_BADARG;
    }
    return pointwise_dispatch((const half_t*)x, (const half_t*)Wm, (const half_t*)add, (half_t*)out, nullptr, V, Cin,
                              Cout, false, false, pw_blocks(V), (hipStream_t)stream, scale, shift);
}
