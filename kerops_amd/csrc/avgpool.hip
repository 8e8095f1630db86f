// 2x2x2 stride-2 ceil-mode average pool with per-channel statistics of the pooled
// values, and its backward, on [N][H][W][D][C] fp16 (gfx950).
//
// One thread produces one chunk of V = min(8, C) channels of one pooled voxel: it reads
// the (up to) eight input chunks of the window as 16-byte accesses, adds the D pair first
// and then the four (h, w) rows in the order (0,0) (0,1) (1,0) (1,1), divides by the number
// of voxels that exist in the window and stores the RNE-rounded fp16 chunk.  Consecutive
// lanes take consecutive (d_out, channel-group) chunks, so the two D-taps of a wavefront
// together cover contiguous input memory.  The statistics use the unrounded fp32 pooled
// values and the same deterministic two-pass reduction as the other per-channel sums.
#include <type_traits>

#include "common.hpp"

namespace kerops {

struct PoolDims {
    int N, H, W, D, Ho, Wo, Do, C, CG;
};

// acc + float(half SEL of the packed pair), one instruction (the mixed-precision fused multiply-add with the factor
// 1.0: the product is exact, the sum is rounded once, i.e. the bits of a conversion followed by an addition)
template <int SEL>
__device__ __forceinline__ float add_half_of(uint32_t pair, float acc)
{
    float r;
    if constexpr (SEL == 0)
        asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pair), "v"(acc));
    else
        asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pair), "v"(acc));
    return r;
}

// BNRELU: every voxel that exists is first mapped to fp16(max(x * bw[c] + bb[c], 0)), exactly what
// bnrelu_fwd_kernel would have stored, so the fused op equals ApplyBNReLU followed by the pool bit for bit
// while the full-size intermediate is neither written nor read.
// NTLD: the input loads carry the streaming hint.  A load instruction of a wavefront takes one of the two D taps,
// i.e. every second voxel row: where a voxel row is a whole 128-byte line (64 channels and more) each instruction
// fetches whole lines and the hint wins (0.399 against 0.427 ms at C = 64); with narrower rows the two taps share
// their lines, which the hint would fetch twice, and cached loads win (C = 8: 0.053 against 0.062 ms, C = 16: 0.111
// against 0.118, C = 32: 0.219 against 0.220).
template <int V, int U, bool BNRELU, bool NTLD>
__global__ __launch_bounds__(kStreamMaxThreads) void avgpool_fwd_kernel(const half_t* __restrict__ x,
                                                                        const float* __restrict__ bw,
                                                                        const float* __restrict__ bb,
                                                                        half_t* __restrict__ y, float* __restrict__ ws,
                                                                        const PoolDims p, int64_t nchunks,
                                                                        int segments)
{
    typedef typename HVec<V>::type hv;
    __shared__ float red[4 * 2 * 64 * V];
    const ChunkWalk<U> wk(nchunks, segments != 0);
    float acc[2][V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[0][j] = acc[1][j] = 0.0f;
    // every stride of the walk is a multiple of the number of channel groups: a thread keeps its channel group
    float cw[V], cb[V];
    if (BNRELU) {
        const int cg0 = (int)(wk.first % p.CG);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            cw[j] = bw[cg0 * V + j];
            cb[j] = bb[cg0 * V + j];
        }
    }
    const int64_t sD = p.CG, sW = (int64_t)p.D * p.CG, sH = (int64_t)p.W * sW, sN = (int64_t)p.H * sH;  // in chunks

    struct Window {
        hv v[2][2][2];
        bool h1, w1, d1;
    };
    // all eight loads of a window are issued before the first value is touched
    auto load_window = [&](int64_t i, Window& wn) {
        int64_t r = i;
        const int cg = (int)(r % p.CG);
        r /= p.CG;
        const int dO = (int)(r % p.Do);
        r /= p.Do;
        const int wO = (int)(r % p.Wo);
        r /= p.Wo;
        const int hO = (int)(r % p.Ho);
        const int n = (int)(r / p.Ho);
        wn.h1 = 2 * hO + 1 < p.H;
        wn.w1 = 2 * wO + 1 < p.W;
        wn.d1 = 2 * dO + 1 < p.D;
        const int64_t base = n * sN + (2 * hO) * sH + (2 * wO) * sW + (2 * dO) * sD + cg;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const bool ok = (a == 0 || wn.h1) && (b == 0 || wn.w1) && (e == 0 || wn.d1);
                    hv t;
#pragma unroll
                    for (int j = 0; j < V; ++j) t[j] = (half_t)0;
                    if (ok) {
                        if constexpr (NTLD) t = ld_stream<V>(x, base + a * sH + b * sW + e * sD);
                        else t = *reinterpret_cast<const hv*>(x + (base + a * sH + b * sW + e * sD) * V);
                    }
                    wn.v[a][b][e] = t;
                }
    };
    auto finish_window = [&](int64_t i, Window& wn) {
        if (BNRELU) {
            hv zero;
#pragma unroll
            for (int j = 0; j < V; ++j) zero[j] = (half_t)0;
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const bool ok = (a == 0 || wn.h1) && (b == 0 || wn.w1) && (e == 0 || wn.d1);
                        // fp16(max(v, 0)) = max(fp16(v), 0): rounding keeps the sign and the order, so the ReLU runs
                        // on the rounded pairs (one packed instruction for two channels)
                        // (fp16 of the fp32 result, as ApplyBNReLU stores it: two roundings)
                        hv r;
#pragma unroll
                        for (int j = 0; j < V; ++j)
                            r[j] = (half_t)as_fp32_value(__builtin_fmaf((float)wn.v[a][b][e][j], cw[j], cb[j]));
                        if constexpr (V >= 2) r = __builtin_elementwise_max(r, zero);
                        else r[0] = r[0] > (half_t)0 ? r[0] : (half_t)0;
                        wn.v[a][b][e] = ok ? r : zero;
                    }
        }
        // the window holds 2^k voxels, k = 0..3: the product with 2^-k (built from its exponent bits) is the
        // correctly rounded quotient
        const uint32_t k = (uint32_t)wn.h1 + (uint32_t)wn.w1 + (uint32_t)wn.d1;
        const float inv = __builtin_bit_cast(float, (127u - k) << 23);
        hv o;
        if constexpr (V >= 2) {
            // a (h, w) row: the two D taps of a channel are float(tap 0) + float(tap 1), the second conversion and the
            // addition in one instruction
            uint32_t wd[2][2][2][V / 2];
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int e = 0; e < 2; ++e) __builtin_memcpy(wd[a][b][e], &wn.v[a][b][e], V * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                float s = 0.0f;
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        const float t0 = (float)wn.v[a][b][0][j];
                        s += (j % 2 == 0) ? add_half_of<0>(wd[a][b][1][j / 2], t0) : add_half_of<1>(wd[a][b][1][j / 2], t0);
                    }
                const float m = s * inv;
                o[j] = (half_t)m;
                acc[0][j] += m;
                acc[1][j] = __builtin_fmaf(m, m, acc[1][j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                float s = 0.0f;
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int b = 0; b < 2; ++b) s += (float)wn.v[a][b][0][j] + (float)wn.v[a][b][1][j];
                const float m = s * inv;
                o[j] = (half_t)m;
                acc[0][j] += m;
                acc[1][j] = __builtin_fmaf(m, m, acc[1][j]);
            }
        }
        st_stream<V>(y, i, o);
    };
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        Window wn[U];
#pragma unroll
        for (int u = 0; u < U; ++u) load_window(i + u * wk.su, wn[u]);
#pragma unroll
        for (int u = 0; u < U; ++u) finish_window(i + u * wk.su, wn[u]);
    }
    for (int64_t i = wk.tail; i < nchunks; i += wk.T) {
        Window wn;
        load_window(i, wn);
        finish_window(i, wn);
    }
    block_channel_partials_any<2, V>(acc, p.CG, red, ws + (int64_t)blockIdx.x * 2 * p.CG * V);
}

// PERM (16-byte chunks, even D, whole wavefronts inside one pooled row, fewer than 64 channels): a wavefront's 64
// results belong to 64 / CG consecutive pooled positions of one pooled row, so each of the four (h, w) rows of their
// windows is one run of 128 consecutive output chunks in which every result appears twice (both D taps).  The
// results are redistributed over the lanes (ds_bpermute: output chunk j of the run comes from lane (j / 2CG) CG +
// j % CG) and every store instruction writes 1 KB of consecutive memory; stored straight from the lane that computed
// them, an instruction would write every second voxel row, i.e. parts of 128-byte lines where a voxel row is
// narrower than a line.
template <int V, int U, bool PERM>
__global__ __launch_bounds__(kStreamMaxThreads) void avgpool_bwd_kernel(const half_t* __restrict__ inpgrad,
                                                                        const float* __restrict__ meangrad,
                                                                        const float* __restrict__ sqmeangrad,
                                                                        const half_t* __restrict__ output,
                                                                        half_t* __restrict__ dx, const PoolDims p,
                                                                        int64_t nchunks, float fMo, int segments)
{
    typedef typename HVec<V>::type hv;
    const ChunkWalk<U> wk(nchunks, segments != 0);
    const int64_t sD = p.CG, sW = (int64_t)p.D * p.CG, sH = (int64_t)p.W * sW, sN = (int64_t)p.H * sH;
    const int cg0 = (int)(wk.first % p.CG);
    float mg[V], sg[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        mg[j] = __fdiv_rn(meangrad[cg0 * V + j], fMo);
        sg[j] = sqmeangrad[cg0 * V + j];
    }
    const int lane = threadIdx.x % kWave;
    const int src0 = ((lane / (2 * p.CG)) * p.CG + lane % p.CG) * 4;  // PERM: byte index of the source lane, first run half
    auto one = [&](int64_t i, const hv& g, const hv& o, auto whole_wave) {
        int64_t r = i / p.CG;
        const int dO = (int)(r % p.Do);
        r /= p.Do;
        const int wO = (int)(r % p.Wo);
        r /= p.Wo;
        const int hO = (int)(r % p.Ho);
        const int n = (int)(r / p.Ho);
        const bool h1 = 2 * hO + 1 < p.H, w1 = 2 * wO + 1 < p.W, d1 = 2 * dO + 1 < p.D;
        const float cnt = (float)((h1 ? 2 : 1) * (w1 ? 2 : 1) * (d1 ? 2 : 1));
        hv res;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float s = __fdiv_rn(__fmul_rn(__fmul_rn(2.0f, (float)o[j]), sg[j]), fMo);
            const float t = __fadd_rn(__fadd_rn((float)g[j], mg[j]), s);
            res[j] = (half_t)__fdiv_rn(t, cnt);
        }
        const int64_t base = n * sN + (2 * hO) * sH + (2 * wO) * sW + (2 * dO) * sD + cg0;
        if constexpr (PERM && decltype(whole_wave)::value) {
            // lane 0 holds the first pooled position of the run and channel group 0
            const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)(uint64_t)base);
            const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)base >> 32));
            const int64_t run0 = (int64_t)(((uint64_t)bhi << 32) | blo);
            constexpr int NDW = (int)(sizeof(hv) + 3) / 4;  // (4 dwords: this path is built for 16-byte chunks)
            uint32_t rv[NDW] = {};
            __builtin_memcpy(rv, &res, sizeof(hv));
#pragma unroll
            for (int e = 0; e < 2; ++e) {  // the two halves of the run
                uint32_t pv[NDW];
#pragma unroll
                for (int q = 0; q < NDW; ++q) pv[q] = (uint32_t)__builtin_amdgcn_ds_bpermute(src0 + e * 128, (int)rv[q]);
                hv out;
                __builtin_memcpy(&out, pv, sizeof(hv));
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int b = 0; b < 2; ++b)
                        if ((a == 0 || h1) && (b == 0 || w1))  // wavefront-uniform
                            st_stream<V>(dx, run0 + a * sH + b * sW + e * 64 + lane, out);
            }
        } else {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const bool ok = (a == 0 || h1) && (b == 0 || w1) && (e == 0 || d1);
                        if (ok) st_stream<V>(dx, base + a * sH + b * sW + e * sD, res);
                    }
        }
    };
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        hv g[U], o[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            g[u] = ld_stream<V>(inpgrad, i + u * wk.su);
            o[u] = ld_stream<V>(output, i + u * wk.su);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) one(i + u * wk.su, g[u], o[u], std::true_type{});
    }
    // (the last, partly filled step: every lane stores its own result)
    for (int64_t i = wk.tail; i < nchunks; i += wk.T)
        one(i, ld_stream<V>(inpgrad, i), ld_stream<V>(output, i), std::false_type{});
}

// Launch shape (blocks, waves, segment) as for the flat stream kernels; segment counts output chunks per thread and
// step: 1 = interleaved (one window per thread in flight), 2 = contiguous runs of two chunks per thread (two
// windows, 16 loads, in flight).  Built-in choices measured at (1,64,350,350,128).
struct PoolDefault {
    int blocks, waves, segment;
};
constexpr PoolDefault kDefPoolFwd{256, 4, 1};
constexpr PoolDefault kDefPoolFwdBnRelu{256, 4, 2};
constexpr PoolDefault kDefPoolBwd{256, 4, 1};
constexpr int kMaxDefaultBlocks = 4096;  // workspace queries with blocks = 0 size for this many partials

static int pool_plan(const char* op, const PoolDefault& def, int N, int H, int W, int D, int C, int blocks, int waves,
                     int segment, PoolDims* p, int64_t* nchunks, StreamShape* sh)
{
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0 || C <= 0 || !is_pow2(C)) {
        set_error("%s: extents must be positive and C a power of two", op);
        return KEROPS_E_BADARG;
    }
    if (C > kMaxReduceChannels) {
        set_error("%s: built for C <= %d (got %d)", op, kMaxReduceChannels, C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    if (volume_exceeds_i64(N, H, W, D, C)) {
        set_error("%s: tensor too large", op);
        return KEROPS_E_BADARG;
    }
    if (waves == 0) waves = def.waves;
    if (segment == 0) segment = def.segment;
    if (!(waves == 4 || waves == 8 || waves == 16)) {
        set_error("%s: waves must be 4, 8 or 16 wavefronts per workgroup (got %d)", op, waves);
        return KEROPS_E_BADARG;
    }
    if (!(segment == 1 || segment == 2)) {
        set_error("%s: segment must be 1 (interleaved) or 2 (got %d)", op, segment);
        return KEROPS_E_BADARG;
    }
    if (blocks > 65536) {
        set_error("%s: blocks must be <= 65536", op);
        return KEROPS_E_BADARG;
    }
    const int V = C >= 8 ? 8 : C;
    p->N = N;
    p->H = H;
    p->W = W;
    p->D = D;
    p->Ho = ceil_div(H, 2);
    p->Wo = ceil_div(W, 2);
    p->Do = ceil_div(D, 2);
    p->C = C;
    p->CG = C / V;
    *nchunks = (int64_t)N * p->Ho * p->Wo * p->Do * p->CG;
    sh->threads = waves * kWave;
    sh->segment = segment;
    // the built-in workgroup counts were measured on 256 compute units: scale them to the device at hand
    // (never beyond what a workspace query with blocks = 0 sizes for)
    if (blocks <= 0)
        blocks = std::min(kMaxDefaultBlocks, std::max(1, (int)((int64_t)def.blocks * device_geometry().cus / 256)));
    sh->blocks = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div64(*nchunks, (int64_t)sh->threads * segment), blocks));
    return KEROPS_OK;
}

}  // namespace kerops

using namespace kerops;

extern "C" int64_t kerops_avgpool_ceil_stats_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                                             int32_t blocks)
{
    PoolDims p;
    int64_t nchunks = 0;
    StreamShape sh;
    int rc = pool_plan("avgpool_ceil_stats", kDefPoolFwd, N, H, W, D, C, blocks, 0, 0, &p, &nchunks, &sh);
    if (rc != KEROPS_OK) return rc;
    if (blocks <= 0) blocks = kMaxDefaultBlocks;
    return (int64_t)blocks * 2 * C * (int64_t)sizeof(float);
}

static int pool_fwd_run(const char* op, const void* x, const float* bw, const float* bb, void* y, float* mean,
                        float* sqmean, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C, void* workspace,
                        int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    PoolDims p;
    int64_t nchunks = 0;
    StreamShape sh;
    int rc = pool_plan(op, bw ? kDefPoolFwdBnRelu : kDefPoolFwd, N, H, W, D, C, blocks, waves, segment, &p, &nchunks,
                       &sh);
    if (rc != KEROPS_OK) return rc;
    if (!x || !y || !mean || !sqmean || !aligned16(x) || !aligned16(y)) {
        set_error("%s: null or misaligned pointer", op);
        return KEROPS_E_BADARG;
    }
    const int64_t need = (int64_t)sh.blocks * 2 * C * (int64_t)sizeof(float);
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("%s: workspace of %lld bytes required, %lld given", op, (long long)need, (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    hipStream_t s = (hipStream_t)stream;
    float* ws = (float*)workspace;
    const int seg = sh.segment != 1;
    const bool ntld = C >= 64;  // voxel rows of whole 128-byte lines
#define KEROPS_POOL_GO(Uv, B)                                                                                      \
    KEROPS_DISPATCH_V(C, {                                                                                         \
        if (ntld)                                                                                                  \
            hipLaunchKernelGGL((avgpool_fwd_kernel<V, Uv, B, true>), dim3(sh.blocks), dim3(sh.threads), 0, s,      \
                               (const half_t*)x, bw, bb, (half_t*)y, ws, p, nchunks, seg);                         \
        else                                                                                                       \
            hipLaunchKernelGGL((avgpool_fwd_kernel<V, Uv, B, false>), dim3(sh.blocks), dim3(sh.threads), 0, s,     \
                               (const half_t*)x, bw, bb, (half_t*)y, ws, p, nchunks, seg);                         \
    })
    if (bw) {
        if (sh.segment == 2) KEROPS_POOL_GO(2, true);
        else KEROPS_POOL_GO(1, true);
    } else {
        if (sh.segment == 2) KEROPS_POOL_GO(2, false);
        else KEROPS_POOL_GO(1, false);
    }
#undef KEROPS_POOL_GO
    rc = check_launch(op);
    if (rc != KEROPS_OK) return rc;
    const double Mo = (double)N * p.Ho * p.Wo * p.Do;
    launch_reduce_rows(ws, sh.blocks, 2 * C, mean, sqmean, C, 1.0 / Mo, s);
    return check_launch(op);
}

extern "C" int kerops_avgpool_ceil_stats_f16(const void* x, void* y, float* mean, float* sqmean, int32_t N, int32_t H,
                                             int32_t W, int32_t D, int32_t C, void* workspace,
                                             int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment,
                                             void* stream)
{
    return pool_fwd_run("avgpool_ceil_stats", x, nullptr, nullptr, y, mean, sqmean, N, H, W, D, C, workspace,
                        workspace_bytes, blocks, waves, segment, stream);
}

extern "C" int kerops_bnrelu_avgpool_ceil_stats_f16(const void* x, const float* weight, const float* bias, void* y,
                                                    float* mean, float* sqmean, int32_t N, int32_t H, int32_t W,
                                                    int32_t D, int32_t C, void* workspace, int64_t workspace_bytes,
                                                    int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    if (!weight || !bias) {
        set_error("bnrelu_avgpool_ceil_stats: null weight or bias");
        return KEROPS_E_BADARG;
    }
    return pool_fwd_run("bnrelu_avgpool_ceil_stats", x, weight, bias, y, mean, sqmean, N, H, W, D, C, workspace,
                        workspace_bytes, blocks, waves, segment, stream);
}

extern "C" int kerops_avgpool_ceil_stats_bwd_f16(const void* inpgrad, const float* meangrad, const float* sqmeangrad,
                                                 const void* output, void* dx, int32_t N, int32_t H, int32_t W,
                                                 int32_t D, int32_t C, int32_t blocks, int32_t waves, int32_t segment,
                                                 void* stream)
{
    PoolDims p;
    int64_t nchunks = 0;
    StreamShape sh;
    int rc = pool_plan("avgpool_ceil_stats_bwd", kDefPoolBwd, N, H, W, D, C, blocks, waves, segment, &p, &nchunks, &sh);
    if (rc != KEROPS_OK) return rc;
    if (!inpgrad || !meangrad || !sqmeangrad || !output || !dx || !aligned16(inpgrad) || !aligned16(output) ||
        !aligned16(dx)) {
        set_error("avgpool_ceil_stats_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    const float fMo = (float)((int64_t)N * p.Ho * p.Wo * p.Do);
    const int seg = sh.segment != 1;
    // redistribute the results for whole-line stores where a voxel row is narrower than a 128-byte line
    const bool perm = C >= 8 && C < 64 && D % 2 == 0 && ((int64_t)p.Do * p.CG) % kWave == 0;
#define KEROPS_POOLB_GO(Uv)                                                                                          \
    KEROPS_DISPATCH_V(C, {                                                                                           \
        if (perm && V == 8)                                                                                          \
            hipLaunchKernelGGL((avgpool_bwd_kernel<V, Uv, V == 8>), dim3(sh.blocks), dim3(sh.threads), 0,            \
                               (hipStream_t)stream, (const half_t*)inpgrad, meangrad, sqmeangrad,                    \
                               (const half_t*)output, (half_t*)dx, p, nchunks, fMo, seg);                            \
        else                                                                                                         \
            hipLaunchKernelGGL((avgpool_bwd_kernel<V, Uv, false>), dim3(sh.blocks), dim3(sh.threads), 0,             \
                               (hipStream_t)stream, (const half_t*)inpgrad, meangrad, sqmeangrad,                    \
                               (const half_t*)output, (half_t*)dx, p, nchunks, fMo, seg);                            \
    })
    if (sh.segment == 2) KEROPS_POOLB_GO(2);
    else KEROPS_POOLB_GO(1);
#undef KEROPS_POOLB_GO
    return check_launch("avgpool_ceil_stats_bwd");
}
