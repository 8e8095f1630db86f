// Flat per-voxel stream kernels on [M][C] fp16 data (M = N*H*W*D voxels): per-channel
// statistics, BN-ReLU forward/backward, residual add with statistics, the uint8 window
// quantiser pair and the symmetric int8 quantiser.
//
// All of them are HBM-bound.  Each is a persistent grid-stride loop of 256-thread
// workgroups: a thread moves V = min(8, C) consecutive channels per access (16 bytes for
// C >= 8), consecutive lanes take consecutive chunks, and the grid stride is a multiple
// of the number of channel groups, so a thread keeps one channel group for its whole
// life: per-channel parameters sit in registers and per-channel sums are plain
// per-thread fp32 accumulators.  Reductions finish with wavefront shuffles, one LDS
// hop per workgroup, a [workgroups][..] partial buffer and a small fp64 second pass:
// no float atomics, identical bits on every run.
#include "common.hpp"

namespace kerops {

// ------------------------------------------------------------------ Stats
template <int V, bool ADD>
__global__ __launch_bounds__(kStreamThreads) void stats_kernel(const half_t* x, const half_t* y, half_t* z,
                                                               float* __restrict__ ws, int64_t nchunks, int CG)
{
    typedef typename HVec<V>::type hv;
    __shared__ float red[kStreamWaves * 2 * 64 * V];
    const int64_t T = (int64_t)gridDim.x * kStreamThreads;
    float acc[2][V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[0][j] = acc[1][j] = 0.0f;

    auto body = [&](int64_t i) {
        hv v = ld_stream<V>(x, i);
        if (ADD) {
            const hv u = ld_stream<V>(y, i);
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = (half_t)((float)v[j] + (float)u[j]);  // fp16 sum, RNE
            st_stream<V>(z, i, v);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float f = (float)v[j];
            acc[0][j] += f;
            acc[1][j] = __builtin_fmaf(f, f, acc[1][j]);
        }
    };
    int64_t i = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    for (; i + 3 * T < nchunks; i += 4 * T) {
        if (!ADD) {
            const hv v0 = ld_stream<V>(x, i), v1 = ld_stream<V>(x, i + T), v2 = ld_stream<V>(x, i + 2 * T),
                     v3 = ld_stream<V>(x, i + 3 * T);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const float f0 = (float)v0[j], f1 = (float)v1[j], f2 = (float)v2[j], f3 = (float)v3[j];
                acc[0][j] += (f0 + f1) + (f2 + f3);
                acc[1][j] += __builtin_fmaf(f0, f0, f1 * f1) + __builtin_fmaf(f2, f2, f3 * f3);
            }
        } else {
            body(i);
            body(i + T);
            body(i + 2 * T);
            body(i + 3 * T);
        }
    }
    for (; i < nchunks; i += T) body(i);
    block_channel_partials<2, V>(acc, CG, red, ws + (int64_t)blockIdx.x * 2 * CG * V);
}

static int check_reduce_args(const char* op, int64_t M, int C, int* blocks, int64_t* need)
{
    if (M <= 0 || C <= 0 || !is_pow2(C)) {
        set_error("%s: M must be positive and C a power of two (M=%lld C=%d)", op, (long long)M, C);
        return KEROPS_E_BADARG;
    }
    if (C > kMaxReduceChannels) {
        set_error("%s: per-channel reductions are built for C <= %d (got %d)", op, kMaxReduceChannels, C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    const int V = C >= 8 ? 8 : C;
    if (*blocks <= 0) *blocks = stream_blocks_default(M * (C / V));
    if (*blocks > 65536) {
        set_error("%s: blocks must be <= 65536", op);
        return KEROPS_E_BADARG;
    }
    *need = (int64_t)(*blocks) * 2 * C * (int64_t)sizeof(float);
    return KEROPS_OK;
}

static int check_ws(const char* op, const void* ws, int64_t have, int64_t need)
{
    if (!ws || !aligned16(ws) || have < need) {
        set_error("%s: workspace of %lld bytes required, %lld given", op, (long long)need, (long long)have);
        return KEROPS_E_WORKSPACE;
    }
    return KEROPS_OK;
}

// ---------------------------------------------------------- stats backward
template <int V, bool ADD>
__global__ __launch_bounds__(kStreamThreads) void stats_bwd_kernel(const half_t* __restrict__ x,
                                                                   const half_t* __restrict__ add_grad,
                                                                   const float* __restrict__ mean_grad,
                                                                   const float* __restrict__ sqmean_grad,
                                                                   half_t* __restrict__ dx, int64_t nchunks, int CG,
                                                                   float fm)
{
    typedef typename HVec<V>::type hv;
    const int64_t T = (int64_t)gridDim.x * kStreamThreads;
    int64_t i = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    const int cg = (int)(i % CG);
    float sg[V], mg[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        sg[j] = sqmean_grad[cg * V + j];
        mg[j] = __fdiv_rn(mean_grad[cg * V + j], fm);
    }
    auto one = [&](const hv& v, const hv& g) {
        hv o;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float a = __fdiv_rn(__fmul_rn(__fmul_rn(2.0f, (float)v[j]), sg[j]), fm);
            o[j] = ADD ? (half_t)__fadd_rn(__fadd_rn((float)g[j], a), mg[j]) : (half_t)__fadd_rn(a, mg[j]);
        }
        return o;
    };
    constexpr int U = 4;  // chunks in flight per lane and input stream
    for (; i + (U - 1) * T < nchunks; i += U * T) {
        hv v[U], g[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] = ld_stream<V>(x, i + u * T);
            g[u] = ADD ? ld_stream<V>(add_grad, i + u * T) : v[u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) st_stream<V>(dx, i + u * T, one(v[u], g[u]));
    }
    for (; i < nchunks; i += T) {
        const hv v = ld_stream<V>(x, i);
        st_stream<V>(dx, i, one(v, ADD ? ld_stream<V>(add_grad, i) : v));
    }
}

// ---------------------------------------------------------------- BN-ReLU
template <int V>
__global__ __launch_bounds__(kStreamThreads) void bnrelu_fwd_kernel(const half_t* __restrict__ x,
                                                                    const float* __restrict__ wv,
                                                                    const float* __restrict__ bv,
                                                                    half_t* __restrict__ y, int64_t nchunks, int CG)
{
    typedef typename HVec<V>::type hv;
    const int64_t T = (int64_t)gridDim.x * kStreamThreads;
    int64_t i = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    const int cg = (int)(i % CG);
    float w[V], b[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        w[j] = wv[cg * V + j];
        b[j] = bv[cg * V + j];
    }
    auto act = [&](const hv& v) {
        hv o;
#pragma unroll
        for (int j = 0; j < V; ++j) o[j] = (half_t)fmaxf(__builtin_fmaf((float)v[j], w[j], b[j]), 0.0f);
        return o;
    };
    for (; i + 3 * T < nchunks; i += 4 * T) {
        const hv v0 = ld_stream<V>(x, i), v1 = ld_stream<V>(x, i + T), v2 = ld_stream<V>(x, i + 2 * T), v3 = ld_stream<V>(x, i + 3 * T);
        st_stream<V>(y, i, act(v0));
        st_stream<V>(y, i + T, act(v1));
        st_stream<V>(y, i + 2 * T, act(v2));
        st_stream<V>(y, i + 3 * T, act(v3));
    }
    for (; i < nchunks; i += T) st_stream<V>(y, i, act(ld_stream<V>(x, i)));
}

template <int V>
__global__ __launch_bounds__(kStreamThreads) void bnrelu_bwd_kernel(const half_t* __restrict__ x,
                                                                    const float* __restrict__ wv,
                                                                    const float* __restrict__ bv,
                                                                    const half_t* __restrict__ g,
                                                                    half_t* __restrict__ dx, float* __restrict__ ws,
                                                                    int64_t nchunks, int CG)
{
    typedef typename HVec<V>::type hv;
    __shared__ float red[kStreamWaves * 2 * 64 * V];
    const int64_t T = (int64_t)gridDim.x * kStreamThreads;
    int64_t i = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    const int cg = (int)(i % CG);
    float w[V], nb[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        w[j] = wv[cg * V + j];
        nb[j] = -bv[cg * V + j];
    }
    float acc[2][V];  // [0] = dW, [1] = dB
#pragma unroll
    for (int j = 0; j < V; ++j) acc[0][j] = acc[1][j] = 0.0f;
    auto body = [&](int64_t k, const hv& xv, const hv& gv) {
        hv o;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float xf = (float)xv[j];
            const float gm = __fmul_rn((float)gv[j], (__fmul_rn(xf, w[j]) > nb[j]) ? 1.0f : 0.0f);  // keeps the sign of zero
            o[j] = (half_t)__fmul_rn(w[j], gm);
            acc[0][j] = __builtin_fmaf(xf, gm, acc[0][j]);
            acc[1][j] += gm;
        }
        st_stream<V>(dx, k, o);
    };
    for (; i + T < nchunks; i += 2 * T) {
        const hv x0 = ld_stream<V>(x, i), x1 = ld_stream<V>(x, i + T);
        const hv g0 = ld_stream<V>(g, i), g1 = ld_stream<V>(g, i + T);
        body(i, x0, g0);
        body(i + T, x1, g1);
    }
    for (; i < nchunks; i += T) body(i, ld_stream<V>(x, i), ld_stream<V>(g, i));
    block_channel_partials<2, V>(acc, CG, red, ws + (int64_t)blockIdx.x * 2 * CG * V);
}

// ------------------------------------------------------------ quantisers
typedef __bf16 bf16_t;
template <typename T>
__device__ __forceinline__ float to_f32(T v)
{
    return (float)v;
}

// Correctly rounded a / b for a divisor that is constant over the launch, in 3 VALU instructions
// instead of the ~11 of the generic IEEE sequence: with rb = RN(1/b) correctly rounded,
// q0 = RN(a*rb), e = a - q0*b (exact in one FMA), q = RN(q0 + e*rb) is the correctly rounded
// quotient (Markstein).  Valid when nothing over/underflows on the way; the callers guarantee the
// operand ranges (see the launchers) and fall back to the IEEE division otherwise.
__device__ __forceinline__ float div_by_const(float a, float b, float rb)
{
    const float q0 = __fmul_rn(a, rb);
    const float e = __builtin_fmaf(-q0, b, a);
    return __builtin_fmaf(e, rb, q0);
}

template <bool FAST>
__device__ __forceinline__ uint32_t quant_u8_one(float t, float window, float two_w, float r_two_w)
{
    t = fminf(fmaxf(t, -window), window);
    t = __fadd_rn(t, window);
    t = FAST ? div_by_const(t, two_w, r_two_w) : __fdiv_rn(t, two_w);
    t = __fmul_rn(t, 255.0f);
    return (uint32_t)t;  // truncation toward zero
}

// The quantisers move 16 bytes per lane on their wide side (8 two-byte or 4 four-byte elements) and the matching
// 8 or 4 bytes on the byte side, consecutive lanes on consecutive pieces: every load and every store instruction of
// a wavefront covers one contiguous run of whole 128-byte lines (1 KiB wide side, 512 or 256 bytes byte side).
// A lane that took 16 bytes of the byte side instead would touch the wide side with two or four accesses that
// interleave with its neighbours' (alternate 16-byte pieces per instruction): measured, that wrote 1.135x the
// tensor size to HBM in partial lines.
template <typename T>
struct QuantUnit {
    static constexpr int E = 16 / (int)sizeof(T);  // elements of one lane and step
    typedef T wide_t __attribute__((ext_vector_type(E)));
    typedef uint32_t bytes_t __attribute__((ext_vector_type(E / 4)));
};
template <>
struct QuantUnit<float> {
    static constexpr int E = 4;
    typedef float wide_t __attribute__((ext_vector_type(4)));
    typedef uint32_t bytes_t;
};
__device__ __forceinline__ uint32_t bytes_word(const uint32_t& v, int) { return v; }
__device__ __forceinline__ uint32_t bytes_word(const u32x2_t& v, int k) { return v[k]; }
__device__ __forceinline__ void set_bytes_word(uint32_t& v, int, uint32_t w) { v = w; }
__device__ __forceinline__ void set_bytes_word(u32x2_t& v, int k, uint32_t w) { v[k] = w; }

constexpr int kQuantInFlight = 4;  // steps in flight per lane

template <typename T, bool FAST>
__global__ __launch_bounds__(kStreamThreads) void quant_u8_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                                  int64_t numel, float window, float r_two_w)
{
    typedef QuantUnit<T> QU;
    constexpr int E = QU::E, U = kQuantInFlight;
    const float two_w = __fmul_rn(2.0f, window);
    const int64_t nunits = numel / E;
    const int64_t Tn = (int64_t)gridDim.x * kStreamThreads;
    const int64_t gid = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    auto one = [&](const typename QU::wide_t& v) {
        typename QU::bytes_t o;
#pragma unroll
        for (int k = 0; k < E / 4; ++k) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w |= quant_u8_one<FAST>(to_f32(v[4 * k + j]), window, two_w, r_two_w) << (8 * j);
            set_bytes_word(o, k, w);
        }
        return o;
    };
    const typename QU::wide_t* xv = reinterpret_cast<const typename QU::wide_t*>(x);
    typename QU::bytes_t* qv = reinterpret_cast<typename QU::bytes_t*>(q);
    int64_t i = gid;
    for (; i + (U - 1) * Tn < nunits; i += U * Tn) {
        typename QU::wide_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(xv + i + u * Tn);
#pragma unroll
        for (int u = 0; u < U; ++u) __builtin_nontemporal_store(one(v[u]), qv + i + u * Tn);
    }
    for (; i < nunits; i += Tn) __builtin_nontemporal_store(one(__builtin_nontemporal_load(xv + i)), qv + i);
    if (gid == 0) {
        for (int64_t k = nunits * E; k < numel; ++k)
            q[k] = (uint8_t)quant_u8_one<FAST>(to_f32(x[k]), window, two_w, r_two_w);
    }
}

template <typename T>
__global__ __launch_bounds__(kStreamThreads) void dequant_u8_kernel(const uint8_t* __restrict__ q,
                                                                    T* __restrict__ out, int64_t numel, float window)
{
    typedef QuantUnit<T> QU;
    constexpr int E = QU::E, U = kQuantInFlight;
    const float scale = __fdiv_rn(__fmul_rn(2.0f, window), 255.0f);
    const int64_t nunits = numel / E;
    const int64_t Tn = (int64_t)gridDim.x * kStreamThreads;
    const int64_t gid = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    auto one = [&](const typename QU::bytes_t& b) {
        typename QU::wide_t o;
#pragma unroll
        for (int j = 0; j < E; ++j)
            o[j] = (T)__fsub_rn(__fmul_rn((float)((bytes_word(b, j / 4) >> (8 * (j % 4))) & 0xffu), scale), window);
        return o;
    };
    const typename QU::bytes_t* qv = reinterpret_cast<const typename QU::bytes_t*>(q);
    typename QU::wide_t* ov = reinterpret_cast<typename QU::wide_t*>(out);
    int64_t i = gid;
    for (; i + (U - 1) * Tn < nunits; i += U * Tn) {
        typename QU::bytes_t b[U];
#pragma unroll
        for (int u = 0; u < U; ++u) b[u] = __builtin_nontemporal_load(qv + i + u * Tn);
#pragma unroll
        for (int u = 0; u < U; ++u) __builtin_nontemporal_store(one(b[u]), ov + i + u * Tn);
    }
    for (; i < nunits; i += Tn) __builtin_nontemporal_store(one(__builtin_nontemporal_load(qv + i)), ov + i);
    if (gid == 0) {
        for (int64_t k = nunits * E; k < numel; ++k)
            out[k] = (T)__fsub_rn(__fmul_rn((float)q[k], scale), window);
    }
}

// 16 consecutive fp16 values per lane (two 16-byte loads) for one 16-byte store of bytes: the int8 pass
template <typename T>
__device__ __forceinline__ void load16(const T* p, float (&f)[16])
{
    typedef T tv8 __attribute__((ext_vector_type(8)));
    const tv8 a = __builtin_nontemporal_load(reinterpret_cast<const tv8*>(p));
    const tv8 b = __builtin_nontemporal_load(reinterpret_cast<const tv8*>(p + 8));
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        f[j] = (float)a[j];
        f[8 + j] = (float)b[j];
    }
}
__device__ __forceinline__ u32x4_t pack16(const uint32_t (&b)[16])
{
    u32x4_t o;
#pragma unroll
    for (int w = 0; w < 4; ++w) o[w] = b[4 * w] | (b[4 * w + 1] << 8) | (b[4 * w + 2] << 16) | (b[4 * w + 3] << 24);
    return o;
}

__global__ __launch_bounds__(kStreamThreads) void absmax_kernel(const half_t* __restrict__ y, float* __restrict__ ws,
                                                                int64_t numel)
{
    __shared__ float red[kStreamWaves];
    const int64_t nchunks = numel / 8;
    const int64_t Tn = (int64_t)gridDim.x * kStreamThreads;
    const int64_t gid = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    float m = 0.0f;
    int64_t i = gid;
    for (; i + 3 * Tn < nchunks; i += 4 * Tn) {
        const half8_t v0 = load_c8_nt(y + i * 8), v1 = load_c8_nt(y + (i + Tn) * 8), v2 = load_c8_nt(y + (i + 2 * Tn) * 8),
                      v3 = load_c8_nt(y + (i + 3 * Tn) * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            m = fmaxf(m, fmaxf(fmaxf(fabsf((float)v0[j]), fabsf((float)v1[j])),
                               fmaxf(fabsf((float)v2[j]), fabsf((float)v3[j]))));
        }
    }
    for (; i < nchunks; i += Tn) {
        const half8_t v = load_c8_nt(y + i * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf((float)v[j]));
    }
    if (gid == 0) {
        for (int64_t k = nchunks * 8; k < numel; ++k) m = fmaxf(m, fabsf((float)y[k]));
    }
    m = wave_max(m);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = red[0];
#pragma unroll
        for (int wv = 1; wv < kStreamWaves; ++wv) r = fmaxf(r, red[wv]);
        ws[blockIdx.x] = r;
    }
}

__global__ __launch_bounds__(kStreamThreads) void absmax_final_kernel(const float* __restrict__ ws, int n,
                                                                      float* __restrict__ out)
{
    __shared__ float red[kStreamWaves];
    float m = 0.0f;
    for (int i = threadIdx.x; i < n; i += kStreamThreads) m = fmaxf(m, ws[i]);
    m = wave_max(m);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = red[0];
#pragma unroll
        for (int wv = 1; wv < kStreamWaves; ++wv) r = fmaxf(r, red[wv]);
        out[0] = r;
    }
}

__device__ __forceinline__ uint32_t quant_i8_one(float v, float scale, float rscale)
{
    // |v| <= 65504 and scale = absmax/127 >= 2^-31: no overflow; a quotient that underflows rounds to 0
    float t = rintf(div_by_const(v, scale, rscale));  // round half to even
    t = fminf(fmaxf(t, -127.0f), 127.0f);
    return (uint32_t)((int)t) & 0xffu;
}

__global__ __launch_bounds__(kStreamThreads) void quant_i8_kernel(const half_t* __restrict__ y,
                                                                  const float* __restrict__ absmax,
                                                                  int8_t* __restrict__ q, int64_t numel)
{
    const float scale = __fdiv_rn(absmax[0], 127.0f);
    const bool zero = (scale == 0.0f);
    const float rscale = __fdiv_rn(1.0f, zero ? 1.0f : scale);  // correctly rounded reciprocal, once per thread
    const int64_t ngroups = numel / 16;
    const int64_t Tn = (int64_t)gridDim.x * kStreamThreads;
    const int64_t gid = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
    for (int64_t i = gid; i < ngroups; i += Tn) {
        float f[16];
        load16<half_t>(y + i * 16, f);
        uint32_t b[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) b[j] = zero ? 0u : quant_i8_one(f[j], scale, rscale);
        __builtin_nontemporal_store(pack16(b), reinterpret_cast<u32x4_t*>(q + i * 16));
    }
    if (gid == 0) {
        for (int64_t k = ngroups * 16; k < numel; ++k)
            q[k] = zero ? (int8_t)0 : (int8_t)quant_i8_one((float)y[k], scale, rscale);
    }
}

}  // namespace kerops

using namespace kerops;

// ------------------------------------------------------------------ C ABI

extern "C" int64_t kerops_stats_workspace_bytes(int64_t M, int32_t C, int32_t blocks)
{
    int64_t need = 0;
    int rc = check_reduce_args("stats", M, C, &blocks, &need);
    return rc != KEROPS_OK ? rc : need;
}

static int stats_common(const char* op, const void* x, const void* y, void* z, float* mean, float* sqmean, int64_t M,
                        int32_t C, void* workspace, int64_t workspace_bytes, int32_t blocks, void* stream)
{
    int64_t need = 0;
    int rc = check_reduce_args(op, M, C, &blocks, &need);
    if (rc != KEROPS_OK) return rc;
    const bool add = (y != nullptr);
    if (!x || !mean || !sqmean || !aligned16(x) || (add && (!z || !aligned16(y) || !aligned16(z)))) {
        set_error("%s: null or misaligned pointer", op);
        return KEROPS_E_BADARG;
    }
    rc = check_ws(op, workspace, workspace_bytes, need);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    const int64_t nchunks = M * CG;
    float* ws = (float*)workspace;
    KEROPS_DISPATCH_V(C, {
        if (add) {
            hipLaunchKernelGGL((stats_kernel<V, true>), dim3(blocks), dim3(kStreamThreads), 0, s, (const half_t*)x,
                               (const half_t*)y, (half_t*)z, ws, nchunks, CG);
        } else {
            hipLaunchKernelGGL((stats_kernel<V, false>), dim3(blocks), dim3(kStreamThreads), 0, s, (const half_t*)x,
                               (const half_t*)nullptr, (half_t*)nullptr, ws, nchunks, CG);
        }
    });
    rc = check_launch(op);
    if (rc != KEROPS_OK) return rc;
    launch_reduce_rows(ws, blocks, 2 * C, mean, sqmean, C, 1.0 / (double)M, s);
    return check_launch(op);
}

extern "C" int kerops_stats_f16(const void* x, float* mean, float* sqmean, int64_t M, int32_t C, void* workspace,
                                int64_t workspace_bytes, int32_t blocks, void* stream)
{
    return stats_common("stats", x, nullptr, nullptr, mean, sqmean, M, C, workspace, workspace_bytes, blocks, stream);
}

extern "C" int kerops_add_stats_f16(const void* x, const void* y, void* z, float* mean, float* sqmean, int64_t M,
                                    int32_t C, void* workspace, int64_t workspace_bytes, int32_t blocks, void* stream)
{
    if (!y) {
        set_error("add_stats: null pointer");
        return KEROPS_E_BADARG;
    }
    return stats_common("add_stats", x, y, z, mean, sqmean, M, C, workspace, workspace_bytes, blocks, stream);
}

static int check_stream_args(const char* op, int64_t M, int C, int* blocks)
{
    if (M <= 0 || C <= 0 || !is_pow2(C)) {
        set_error("%s: M must be positive and C a power of two (M=%lld C=%d)", op, (long long)M, C);
        return KEROPS_E_BADARG;
    }
    const int V = C >= 8 ? 8 : C;
    if (*blocks <= 0) *blocks = stream_blocks_default(M * (C / V));
    // a thread keeps one channel group only if the grid stride is a multiple of C/V
    const int CG = C / V;
    if (((int64_t)(*blocks) * kStreamThreads) % CG != 0) {
        set_error("%s: blocks*256 must be a multiple of C/8", op);
        return KEROPS_E_BADARG;
    }
    return KEROPS_OK;
}

static int stats_bwd_common(const char* op, const void* x, const void* add_grad, const float* mean_grad,
                            const float* sqmean_grad, void* dx, int64_t M, int32_t C, int32_t blocks, void* stream)
{
    int rc = check_stream_args(op, M, C, &blocks);
    if (rc != KEROPS_OK) return rc;
    if (!x || !mean_grad || !sqmean_grad || !dx || !aligned16(x) || !aligned16(dx) ||
        (add_grad && !aligned16(add_grad))) {
        set_error("%s: null or misaligned pointer", op);
        return KEROPS_E_BADARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    const int64_t nchunks = M * CG;
    KEROPS_DISPATCH_V(C, {
        if (add_grad) {
            hipLaunchKernelGGL((stats_bwd_kernel<V, true>), dim3(blocks), dim3(kStreamThreads), 0, s,
                               (const half_t*)x, (const half_t*)add_grad, mean_grad, sqmean_grad, (half_t*)dx,
                               nchunks, CG, (float)M);
        } else {
            hipLaunchKernelGGL((stats_bwd_kernel<V, false>), dim3(blocks), dim3(kStreamThreads), 0, s,
                               (const half_t*)x, (const half_t*)nullptr, mean_grad, sqmean_grad, (half_t*)dx, nchunks,
                               CG, (float)M);
        }
    });
    return check_launch(op);
}

extern "C" int kerops_stats_bwd_f16(const void* x, const float* mean_grad, const float* sqmean_grad, void* dx,
                                    int64_t M, int32_t C, int32_t blocks, void* stream)
{
    return stats_bwd_common("stats_bwd", x, nullptr, mean_grad, sqmean_grad, dx, M, C, blocks, stream);
}

extern "C" int kerops_add_stats_bwd_f16(const void* add_grad, const float* mean_grad, const float* sqmean_grad,
                                        const void* add_result, void* out, int64_t M, int32_t C, int32_t blocks,
                                        void* stream)
{
    if (!add_grad) {
        set_error("add_stats_bwd: null pointer");
        return KEROPS_E_BADARG;
    }
    return stats_bwd_common("add_stats_bwd", add_result, add_grad, mean_grad, sqmean_grad, out, M, C, blocks, stream);
}

extern "C" int kerops_bnrelu_fwd_f16(const void* x, const float* wv, const float* bv, void* y, int64_t M, int32_t C,
                                     int32_t blocks, void* stream)
{
    int rc = check_stream_args("bnrelu_fwd", M, C, &blocks);
    if (rc != KEROPS_OK) return rc;
    if (!x || !wv || !bv || !y || !aligned16(x) || !aligned16(y)) {
        set_error("bnrelu_fwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    KEROPS_DISPATCH_V(C, {
        hipLaunchKernelGGL((bnrelu_fwd_kernel<V>), dim3(blocks), dim3(kStreamThreads), 0, s, (const half_t*)x, wv, bv,
                           (half_t*)y, M * CG, CG);
    });
    return check_launch("bnrelu_fwd");
}

extern "C" int kerops_bnrelu_bwd_f16(const void* x, const float* wv, const float* bv, const void* g, void* dx,
                                     float* dW, float* dB, int64_t M, int32_t C, void* workspace,
                                     int64_t workspace_bytes, int32_t blocks, void* stream)
{
    int64_t need = 0;
    int rc = check_reduce_args("bnrelu_bwd", M, C, &blocks, &need);
    if (rc != KEROPS_OK) return rc;
    if (!x || !wv || !bv || !g || !dx || !dW || !dB || !aligned16(x) || !aligned16(g) || !aligned16(dx)) {
        set_error("bnrelu_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    rc = check_ws("bnrelu_bwd", workspace, workspace_bytes, need);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    float* ws = (float*)workspace;
    KEROPS_DISPATCH_V(C, {
        hipLaunchKernelGGL((bnrelu_bwd_kernel<V>), dim3(blocks), dim3(kStreamThreads), 0, s, (const half_t*)x, wv, bv,
                           (const half_t*)g, (half_t*)dx, ws, M * CG, CG);
    });
    rc = check_launch("bnrelu_bwd");
    if (rc != KEROPS_OK) return rc;
    launch_reduce_rows(ws, blocks, 2 * C, dW, dB, C, 1.0, s);
    return check_launch("bnrelu_bwd");
}

static int check_flat(const char* op, const void* a, const void* b, int64_t numel, int* blocks)
{
    if (!a || !b || !aligned16(a) || !aligned16(b) || numel <= 0) {
        set_error("%s: null or misaligned pointer, or non-positive numel", op);
        return KEROPS_E_BADARG;
    }
    if (*blocks <= 0) *blocks = stream_blocks_default(ceil_div64(numel, 16), 768);
    return KEROPS_OK;
}

extern "C" int kerops_quant_u8_window(const void* x, int32_t dtype, void* q, int64_t numel, float window,
                                      int32_t blocks, void* stream)
{
    int rc = check_flat("quant_u8_window", x, q, numel, &blocks);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    // 1/(2w) correctly rounded to fp32: the double quotient rounded once more is exact for division
    // (53 >= 2*24 + 2 bits).  The 3-instruction division needs 2w and its quotients to stay normal.
    const float two_w = 2.0f * window;
    const bool fast = window >= 0x1p-60f && window <= 0x1p60f;
    const float r_two_w = fast ? (float)(1.0 / (double)two_w) : 0.0f;
#define KEROPS_QU8_GO(T, F)                                                                                     \
    hipLaunchKernelGGL((quant_u8_kernel<T, F>), dim3(blocks), dim3(kStreamThreads), 0, s, (const T*)x, (uint8_t*)q, \
                       numel, window, r_two_w)
    if (dtype == KEROPS_DTYPE_F16) {
        if (fast) KEROPS_QU8_GO(half_t, true);
        else KEROPS_QU8_GO(half_t, false);
    } else if (dtype == KEROPS_DTYPE_BF16) {
        if (fast) KEROPS_QU8_GO(bf16_t, true);
        else KEROPS_QU8_GO(bf16_t, false);
    } else if (dtype == KEROPS_DTYPE_F32) {
        if (fast) KEROPS_QU8_GO(float, true);
        else KEROPS_QU8_GO(float, false);
    } else {
        set_error("quant_u8_window: unknown dtype tag %d", dtype);
        return KEROPS_E_BADARG;
    }
#undef KEROPS_QU8_GO
    return check_launch("quant_u8_window");
}

extern "C" int kerops_dequant_u8_window(const void* q, void* out, int32_t dtype, int64_t numel, float window,
                                        int32_t blocks, void* stream)
{
    int rc = check_flat("dequant_u8_window", q, out, numel, &blocks);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == KEROPS_DTYPE_F16) {
        hipLaunchKernelGGL((dequant_u8_kernel<half_t>), dim3(blocks), dim3(kStreamThreads), 0, s, (const uint8_t*)q,
                           (half_t*)out, numel, window);
    } else if (dtype == KEROPS_DTYPE_BF16) {
        hipLaunchKernelGGL((dequant_u8_kernel<bf16_t>), dim3(blocks), dim3(kStreamThreads), 0, s, (const uint8_t*)q,
                           (bf16_t*)out, numel, window);
    } else if (dtype == KEROPS_DTYPE_F32) {
        hipLaunchKernelGGL((dequant_u8_kernel<float>), dim3(blocks), dim3(kStreamThreads), 0, s, (const uint8_t*)q,
                           (float*)out, numel, window);
    } else {
        set_error("dequant_u8_window: unknown dtype tag %d", dtype);
        return KEROPS_E_BADARG;
    }
    return check_launch("dequant_u8_window");
}

extern "C" int64_t kerops_absmax_workspace_bytes(int32_t blocks)
{
    if (blocks <= 0) blocks = 768;
    return (int64_t)blocks * (int64_t)sizeof(float);
}

extern "C" int kerops_absmax_f16(const void* y, float* absmax, int64_t numel, void* workspace,
                                 int64_t workspace_bytes, int32_t blocks, void* stream)
{
    if (blocks <= 0) blocks = 768;
    int b = blocks;
    int rc = check_flat("absmax", y, absmax, numel, &b);
    if (rc != KEROPS_OK) return rc;
    rc = check_ws("absmax", workspace, workspace_bytes, (int64_t)blocks * 4);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(absmax_kernel, dim3(blocks), dim3(kStreamThreads), 0, s, (const half_t*)y, (float*)workspace,
                       numel);
    rc = check_launch("absmax");
    if (rc != KEROPS_OK) return rc;
    hipLaunchKernelGGL(absmax_final_kernel, dim3(1), dim3(kStreamThreads), 0, s, (const float*)workspace, blocks,
                       absmax);
    return check_launch("absmax");
}

extern "C" int kerops_quant_i8_sym_f16(const void* y, const float* absmax, void* q, int64_t numel, int32_t blocks,
                                       void* stream)
{
    int rc = check_flat("quant_i8_sym", y, q, numel, &blocks);
    if (rc != KEROPS_OK) return rc;
    if (!absmax) {
        set_error("quant_i8_sym: null absmax");
        return KEROPS_E_BADARG;
    }
    hipLaunchKernelGGL(quant_i8_kernel, dim3(blocks), dim3(kStreamThreads), 0, (hipStream_t)stream,
                       (const half_t*)y, absmax, (int8_t*)q, numel);
    return check_launch("quant_i8_sym");
}
