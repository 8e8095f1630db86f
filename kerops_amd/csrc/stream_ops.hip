// Flat per-voxel stream kernels on [M][C] fp16 data (M = N*H*W*D voxels): per-channel
// statistics, BN-ReLU forward/backward, residual add with statistics, the uint8 window
// quantiser pair and the symmetric int8 quantiser.
//
// All of them are HBM-bound.  Each is a persistent loop of 256- or 1024-thread workgroups
// over steps of U chunks per thread (ChunkWalk in common.hpp: interleaved, or one contiguous
// segment per workgroup and step): a thread moves V = min(8, C) consecutive channels per
// access (16 bytes for C >= 8), consecutive lanes take consecutive chunks, and every stride
// of the walk is a multiple of the number of channel groups, so a thread keeps one channel
// group for its whole life: per-channel parameters sit in registers and per-channel sums
// are plain per-thread fp32 accumulators.  Reductions finish with wavefront shuffles, one LDS
// hop per workgroup, a [workgroups][..] partial buffer and a small fp64 second pass:
// no float atomics, identical bits on every run.
#include "common.hpp"

namespace kerops {

// ------------------------------------------------------------------ Stats
template <int V, int U, bool ADD>
__global__ __launch_bounds__(kStreamMaxThreads) void stats_kernel(const half_t* x, const half_t* y, half_t* z,
                                                                  float* __restrict__ ws, int64_t nchunks, int CG,
                                                                  int segments)
{
    typedef typename HVec<V>::type hv;
    __shared__ float red[4 * 2 * 64 * V];
    const ChunkWalk<U> wk(nchunks, segments != 0);
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
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        hv v[U], w[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] = ld_stream<V>(x, i + u * wk.su);
            w[u] = ADD ? ld_stream<V>(y, i + u * wk.su) : v[u];
        }
        if (ADD) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int j = 0; j < V; ++j) v[u][j] = (half_t)((float)v[u][j] + (float)w[u][j]);  // fp16 sum, RNE
                st_stream<V>(z, i + u * wk.su, v[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u += 4) {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const float f0 = (float)v[u][j], f1 = (float)v[u + 1][j], f2 = (float)v[u + 2][j],
                            f3 = (float)v[u + 3][j];
                acc[0][j] += (f0 + f1) + (f2 + f3);
                acc[1][j] += __builtin_fmaf(f0, f0, f1 * f1) + __builtin_fmaf(f2, f2, f3 * f3);
            }
        }
    }
    for (int64_t i = wk.tail; i < nchunks; i += wk.T) body(i);
    block_channel_partials_any<2, V>(acc, CG, red, ws + (int64_t)blockIdx.x * 2 * CG * V);
}

// ---------------------------------------------------------- stats backward
template <int V, int U, bool ADD>
__global__ __launch_bounds__(kStreamMaxThreads) void stats_bwd_kernel(const half_t* __restrict__ x,
                                                                      const half_t* __restrict__ add_grad,
                                                                      const float* __restrict__ mean_grad,
                                                                      const float* __restrict__ sqmean_grad,
                                                                      half_t* __restrict__ dx, int64_t nchunks, int CG,
                                                                      float fm, int segments)
{
    typedef typename HVec<V>::type hv;
    const ChunkWalk<U> wk(nchunks, segments != 0);
    const int cg = (int)(wk.first % CG);
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
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        hv v[U], g[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] = ld_stream<V>(x, i + u * wk.su);
            g[u] = ADD ? ld_stream<V>(add_grad, i + u * wk.su) : v[u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) st_stream<V>(dx, i + u * wk.su, one(v[u], g[u]));
    }
    for (int64_t i = wk.tail; i < nchunks; i += wk.T) {
        const hv v = ld_stream<V>(x, i);
        st_stream<V>(dx, i, one(v, ADD ? ld_stream<V>(add_grad, i) : v));
    }
}

// ---------------------------------------------------------------- BN-ReLU
template <int V, int U>
__global__ __launch_bounds__(kStreamMaxThreads) void bnrelu_fwd_kernel(const half_t* __restrict__ x,
                                                                       const float* __restrict__ wv,
                                                                       const float* __restrict__ bv,
                                                                       half_t* __restrict__ y, int64_t nchunks, int CG,
                                                                       int segments)
{
    typedef typename HVec<V>::type hv;
    const ChunkWalk<U> wk(nchunks, segments != 0);
    const int cg = (int)(wk.first % CG);
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
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        hv v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = ld_stream<V>(x, i + u * wk.su);
#pragma unroll
        for (int u = 0; u < U; ++u) st_stream<V>(y, i + u * wk.su, act(v[u]));
    }
    for (int64_t i = wk.tail; i < nchunks; i += wk.T) st_stream<V>(y, i, act(ld_stream<V>(x, i)));
}

template <int V, int U>
__global__ __launch_bounds__(kStreamMaxThreads) void bnrelu_bwd_kernel(const half_t* __restrict__ x,
                                                                       const float* __restrict__ wv,
                                                                       const float* __restrict__ bv,
                                                                       const half_t* __restrict__ g,
                                                                       half_t* __restrict__ dx, float* __restrict__ ws,
                                                                       int64_t nchunks, int CG, int segments)
{
    typedef typename HVec<V>::type hv;
    __shared__ float red[4 * 2 * 64 * V];
    const ChunkWalk<U> wk(nchunks, segments != 0);
    const int cg = (int)(wk.first % CG);
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
            // (one channel per lane: the compiler would otherwise round the exact product once; with two and more it
            // converts pairs of fp32 products, and the opaque value only costs registers)
            o[j] = (half_t)(V == 1 ? as_fp32_value(__fmul_rn(w[j], gm)) : __fmul_rn(w[j], gm));
            acc[0][j] = __builtin_fmaf(xf, gm, acc[0][j]);
            acc[1][j] += gm;
        }
        st_stream<V>(dx, k, o);
    };
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        hv xv[U], gv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            xv[u] = ld_stream<V>(x, i + u * wk.su);
            gv[u] = ld_stream<V>(g, i + u * wk.su);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) body(i + u * wk.su, xv[u], gv[u]);
    }
    for (int64_t i = wk.tail; i < nchunks; i += wk.T) body(i, ld_stream<V>(x, i), ld_stream<V>(g, i));
    block_channel_partials_any<2, V>(acc, CG, red, ws + (int64_t)blockIdx.x * 2 * CG * V);
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

template <typename T, int U, bool FAST>
__global__ __launch_bounds__(kStreamMaxThreads) void quant_u8_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                                     int64_t numel, float window, float r_two_w,
                                                                     int segments)
{
    typedef QuantUnit<T> QU;
    constexpr int E = QU::E;
    const float two_w = __fmul_rn(2.0f, window);
    const int64_t nunits = numel / E;
    const ChunkWalk<U> wk(nunits, segments != 0);
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
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        typename QU::wide_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(xv + i + u * wk.su);
#pragma unroll
        for (int u = 0; u < U; ++u) __builtin_nontemporal_store(one(v[u]), qv + i + u * wk.su);
    }
    for (int64_t i = wk.tail; i < nunits; i += wk.T)
        __builtin_nontemporal_store(one(__builtin_nontemporal_load(xv + i)), qv + i);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (int64_t k = nunits * E; k < numel; ++k)
            q[k] = (uint8_t)quant_u8_one<FAST>(to_f32(x[k]), window, two_w, r_two_w);
    }
}

template <typename T, int U>
__global__ __launch_bounds__(kStreamMaxThreads) void dequant_u8_kernel(const uint8_t* __restrict__ q,
                                                                       T* __restrict__ out, int64_t numel,
                                                                       float window, int segments)
{
    typedef QuantUnit<T> QU;
    constexpr int E = QU::E;
    const float scale = __fdiv_rn(__fmul_rn(2.0f, window), 255.0f);
    const int64_t nunits = numel / E;
    const ChunkWalk<U> wk(nunits, segments != 0);
    auto one = [&](const typename QU::bytes_t& b) {
        typename QU::wide_t o;
#pragma unroll
        for (int j = 0; j < E; ++j)
            o[j] = (T)__fsub_rn(__fmul_rn((float)((bytes_word(b, j / 4) >> (8 * (j % 4))) & 0xffu), scale), window);
        return o;
    };
    const typename QU::bytes_t* qv = reinterpret_cast<const typename QU::bytes_t*>(q);
    typename QU::wide_t* ov = reinterpret_cast<typename QU::wide_t*>(out);
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        typename QU::bytes_t b[U];
#pragma unroll
        for (int u = 0; u < U; ++u) b[u] = __builtin_nontemporal_load(qv + i + u * wk.su);
#pragma unroll
        for (int u = 0; u < U; ++u) __builtin_nontemporal_store(one(b[u]), ov + i + u * wk.su);
    }
    for (int64_t i = wk.tail; i < nunits; i += wk.T)
        __builtin_nontemporal_store(one(__builtin_nontemporal_load(qv + i)), ov + i);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (int64_t k = nunits * E; k < numel; ++k)
            out[k] = (T)__fsub_rn(__fmul_rn((float)q[k], scale), window);
    }
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

template <int U>
__global__ __launch_bounds__(kStreamMaxThreads) void quant_i8_kernel(const half_t* __restrict__ y,
                                                                     const float* __restrict__ absmax,
                                                                     int8_t* __restrict__ q,
                                                                     float* __restrict__ scale_out, int64_t numel,
                                                                     int segments)
{
    const float scale = __fdiv_rn(absmax[0], 127.0f);
    const bool zero = (scale == 0.0f);
    const float rscale = __fdiv_rn(1.0f, zero ? 1.0f : scale);  // correctly rounded reciprocal, once per thread
    const int64_t nunits = numel / 8;  // 16 bytes in, 8 bytes out per lane and access
    const ChunkWalk<U> wk(nunits, segments != 0);
    auto one = [&](const half8_t& v) {
        u32x2_t o;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) w |= (zero ? 0u : quant_i8_one((float)v[4 * k + j], scale, rscale)) << (8 * j);
            o[k] = w;
        }
        return o;
    };
    const half8_t* yv = reinterpret_cast<const half8_t*>(y);
    u32x2_t* qv = reinterpret_cast<u32x2_t*>(q);
    for (int64_t k = 0; k < wk.nfull; ++k) {
        const int64_t i = k * wk.step + wk.first;
        half8_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(yv + i + u * wk.su);
#pragma unroll
        for (int u = 0; u < U; ++u) __builtin_nontemporal_store(one(v[u]), qv + i + u * wk.su);
    }
    for (int64_t i = wk.tail; i < nunits; i += wk.T)
        __builtin_nontemporal_store(one(__builtin_nontemporal_load(yv + i)), qv + i);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        for (int64_t k = nunits * 8; k < numel; ++k)
            q[k] = zero ? (int8_t)0 : (int8_t)quant_i8_one((float)y[k], scale, rscale);
        if (scale_out) scale_out[0] = scale;  // absmax / 127, correctly rounded: what the caller dequantises with
    }
}

}  // namespace kerops

using namespace kerops;

// ------------------------------------------------------------------ C ABI
//
// Launch shape of an entry point: (blocks, waves, segment), 0 = the built-in choice below.
//   blocks   workgroups of the persistent loop
//   waves    wavefronts per workgroup: 4, 8 or 16
//   segment  1 = interleaved walk, 4 or 8 = each workgroup step covers one contiguous run of that many
//            chunks per thread (with C < 8 a request for 8 runs as 4)
// Built-in choices: measured on MI355X at (1,64,350,350,128) with `python -m kerops_amd.tune --streams`.
namespace {

struct StreamDefault {
    int blocks, waves, segment;
};
constexpr StreamDefault kDefStats{256, 4, 8};
constexpr StreamDefault kDefAddStats{1280, 16, 8};
constexpr StreamDefault kDefStatsBwd{4096, 16, 4};
constexpr StreamDefault kDefAddStatsBwd{512, 4, 4};
constexpr StreamDefault kDefBnReluFwd{1280, 16, 4};
constexpr StreamDefault kDefBnReluBwd{1536, 16, 4};
constexpr StreamDefault kDefQuantU8{256, 4, 8};
constexpr StreamDefault kDefDequantU8{512, 4, 4};
constexpr StreamDefault kDefQuantI8{4096, 16, 4};
constexpr int kMaxStreamBlocks = 65536;
constexpr int kMaxDefaultBlocks = 4096;  // workspace queries with blocks = 0 size for this many partials

int resolve_shape(const char* op, const StreamDefault& def, int64_t work_items, bool wide8, int blocks, int waves,
                  int segment, StreamShape* out)
{
    if (waves == 0) waves = def.waves;
    if (segment == 0) segment = def.segment;
    if (segment == 8 && !wide8) segment = 4;  // narrow chunks (C < 8) are built with four per thread only
    if (!(waves == 4 || waves == 8 || waves == 16)) {
        set_error("%s: waves must be 4, 8 or 16 wavefronts per workgroup (got %d)", op, waves);
        return KEROPS_E_BADARG;
    }
    if (!(segment == 1 || segment == 4 || segment == 8)) {
        set_error("%s: segment must be 1 (interleaved), 4 or 8 (got %d)", op, segment);
        return KEROPS_E_BADARG;
    }
    out->threads = waves * kWave;
    out->segment = segment;
    if (blocks > kMaxStreamBlocks) {
        set_error("%s: blocks must be <= %d", op, kMaxStreamBlocks);
        return KEROPS_E_BADARG;
    }
    // the built-in workgroup counts were measured on 256 compute units: scale them to the device at hand
    // (never beyond what a workspace query with blocks = 0 sizes for)
    if (blocks <= 0)
        blocks = std::min(kMaxDefaultBlocks, std::max(1, (int)((int64_t)def.blocks * device_geometry().cus / 256)));
    // never more workgroups than steps of work (small tensors)
    const int64_t per_step = (int64_t)out->threads * out->unroll();
    out->blocks = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div64(work_items, per_step), blocks));
    return KEROPS_OK;
}

int check_channels(const char* op, int64_t M, int C, bool reduces)
{
    if (M <= 0 || C <= 0 || !is_pow2(C)) {
        set_error("%s: M must be positive and C a power of two (M=%lld C=%d)", op, (long long)M, C);
        return KEROPS_E_BADARG;
    }
    if (reduces && C > kMaxReduceChannels) {
        set_error("%s: per-channel reductions are built for C <= %d (got %d)", op, kMaxReduceChannels, C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    if (C / (C >= 8 ? 8 : C) > 256) {  // a thread keeps its channel group: threads % (C/8) == 0
        set_error("%s: built for C <= 2048 (got %d)", op, C);
        return KEROPS_E_UNSUPPORTED_C;
    }
    return KEROPS_OK;
}

int check_ws(const char* op, const void* ws, int64_t have, int64_t need)
{
    if (!ws || !aligned16(ws) || have < need) {
        set_error("%s: workspace of %lld bytes required, %lld given", op, (long long)need, (long long)have);
        return KEROPS_E_WORKSPACE;
    }
    return KEROPS_OK;
}

// Runs the statement list with constexpr V = min(8, C) and U = 4 or 8 (8 only with V = 8) in scope.
#define KEROPS_DISPATCH_VU(C, shape, ...)          \
    do {                                           \
        if ((C) >= 8 && (shape).unroll() == 8) {   \
            constexpr int V = 8, U = 8;            \
            __VA_ARGS__;                           \
        } else {                                   \
            constexpr int U = 4;                   \
            KEROPS_DISPATCH_V(C, __VA_ARGS__);     \
        }                                          \
    } while (0)

}  // namespace

extern "C" int64_t kerops_stats_workspace_bytes(int64_t M, int32_t C, int32_t blocks)
{
    int rc = check_channels("stats", M, C, true);
    if (rc != KEROPS_OK) return rc;
    if (blocks > kMaxStreamBlocks) {
        set_error("stats: blocks must be <= %d", kMaxStreamBlocks);
        return KEROPS_E_BADARG;
    }
    if (blocks <= 0) blocks = kMaxDefaultBlocks;
    return (int64_t)blocks * 2 * C * (int64_t)sizeof(float);
}

static int stats_common(const char* op, const StreamDefault& def, const void* x, const void* y, void* z, float* mean,
                        float* sqmean, int64_t M, int32_t C, void* workspace, int64_t workspace_bytes, int32_t blocks,
                        int32_t waves, int32_t segment, void* stream)
{
    int rc = check_channels(op, M, C, true);
    if (rc != KEROPS_OK) return rc;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    const int64_t nchunks = M * CG;
    StreamShape sh;
    rc = resolve_shape(op, def, nchunks, Vr == 8, blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    const bool add = (y != nullptr);
    if (!x || !mean || !sqmean || !aligned16(x) || (add && (!z || !aligned16(y) || !aligned16(z)))) {
        set_error("%s: null or misaligned pointer", op);
        return KEROPS_E_BADARG;
    }
    rc = check_ws(op, workspace, workspace_bytes, (int64_t)sh.blocks * 2 * C * (int64_t)sizeof(float));
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    float* ws = (float*)workspace;
    const int seg = sh.segment != 1;
    KEROPS_DISPATCH_VU(C, sh, {
        if (add) {
            hipLaunchKernelGGL((stats_kernel<V, U, true>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const half_t*)x,
                               (const half_t*)y, (half_t*)z, ws, nchunks, CG, seg);
        } else {
            hipLaunchKernelGGL((stats_kernel<V, U, false>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const half_t*)x,
                               (const half_t*)nullptr, (half_t*)nullptr, ws, nchunks, CG, seg);
        }
    });
    rc = check_launch(op);
    if (rc != KEROPS_OK) return rc;
    launch_reduce_rows(ws, sh.blocks, 2 * C, mean, sqmean, C, 1.0 / (double)M, s);
    return check_launch(op);
}

extern "C" int kerops_stats_f16(const void* x, float* mean, float* sqmean, int64_t M, int32_t C, void* workspace,
                                int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    return stats_common("stats", kDefStats, x, nullptr, nullptr, mean, sqmean, M, C, workspace, workspace_bytes, blocks,
                        waves, segment, stream);
}

extern "C" int kerops_add_stats_f16(const void* x, const void* y, void* z, float* mean, float* sqmean, int64_t M,
                                    int32_t C, void* workspace, int64_t workspace_bytes, int32_t blocks, int32_t waves,
                                    int32_t segment, void* stream)
{
    if (!y) {
        set_error("add_stats: null pointer");
        return KEROPS_E_BADARG;
    }
    return stats_common("add_stats", kDefAddStats, x, y, z, mean, sqmean, M, C, workspace, workspace_bytes, blocks,
                        waves, segment, stream);
}

static int stats_bwd_common(const char* op, const StreamDefault& def, const void* x, const void* add_grad,
                            const float* mean_grad, const float* sqmean_grad, void* dx, int64_t M, int32_t C,
                            int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    int rc = check_channels(op, M, C, false);
    if (rc != KEROPS_OK) return rc;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    const int64_t nchunks = M * CG;
    StreamShape sh;
    rc = resolve_shape(op, def, nchunks, Vr == 8, blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    if (!x || !mean_grad || !sqmean_grad || !dx || !aligned16(x) || !aligned16(dx) ||
        (add_grad && !aligned16(add_grad))) {
        set_error("%s: null or misaligned pointer", op);
        return KEROPS_E_BADARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int seg = sh.segment != 1;
    KEROPS_DISPATCH_VU(C, sh, {
        if (add_grad) {
            hipLaunchKernelGGL((stats_bwd_kernel<V, U, true>), dim3(sh.blocks), dim3(sh.threads), 0, s,
                               (const half_t*)x, (const half_t*)add_grad, mean_grad, sqmean_grad, (half_t*)dx,
                               nchunks, CG, (float)M, seg);
        } else {
            hipLaunchKernelGGL((stats_bwd_kernel<V, U, false>), dim3(sh.blocks), dim3(sh.threads), 0, s,
                               (const half_t*)x, (const half_t*)nullptr, mean_grad, sqmean_grad, (half_t*)dx, nchunks,
                               CG, (float)M, seg);
        }
    });
    return check_launch(op);
}

extern "C" int kerops_stats_bwd_f16(const void* x, const float* mean_grad, const float* sqmean_grad, void* dx,
                                    int64_t M, int32_t C, int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    return stats_bwd_common("stats_bwd", kDefStatsBwd, x, nullptr, mean_grad, sqmean_grad, dx, M, C, blocks, waves,
                            segment, stream);
}

extern "C" int kerops_add_stats_bwd_f16(const void* add_grad, const float* mean_grad, const float* sqmean_grad,
                                        const void* add_result, void* out, int64_t M, int32_t C, int32_t blocks,
                                        int32_t waves, int32_t segment, void* stream)
{
    if (!add_grad) {
        set_error("add_stats_bwd: null pointer");
        return KEROPS_E_BADARG;
    }
    return stats_bwd_common("add_stats_bwd", kDefAddStatsBwd, add_result, add_grad, mean_grad, sqmean_grad, out, M, C,
                            blocks, waves, segment, stream);
}

extern "C" int kerops_bnrelu_fwd_f16(const void* x, const float* wv, const float* bv, void* y, int64_t M, int32_t C,
                                     int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    int rc = check_channels("bnrelu_fwd", M, C, false);
    if (rc != KEROPS_OK) return rc;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    StreamShape sh;
    rc = resolve_shape("bnrelu_fwd", kDefBnReluFwd, M * CG, Vr == 8, blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    if (!x || !wv || !bv || !y || !aligned16(x) || !aligned16(y)) {
        set_error("bnrelu_fwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int seg = sh.segment != 1;
    KEROPS_DISPATCH_VU(C, sh, {
        hipLaunchKernelGGL((bnrelu_fwd_kernel<V, U>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const half_t*)x, wv,
                           bv, (half_t*)y, M * CG, CG, seg);
    });
    return check_launch("bnrelu_fwd");
}

extern "C" int kerops_bnrelu_bwd_f16(const void* x, const float* wv, const float* bv, const void* g, void* dx,
                                     float* dW, float* dB, int64_t M, int32_t C, void* workspace,
                                     int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment,
                                     void* stream)
{
    int rc = check_channels("bnrelu_bwd", M, C, true);
    if (rc != KEROPS_OK) return rc;
    const int Vr = C >= 8 ? 8 : C;
    const int CG = C / Vr;
    StreamShape sh;
    rc = resolve_shape("bnrelu_bwd", kDefBnReluBwd, M * CG, Vr == 8, blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    if (!x || !wv || !bv || !g || !dx || !dW || !dB || !aligned16(x) || !aligned16(g) || !aligned16(dx)) {
        set_error("bnrelu_bwd: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    rc = check_ws("bnrelu_bwd", workspace, workspace_bytes, (int64_t)sh.blocks * 2 * C * (int64_t)sizeof(float));
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    float* ws = (float*)workspace;
    const int seg = sh.segment != 1;
    KEROPS_DISPATCH_VU(C, sh, {
        hipLaunchKernelGGL((bnrelu_bwd_kernel<V, U>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const half_t*)x, wv,
                           bv, (const half_t*)g, (half_t*)dx, ws, M * CG, CG, seg);
    });
    rc = check_launch("bnrelu_bwd");
    if (rc != KEROPS_OK) return rc;
    launch_reduce_rows(ws, sh.blocks, 2 * C, dW, dB, C, 1.0, s);
    return check_launch("bnrelu_bwd");
}

static int check_flat(const char* op, const StreamDefault& def, const void* a, const void* b, int64_t numel,
                      int64_t units, int blocks, int waves, int segment, StreamShape* sh)
{
    if (!a || !b || !aligned16(a) || !aligned16(b) || numel <= 0) {
        set_error("%s: null or misaligned pointer, or non-positive numel", op);
        return KEROPS_E_BADARG;
    }
    return resolve_shape(op, def, units, true, blocks, waves, segment, sh);
}

extern "C" int kerops_quant_u8_window(const void* x, int32_t dtype, void* q, int64_t numel, float window,
                                      int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    if (!(dtype == KEROPS_DTYPE_F16 || dtype == KEROPS_DTYPE_BF16 || dtype == KEROPS_DTYPE_F32)) {
        set_error("quant_u8_window: unknown dtype tag %d", dtype);
        return KEROPS_E_BADARG;
    }
    StreamShape sh;
    int rc = check_flat("quant_u8_window", kDefQuantU8, x, q, numel, numel / (dtype == KEROPS_DTYPE_F32 ? 4 : 8), blocks,
                        waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    // 1/(2w) correctly rounded to fp32: the double quotient rounded once more is exact for division
    // (53 >= 2*24 + 2 bits).  The 3-instruction division needs 2w and its quotients to stay normal.
    const float two_w = 2.0f * window;
    const bool fast = window >= 0x1p-60f && window <= 0x1p60f;
    const float r_two_w = fast ? (float)(1.0 / (double)two_w) : 0.0f;
    const int seg = sh.segment != 1;
#define KEROPS_QU8_GO(T, Uv, F)                                                                                  \
    hipLaunchKernelGGL((quant_u8_kernel<T, Uv, F>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const T*)x, (uint8_t*)q, \
                       numel, window, r_two_w, seg)
#define KEROPS_QU8_T(T)                            \
    if (sh.unroll() == 8) {                        \
        if (fast) KEROPS_QU8_GO(T, 8, true);       \
        else KEROPS_QU8_GO(T, 8, false);           \
    } else {                                       \
        if (fast) KEROPS_QU8_GO(T, 4, true);       \
        else KEROPS_QU8_GO(T, 4, false);           \
    }
    if (dtype == KEROPS_DTYPE_F16) {
        KEROPS_QU8_T(half_t)
    } else if (dtype == KEROPS_DTYPE_BF16) {
        KEROPS_QU8_T(bf16_t)
    } else {
        KEROPS_QU8_T(float)
    }
#undef KEROPS_QU8_T
#undef KEROPS_QU8_GO
    return check_launch("quant_u8_window");
}

extern "C" int kerops_dequant_u8_window(const void* q, void* out, int32_t dtype, int64_t numel, float window,
                                        int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    if (!(dtype == KEROPS_DTYPE_F16 || dtype == KEROPS_DTYPE_BF16 || dtype == KEROPS_DTYPE_F32)) {
        set_error("dequant_u8_window: unknown dtype tag %d", dtype);
        return KEROPS_E_BADARG;
    }
    StreamShape sh;
    int rc = check_flat("dequant_u8_window", kDefDequantU8, q, out, numel, numel / (dtype == KEROPS_DTYPE_F32 ? 4 : 8),
                        blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const int seg = sh.segment != 1;
#define KEROPS_DQ_T(T)                                                                                              \
    if (sh.unroll() == 8) {                                                                                         \
        hipLaunchKernelGGL((dequant_u8_kernel<T, 8>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const uint8_t*)q,   \
                           (T*)out, numel, window, seg);                                                            \
    } else {                                                                                                        \
        hipLaunchKernelGGL((dequant_u8_kernel<T, 4>), dim3(sh.blocks), dim3(sh.threads), 0, s, (const uint8_t*)q,   \
                           (T*)out, numel, window, seg);                                                            \
    }
    if (dtype == KEROPS_DTYPE_F16) {
        KEROPS_DQ_T(half_t)
    } else if (dtype == KEROPS_DTYPE_BF16) {
        KEROPS_DQ_T(bf16_t)
    } else {
        KEROPS_DQ_T(float)
    }
#undef KEROPS_DQ_T
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
    if (!y || !absmax || !aligned16(y) || numel <= 0) {
        set_error("absmax: null or misaligned pointer, or non-positive numel");
        return KEROPS_E_BADARG;
    }
    if (blocks > kMaxStreamBlocks) {
        set_error("absmax: blocks must be <= %d", kMaxStreamBlocks);
        return KEROPS_E_BADARG;
    }
    int rc = check_ws("absmax", workspace, workspace_bytes, (int64_t)blocks * 4);
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

extern "C" int kerops_quant_i8_sym_f16(const void* y, const float* absmax, void* q, float* scale, int64_t numel,
                                       int32_t blocks, int32_t waves, int32_t segment, void* stream)
{
    StreamShape sh;
    int rc = check_flat("quant_i8_sym", kDefQuantI8, y, q, numel, numel / 8, blocks, waves, segment, &sh);
    if (rc != KEROPS_OK) return rc;
    if (!absmax) {
        set_error("quant_i8_sym: null absmax");
        return KEROPS_E_BADARG;
    }
    const int seg = sh.segment != 1;
    if (sh.unroll() == 8) {
        hipLaunchKernelGGL(quant_i8_kernel<8>, dim3(sh.blocks), dim3(sh.threads), 0, (hipStream_t)stream,
                           (const half_t*)y, absmax, (int8_t*)q, scale, numel, seg);
    } else {
        hipLaunchKernelGGL(quant_i8_kernel<4>, dim3(sh.blocks), dim3(sh.threads), 0, (hipStream_t)stream,
                           (const half_t*)y, absmax, (int8_t*)q, scale, numel, seg);
    }
    return check_launch("quant_i8_sym");
}
