/*
 * CPU oracle for the channels-last 3D depthwise-conv hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, what each op of
 * the reference computes.  It is compiled by oracle/build_oracle.py into
 * oracle/_build/liboracle.so and may be loaded only by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, always as
 * the checker and never as the product path.  The product (kerops_amd) never
 * imports, links or calls anything in this directory.
 *
 * Layout conventions (kerops/ops/conv/dwconv.py:29,37-38 of the reference):
 * a tensor of torch shape (N, C, H, W, D) in channels_last_3d is the dense
 * array [N][H][W][D][C]; fp16 values travel as their uint16 bit patterns.
 * The depthwise weight is [3][3][3][C] = [kH][kW][kD][C]
 * (kerops/ops/conv/dwconv.py:32, kerops/kernels/dw_conv.py:36-47).
 *
 * Arithmetic policy: the reference kernels mix fp16 products, fp16 partial
 * sums and fp32 accumulators (kerops/kernels/dw_conv.py:49-52,71-121,185-193);
 * those incidental roundings are below every tolerance its tests state.  The
 * oracle therefore evaluates the defining sums in fp32 (wide == 0, the same
 * precision torch's CPU conv3d uses) or fp64 (wide == 1), and rounds once at
 * the end.  The byte/integer ops (quantisers) follow the reference's fp32
 * step order exactly, with no fused multiply-add.
 *
 * Pinning (see tests/test_oracle_*.py): every function below is checked
 * against the torch CPU routine the reference's own tests use as ground truth,
 * plus closed forms / brute force that fail on a flipped tap, a wrong sign or
 * a transposed axis.  The two window quantisers have no test in the reference
 * at all; their parity is pinned only by closed forms and an exhaustive sweep
 * of all fp16 bit patterns against a numpy restatement ("parity unpinned" with
 * respect to the reference itself).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 */

static inline float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* float -> half, round to nearest even (IEEE 754 binary16) */
static inline uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* result is subnormal or zero: below 2^-14 */
        if (ax < 0x33000000u) { /* < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
            return (uint16_t)sign;
        }
        uint32_t e = ax >> 23;               /* biased exponent, 102..112 */
        uint32_t man = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;           /* 14..24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) {
            ++q;
        }
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - 112u;
    uint32_t man = ax & 0x7fffffu;
    uint32_t q = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) {
        ++q; /* carry into the exponent is the correct behaviour */
    }
    return (uint16_t)(sign | q);
}

void oracle_h2f_array(const uint16_t *h, float *f, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        f[i] = h2f(h[i]);
    }
}

void oracle_f2h_array(const float *f, uint16_t *h, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        h[i] = f2h(f[i]);
    }
}

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------ DWConv fprop
 * y[n,h,w,d,c] = sum_{kh,kw,kd} x[n,h+kh-1,w+kw-1,d+kd-1,c] * wt[kh,kw,kd,c]
 * zero padding 1, stride 1, no bias, cross-correlation (no kernel flip):
 * kerops/kernels/dw_conv.py:62-130 walks the 4x4 (h,w) neighbourhood of a 2x2
 * output cell and pairs input offset i (resp. j) with weight row kh = i - out_h
 * + 1; kerops/ops/conv/dwconv.py:25-63 fixes layouts and the fp16 output.
 * y32 (optional) receives the unrounded sums, y16 (optional) the fp16 result.
 */
void oracle_dwconv_fwd(const uint16_t *x, const uint16_t *wt, float *y32, uint16_t *y16, int N, int H, int W, int D,
                       int C, int wide)
{
    int64_t total = (int64_t)N * H * W * D * C;
    float *xf = (float *)malloc((size_t)total * sizeof(float));
    float *wf = (float *)malloc((size_t)27 * C * sizeof(float));
    oracle_h2f_array(wt, wf, (int64_t)27 * C);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < total; ++i) {
        xf[i] = h2f(x[i]);
    }
    int64_t sD = C, sW = (int64_t)D * C, sH = (int64_t)W * D * C, sN = (int64_t)H * W * D * C;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int h = 0; h < H; ++h) {
            float *acc = (float *)malloc((size_t)C * sizeof(float));
            double *accd = (double *)malloc((size_t)C * sizeof(double));
            for (int w = 0; w < W; ++w) {
                for (int d = 0; d < D; ++d) {
                    for (int c = 0; c < C; ++c) {
                        acc[c] = 0.0f;
                        accd[c] = 0.0;
                    }
                    for (int kh = 0; kh < 3; ++kh) {
                        int hh = h + kh - 1;
                        if (hh < 0 || hh >= H) continue;
                        for (int kw = 0; kw < 3; ++kw) {
                            int ww = w + kw - 1;
                            if (ww < 0 || ww >= W) continue;
                            for (int kd = 0; kd < 3; ++kd) {
                                int dd = d + kd - 1;
                                if (dd < 0 || dd >= D) continue;
                                const float *xp = xf + n * sN + hh * sH + ww * sW + dd * sD;
                                const float *wp = wf + (size_t)((kh * 3 + kw) * 3 + kd) * C;
                                if (wide) {
                                    for (int c = 0; c < C; ++c) accd[c] += (double)xp[c] * (double)wp[c];
                                } else {
                                    for (int c = 0; c < C; ++c) acc[c] += xp[c] * wp[c];
                                }
                            }
                        }
                    }
                    int64_t o = n * sN + h * sH + w * sW + d * sD;
                    for (int c = 0; c < C; ++c) {
                        float v = wide ? (float)accd[c] : acc[c];
                        if (y32) y32[o + c] = v;
                        if (y16) y16[o + c] = f2h(v);
                    }
                }
            }
            free(acc);
            free(accd);
        }
    }
    free(xf);
    free(wf);
}

/* ------------------------------------------------------------ DWConv wgrad
 * gw[kh,kw,kd,c] = sum_{n,h,w,d} g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]
 * (out-of-range x is zero): kerops/kernels/dw_conv.py:198-277, tap bookkeeping
 * kh = a - i + 1 at :224-275; contracts at kerops/ops/conv/dwconv_wgrad.py:31-79.
 * Accumulated in fp64, one partial per (n,h) row combined in a fixed order.
 */
void oracle_dwconv_wgrad(const uint16_t *x, const uint16_t *g, double *gw, int N, int H, int W, int D, int C)
{
    int64_t sD = C, sW = (int64_t)D * C, sH = (int64_t)W * D * C, sN = (int64_t)H * W * D * C;
    int rows = N * H;
    double *part = (double *)calloc((size_t)rows * 27 * C, sizeof(double));
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        int n = r / H, h = r % H;
        double *p = part + (size_t)r * 27 * C;
        for (int w = 0; w < W; ++w) {
            for (int d = 0; d < D; ++d) {
                const uint16_t *gp = g + n * sN + h * sH + w * sW + d * sD;
                for (int kh = 0; kh < 3; ++kh) {
                    int hh = h + kh - 1;
                    if (hh < 0 || hh >= H) continue;
                    for (int kw = 0; kw < 3; ++kw) {
                        int ww = w + kw - 1;
                        if (ww < 0 || ww >= W) continue;
                        for (int kd = 0; kd < 3; ++kd) {
                            int dd = d + kd - 1;
                            if (dd < 0 || dd >= D) continue;
                            const uint16_t *xp = x + n * sN + hh * sH + ww * sW + dd * sD;
                            double *pp = p + (size_t)((kh * 3 + kw) * 3 + kd) * C;
                            for (int c = 0; c < C; ++c) pp[c] += (double)h2f(gp[c]) * (double)h2f(xp[c]);
                        }
                    }
                }
            }
        }
    }
    for (int i = 0; i < 27 * C; ++i) gw[i] = 0.0;
    for (int r = 0; r < rows; ++r) {
        for (int i = 0; i < 27 * C; ++i) gw[i] += part[(size_t)r * 27 * C + i];
    }
    free(part);
}

/* ------------------------------------------------------------------ Stats
 * mean[c] = sum x / M, sqmean[c] = sum x^2 / M over M = numel / C voxels:
 * kerops/kernels/stats.py:6-23, kerops/ops/stats.py:11-31.  fp64 sums.
 */
void oracle_stats(const uint16_t *x, double *mean, double *sqmean, int64_t M, int C)
{
    for (int c = 0; c < C; ++c) {
        mean[c] = 0.0;
        sqmean[c] = 0.0;
    }
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            double t = (double)h2f(x[v * C + c]);
            mean[c] += t;
            sqmean[c] += t * t;
        }
    }
    for (int c = 0; c < C; ++c) {
        mean[c] /= (double)M;
        sqmean[c] /= (double)M;
    }
}

/* dx = 2*x*g_sq/M + g_mean/M -> fp16: kerops/kernels/stats.py:26-51 */
void oracle_stats_bwd(const uint16_t *x, const float *mean_grad, const float *sqmean_grad, uint16_t *dx, int64_t M,
                      int C)
{
    float fm = (float)M;
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            float t = h2f(x[v * C + c]);
            float a = (2.0f * t) * sqmean_grad[c];
            a = a / fm;
            float b = mean_grad[c] / fm;
            dx[v * C + c] = f2h(a + b);
        }
    }
}

/* AddStats: z = x + y rounded to fp16, stats of the rounded z:
 * kerops/kernels/addition.py:6-37 (sum formed in fp16 at :30). */
void oracle_add_stats(const uint16_t *x, const uint16_t *y, uint16_t *z, double *mean, double *sqmean, int64_t M,
                      int C)
{
    for (int c = 0; c < C; ++c) {
        mean[c] = 0.0;
        sqmean[c] = 0.0;
    }
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            uint16_t s = f2h(h2f(x[v * C + c]) + h2f(y[v * C + c]));
            z[v * C + c] = s;
            double t = (double)h2f(s);
            mean[c] += t;
            sqmean[c] += t * t;
        }
    }
    for (int c = 0; c < C; ++c) {
        mean[c] /= (double)M;
        sqmean[c] /= (double)M;
    }
}

/* dz = g + 2*z*g_sq/M + g_mean/M -> fp16: kerops/kernels/addition.py:41-75 */
void oracle_add_stats_bwd(const uint16_t *add_grad, const float *mean_grad, const float *sqmean_grad,
                          const uint16_t *add_result, uint16_t *out, int64_t M, int C)
{
    float fm = (float)M;
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            float s = h2f(add_result[v * C + c]);
            float a = ((2.0f * s) * sqmean_grad[c]) / fm;
            float b = mean_grad[c] / fm;
            out[v * C + c] = f2h((h2f(add_grad[v * C + c]) + a) + b);
        }
    }
}

/* ---------------------------------------------------------------- BN-ReLU
 * y = max(float(x)*W[c] + B[c], 0) -> fp16: kerops/kernels/bnrelu.py:6-31.
 * The multiply-add is evaluated in fp64 then rounded to fp32 (i.e. as a fused
 * multiply-add), which is what both Triton and hipcc emit for x*w+b.
 */
void oracle_bnrelu_fwd(const uint16_t *x, const float *wv, const float *bv, uint16_t *y, int64_t M, int C)
{
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            float t = fmaf(h2f(x[v * C + c]), wv[c], bv[c]);
            y[v * C + c] = f2h(t > 0.0f ? t : 0.0f);
        }
    }
}

/* m = (x*W > -B); g' = g*m; dx = W*g' (fp16); dB = sum g'; dW = sum x*g':
 * kerops/kernels/bnrelu.py:35-71.  Sums in fp64. */
void oracle_bnrelu_bwd(const uint16_t *x, const float *wv, const float *bv, const uint16_t *g, uint16_t *dx,
                       double *dW, double *dB, int64_t M, int C)
{
    for (int c = 0; c < C; ++c) {
        dW[c] = 0.0;
        dB[c] = 0.0;
    }
    for (int64_t v = 0; v < M; ++v) {
        for (int c = 0; c < C; ++c) {
            float xi = h2f(x[v * C + c]);
            float gi = h2f(g[v * C + c]);
            float keep = (xi * wv[c] > -bv[c]) ? 1.0f : 0.0f;
            float gm = gi * keep;
            dx[v * C + c] = f2h(wv[c] * gm);
            dB[c] += (double)gm;
            dW[c] += (double)xi * (double)gm;
        }
    }
}

/* --------------------------------------------------- AvgPoolCeilStats
 * 2x2x2 stride-2 average pool, ceil_mode: the divisor of an edge window is
 * the number of voxels that exist in it (norm_step * num_norm at
 * kerops/kernels/avgpool.py:45-46,86); mean / sqmean are taken over the fp32
 * pooled values before they are rounded to fp16 (:89-93).
 * Output is dense [N][Ho][Wo][Do][C].
 */
void oracle_avgpool_ceil_stats(const uint16_t *x, float *y32, uint16_t *y16, double *mean, double *sqmean, int N,
                               int H, int W, int D, int C)
{
    int Ho = (H + 1) / 2, Wo = (W + 1) / 2, Do = (D + 1) / 2;
    int64_t sD = C, sW = (int64_t)D * C, sH = (int64_t)W * D * C, sN = (int64_t)H * W * D * C;
    for (int c = 0; c < C; ++c) {
        mean[c] = 0.0;
        sqmean[c] = 0.0;
    }
    int64_t Mo = (int64_t)N * Ho * Wo * Do;
    for (int n = 0; n < N; ++n)
        for (int h = 0; h < Ho; ++h)
            for (int w = 0; w < Wo; ++w)
                for (int d = 0; d < Do; ++d) {
                    int cnt = 0;
                    for (int a = 0; a < 2; ++a)
                        for (int b = 0; b < 2; ++b)
                            for (int e = 0; e < 2; ++e)
                                if (2 * h + a < H && 2 * w + b < W && 2 * d + e < D) ++cnt;
                    int64_t o = ((((int64_t)n * Ho + h) * Wo + w) * Do + d) * C;
                    for (int c = 0; c < C; ++c) {
                        float s = 0.0f;
                        /* same association as the kernel: pair sum along D first, rows added in
                         * the order (h0,w0), (h0,w1), (h1,w0), (h1,w1); all partial sums of <= 8
                         * fp16 values are exact in fp32 unless exponents differ by > 13 */
                        for (int a = 0; a < 2; ++a)
                            for (int b = 0; b < 2; ++b) {
                                int hh = 2 * h + a, ww = 2 * w + b;
                                if (hh >= H || ww >= W) continue;
                                float p = 0.0f;
                                for (int e = 0; e < 2; ++e) {
                                    int dd = 2 * d + e;
                                    if (dd < D) p += h2f(x[n * sN + hh * sH + ww * sW + dd * sD + c]);
                                }
                                s += p;
                            }
                        float v = s / (float)cnt;
                        if (y32) y32[o + c] = v;
                        if (y16) y16[o + c] = f2h(v);
                        mean[c] += (double)v;
                        sqmean[c] += (double)v * (double)v;
                    }
                }
    for (int c = 0; c < C; ++c) {
        mean[c] /= (double)Mo;
        sqmean[c] /= (double)Mo;
    }
}

/* dx[window] = (g_pool + g_mean/Mo + 2*y*g_sq/Mo) / count, written to every
 * existing voxel of the window: kerops/kernels/avgpool.py:97-185.
 * inpgrad / output are the pooled-size fp16 tensors, dx has the input size. */
void oracle_avgpool_ceil_stats_bwd(const uint16_t *inpgrad, const float *meangrad, const float *sqmeangrad,
                                   const uint16_t *output, uint16_t *dx, int N, int H, int W, int D, int C)
{
    int Ho = (H + 1) / 2, Wo = (W + 1) / 2, Do = (D + 1) / 2;
    int64_t sD = C, sW = (int64_t)D * C, sH = (int64_t)W * D * C, sN = (int64_t)H * W * D * C;
    float Mo = (float)((int64_t)N * Ho * Wo * Do);
    for (int n = 0; n < N; ++n)
        for (int h = 0; h < Ho; ++h)
            for (int w = 0; w < Wo; ++w)
                for (int d = 0; d < Do; ++d) {
                    int cnt = 0;
                    for (int a = 0; a < 2; ++a)
                        for (int b = 0; b < 2; ++b)
                            for (int e = 0; e < 2; ++e)
                                if (2 * h + a < H && 2 * w + b < W && 2 * d + e < D) ++cnt;
                    int64_t o = ((((int64_t)n * Ho + h) * Wo + w) * Do + d) * C;
                    for (int c = 0; c < C; ++c) {
                        float mg = meangrad[c] / Mo;
                        float sg = ((2.0f * h2f(output[o + c])) * sqmeangrad[c]) / Mo;
                        float gsum = (h2f(inpgrad[o + c]) + mg) + sg;
                        uint16_t r = f2h(gsum / (float)cnt);
                        for (int a = 0; a < 2; ++a)
                            for (int b = 0; b < 2; ++b)
                                for (int e = 0; e < 2; ++e) {
                                    int hh = 2 * h + a, ww = 2 * w + b, dd = 2 * d + e;
                                    if (hh < H && ww < W && dd < D) dx[n * sN + hh * sH + ww * sW + dd * sD + c] = r;
                                }
                    }
                }
}

/* ------------------------------------------------------------ quantisers
 * uint8 window quantiser, kerops/kernels/quantization.py:21-25 step by step in
 * fp32: clip to [-w, w]; (t + w) / (2*w); * 255; truncate to uint8.
 * Compile this file with -ffp-contract=off: no step may be fused.
 */
void oracle_quant_u8_window_f32(const float *x, uint8_t *q, int64_t n, float window)
{
    volatile float two_w = 2.0f * window;
    for (int64_t i = 0; i < n; ++i) {
        float t = x[i];
        t = fminf(fmaxf(t, -window), window);
        volatile float u = t + window;
        volatile float r = u / two_w;
        volatile float s = r * 255.0f;
        q[i] = (uint8_t)s; /* C float->integer conversion truncates toward zero */
    }
}

void oracle_quant_u8_window_f16(const uint16_t *x, uint8_t *q, int64_t n, float window)
{
    volatile float two_w = 2.0f * window;
    for (int64_t i = 0; i < n; ++i) {
        float t = h2f(x[i]);
        t = fminf(fmaxf(t, -window), window);
        volatile float u = t + window;
        volatile float r = u / two_w;
        volatile float s = r * 255.0f;
        q[i] = (uint8_t)s;
    }
}

/* x = float(u8) * (2*w/255) - w: kerops/kernels/quantization.py:46-47; the
 * scale 2*w/255 is formed once in fp32, then one multiply and one subtract. */
void oracle_dequant_u8_window_f32(const uint8_t *q, float *x, int64_t n, float window)
{
    volatile float two_w = 2.0f * window;
    volatile float scale = two_w / 255.0f;
    for (int64_t i = 0; i < n; ++i) {
        volatile float m = (float)q[i] * scale;
        x[i] = m - window;
    }
}

void oracle_dequant_u8_window_f16(const uint8_t *q, uint16_t *x, int64_t n, float window)
{
    volatile float two_w = 2.0f * window;
    volatile float scale = two_w / 255.0f;
    for (int64_t i = 0; i < n; ++i) {
        volatile float m = (float)q[i] * scale;
        x[i] = f2h(m - window);
    }
}

/* Symmetric per-tensor int8 quantiser of the fused-block config (no reference
 * counterpart): absmax over the tensor; scale = absmax / 127 in fp32;
 * q = clamp(rint_half_even(float(y) / scale), -127, 127); scale == 0 -> q = 0. */
float oracle_absmax_f16(const uint16_t *y, int64_t n)
{
    float m = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(h2f(y[i]));
        if (a > m) m = a;
    }
    return m;
}

void oracle_quant_i8_sym_f16(const uint16_t *y, int8_t *q, int64_t n, float absmax)
{
    volatile float scale = absmax / 127.0f;
    for (int64_t i = 0; i < n; ++i) {
        if (scale == 0.0f) {
            q[i] = 0;
            continue;
        }
        volatile float r = h2f(y[i]) / scale;
        float t = nearbyintf(r); /* default rounding mode: to nearest, ties to even */
        if (t > 127.0f) t = 127.0f;
        if (t < -127.0f) t = -127.0f;
        q[i] = (int8_t)t;
    }
}

/* ----------------------------------------------------- pointwise 1x1x1 ops
 * out[v, co] = fp16( sum_ci relu(x[v,ci]) * Wm[ci,co] ) + add[v,co] (fp16 add):
 * kerops/kernels/linear.py:6-45 (ReLU at :39, dot with fp32 accumulate, cast,
 * then the fp16 residual add at :40).  fp64 accumulate here.
 * relu_in == 0 skips the ReLU; add == NULL skips the residual.
 */
void oracle_pointwise(const uint16_t *x, const uint16_t *Wm, const uint16_t *add, uint16_t *out, int64_t V, int Cin,
                      int Cout, int relu_in)
{
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < V; ++v) {
        for (int co = 0; co < Cout; ++co) {
            double s = 0.0;
            for (int ci = 0; ci < Cin; ++ci) {
                float xv = h2f(x[v * Cin + ci]);
                if (relu_in && xv < 0.0f) xv = 0.0f;
                s += (double)xv * (double)h2f(Wm[(int64_t)ci * Cout + co]);
            }
            uint16_t r = f2h((float)s);
            if (add) r = f2h(h2f(r) + h2f(add[v * Cout + co]));
            out[v * Cout + co] = r;
        }
    }
}

/* Backward of the ReLU-linear op: kerops/kernels/linear.py:48-98 (dot products with fp32 accumulate;
 * input_grad rounded to fp16 then masked by input > 0 at :92; weight_grad accumulated over voxels at
 * :89-91).  fp64 accumulate here; dW is returned in fp64.
 *   dx[v,ci] = x[v,ci] > 0 ? fp16(sum_co g[v,co] * Wm[ci,co]) : 0
 *   dW[ci,co] = sum_v relu(x[v,ci]) * g[v,co]
 */
void oracle_relu_linear_bwd(const uint16_t *x, const uint16_t *g, const uint16_t *Wm, uint16_t *dx, double *dW,
                            int64_t V, int Cin, int Cout)
{
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < V; ++v) {
        for (int ci = 0; ci < Cin; ++ci) {
            double s = 0.0;
            for (int co = 0; co < Cout; ++co)
                s += (double)h2f(g[v * Cout + co]) * (double)h2f(Wm[(int64_t)ci * Cout + co]);
            dx[v * Cin + ci] = h2f(x[v * Cin + ci]) > 0.0f ? f2h((float)s) : (uint16_t)0;
        }
    }
#pragma omp parallel for schedule(static)
    for (int ci = 0; ci < Cin; ++ci) {
        for (int co = 0; co < Cout; ++co) {
            double s = 0.0;
            for (int64_t v = 0; v < V; ++v) {
                const float xv = h2f(x[v * Cin + ci]);
                if (xv > 0.0f) s += (double)xv * (double)h2f(g[v * Cout + co]);
            }
            dW[(int64_t)ci * Cout + co] = s;
        }
    }
}

/* Inverted-bottleneck pointwise block: kerops/kernels/linear.py:102-146.
 *   hid = relu(fp16(x @ Wup) + bias)   (dot with wide accumulate, cast to fp16, fp16 add at :139, ReLU :140)
 *   out = fp16(hid @ Wdown) + add      (:141)
 * fp64 accumulate here; hid16 (optional) receives the hidden activation [V][2C].
 */
void oracle_lin_brelu_lin_add(const uint16_t *x, const uint16_t *Wup, const uint16_t *Wdown, const uint16_t *bias,
                              const uint16_t *add, uint16_t *hid16, uint16_t *out, int64_t V, int C)
{
    const int HID = 2 * C;
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < V; ++v) {
        float hid[256];
        for (int hcn = 0; hcn < HID; ++hcn) {
            double s = 0.0;
            for (int ci = 0; ci < C; ++ci) s += (double)h2f(x[v * C + ci]) * (double)h2f(Wup[(int64_t)ci * HID + hcn]);
            float hv = h2f(f2h(h2f(f2h((float)s)) + h2f(bias[hcn])));
            if (!(hv > 0.0f)) hv = 0.0f;
            hid[hcn] = hv;
            if (hid16) hid16[v * HID + hcn] = f2h(hv);
        }
        for (int co = 0; co < C; ++co) {
            double s = 0.0;
            for (int hcn = 0; hcn < HID; ++hcn) s += (double)hid[hcn] * (double)h2f(Wdown[(int64_t)hcn * C + co]);
            out[v * C + co] = f2h(h2f(f2h((float)s)) + h2f(add[v * C + co]));
        }
    }
}

/* Backward of the inverted-bottleneck block: kerops/kernels/linear.py:149-230.
 *   linup = fp16(x @ Wup) + bias (fp16 add, :196-198); hid = relu(linup) (:199)
 *   dWdown[h,c] = sum_v hid[v,h] g[v,c] (:201-203)
 *   lg[v,h] = linup > 0 ? fp16(sum_c Wdown[h,c] g[v,c]) : 0 (:205-207)
 *   dWup[c,h] = sum_v x[v,c] lg[v,h] (:208-210);  dbias[h] = sum_v lg[v,h] (:211)
 *   dx[v,c] = fp16(sum_h Wup[c,h] lg[v,h]) (:213-214)
 * fp64 accumulate here; the weight / bias gradients are returned in fp64.
 */
void oracle_lin_brelu_lin_bwd(const uint16_t *x, const uint16_t *g, const uint16_t *Wup, const uint16_t *Wdown,
                              const uint16_t *bias, uint16_t *dx, double *dWup, double *dWdown, double *dbias,
                              int64_t V, int C)
{
    const int H = 2 * C;
    float *hid = (float *)malloc((size_t)V * H * sizeof(float));
    float *lg = (float *)malloc((size_t)V * H * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < V; ++v) {
        for (int h = 0; h < H; ++h) {
            double s = 0.0, d = 0.0;
            for (int c = 0; c < C; ++c) {
                s += (double)h2f(x[v * C + c]) * (double)h2f(Wup[(int64_t)c * H + h]);
                d += (double)h2f(g[v * C + c]) * (double)h2f(Wdown[(int64_t)h * C + c]);
            }
            const float lin = h2f(f2h(h2f(f2h((float)s)) + h2f(bias[h])));
            const int pos = lin > 0.0f;
            hid[v * H + h] = pos ? lin : 0.0f;
            lg[v * H + h] = pos ? h2f(f2h((float)d)) : 0.0f;
        }
        for (int c = 0; c < C; ++c) {
            double s = 0.0;
            for (int h = 0; h < H; ++h) s += (double)h2f(Wup[(int64_t)c * H + h]) * (double)lg[v * H + h];
            dx[v * C + c] = f2h((float)s);
        }
    }
#pragma omp parallel for schedule(static)
    for (int h = 0; h < H; ++h) {
        double sb = 0.0;
        for (int64_t v = 0; v < V; ++v) sb += (double)lg[v * H + h];
        dbias[h] = sb;
        for (int c = 0; c < C; ++c) {
            double sd = 0.0, su = 0.0;
            for (int64_t v = 0; v < V; ++v) {
                sd += (double)hid[v * H + h] * (double)h2f(g[v * C + c]);
                su += (double)h2f(x[v * C + c]) * (double)lg[v * H + h];
            }
            dWdown[(int64_t)h * C + c] = sd;
            dWup[(int64_t)c * H + h] = su;
        }
    }
    free(hid);
    free(lg);
}

/* Fused depthwise-separable block of config 5 (composition of the pieces above;
 * no single reference counterpart): t = fp16(relu(dwconv(x) * scale[c] +
 * shift[c])) with the depthwise sum and the affine step in fp32; y = fp16(t @ Wm).
 * t16 (optional) receives the intermediate. */
void oracle_dwsep_block(const uint16_t *x, const uint16_t *wt, const float *scale, const float *shift,
                        const uint16_t *Wm, uint16_t *t16, uint16_t *y, int N, int H, int W, int D, int Cin, int Cout)
{
    int64_t V = (int64_t)N * H * W * D;
    float *acc = (float *)malloc((size_t)V * Cin * sizeof(float));
    uint16_t *t = t16 ? t16 : (uint16_t *)malloc((size_t)V * Cin * sizeof(uint16_t));
    oracle_dwconv_fwd(x, wt, acc, NULL, N, H, W, D, Cin, 1);
    for (int64_t v = 0; v < V; ++v) {
        for (int c = 0; c < Cin; ++c) {
            float a = fmaf(acc[v * Cin + c], scale[c], shift[c]);
            t[v * Cin + c] = f2h(a > 0.0f ? a : 0.0f);
        }
    }
    oracle_pointwise(t, Wm, NULL, y, V, Cin, Cout, 0);
    free(acc);
    if (!t16) free(t);
}
