/*
 * C ABI of libkerops_hip.so -- hand-written gfx950 (MI355X) kernels for the
 * channels-last 3D depthwise-conv path of neuro-ml/kerops.
 *
 * The reference has no FFI: its boundary is the launch of a Triton kernel from
 * a Python op (`kernel[grid](tensors..., ints..., constexprs..., num_warps=)`).
 * Each entry point below replaces one such launch site (cited per function,
 * paths relative to the reference tree) together with the torch glue around it
 * (per-sample launch loops, zero-filled partial buffers, torch.sum reductions).
 *
 * Conventions
 *  - Activations are dense [N][H][W][D][C] fp16 arrays: the memory of a torch
 *    (N, C, H, W, D) tensor in channels_last_3d.  H, W, D are the reference's axis
 *    names in torch-shape order; D is the innermost spatial axis.
 *  - Every pointer is a device pointer, 16-byte aligned.  C is a power of two.
 *  - The caller owns every buffer, including the workspace whose size the
 *    matching *_workspace_bytes function returns.  The library allocates nothing
 *    and keeps no device state (the one exception is the fixed array behind
 *    kerops_dwconv_wgrad_noalloc_f16); workspaces need not be zeroed.  A workspace
 *    query with blocks = 0 returns a size that covers every built-in launch shape.
 *  - All work is enqueued on `stream` (a hipStream_t, NULL = default stream); no
 *    entry point synchronises with the host.
 *  - Return value: KEROPS_OK or a negative KEROPS_E_* code; the text of the last
 *    failure on the calling thread is available from kerops_last_error_string().
 *    Nothing throws.
 *  - Trailing `tile_*`, `h_chunk`, `lane_channels`, `blocks`, `waves` and `segment`
 *    arguments are launch-shape knobs (patch extents along W and D, rows of H one
 *    workgroup marches over, channels one lane owns; for the flat stream kernels the
 *    workgroup count, the wavefronts per workgroup (4, 8 or 16) and the walk: segment
 *    1 = a workgroup's 16-byte chunks are interleaved with the other workgroups',
 *    4 or 8 = every step of a workgroup covers one contiguous run of that many chunks
 *    per thread (with C < 8 a request for 8 runs as 4); the pooling kernels count output chunks and take 1 or 2);
 *    0 selects the built-in choice for gfx950, an unbuilt combination
 *    returns KEROPS_E_BADARG.
 *    For kerops_dwconv_fwd_f16 and kerops_dwconv_wgrad_f16 with the matrix-core
 *    kernels, h_chunk > 0 cuts H into uniform chunks of that many rows, one per
 *    workgroup; h_chunk = 0 is the balanced split: as many workgroups as the GPU
 *    holds at once, in groups that each own an equal, contiguous share of the
 *    (bundle of neighbouring patches, row) sequence and march over it in step;
 *    h_chunk = -g selects that split with groups of g workgroups (for the weight
 *    gradient g must be a multiple of C / 64 when C > 64).
 */
#ifndef KEROPS_HIP_H
#define KEROPS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KEROPS_OK 0
#define KEROPS_E_BADARG (-1)        /* null/misaligned pointer, non-positive size, bad knob */
#define KEROPS_E_UNSUPPORTED_C (-2) /* channel count the kernel family does not cover */
#define KEROPS_E_WORKSPACE (-3)     /* workspace missing or smaller than *_workspace_bytes */
#define KEROPS_E_LAUNCH (-4)        /* HIP reported a launch error */

#define KEROPS_DTYPE_F16 0
#define KEROPS_DTYPE_F32 1
#define KEROPS_DTYPE_BF16 2

/* Version of this interface: bumped whenever an entry point is added or a signature changes, so a
 * caller built against an older header can detect the mismatch before passing arguments
 * (kerops_hip_version() of the loaded library must equal the KEROPS_HIP_VERSION it was compiled
 * against).  100: first interface; 200: launch-shape knobs (waves, segment) on the stream entry points,
 * kerops_dwconv_wgrad_noalloc_f16, KEROPS_DTYPE_BF16; 210: the *_f16_out variants (weight gradients written as fp16 by the
 * reduction kernels), scale output of kerops_quant_i8_sym_f16. */
#define KEROPS_HIP_VERSION 210

int kerops_hip_version(void);
const char* kerops_last_error_string(void);

/* Depthwise 3x3x3 cross-correlation, zero padding 1, stride 1, no bias, fp32
 * accumulation of all 27 taps, one RNE rounding to fp16:
 *   y[n,h,w,d,c] = sum_{kh,kw,kd} x[n,h+kh-1,w+kw-1,d+kd-1,c] * wt[kh,kw,kd,c]
 * wt is [3][3][3][C] fp16.  C in {8,16,32,64,128}.
 * lane_channels selects the kernel family: 16 = matrix-core kernels (one 4x4x4
 * MFMA block per channel; the built-in choice), 2 or 4 = vector kernels with that
 * many channels per lane.
 * Replaces the `_DWConv_cl3d_impl[grid](...)` launch and its per-sample Python
 * loop: kerops/ops/conv/dwconv.py:47-61 (kernel kerops/kernels/dw_conv.py:6-142). */
int kerops_dwconv_fwd_f16(const void* x, const void* wt, void* y, int32_t N, int32_t H, int32_t W, int32_t D,
                          int32_t C, int32_t tile_w, int32_t tile_d, int32_t h_chunk, int32_t lane_channels,
                          void* stream);

/* Depthwise convolution as above plus the per-channel batch statistics of its output in the same pass
 * (an addition, no single reference counterpart: it stands for kerops_dwconv_fwd_f16 followed by
 * kerops_stats_f16 on y, i.e. kerops/ops/conv/dwconv.py:20-63 then kerops/ops/stats.py:11-38, and saves the
 * second pass over y):
 *   mean[c] = sum y / (N*H*W*D),  sqmean[c] = sum y*y / (N*H*W*D),  y as stored (fp16), fp32 sums per
 *   workgroup in the workspace, added in a fixed order in fp64 by a second kernel (deterministic).
 * Runs the matrix-core kernel at its built-in launch shape.  C in {8,16,32,64,128}. */
int64_t kerops_dwconv_stats_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C);
int kerops_dwconv_stats_f16(const void* x, const void* wt, void* y, float* mean, float* sqmean, void* workspace,
                            int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                            void* stream);

/* Depthwise weight gradient, fp32 end to end:
 *   gw[kh,kw,kd,c] = sum_{n,h,w,d} g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]
 * gw is [3][3][3][C] fp32.  Deterministic: per-workgroup partials go to the
 * workspace and a second kernel adds them in a fixed order.
 * lane_channels selects the kernel family: 32 = matrix-core kernel (one 4x4x4
 * MFMA block per channel) with planes loaded straight into LDS and 8-byte operand
 * reads, on 8-row patches of 512 16-byte chunks (tile_w 8, tile_d 64 / 32 / 16 / 8 for
 * C = 8 / 16 / 32 / 64 and more; the built-in choice) or 4-row patches of 256; 33 / 34 / 35 = the same with one / two /
 * one x and two g planes in flight ahead of the arithmetic; 16 = matrix-core kernels
 * staged through registers; 2 = vector kernels (two channels per lane, 2-way fp16
 * dot products).
 * Replaces the zero-filled partial buffer, the `_DWConv_wgrad_cl3d_impl[grid](...)`
 * launches and the trailing `grad_w.sum(dim=(0, 1))`:
 * kerops/ops/conv/dwconv_wgrad.py:54-77 (kernel kerops/kernels/dw_conv.py:147-287). */
int64_t kerops_dwconv_wgrad_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C, int32_t tile_w,
                                            int32_t tile_d, int32_t h_chunk, int32_t lane_channels);
int kerops_dwconv_wgrad_f16(const void* x, const void* g, float* gw, void* workspace, int64_t workspace_bytes,
                            int32_t N, int32_t H, int32_t W, int32_t D, int32_t C, int32_t tile_w, int32_t tile_d,
                            int32_t h_chunk, int32_t lane_channels, void* stream);
/* kerops_dwconv_wgrad_f16 with the type of the result chosen by the caller: gw_dtype = KEROPS_DTYPE_F32 (gw is
 * float[27*C], the same bits as kerops_dwconv_wgrad_f16) or KEROPS_DTYPE_F16 (gw is fp16[27*C]: the fp32 sum rounded
 * once, to nearest even, by the reduction kernel).  The reference returns an fp16 [3,3,3,C] tensor
 * (kerops/ops/conv/dwconv_wgrad.py:54,77-79); this entry point gives that type without a cast kernel after the call. */
int kerops_dwconv_wgrad_f16_out(const void* x, const void* g, void* gw, int32_t gw_dtype, void* workspace,
                                int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                int32_t tile_w, int32_t tile_d, int32_t h_chunk, int32_t lane_channels, void* stream);

/* kerops_dwconv_wgrad_f16 at its built-in launch shape for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * op allocates its partial buffer with torch on every call, kerops/ops/conv/dwconv_wgrad.py:54).  No workspace
 * argument: the per-workgroup partials go to a 4 MiB device array that is part of the library (each GPU the
 * library runs on holds its copy until the process ends); the entry point calls no hipMalloc, hipFree or other
 * allocating routine.  The built-in launch shapes need at most 3.5 MB whatever the tensor size; a shape that
 * would need more than 4 MiB returns KEROPS_E_WORKSPACE.  Same result, bit for bit, as kerops_dwconv_wgrad_f16
 * with tile_w = tile_d = h_chunk = lane_channels = 0.  Calls on one GPU share the array: calls that overlap on
 * one GPU (different streams) race.  The first call on a device looks up the array's address
 * (hipGetSymbolAddress) and should be made outside graph capture. */
int kerops_dwconv_wgrad_noalloc_f16(const void* x, const void* g, float* gw, int32_t N, int32_t H, int32_t W,
                                    int32_t D, int32_t C, void* stream);

/* Backward of the depthwise convolution in one pass over x and g (no reference counterpart: the reference has
 * no input gradient, TODO at kerops/kernels/dw_conv.py:145, and computes the weight gradient separately,
 * kerops/ops/conv/dwconv_wgrad.py:25-79):
 *   dx[n,h,w,d,c] = sum_{kh,kw,kd} g[n,h-kh+1,w-kw+1,d-kd+1,c] * wt[kh,kw,kd,c]      (fp16, one rounding)
 *   gw[kh,kw,kd,c] = sum_{n,h,w,d} g[n,h,w,d,c] * x[n,h+kh-1,w+kw-1,d+kd-1,c]        (fp32, deterministic)
 * Every plane of g is staged once and feeds both products, which saves one of the two reads of g that
 * kerops_dwconv_fwd_f16(g, flipped wt) + kerops_dwconv_wgrad_f16 need.  C in {8,16,32,64,128}.
 * The environment variable KEROPS_BWD_STAGING=registers (read at every call of either function) selects the
 * earlier kernel that stages the planes through registers; dx is bit-identical, gw differs in the last bits. */
int64_t kerops_dwconv_bwd_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C, int32_t h_chunk);
int kerops_dwconv_bwd_f16(const void* x, const void* g, const void* wt, void* dx, float* gw, void* workspace,
                          int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                          int32_t h_chunk, void* stream);
/* kerops_dwconv_bwd_f16 with gw written as gw_dtype (KEROPS_DTYPE_F32 or KEROPS_DTYPE_F16, rounded once), as in
 * kerops_dwconv_wgrad_f16_out. */
int kerops_dwconv_bwd_f16_out(const void* x, const void* g, const void* wt, void* dx, void* gw, int32_t gw_dtype,
                              void* workspace, int64_t workspace_bytes, int32_t N, int32_t H, int32_t W, int32_t D,
                              int32_t C, int32_t h_chunk, void* stream);

/* Per-channel mean and mean of squares over M = numel / C voxels, fp32.
 * Replaces the zero-fill of mean/sqmean and the `_Stats_cl3d_impl[(grid,)](...)`
 * launch: kerops/ops/stats.py:27-31 (kernel kerops/kernels/stats.py:6-23).
 * Two-pass and deterministic instead of float atomics. */
int64_t kerops_stats_workspace_bytes(int64_t M, int32_t C, int32_t blocks);
int kerops_stats_f16(const void* x, float* mean, float* sqmean, int64_t M, int32_t C, void* workspace,
                     int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* dx = 2*x*sqmean_grad[c]/M + mean_grad[c]/M, fp16.
 * Replaces `_Stats_cl3d_backward_impl[(grid,)](...)`: kerops/ops/stats.py:52-63
 * (kernel kerops/kernels/stats.py:26-51). */
int kerops_stats_bwd_f16(const void* x, const float* mean_grad, const float* sqmean_grad, void* dx, int64_t M,
                         int32_t C, int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* z = fp16(x + y) and the per-channel mean / mean of squares of z.
 * Replaces `_AddStats_cl3d_impl[(grid,)](...)`: kerops/ops/addition.py:35-48
 * (kernel kerops/kernels/addition.py:6-37).  z may alias x (the inplace mode).
 * Workspace as for kerops_stats_f16. */
int kerops_add_stats_f16(const void* x, const void* y, void* z, float* mean, float* sqmean, int64_t M, int32_t C,
                         void* workspace, int64_t workspace_bytes, int32_t blocks, int32_t waves, int32_t segment,
                         void* stream);

/* out = fp16(add_grad + 2*add_result*sqmean_grad[c]/M + mean_grad[c]/M).
 * Replaces `_AddStats_cl3d_backward_impl[(grid,)](...)`: kerops/ops/addition.py:75-88
 * (kernel kerops/kernels/addition.py:41-75). */
int kerops_add_stats_bwd_f16(const void* add_grad, const float* mean_grad, const float* sqmean_grad,
                             const void* add_result, void* out, int64_t M, int32_t C, int32_t blocks, int32_t waves,
                             int32_t segment, void* stream);

/* y = fp16(max(float(x) * wv[c] + bv[c], 0)); wv, bv are fp32 [C].
 * Replaces `_ApplyBNReLU_cl3d_impl[(grid,)](...)`: kerops/ops/bnrelu.py:30-41
 * (kernel kerops/kernels/bnrelu.py:6-31). */
int kerops_bnrelu_fwd_f16(const void* x, const float* wv, const float* bv, void* y, int64_t M, int32_t C,
                          int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* keep = (x*wv[c] > -bv[c]); g' = g*keep; dx = fp16(wv[c]*g'); dW[c] = sum x*g';
 * dB[c] = sum g' (fp32, deterministic two-pass).
 * Replaces the zero-fill of the two gradients and
 * `_ApplyBNReLU_cl3d_backward_impl[(grid,)](...)`: kerops/ops/bnrelu.py:64-82
 * (kernel kerops/kernels/bnrelu.py:35-71).  Workspace as for kerops_stats_f16. */
int kerops_bnrelu_bwd_f16(const void* x, const float* wv, const float* bv, const void* g, void* dx, float* dW,
                          float* dB, int64_t M, int32_t C, void* workspace, int64_t workspace_bytes, int32_t blocks,
                          int32_t waves, int32_t segment, void* stream);

/* 2x2x2 stride-2 average pool with ceil_mode (edge windows divide by the number
 * of existing voxels), y dense [N][ceil(H/2)][ceil(W/2)][ceil(D/2)][C] fp16, plus
 * mean / mean of squares of the fp32 pooled values.
 * Replaces the zero-fill of mean/sqmean and
 * `_AvgPoolCeilStats_cl3d_impl[(N, H/2, W/2)](...)`: kerops/ops/avgpool.py:33-60
 * (kernel kerops/kernels/avgpool.py:6-93). */
int64_t kerops_avgpool_ceil_stats_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                                  int32_t blocks);
int kerops_avgpool_ceil_stats_f16(const void* x, void* y, float* mean, float* sqmean, int32_t N, int32_t H,
                                  int32_t W, int32_t D, int32_t C, void* workspace, int64_t workspace_bytes,
                                  int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* ApplyBNReLU and AvgPoolCeilStats in one pass (no single reference counterpart; the reference composes
 * the two ops, tests/ops/test_bn_relu.py:26-30 and tests/ops/test_avgpool.py): every existing voxel is
 * mapped to fp16(max(x * weight[c] + bias[c], 0)) before the pool, so the result equals the composition
 * bit for bit while the full-size intermediate never reaches memory.  Workspace as for
 * kerops_avgpool_ceil_stats_f16. */
int kerops_bnrelu_avgpool_ceil_stats_f16(const void* x, const float* weight, const float* bias, void* y, float* mean,
                                         float* sqmean, int32_t N, int32_t H, int32_t W, int32_t D, int32_t C,
                                         void* workspace, int64_t workspace_bytes, int32_t blocks, int32_t waves,
                                         int32_t segment, void* stream);

/* dx[every existing voxel of a window] =
 *   fp16((inpgrad + meangrad[c]/Mo + 2*output*sqmeangrad[c]/Mo) / count),
 * Mo = N*ceil(H/2)*ceil(W/2)*ceil(D/2); (N,H,W,D) is the shape of dx.
 * Replaces the zero-filled outgrad and
 * `_AvgPoolCeilStats_cl3d_backward_impl[(N, H/2, W/2)](...)`:
 * kerops/ops/avgpool.py:93-122 (kernel kerops/kernels/avgpool.py:97-185). */
int kerops_avgpool_ceil_stats_bwd_f16(const void* inpgrad, const float* meangrad, const float* sqmeangrad,
                                      const void* output, void* dx, int32_t N, int32_t H, int32_t W, int32_t D,
                                      int32_t C, int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* u8 = (uint8)(((clip(float(x), -window, window) + window) / (2*window)) * 255),
 * each step one IEEE fp32 operation, conversion by truncation.  dtype is the
 * KEROPS_DTYPE_* tag of x (fp16, fp32 or bf16; the reference kernel converts whatever
 * floating type it is given to fp32 first).  Flat over numel elements.
 * Replaces `_QuantUint8Window_impl[(numblocks,)](...)`:
 * kerops/ops/quantization.py:19 (kernel kerops/kernels/quantization.py:6-27). */
int kerops_quant_u8_window(const void* x, int32_t dtype, void* q, int64_t numel, float window, int32_t blocks,
                           int32_t waves, int32_t segment, void* stream);

/* out = float(u8) * (2*window/255) - window (scale formed once in fp32; one
 * multiply, one subtract), stored as dtype (fp16, fp32 or bf16; one RNE rounding).
 * Replaces `_DequantUint8Window_impl[(numblocks,)](...)`:
 * kerops/ops/quantization.py:34 (kernel kerops/kernels/quantization.py:31-49). */
int kerops_dequant_u8_window(const void* q, void* out, int32_t dtype, int64_t numel, float window, int32_t blocks,
                             int32_t waves, int32_t segment, void* stream);

/* max |y| over numel fp16 values, written to *absmax (device fp32).  No reference
 * counterpart: first pass of the symmetric int8 quantiser of the fused-block
 * configuration.  Workspace: kerops_absmax_workspace_bytes(blocks). */
int64_t kerops_absmax_workspace_bytes(int32_t blocks);
int kerops_absmax_f16(const void* y, float* absmax, int64_t numel, void* workspace, int64_t workspace_bytes,
                      int32_t blocks, void* stream);

/* q = clamp(rint_half_even(float(y) / (absmax/127)), -127, 127) as int8, with
 * absmax read from device memory; absmax == 0 gives q = 0.  scale (device fp32, may be
 * null) receives absmax/127, the factor that dequantises q.  No reference
 * counterpart: second pass of the symmetric int8 quantiser. */
int kerops_quant_i8_sym_f16(const void* y, const float* absmax, void* q, float* scale, int64_t numel,
                            int32_t blocks, int32_t waves, int32_t segment, void* stream);

/* Pointwise (1x1x1) channel mixing on MFMA:
 *   out[v, co] = fp16(sum_ci act(x[v, ci]) * Wm[ci, co]) (+ add[v, co], fp16 add)
 * x dense [V][Cin] fp16, Wm [Cin][Cout] fp16, add/out dense [V][Cout] fp16;
 * act = ReLU when relu_in != 0; add may be NULL.  Cin, Cout in {16,32,64,128}.
 * Replaces `_ReLULinearAdd[(grid,)](...)`: kerops/ops/linear/relu_linear_add.py:46-50
 * (kernel kerops/kernels/linear.py:6-45). */
int kerops_pointwise_f16(const void* x, const void* Wm, const void* add, void* out, int64_t V, int32_t Cin,
                         int32_t Cout, int32_t relu_in, void* stream);

/* Batch-norm affine map + ReLU + pointwise product + residual in one pass (an addition, no single reference
 * counterpart: it stands for kerops_bnrelu_fwd_f16 followed by kerops_pointwise_f16 with relu_in, i.e.
 * kerops/ops/bnrelu.py:11-42 then kerops/ops/linear/relu_linear_add.py:20-52, bit-identical to that composition,
 * without writing and re-reading the normalised activation):
 *   out[v, co] = fp16( sum_ci fp16(max(fma(x[v, ci], scale[ci], shift[ci]), 0)) * Wm[ci, co] ) + add[v, co]
 * scale, shift: [Cin] fp32.  add may be null.  Cin, Cout in {16,32,64,128}. */
int kerops_bnrelu_pointwise_f16(const void* x, const float* scale, const float* shift, const void* Wm,
                                const void* add, void* out, int64_t V, int32_t Cin, int32_t Cout, void* stream);

/* Backward of the ReLU-linear op, one pass over x and grad on MFMA:
 *   dx[v, ci] = x[v, ci] > 0 ? fp16(sum_co g[v, co] * Wm[ci, co]) : 0
 *   dW[ci, co] = sum_v relu(x[v, ci]) * g[v, co]         (fp32, deterministic)
 * x/dx dense [V][Cin] fp16, g dense [V][Cout] fp16, Wm [Cin][Cout] fp16, dW [Cin][Cout] fp32.
 * Cin, Cout in {16,32,64,128}.  Replaces the zero-filled partial buffer, the
 * `_ReLULinearAddBackward[(grid,)](...)` launch and the trailing `weight_grad.sum(dim=0)`:
 * kerops/ops/linear/relu_linear_backward.py:52-70 (kernel kerops/kernels/linear.py:48-98). */
int64_t kerops_relu_linear_bwd_workspace_bytes(int64_t V, int32_t Cin, int32_t Cout);
int kerops_relu_linear_bwd_f16(const void* x, const void* g, const void* Wm, void* dx, float* dW, void* workspace,
                               int64_t workspace_bytes, int64_t V, int32_t Cin, int32_t Cout, void* stream);
/* kerops_relu_linear_bwd_f16 with dW written as dw_dtype: KEROPS_DTYPE_F32, or KEROPS_DTYPE_F16 = the fp32 result
 * rounded once by the reduction kernel (the reference returns fp16, kerops/ops/linear/relu_linear_backward.py:70). */
int kerops_relu_linear_bwd_f16_out(const void* x, const void* g, const void* Wm, void* dx, void* dW, int32_t dw_dtype,
                                   void* workspace, int64_t workspace_bytes, int64_t V, int32_t Cin, int32_t Cout,
                                   void* stream);

/* Inverted-bottleneck pointwise block on MFMA, the hidden activation stays in registers:
 *   hid = relu(fp16(x @ Wup) + bias);  out = fp16(hid @ Wdown) + add       (fp16 adds)
 * x/add/out dense [V][C] fp16, Wup [C][2C], Wdown [2C][C], bias [2C] fp16.  C in {16,32,64}.
 * Replaces `_LinBReLULinAdd[(grid,)](...)`: kerops/ops/linear/linear_bias_relu_linear_add.py:58-71
 * (kernel kerops/kernels/linear.py:102-146). */
int kerops_lin_brelu_lin_add_f16(const void* x, const void* Wup, const void* Wdown, const void* bias, const void* add,
                                 void* out, int64_t V, int32_t C, void* stream);

/* Backward of the inverted-bottleneck block, one pass over x and grad on MFMA:
 *   linup = fp16(x @ Wup) + bias;  lg = linup > 0 ? fp16(g @ Wdown^T) : 0
 *   dx = fp16(lg @ Wup^T);  dWup = x^T lg;  dWdown = relu(linup)^T g;  dbias = sum_v lg   (fp32, deterministic)
 * x/g/dx dense [V][C] fp16; dWup [C][2C], dWdown [2C][C], dbias [2C] fp32.  C in {16,32,64}.
 * Replaces the zero-filled partial buffers, the `_LinBReLULinBackward[(grid,)](...)` launch and the three
 * trailing `.sum(dim=0)`: kerops/ops/linear/linear_bias_relu_linear_backward.py:48-71
 * (kernel kerops/kernels/linear.py:149-230). */
int64_t kerops_lin_brelu_lin_bwd_workspace_bytes(int64_t V, int32_t C);
int kerops_lin_brelu_lin_bwd_f16(const void* x, const void* g, const void* Wup, const void* Wdown, const void* bias,
                                 void* dx, float* dWup, float* dWdown, float* dbias, void* workspace,
                                 int64_t workspace_bytes, int64_t V, int32_t C, void* stream);
/* kerops_lin_brelu_lin_bwd_f16 with dWup, dWdown and dbias written as grad_dtype: KEROPS_DTYPE_F32, or
 * KEROPS_DTYPE_F16 = the fp32 results rounded once by the reduction kernel (the reference returns fp16,
 * kerops/ops/linear/linear_bias_relu_linear_backward.py:71-73). */
int kerops_lin_brelu_lin_bwd_f16_out(const void* x, const void* g, const void* Wup, const void* Wdown, const void* bias,
                                     void* dx, void* dWup, void* dWdown, void* dbias, int32_t grad_dtype,
                                     void* workspace, int64_t workspace_bytes, int64_t V, int32_t C, void* stream);

/* Fused depthwise-separable block (no single reference counterpart; composition
 * of DWConv, a folded inference BN, ReLU and the pointwise GEMM above):
 *   t = fp16(relu(dwconv(x, wt) * scale[c] + shift[c]));  y = fp16(t @ Wm)
 * and the running max |y| written to *absmax (device fp32) for the int8 pass.
 * x [N][H][W][D][Cin], y [N][H][W][D][Cout].  Cin = 64, Cout = 128 built in.
 * Workspace: kerops_dwsep_block_workspace_bytes(...). */
int64_t kerops_dwsep_block_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t Cin, int32_t Cout);
int kerops_dwsep_block_f16(const void* x, const void* wt, const float* scale, const float* shift, const void* Wm,
                           void* y, float* absmax, int32_t N, int32_t H, int32_t W, int32_t D, int32_t Cin,
                           int32_t Cout, void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* KEROPS_HIP_H */
