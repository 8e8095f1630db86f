// Depthwise-separable block: DWConv 3x3x3 -> folded inference BN (scale, shift) -> ReLU ->
// pointwise 1x1x1 GEMM on the matrix cores, plus max|y| for the symmetric int8 pass.
//
//   t = fp16(max(dwconv(x, wt) * scale[c] + shift[c], 0))   (fp32 accumulate, one rounding)
//   y = fp16(t @ Wm)                                          (fp32 accumulate, one rounding)
//
// Cout in {64, 128}: one kernel.  The matrix-core depthwise kernel hands every finished output plane of
// its 8x8 patch (64 positions x 64 channels, rounded to fp16) through an LDS tile to the pointwise GEMM
// on the 32x32x16 matrix instruction; t never reaches memory and the workspace only holds one max|y|
// per workgroup.  Other Cout: two kernels (depthwise with the affine+ReLU epilogue, then the
// pointwise kernel with the running max), t goes through the caller's workspace.
#include "common.hpp"

using namespace kerops;

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

extern "C" int64_t kerops_dwsep_block_workspace_bytes(int32_t N, int32_t H, int32_t W, int32_t D, int32_t Cin,
                                                      int32_t Cout)
{
    if (N <= 0 || H <= 0 || W <= 0 || D <= 0) {
        set_error("dwsep_block: non-positive extent");
        return KEROPS_E_BADARG;
    }
    if (Cin != 64 || !(Cout == 16 || Cout == 32 || Cout == 64 || Cout == 128)) {
        set_error("dwsep_block: built for Cin = 64 and Cout in {16,32,64,128} (got %d -> %d)", Cin, Cout);
        return KEROPS_E_UNSUPPORTED_C;
    }
    // 32-bit offsets inside a plane of x and of y, 64-bit plane bases (as for every convolution entry point)
    if (plane_exceeds_i32(W, D, Cin) || plane_exceeds_i32(W, D, Cout) || volume_exceeds_i64(N, H, W, D, Cout)) {
        set_error("dwsep_block: one (W,D,C) plane must stay below 2^31 elements and the volume below 2^60");
        return KEROPS_E_BADARG;
    }
    if (Cout >= 64) {
        const int nb = dwsep_fused_blocks(N, H, W, D);
        if (nb < 0) return KEROPS_E_BADARG;
        return align256((int64_t)nb * 4);
    }
    const int64_t V = (int64_t)N * H * W * D;
    return align256(V * Cin * 2) + align256((int64_t)pointwise_blocks(V) * 4);
}

extern "C" int kerops_dwsep_block_f16(const void* x, const void* wt, const float* scale, const float* shift,
                                      const void* Wm, void* y, float* absmax, int32_t N, int32_t H, int32_t W,
                                      int32_t D, int32_t Cin, int32_t Cout, void* workspace, int64_t workspace_bytes,
                                      void* stream)
{
    const int64_t need = kerops_dwsep_block_workspace_bytes(N, H, W, D, Cin, Cout);
    if (need < 0) return (int)need;
    if (!x || !wt || !scale || !shift || !Wm || !y || !absmax || !aligned16(x) || !aligned16(wt) || !aligned16(Wm) ||
        !aligned16(y)) {
        set_error("dwsep_block: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    if (!workspace || !aligned16(workspace) || workspace_bytes < need) {
        set_error("dwsep_block: workspace of %lld bytes required, %lld given", (long long)need,
                  (long long)workspace_bytes);
        return KEROPS_E_WORKSPACE;
    }
    if (Cout >= 64) {
        float* amax_part = (float*)workspace;
        int rc = dwsep_fused_run(x, wt, scale, shift, Wm, y, amax_part, N, H, W, D, Cout, stream);
        if (rc != KEROPS_OK) return rc;
        launch_pw_absmax_final(amax_part, dwsep_fused_blocks(N, H, W, D), absmax, (hipStream_t)stream);
        return check_launch("dwsep_block");
    }
    const int64_t V = (int64_t)N * H * W * D;
    half_t* t = (half_t*)workspace;
    float* amax_ws = (float*)((char*)workspace + align256(V * Cin * 2));
    int rc = dwconv_fwd_run(x, wt, t, scale, shift, N, H, W, D, Cin, 8, 8, 0, 16, stream);
    if (rc != KEROPS_OK) return rc;
    const int blocks = pointwise_blocks(V);
    rc = pointwise_dispatch(t, (const half_t*)Wm, nullptr, (half_t*)y, amax_ws, V, Cin, Cout, false, true, blocks,
                            (hipStream_t)stream);
    if (rc != KEROPS_OK) return rc;
    launch_pw_absmax_final(amax_ws, blocks, absmax, (hipStream_t)stream);
    return check_launch("dwsep_block");
}
