// Library-wide pieces of libkerops_hip.so: version, per-thread error text.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"

namespace kerops {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return KEROPS_E_LAUNCH;
    }
    return KEROPS_OK;
}

}  // namespace kerops

extern "C" int kerops_hip_version(void) { return 100; }

extern "C" const char* kerops_last_error_string(void) { return kerops::g_err; }

namespace kerops {

__global__ __launch_bounds__(256) void reduce_rows_kernel(const float* __restrict__ ws, int nrows, int ncols,
                                                          float* __restrict__ out0, float* __restrict__ out1,
                                                          int split, double scale)
{
    __shared__ double part[16][17];
    const int lo = threadIdx.x % 16;
    const int sl = threadIdx.x / 16;
    const int j = blockIdx.x * 16 + lo;
    double s = 0.0;
    if (j < ncols) {
        for (int r = sl; r < nrows; r += 16) s += (double)ws[(int64_t)r * ncols + j];
    }
    part[sl][lo] = s;
    __syncthreads();
    if (sl == 0 && j < ncols) {
        double v = 0.0;
#pragma unroll
        for (int i = 0; i < 16; ++i) v += part[i][lo];
        v *= scale;
        if (j < split) {
            out0[j] = (float)v;
        } else {
            out1[j - split] = (float)v;
        }
    }
}

void launch_reduce_rows(const float* ws, int nrows, int ncols, float* out0, float* out1, int split, double scale,
                        hipStream_t stream)
{
    hipLaunchKernelGGL(reduce_rows_kernel, dim3(ceil_div(ncols, 16)), dim3(256), 0, stream, ws, nrows, ncols, out0,
                       out1, split, scale);
}

}  // namespace kerops
