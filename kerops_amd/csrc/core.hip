// Library-wide pieces of libkerops_hip.so: version, per-thread error text.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

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

DeviceGeometry device_geometry()
{
    static std::mutex mutex;
    static DeviceGeometry known[64];  // cus == 0: not looked up yet
    const DeviceGeometry fallback{256, 8};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();  // a query without a device must not leave an error behind for the next launch check
        return fallback;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (known[dev].cus == 0) {
        int cus = 0, xcds = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            return fallback;
        }
        if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || xcds <= 0) {
            (void)hipGetLastError();
            xcds = cus >= 64 ? cus / 32 : 1;  // a runtime without the attribute: 32 compute units per die
        }
        known[dev] = DeviceGeometry{cus, xcds};
    }
    return known[dev];
}

}  // namespace kerops

extern "C" int kerops_hip_version(void) { return KEROPS_HIP_VERSION; }

extern "C" const char* kerops_last_error_string(void) { return kerops::g_err; }

namespace kerops {

// Sums the rows of a partial buffer column by column in a fixed order (fp64) and writes scale * sum to out0
// (columns below split) or out1.  A workgroup owns 16 columns; its 64 row slices take interleaved rows with four
// loads in flight each (a single dependent chain over hundreds of rows took longer than the pass it finishes),
// then the slices are combined by a fixed tree in LDS.
// OutT: fp32, or fp16 = the fp32 result rounded once (what a cast of it gives, without the cast's launch).
template <class OutT>
__global__ __launch_bounds__(1024) void reduce_rows_kernel(const float* __restrict__ ws, int nrows, int ncols,
                                                           OutT* __restrict__ out0, OutT* __restrict__ out1,
                                                           int split, double scale)
{
    __shared__ double part[64][17];
    const int lo = threadIdx.x % 16;
    const int sl = threadIdx.x / 16;
    const int j = blockIdx.x * 16 + lo;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    if (j < ncols) {
        int r = sl;
        for (; r + 192 < nrows; r += 256) {
            const float a = ws[(int64_t)r * ncols + j], b = ws[(int64_t)(r + 64) * ncols + j];
            const float c = ws[(int64_t)(r + 128) * ncols + j], d = ws[(int64_t)(r + 192) * ncols + j];
            s0 += (double)a;
            s1 += (double)b;
            s2 += (double)c;
            s3 += (double)d;
        }
        for (; r < nrows; r += 64) s0 += (double)ws[(int64_t)r * ncols + j];
    }
    part[sl][lo] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int w = 32; w > 0; w >>= 1) {
        if (sl < w) part[sl][lo] += part[sl + w][lo];
        __syncthreads();
    }
    if (sl == 0 && j < ncols) {
        const double v = part[0][lo] * scale;
        if (j < split) {
            out0[j] = (OutT)(float)v;
        } else {
            out1[j - split] = (OutT)(float)v;
        }
    }
}

void launch_reduce_rows(const float* ws, int nrows, int ncols, float* out0, float* out1, int split, double scale,
                        hipStream_t stream)
{
    hipLaunchKernelGGL(reduce_rows_kernel<float>, dim3(ceil_div(ncols, 16)), dim3(1024), 0, stream, ws, nrows, ncols,
                       out0, out1, split, scale);
}

void launch_reduce_rows_f16(const float* ws, int nrows, int ncols, half_t* out0, half_t* out1, int split, double scale,
                            hipStream_t stream)
{
    hipLaunchKernelGGL(reduce_rows_kernel<half_t>, dim3(ceil_div(ncols, 16)), dim3(1024), 0, stream, ws, nrows, ncols,
                       out0, out1, split, scale);
}

}  // namespace kerops
