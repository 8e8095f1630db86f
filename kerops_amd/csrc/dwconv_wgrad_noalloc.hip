// The depthwise weight gradient for callers that cannot allocate (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc): kerops_dwconv_wgrad_f16 at its built-in launch shape, with the
// per-workgroup partials in a file-scope device array instead of a caller's workspace.
//
// The balanced split of the H march launches at most 1024 workgroups, each leaving one [27][slab <= 64] fp32
// partial: the built-in shapes need 0.9 MB (C = 8) to 3.5 MB (C >= 32) whatever the tensor size.  Every GPU the
// library runs on holds its own copy of the array until the process ends.  In host code the array's name is only a
// handle, not a device address: the address on the current device comes from hipGetSymbolAddress, once per device,
// and only that pointer is handed to the kernels (as the workspace argument of the existing entry point).
// Calls on one GPU share the array: two calls that overlap on one GPU (different streams) race on the partials.
// Nothing has to start at zero: every workgroup of a launch writes its partial before the reduction reads it.
#include <mutex>

#include "common.hpp"

using namespace kerops;

static constexpr int64_t kScratchBytes = 4 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];  // per device; null until the first call with that device current

static int scratch_of_current_device(void** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("dwconv_wgrad_noalloc: no usable current device (%s)",
                  e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return KEROPS_E_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_error("dwconv_wgrad_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return KEROPS_E_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return KEROPS_OK;
}

extern "C" int kerops_dwconv_wgrad_noalloc_f16(const void* x, const void* g, float* gw, int32_t N, int32_t H,
                                               int32_t W, int32_t D, int32_t C, void* stream)
{
    if (!x || !g || !gw || !aligned16(x) || !aligned16(g) || !aligned16(gw)) {  // before any device call
        set_error("dwconv_wgrad_noalloc: null or misaligned pointer");
        return KEROPS_E_BADARG;
    }
    const int64_t need = kerops_dwconv_wgrad_workspace_bytes(N, H, W, D, C, 0, 0, 0, 0);
    if (need < 0) return (int)need;  // the query has set the error text
    if (need > kScratchBytes) {
        set_error("dwconv_wgrad_noalloc: this shape needs %lld bytes of partials, the built-in buffer holds %lld; "
                  "use kerops_dwconv_wgrad_f16 with a workspace",
                  (long long)need, (long long)kScratchBytes);
        return KEROPS_E_WORKSPACE;
    }
    void* ptr = nullptr;
    const int rc = scratch_of_current_device(&ptr);
    if (rc != KEROPS_OK) return rc;
    return kerops_dwconv_wgrad_f16(x, g, gw, ptr, kScratchBytes, N, H, W, D, C, 0, 0, 0, 0, stream);
}
