// placeholder until the MFMA kernels land
#include "common.hpp"
using namespace kerops;
extern "C" int kerops_pointwise_f16(const void*, const void*, const void*, void*, int64_t, int32_t, int32_t, int32_t,
                                    void*)
{
    set_error("pointwise: not built");
    return KEROPS_E_UNSUPPORTED_C;
}
extern "C" int64_t kerops_dwsep_block_workspace_bytes(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t)
{
    return KEROPS_E_UNSUPPORTED_C;
}
extern "C" int kerops_dwsep_block_f16(const void*, const void*, const float*, const float*, const void*, void*, float*,
                                      int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, void*, int64_t, void*)
{
    set_error("dwsep_block: not built");
    return KEROPS_E_UNSUPPORTED_C;
}
