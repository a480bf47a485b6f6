// Shared host-side helpers of the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "pto_amd.h"

namespace pto_amd {
extern thread_local int g_last_hip_error;

inline int check_launch()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = static_cast<int>(e);
        return PTO_ERR_HIP;
    }
    return PTO_OK;
}

// Dynamic LDS above 64 KiB has to be opted into per kernel.
template <typename K>
inline int allow_lds(K kernel, int bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
        g_last_hip_error = static_cast<int>(e);
        return PTO_ERR_HIP;
    }
    return PTO_OK;
}

// defined in pto_gemm_w8.hip (workgroups of eight wavefronts)
int gemm_f16f32_tile256_w8(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k);
} // namespace pto_amd
