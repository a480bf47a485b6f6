// Shared host-side helpers of the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "pto_amd.h"
#if defined(PTO_ST_HOOKS)
#include "pto_amd_st.h" // test-only entry points (libpto_st.so)
#endif

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

// defined in pto_gemm_w4.hip (256 x 256 / 192 / 128 tiles on four wavefronts, K-steps of 64); PTO_ERR_UNSUPPORTED unless m is a
// multiple of 256, n of one of the widths and k of 128
int gemm_f16f32_w4(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k);
// defined in pto_gemm_mxw4.hip (MXFP8 / MXFP4 on the four-wave engine: 256 x 192 or 256 x 128 tiles, width 0 = chosen by
// rounds); PTO_ERR_UNSUPPORTED unless m >= 256, n >= 128, n % 4 == 0, k % 512 == 0 (fp4, format 4: k % 1024 == 0)
int gemm_mx_w4(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n, int k,
                  int format, int c_fp32, int width);
double mx_w4_time(int m, int n, int k_bytes, int width, bool fp4);
// defined in pto_fa_w8.hip (head_dim 128, workgroups of eight wavefronts = 256 queries, two groups of four waves in
// opposite MFMA / softmax phases)
int fa_fwd_d128_w8(hipStream_t st, void *o, float *lse, const _Float16 *q, const _Float16 *k, const _Float16 *v, int batch, int heads,
                   int seqQ, int seqKv, bool causal, bool oFp32, int causalOff);
// defined in pto_fa_w8m16.hip: the same schedule on v_mfma_f32_16x16x32_f16
int fa_fwd_d128_w8m16(hipStream_t st, void *o, float *lse, const _Float16 *q, const _Float16 *k, const _Float16 *v, int batch, int heads,
                      int seqQ, int seqKv, bool causal, bool oFp32, int causalOff);
} // namespace pto_amd
