// The GEMM kernels of gemm_kernels.hpp instantiated for workgroups of 8 wavefronts (wave grid
// 2 x 4, 512 threads): two waves per SIMD hide each other's LDS and barrier latency.
#define PTO_WAVES_M 2
#define PTO_WAVES_N 4
#include "gemm_kernels.hpp"

namespace pto_amd {
int gemm_compute_units() { return compute_units(); }
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
extern "C" int pto_gemm_f16f32_w8_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k,
                                          int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_gemm<256, 256, 32, 4, 1, 8>(st, c, ha, hb, m, n, k);
    case 1: return launch_gemm<256, 256, 64, 2, 1, 8>(st, c, ha, hb, m, n, k);
    case 2: return launch_gemm<256, 256, 32, 3, 1, 8>(st, c, ha, hb, m, n, k);
    case 3: return launch_gemm<256, 256, 32, 4, 1, 4>(st, c, ha, hb, m, n, k);
    case 4: return launch_gemm<256, 256, 32, 2, 1, 8>(st, c, ha, hb, m, n, k);
    case 5: return launch_gemm<128, 256, 32, 4, 1, 8>(st, c, ha, hb, m, n, k);
    case 30: return launch_gemm_mix<256, 256, 4, 4>(st, c, ha, hb, m, n, k, 1);
    case 31: return launch_gemm_mix<256, 256, 4, 8>(st, c, ha, hb, m, n, k, 1);
    case 32: return launch_gemm_mix<256, 256, 3, 4>(st, c, ha, hb, m, n, k, 1);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
