// The MXFP8 GEMM tile on four wavefronts (gemm_kernels_mxw4.hpp), wave grid 4 x 1, and the choice of its width.
#define PTO_WAVES_M 4
#define PTO_WAVES_N 1
#define PTO_MFMA_M 16
#include "gemm_kernels_mxw4.hpp"

namespace pto_amd {
// Estimated time (microseconds) of the four-wave kernel with 256 x width tiles: rounds over the compute units x (K-steps
// x step time + fixed time), the times as measured at 4096^3, 6144^3 and 8192^3; a huge value where the width does not fit.
double mxfp8_w4_time(int m, int n, int k, int width)
{
    if (m < 256 || n < width || (width != 192 && width != 128))
        return 1e30;
    const int cus = compute_units();
    const long long tiles = (long long)((m + 255) / 256) * ((n + width - 1) / width), rounds = (tiles + cus - 1) / cus;
    return (double)rounds * ((k / 128) * (width == 192 ? 0.99 : 0.70) + (width == 192 ? 11.5 : 9.0));
}

// format: 0 = e4m3 x e4m3, 1 = e5m2 x e5m2, 2 = A e4m3 x B e5m2, 3 = A e5m2 x B e4m3; width: 192 or 128, 0 = the faster by the
// estimate above
int gemm_mxfp8_w4(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n, int k,
                  int format, int c_fp32, int width)
{
    if (format < 0 || format > 3)
        return PTO_ERR_UNSUPPORTED;
    if (width == 0)
        width = n >= 192 && mxfp8_w4_time(m, n, k, 192) <= mxfp8_w4_time(m, n, k, 128) ? 192 : 128;
#define PTO_MXW4_CASE(FMT, FA, FB)                                                                                         \
    if (format == FMT) {                                                                                                  \
        if (width == 192)                                                                                                 \
            return c_fp32 ? launch_gemm_mxw4<FA, FB, float, 192>(st, c, a, b, sa, sb, m, n, k) :                           \
                            launch_gemm_mxw4<FA, FB, bfloat16_t, 192>(st, c, a, b, sa, sb, m, n, k);                       \
        return c_fp32 ? launch_gemm_mxw4<FA, FB, float, 128>(st, c, a, b, sa, sb, m, n, k) :                               \
                        launch_gemm_mxw4<FA, FB, bfloat16_t, 128>(st, c, a, b, sa, sb, m, n, k);                           \
    }
    PTO_MXW4_CASE(0, 0, 0)
    PTO_MXW4_CASE(1, 1, 1)
    PTO_MXW4_CASE(2, 0, 1)
    PTO_MXW4_CASE(3, 1, 0)
#undef PTO_MXW4_CASE
    return PTO_ERR_UNSUPPORTED;
}
} // namespace pto_amd
