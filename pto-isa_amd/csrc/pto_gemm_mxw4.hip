// The MXFP8 / MXFP4 GEMM tile on four wavefronts (gemm_kernels_mxw4.hpp), wave grid 4 x 1, and the choice of its width.
#define PTO_WAVES_M 4
#define PTO_WAVES_N 1
#define PTO_MFMA_M 16
#include "gemm_kernels_mxw4.hpp"

namespace pto_amd {
// Estimated time (microseconds) of the four-wave kernel with 256 x width tiles: rounds over the compute units x (K-steps
// of 128 bytes x step time + fixed time), the times as measured at 4096^3, 6144^3 and 8192^3; a last round that does not
// fill the chip counts as half a round plus half its share of the compute units (the others finish early and the clock
// rises).  A huge value where the width does not fit.  k_bytes: bytes of a row of A (k for fp8, k / 2 for fp4).
double mx_w4_time(int m, int n, int k_bytes, int width, bool fp4)
{
    if (m < 256 || n < width || (width != 192 && width != 128))
        return 1e30;
    const int cus = compute_units();
    const long long tiles = (long long)((m + 255) / 256) * ((n + width - 1) / width), full = tiles / cus, rest = tiles - full * cus;
    const double rounds = (double)full + (rest ? 0.5 + 0.5 * (double)rest / cus : 0.0);
    const double step = width == 192 ? (fp4 ? 1.16 : 1.0) : 0.78, fixed = width == 192 ? 11.0 : (fp4 ? 8.7 : 6.0);
    return rounds * ((k_bytes / 128) * step + fixed);
}

// format: 0 = e4m3 x e4m3, 1 = e5m2 x e5m2, 2 = A e4m3 x B e5m2, 3 = A e5m2 x B e4m3, 4 = e2m1 x e2m1 (k then counts 4-bit
// elements, two per byte); width: 192 or 128, 0 = the faster by the estimate above
int gemm_mx_w4(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n, int k,
                  int format, int c_fp32, int width)
{
    if (format < 0 || format > 4)
        return PTO_ERR_UNSUPPORTED;
    const int kBytes = format == 4 ? k / 2 : k;
    if (width == 0)
        width = n >= 192 && mx_w4_time(m, n, kBytes, 192, format == 4) <= mx_w4_time(m, n, kBytes, 128, format == 4) ? 192 : 128;
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
    PTO_MXW4_CASE(4, 4, 4)
#undef PTO_MXW4_CASE
    return PTO_ERR_UNSUPPORTED;
}
} // namespace pto_amd
