// The 256 x BN GEMM tile on four wavefronts (gemm_kernels_w4.hpp), wave grid 4 x 1, and the choice of BN.
#define PTO_WAVES_M 4
#define PTO_WAVES_N 1
#define PTO_MFMA_M 16
#include "gemm_kernels_w4.hpp"

namespace pto_amd {
// Tiles are dealt to the compute units one workgroup at a time, so a problem takes ceil(tiles / units) rounds of one
// tile's time, and a tile's time is its K-steps times the step time of its width plus what does not depend on k (two
// copy round trips before the first MFMA, the store of C).  The narrower tiles move more operand bytes per flop and run
// their step at a lower rate, but cut m x n into more pieces: 6144^2 is 2.25 rounds of 256 x 256 and exactly 3 of
// 256 x 192.  Times in microseconds as measured at 6144^3 and 7680^3 (96 and 120 K-steps); only their ratios matter.
int gemm_f16f32_w4(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    if (m < kW4TileM || n % 4 || k % 128 || k < 128)
        return PTO_ERR_UNSUPPORTED;
    struct Width { int bn; double step, fixed; };
    const Width widths[3] = {{256, 1.31, 10.0}, {192, 1.03, 10.0}, {128, 0.70, 7.0}};
    const int cus = compute_units();
    int best = -1;
    double bestTime = 0.0;
    for (int i = 0; i < 3; ++i) {
        if (n < widths[i].bn)
            continue;
        const long long tiles = (long long)((m + kW4TileM - 1) / kW4TileM) * ((n + widths[i].bn - 1) / widths[i].bn);
        const long long rounds = (tiles + cus - 1) / cus;
        const double time = (double)rounds * ((k / 64) * widths[i].step + widths[i].fixed);
        if (best < 0 || time < bestTime) {
            best = i;
            bestTime = time;
        }
    }
    switch (best) {
    case 0: return launch_gemm_w4<256>(st, c, a, b, m, n, k);
    case 1: return launch_gemm_w4<192>(st, c, a, b, m, n, k);
    case 2: return launch_gemm_w4<128>(st, c, a, b, m, n, k);
    default: return PTO_ERR_UNSUPPORTED;
    }
}
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
// tile width by number: 0 = 256, 1 = 192, 2 = 128
extern "C" int pto_gemm_f16f32_w4_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k, int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_gemm_w4<256>(st, c, ha, hb, m, n, k);
    case 1: return launch_gemm_w4<192>(st, c, ha, hb, m, n, k);
    case 2: return launch_gemm_w4<128>(st, c, ha, hb, m, n, k);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
