// The 256 x BN and 192 x BN GEMM tiles on four wavefronts (gemm_kernels_w4.hpp), wave grid 4 x 1, and the choice among them.
#define PTO_WAVES_M 4
#define PTO_WAVES_N 1
#define PTO_MFMA_M 16
#include "gemm_kernels_w4.hpp"

namespace pto_amd {
// Tiles are dealt to the compute units one workgroup at a time, so a problem takes ceil(tiles / units) rounds of one
// tile's time, and a tile's time is its K-steps times the step time of its shape plus what does not depend on k (two
// copy round trips before the first MFMA, the store of C).  The smaller tiles move more operand bytes per flop and run
// their step at a lower rate, but cut m x n into more pieces: 6144^2 is 2.25 rounds of 256 x 256 and exactly 3 of
// 256 x 192; 3072^2 is three quarters of a round of 256 x 192 and exactly one of 192 x 192.  Times in microseconds as
// measured at 3072^3, 6144^3 and 7680^3 (48, 96 and 120 K-steps); only their ratios matter.
int gemm_f16f32_w4(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    if (n % 4 || k % 128 || k < 128)
        return PTO_ERR_UNSUPPORTED;
    using Launch = int (*)(hipStream_t, float *, const half *, const half *, int, int, int);
    struct Shape { int tm, bn; double step, fixed; Launch launch; };
    static const Shape shapes[6] = {{256, 256, 1.31, 10.0, launch_gemm_w4<256, 4>}, {256, 192, 1.03, 10.0, launch_gemm_w4<192, 4>},
                                    {256, 128, 0.70, 7.0, launch_gemm_w4<128, 4>},  {192, 256, 1.04, 10.0, launch_gemm_w4<256, 3>},
                                    {192, 192, 0.80, 10.0, launch_gemm_w4<192, 3>}, {192, 128, 0.56, 7.0, launch_gemm_w4<128, 3>}};
    const int cus = compute_units();
    const Shape *best = nullptr;
    double bestTime = 0.0;
    for (const Shape &s : shapes) {
        if (m < s.tm || n < s.bn)
            continue;
        const long long tiles = (long long)((m + s.tm - 1) / s.tm) * ((n + s.bn - 1) / s.bn), rounds = (tiles + cus - 1) / cus;
        const double time = (double)rounds * ((k / 64) * s.step + s.fixed);
        if (best == nullptr || time < bestTime) {
            best = &s;
            bestTime = time;
        }
    }
    return best != nullptr ? best->launch(st, c, a, b, m, n, k) : PTO_ERR_UNSUPPORTED;
}
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
// tile shape by number: 0 .. 2 = 256 rows x 256 / 192 / 128 columns, 3 .. 5 = 192 rows x the same widths
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
    case 3: return launch_gemm_w4<256, 3>(st, c, ha, hb, m, n, k);
    case 4: return launch_gemm_w4<192, 3>(st, c, ha, hb, m, n, k);
    case 5: return launch_gemm_w4<128, 3>(st, c, ha, hb, m, n, k);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
