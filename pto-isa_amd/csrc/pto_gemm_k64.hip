// The GEMM tile with K-steps of 64 (whole 128-byte lines per row and step, gemm_kernels_k64.hpp) for workgroups of eight
// wavefronts on v_mfma_f32_16x16x32_f16, wave grid 4 x 2: at 384 x 192 a wave owns 96 x 96 of C, which takes 12 fragment
// reads per 32-wide K half for its 36 MFMAs (192 x 48 per wave on a 2 x 4 grid takes 15, and two fragment sets of that size
// do not fit the 256 registers of a wave next to the 144 accumulators).
#define PTO_WAVES_M 4
#define PTO_WAVES_N 2
#define PTO_MFMA_M 16
#include "gemm_kernels_k64.hpp"

namespace pto_amd {
// Picks the tile shape that keeps the compute units busiest: the fraction of the rounds' tile slots that hold a tile, times
// the shape's own efficiency (256 x 192 moves more operand bytes per flop: 1250 against 1340 TFLOP/s at 6144^3, where both
// shapes fill whole rounds).  The kernel has no quarter tiles for a partial last round, so below 0.85 the caller's other
// kernels take the problem (PTO_ERR_UNSUPPORTED).  Measured against them (interleaved runs, TFLOP/s): 6144^3 1336 / 1254,
// 8192^3 1329 / 1298, 4096^3 1290 / 1235, 7680^3 (3.5 rounds of 256 x 256) 1225 / 1207, 9216^3 (4.5 rounds of 384 x 192)
// 1187 / 1140.
int gemm_f16f32_k64(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    const int cus = compute_units();
    if (k % 128)
        return PTO_ERR_UNSUPPORTED;
    struct Shape { int bm, bn; double eff; };
    const Shape shapes[3] = {{256, 256, 1.0}, {384, 192, 1.0}, {256, 192, 0.93}};
    int best = -1;
    double bestScore = 0.85;
    for (int i = 0; i < 3; ++i) {
        if (m % shapes[i].bm || n % shapes[i].bn)
            continue;
        const long long tiles = (long long)(m / shapes[i].bm) * (n / shapes[i].bn), rounds = (tiles + cus - 1) / cus;
        const double score = shapes[i].eff * (double)tiles / (double)(rounds * cus);
        if (score > bestScore + 1e-9) {
            bestScore = score;
            best = i;
        }
    }
    switch (best) {
    case 0: return launch_gemm_k64<256, 256, 4>(st, c, a, b, m, n, k);
    case 1: return launch_gemm_k64<384, 192, 4>(st, c, a, b, m, n, k);
    case 2: return launch_gemm_k64<256, 192, 4>(st, c, a, b, m, n, k);
    default: return PTO_ERR_UNSUPPORTED;
    }
}
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
extern "C" int pto_gemm_f16f32_k64_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k,
                                           int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_gemm_k64<384, 192, 4>(st, c, ha, hb, m, n, k);
    case 1: return launch_gemm_k64<256, 256, 4>(st, c, ha, hb, m, n, k);
    case 2: return launch_gemm_k64<256, 192, 4>(st, c, ha, hb, m, n, k);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
