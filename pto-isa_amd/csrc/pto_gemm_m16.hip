// The 256 x 256 GEMM tile for workgroups of 8 wavefronts (wave grid 2 x 4) on v_mfma_f32_16x16x32_f16: same flops
// per cycle as the 32 x 32 x 16 form, half the accumulator register traffic per flop, and a higher sustained clock
// under the chip's power limit.
#define PTO_WAVES_M 2
#define PTO_WAVES_N 4
#define PTO_MFMA_M 16
#include "gemm_kernels.hpp"

namespace pto_amd {
// 256 x 256 C tiles, eight wavefronts per workgroup (128 x 64 of C per wave), 16 x 16 x 32 MFMAs: the default for
// large problems.
int gemm_f16f32_tile256_w8(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    // A problem whose 256 x 256 tiles do not even fill one round: 256 x 192 tiles put more compute units to work
    // (3072^3: 192 instead of 144 workgroups, measured +12 %).  With several rounds the square tile wins (less operand
    // traffic per flop) even where the narrower one would divide the rounds evenly (6144^3: -4 %, 7680^3: -9 %).
    const int cus = compute_units();
    if (n % 192 == 0 && (m / 256) * (n / 256) < cus && (m / 256) * (n / 192) <= cus)
        return launch_gemm_mix<256, 192, 4, 4, true>(st, c, a, b, m, n, k, 0);
    return launch_gemm_mix<256, 256, 4, 4, true>(st, c, a, b, m, n, k, 1);
}
// 384 x 192 C tiles (the operand traffic per flop of the 256 x 256 tile, 144 accumulator registers per wave, 144 KiB of
// LDS) for problems that they cut into whole rounds over the compute units while 256 x 256 tiles leave a partial round:
// 6144 x 6144 = 512 tiles = two rounds on 256 compute units (interleaved runs: 1274 against 1261 TFLOP/s for the four-wave
// kernel with its quarter-tile round; slower wherever the rounds are not whole).  PTO_ERR_UNSUPPORTED: not such a problem.
int gemm_f16f32_tile384x192_w8(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    const int cus = compute_units();
    if (m % 384 || n % 192 || m % 256 || n % 256)
        return PTO_ERR_UNSUPPORTED;
    const long long t384 = (long long)(m / 384) * (n / 192), t256 = (long long)(m / 256) * (n / 256);
    if (t384 % cus != 0 || t256 % cus == 0)
        return PTO_ERR_UNSUPPORTED;
    return launch_gemm_mix<384, 192, 4, 4, true>(st, c, a, b, m, n, k, 0);
}
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
extern "C" int pto_gemm_f16f32_m16_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k,
                                           int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_gemm_mix<256, 256, 4, 4, true>(st, c, ha, hb, m, n, k, 1);
    case 2: return launch_gemm_mix<256, 256, 4, 8, true>(st, c, ha, hb, m, n, k, 1);
    case 3: return launch_gemm_mix<256, 256, 4, 4, true>(st, c, ha, hb, m, n, k, 0);
    case 10: return launch_gemm_mix<256, 192, 4, 4, true>(st, c, ha, hb, m, n, k, 0);
    case 11: return launch_gemm_mix<256, 192, 4, 8, true>(st, c, ha, hb, m, n, k, 0);
    case 12: return launch_gemm_mix<384, 192, 4, 4, true>(st, c, ha, hb, m, n, k, 0);
    case 14: return launch_gemm_mix<384, 192, 4, 8, true>(st, c, ha, hb, m, n, k, 0);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
