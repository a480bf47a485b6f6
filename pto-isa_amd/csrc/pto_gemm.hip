// fp16 x fp16 -> fp32 GEMM for MI355X written with PTO tile instructions:
//   TLOAD (HBM -> LDS, async 16-byte copies)  ->  TEXTRACT (LDS -> MFMA operand fragments)
//   ->  TMATMUL / TMATMUL_ACC (v_mfma_f32_32x32x16_f16)  ->  TSTORE (accumulators -> HBM).
//
// Same decomposition as the reference's manual kernel
// (kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp:67-230): each "core" owns
// BM x BN blocks of C, walks K in steps of BK, double-buffers the staged A / B panels and
// synchronises the stages with set_flag / wait_flag.  Differences that the hardware asks for:
// the stages are software-pipelined in program order (one instruction stream per wavefront: the
// TLOAD of step i+1 is issued before the TEXTRACT / TMATMUL of step i), one workgroup per C block
// instead of a 24-core loop nest, and an XCD-aware block -> tile map.
#include "gemm_kernels.hpp"

#if defined(PTO_ST_HOOKS)
// Tuning hook (not part of the public header): the same GEMM with another tiling / pipeline depth.
extern "C" int pto_gemm_f16f32_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k,
                                       int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_gemm<128, 256, 64, 2, 1, 8>(st, c, ha, hb, m, n, k);
    case 1: return launch_gemm<128, 256, 32, 2, 2, 8>(st, c, ha, hb, m, n, k);
    case 2: return launch_gemm<128, 256, 32, 3, 2, 8>(st, c, ha, hb, m, n, k);
    case 3: return launch_gemm<128, 256, 64, 3, 1, 8>(st, c, ha, hb, m, n, k);
    case 4: return launch_gemm<128, 256, 32, 4, 2, 8>(st, c, ha, hb, m, n, k);
    case 5: return launch_gemm<128, 256, 32, 3, 2, 4>(st, c, ha, hb, m, n, k);
    case 6: return launch_gemm<128, 256, 32, 3, 2, 16>(st, c, ha, hb, m, n, k);
    case 7: return launch_gemm<256, 256, 32, 4, 1, 8>(st, c, ha, hb, m, n, k);
    case 8: return launch_gemm<256, 256, 64, 2, 1, 8>(st, c, ha, hb, m, n, k);
    case 9: return launch_gemm<256, 256, 32, 3, 1, 8>(st, c, ha, hb, m, n, k);
    case 10: return launch_gemm<256, 256, 32, 4, 1, 4>(st, c, ha, hb, m, n, k);
    case 11: return launch_gemm<256, 256, 32, 2, 1, 8>(st, c, ha, hb, m, n, k);
    case 30: return launch_gemm_mix<256, 256, 4, 8>(st, c, ha, hb, m, n, k, 2);
    case 31: return launch_gemm_mix<256, 256, 3, 8>(st, c, ha, hb, m, n, k, 2);
    case 32: return launch_gemm_mix<256, 256, 4, 4>(st, c, ha, hb, m, n, k, 2);
    case 33: return launch_gemm_mix<256, 256, 4, 8>(st, c, ha, hb, m, n, k, 0);
    case 35: return launch_gemm_mix<256, 256, 4, 4>(st, c, ha, hb, m, n, k, 3);
    case 36: return launch_gemm_mix<256, 256, 4, 8>(st, c, ha, hb, m, n, k, 3);
    case 34: return launch_gemm_mix<256, 256, 4, 4>(st, c, ha, hb, m, n, k, 0);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS

extern "C" int pto_gemm_f16f32(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    // Large problems: 256 x 256 C tiles (two thirds of the operand traffic per flop of the 128 x 256
    // block), one workgroup of eight wavefronts per compute unit.  Problems with too few such tiles
    // to fill the machine, or with extents that are not multiples of them: the 128 x 256 block of
    // the reference kernel, two workgroups of four wavefronts per compute unit.
    const bool big = m % 256 == 0 && n % 256 == 0 && k % 128 == 0 && k / 32 >= 8 &&
                     (long long)(m / 256) * (n / 256) * 2 >= compute_units();
    if (big) {
        // tiles that (nearly) fill whole rounds over the compute units: the kernel with K-steps of 64 (every operand row a
        // whole 128-byte line per step; interleaved runs: 6144^3 1336 against 1254 TFLOP/s, 8192^3 1329 against 1298)
        const int rc64 = pto_amd::gemm_f16f32_k64(st, c, ha, hb, m, n, k);
        if (rc64 != PTO_ERR_UNSUPPORTED)
            return rc64;
        // otherwise four wavefronts with the K-step written fragment by fragment where that kernel has a tile shape for
        // the problem and is the faster one (uneven rounds, or 192 x 192 tiles for a single round), else eight wavefronts
        const int rc384 = pto_amd::gemm_f16f32_tile384x192_w8(st, c, ha, hb, m, n, k); // whole rounds of 384 x 192 tiles, k % 128 != 0
        if (rc384 != PTO_ERR_UNSUPPORTED)
            return rc384;
        const int rc = pto_amd::gemm_f16f32_tile256_w4(st, c, ha, hb, m, n, k);
        if (rc != PTO_ERR_UNSUPPORTED)
            return rc;
        return pto_amd::gemm_f16f32_tile256_w8(st, c, ha, hb, m, n, k);
    }
    return launch_gemm<128, 256, 32, 3, 2, 8>(st, c, ha, hb, m, n, k);
}
