// fp16 x fp16 -> fp32 GEMM for MI355X written with PTO tile instructions:
//   TLOAD (HBM -> LDS, async 16-byte copies)  ->  TEXTRACT (LDS -> MFMA operand fragments)
//   ->  TMATMUL / TMATMUL_ACC (v_mfma_f32_32x32x16_f16)  ->  TSTORE (accumulators -> HBM);
// and the entry point that picks between it and the four-wave kernel of pto_gemm_w4.hip.
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
    // Tiles of 256 or 192 rows on four wavefronts with K-steps of 64, the shape chosen by the number of rounds it gives
    // (pto_gemm_w4.hip; m >= 192, n >= 128, n % 4 == 0, k % 128 == 0): faster than the kernel below at every size measured
    // (512^3: 30 against 23 TFLOP/s, 2048^3: 756 against 440, 6144^3: 1450 against 1130).  Other K extents: the 128 x 256
    // block of the reference kernel written with the tile instructions, K-steps of 32, two workgroups of four wavefronts
    // per compute unit (m % 128 == 0, n % 256 == 0, k % 32 == 0).
    const int rc = pto_amd::gemm_f16f32_w4(st, c, ha, hb, m, n, k);
    if (rc != PTO_ERR_UNSUPPORTED)
        return rc;
    return launch_gemm<128, 256, 32, 3, 2, 8>(st, c, ha, hb, m, n, k);
}
