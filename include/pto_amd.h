/*
 * pto_amd.h -- C ABI of the MI355X (gfx950) back end for the PTO tile compute path.
 *
 * Every entry point is stream-ordered and asynchronous, takes raw device pointers owned by the
 * caller and allocates nothing.  `stream` is a hipStream_t passed as void* (NULL = default stream),
 * like the `void *stream` of the reference's launch wrappers.  Return value: PTO_OK, or a negative
 * PTO_ERR_* code; nothing is launched when an error is returned.
 *
 * Reference interfaces these replace (cannmirror/pto-isa, file:line):
 *   pto_gemm_f16f32      LaunchGEMME2E<T>(uint8_t *out, uint8_t *src0, uint8_t *src1, void *stream)
 *                        kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp:243-264, and the
 *                        ctypes entry call_kernel(blockDim, stream, out, src0, src1) demos/torch_jit/gemm/gemm_kernel.cpp:259-262
 *   pto_gemm_mxfp8       LaunchMxMatmul(uint8_t *out, uint8_t *src0, uint8_t *src1, uint8_t *src2, uint8_t *src3, void *stream)
 *                        kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp:344-364
 *   pto_quant_mxfp8_f32  TQUANT<QuantType::MXFP8>(dst, src, &exp, &max, &scaling) include/pto/common/pto_instr.hpp:1481-1490,
 *                        include/pto/npu/a5/TQuant.hpp:262-322, as launched by runTQuant<rows, cols, 0>
 *                        tests/npu/a5/src/st/testcase/tquant/tquant_kernel.cpp:27-80 (TLOAD -> TQUANT -> TSTORE of both outputs)
 *   pto_topk_f32         launchTopk<float>(uint8_t *out, uint8_t *index, uint8_t *src, uint8_t *inIdx, void *stream)
 *                        kernels/manual/a2a3/topk/topk_kernel.cpp:334-345
 *   pto_mla_attention_*  mla_pto(q, k, v, wq, wk, wv, wo, out) demos/cpu/mla_attention_demo/mla_attention_demo.cpp:227-397
 *   pto_fa_fwd_f16       LaunchTFA<...>(...) kernels/manual/common/flash_atten/fa_performance_kernel.h:28-41 and
 *                        call_kernel(...) demos/torch_jit/flash_atten/fa_kernel.cpp:1017-1092
 *   pto_tcvt_*           runTCVT / launchTCVT tests/cpu/st/testcase/tcvt/tcvt_kernel.cpp:18-66 (TLOAD -> TCVT -> TSTORE)
 *   pto_gather_rows      MGATHER include/pto/common/pto_instr.hpp:1328-1334 with idx[i,j] = idx[i]*cols + j
 *                        (test kernels tests/cpu/st/testcase/mgather/, tgather/tgather_kernel.cpp:224-)
 */
#ifndef PTO_AMD_H
#define PTO_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTO_OK 0
#define PTO_ERR_BAD_ARG (-1)     /* null pointer, non-positive extent, unknown enum value */
#define PTO_ERR_UNSUPPORTED (-2) /* shape not a multiple of the tile the kernel is built for */
#define PTO_ERR_HIP (-3)         /* the HIP runtime refused the launch; see pto_last_hip_error() */
#define PTO_ERR_WORKSPACE (-4)   /* workspace missing or too small */

/* rounding modes of TCVT: values of pto::RoundMode (include/pto/common/type.hpp:167-176) */
#define PTO_CAST_RINT 1
#define PTO_CAST_ROUND 2
#define PTO_CAST_FLOOR 3
#define PTO_CAST_CEIL 4
#define PTO_CAST_TRUNC 5
#define PTO_CAST_ODD 6

/* Library / device checks: 0 when a gfx950 device is current and usable. */
int pto_init(void);
const char *pto_version(void);
/* hipError_t of the last failing HIP call made by this library on the calling thread (0 = none) */
int pto_last_hip_error(void);

/* C[m,n] fp32 row-major = A[m,k] fp16 row-major x B, where B is stored [n,k] fp16 (a column-major
 * k x n operand), fp32 accumulation.  Accepted extents: m % 128 == 0, n % 256 == 0, k % 32 == 0 (multiples of the
 * 128 x 256 block of the reference kernel), or any m >= 192 and n >= 128 with n % 4 == 0 and k % 128 == 0 (256- or 192-row
 * tiles whose last row / column of tiles is moved back to end with the matrix).  Anything else: PTO_ERR_UNSUPPORTED. */
int pto_gemm_f16f32(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k);

/* MXFP8 GEMM: C[m,n] row-major = (A .* 2^(scale_a - 127)) x (B .* 2^(scale_b - 127)) with fp32 accumulation.
 * a [m,k] and b stored [n,k] (a column-major k x n operand) hold 8-bit floats: format 0 = e4m3 (OCP, no infinities),
 * 1 = e5m2 for both operands; 2 = a in e4m3 and b in e5m2, 3 = a in e5m2 and b in e4m3 (the matrix instruction takes a
 * format per operand).  scale_a [m,k/32] and scale_b stored [n,k/32] hold one e8m0 exponent per row
 * (column) and 32 consecutive k (the reference's x1_gm / x2_gm / x1_scale_gm / x2_scale_gm files).  c: bf16
 * (c_fp32 == 0, round-to-nearest-even of the fp32 sum) or fp32.  m >= 256, n >= 256 (any value: the last tile row /
 * column is moved back to end at m / n and recomputes what it overlaps; also 128 <= n < 256 when n % 4 == 0),
 * k % 512 == 0. */
int pto_gemm_mxfp8(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a, const uint8_t *scale_b,
                   int m, int n, int k, int format, int c_fp32);

/* MXFP4 GEMM: as pto_gemm_mxfp8 with 4-bit e2m1 operands packed two per byte, element 2i in bits 0-3 (the reference's
 * pack_two_fp4): a [m,k/2] bytes, b stored [n,k/2] bytes (LaunchMxMatmul of
 * kernels/manual/a5/matmul_mxfp4_performance/mxmatmul_performance_kernel.cpp).  Same limits (128 <= n < 256 only
 * when k % 1024 == 0 as well). */
int pto_gemm_mxfp4(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a, const uint8_t *scale_b,
                   int m, int n, int k, int c_fp32);

/* MXFP8 quantisation: src [rows, cols] fp32 contiguous, cols % 32 == 0 -> q [rows, cols] float8_e4m3fn bytes and
 * scale [rows, cols / 32] e8m0 bytes, one per 32 consecutive elements of a row: the operand and scale layout that
 * pto_gemm_mxfp8 takes for A (rows = m, cols = k) and for B stored [n, k].  Per group: E = biased fp32 exponent of the
 * largest |x|, scale byte = E - 8, q = e4m3(clip(x * 2^(127 - scale byte), +-448)) rounded to nearest even, so that the
 * group's largest element lands in [256, 448].  Groups holding an infinity or a NaN: scale byte 0xff, NaN -> NaN (0x7f
 * with the sign), +-inf -> +-448, finite -> +-0.  Groups whose largest |x| is below 2^-119 (all zeros included): scale
 * byte 0, factor 2^127.  src aligned to 16 bytes, q to 4 (else PTO_ERR_UNSUPPORTED). */
int pto_quant_mxfp8_f32(void *stream, uint8_t *q, uint8_t *scale, const float *src, size_t rows, size_t cols);

/* Row-wise top-k.  src [rows, ld] fp32, the first valid_cols columns of every row are scored; in_idx [valid_cols] uint32
 * gives the index reported for a column (the reference passes 0, 1, 2, ...).  Per row the (score, index) pairs are put in
 * descending order of score, equal scores (-0 == +0) in ascending order of index, and the first topk are written:
 * out_score [rows, topk] fp32 (the source bit patterns), out_index [rows, topk] uint32.  valid_cols <= 4096,
 * topk <= valid_cols <= ld.  NaN scores are ordered by their bit patterns (positive NaNs first, negative ones last). */
int pto_topk_f32(void *stream, float *out_score, uint32_t *out_index, const float *src, const uint32_t *in_idx, int rows,
                 int valid_cols, int ld, int topk);

/* Multi-latent attention of the reference's Auto-mode demo (demos/cpu/mla_attention_demo/mla_attention_demo.cpp:227-397,
 * mla_pto(q, k, v, wq, wk, wv, wo, out)) at the demo's sizes: 64 positions, head dim 32, latent dim 16, fp32.
 * q, k, v, out [batch, heads, 64, 32]; wq, wk, wv [32, 16]; wo [16, 32], all contiguous.  Per (batch, head):
 * out = (softmax((q wq) (k wk)^T / 4) (v wv)) wo, one workgroup each, every intermediate a tile. */
int pto_mla_attention_f32_s64_d32_r16(void *stream, float *out, const float *q, const float *k, const float *v, const float *wq,
                                      const float *wk, const float *wv, const float *wo, int batch, int heads);

/* Whole-tile attention of the reference's Auto-mode demo and tflashattn system test
 * (demos/cpu/flash_attention_demo/flash_attention_demo.cpp:169-258, flash_attention_pto(q, k, v, out)): fp32,
 * out = softmax(q k^T / sqrt(head_dim)) v per (batch, head), scores as one [seq, seq] tile, one workgroup per head.
 * q, k, v, out [batch, heads, seq, head_dim] contiguous; (seq, head_dim) = (64, 32) (the demo's) or (128, 64). */
int pto_attention_auto_f32(void *stream, float *out, const float *q, const float *k, const float *v, int batch, int heads, int seq,
                           int head_dim);

/* Flash-attention forward.  q [batch, heads, seq_q, head_dim], k and v [batch, heads, seq_kv, head_dim],
 * fp16, contiguous.  o: fp16 (o_fp32 == 0) or fp32 (o_fp32 != 0) [batch, heads, seq_q, head_dim];
 * lse: NULL or fp32 [batch, heads, seq_q] = max*scale + ln(sum).  scale = 1/sqrt(head_dim) is applied
 * to (x - max) as in the reference's softmax stage (pto_macro_fa_softmax.hpp:82-97).  causal == 1:
 * key j is visible to query i iff j <= i + (seq_kv - seq_q) (the diagonal ends in the last key); seq_kv >= seq_q is
 * required then.  causal == 2: iff j <= i (the diagonal starts in the first key: the rule of the reference's kernel,
 * fa_performance_kernel.cpp:298-299, :757, and of its generator, scripts/gen_data.py:53), any seq_kv.  The two agree
 * when seq_kv == seq_q.
 * head_dim in {64, 128}; seq_q % 128 == 0, seq_kv % 64 == 0.  No workspace: scores and probabilities
 * never leave the compute unit (the reference's caller-provided GM FIFOs have no counterpart). */
int pto_fa_fwd_f16(void *stream, void *o, float *lse, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                   int batch, int heads, int seq_q, int seq_kv, int head_dim, int causal, int o_fp32);

/* Elementwise conversion of n contiguous fp32 values (TLOAD -> TCVT -> TSTORE over 1 x 8192 tiles).
 * fp16: any PTO_CAST_* mode (PTO_CAST_RINT = IEEE round-to-nearest-even).  bf16: PTO_CAST_RINT only.
 * NaN inputs give a quiet NaN that keeps the sign and the top payload bits. */
int pto_tcvt_f32_f16(void *stream, uint16_t *dst, const float *src, size_t n, int round_mode);
int pto_tcvt_f32_bf16(void *stream, uint16_t *dst, const float *src, size_t n, int round_mode);

/* out[i, :] = table[idx[i], :] for i < n_idx; rows whose index is outside [0, table_rows) are zero.
 * elem_bytes in {2, 4}; cols % 8 == 0.  table [table_rows, cols] and out [n_idx, cols] contiguous. */
int pto_gather_rows(void *stream, void *out, const void *table, const int32_t *idx, size_t n_idx,
                    size_t table_rows, size_t cols, int elem_bytes);

/* TGATHER index form on one tile pair (tests/cpu/st/testcase/tgather): dst[r,c] = src0.flat[idx[r,c]],
 * out-of-range -> 0.  src0 [16,1024] fp16, idx and dst [16,128]. */
int pto_tgather_index_f16_16x1024_16x128(void *stream, uint16_t *dst, const uint16_t *src0, const int32_t *idx);

#ifdef __cplusplus
}
#endif
#endif /* PTO_AMD_H */
