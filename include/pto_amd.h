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
 * k x n operand), fp32 accumulation.  m % 128 == 0, n % 256 == 0, k % 32 == 0 (multiples of the
 * 128 x 256 block of the reference kernel; C is tiled 256 x 256 when m allows it). */
int pto_gemm_f16f32(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k);

/* MXFP8 GEMM: C[m,n] row-major = (A .* 2^(scale_a - 127)) x (B .* 2^(scale_b - 127)) with fp32 accumulation.
 * a [m,k] and b stored [n,k] (a column-major k x n operand) hold 8-bit floats: format 0 = e4m3 (OCP, no infinities),
 * 1 = e5m2, the same for both operands.  scale_a [m,k/32] and scale_b stored [n,k/32] hold one e8m0 exponent per row
 * (column) and 32 consecutive k (the reference's x1_gm / x2_gm / x1_scale_gm / x2_scale_gm files).  c: bf16
 * (c_fp32 == 0, round-to-nearest-even of the fp32 sum) or fp32.  m >= 256, n >= 256 (any value: the last tile row /
 * column is moved back to end at m / n and recomputes what it overlaps), k % 512 == 0. */
int pto_gemm_mxfp8(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a, const uint8_t *scale_b,
                   int m, int n, int k, int format, int c_fp32);

/* MXFP4 GEMM: as pto_gemm_mxfp8 with 4-bit e2m1 operands packed two per byte, element 2i in bits 0-3 (the reference's
 * pack_two_fp4): a [m,k/2] bytes, b stored [n,k/2] bytes (LaunchMxMatmul of
 * kernels/manual/a5/matmul_mxfp4_performance/mxmatmul_performance_kernel.cpp).  Same limits. */
int pto_gemm_mxfp4(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a, const uint8_t *scale_b,
                   int m, int n, int k, int c_fp32);

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

/* ---- single-tile instruction programs -------------------------------------------------------
 * One workgroup runs a short PTO program on one or a few tiles: the counterparts of the reference's
 * per-instruction system-test kernels (tests/cpu/st/testcase/<op>/<op>_kernel.cpp), here so that
 * every instruction of the path can be driven through the C ABI. */

/* One streaming-softmax step on a [64,256] fp32 score tile (pto_macro_fa_softmax.hpp:82-97, 141-183).
 * first != 0: max = rowmax(x), p = exp(scale (x - max)), sum = rowsum(p), alpha = 1.
 * first == 0: max' = max(max_in, rowmax x), alpha = exp(scale (max_in - max')), p = exp(scale (x - max')),
 *             sum' = alpha sum_in + rowsum(p).   x_exp = fp16(p) under round_mode.  Vectors are [64] fp32. */
int pto_st_softmax_step_f32_64x256(void *stream, uint16_t *x_exp, float *max_out, float *sum_out, float *alpha_out,
                                   const float *x, const float *max_in, const float *sum_in, float scale, int first,
                                   int round_mode);
/* Rescale-accumulate step on [64,128] fp32 tiles (pto_macro_fa_gu.hpp:33-56): o = o_prev alpha + pv; last: o /= sum. */
int pto_st_gu_step_f32_64x128(void *stream, float *o_out, const float *o_prev, const float *pv, const float *alpha,
                              const float *sum, int last);
/* out = x + tri(diagonal) * value on a [64,128] fp32 tile; upper != 0: TTRI upper form (cpu/TTRI.hpp:31-63). */
int pto_st_tri_mask_f32_64x128(void *stream, float *out, const float *x, int diagonal, float value, int upper);
/* TGATHER mask form on a [16,64] tile of 16-bit elements -> [16, 64/div] (tgather_kernel.cpp:18-42); pattern 1..7. */
int pto_st_tgather_mask_b16_16x64(void *stream, uint16_t *out, const uint16_t *src, int pattern);
/* MGATHER element form: out[8,128] = gm[idx[8,128]] (tests/cpu/st/testcase/mgather). */
int pto_st_mgather_b16_8x128(void *stream, uint16_t *out, const uint16_t *gm, const int32_t *idx, int gm_elems);
/* TLOAD of a [10,20] fp32 region into a [16,32] tile with PadValue::Max; the whole tile image comes back
 * (tload/main.cpp:138-183, PADMAX case). */
int pto_st_tload_pad_f32_16x32(void *stream, float *image, const float *gm);
/* TLOAD of the 5-D view shape [1,2,3,4,8], strides [1000,400,100,10,1] into a [24,8] tile; TSTORE to a dense
 * [24,8] buffer and back through the same 5-D strides (tload/ and tstore/ 5-D cases). */
int pto_st_tload_5d_f32(void *stream, float *dense, float *strided, const float *gm);
/* TEXTRACT windows (docs/isa/TEXTRACT.md:14-18): out_left[128,256] = a[:, col0:col0+64] x eye,
 * out_right[128,256] = eye x b[row0:row0+64, :].  a [128,256] fp16 row-major; b_t [256][256] (column-major b);
 * eye_b [256][64] column-major 64 x 256 with eye(k,n) = (k == n); eye_a [128,64] with eye(r,k) = (r == k). */
int pto_st_textract_windows_f16(void *stream, float *out_left, float *out_right, const uint16_t *a, const uint16_t *b_t,
                                const uint16_t *eye_b, const uint16_t *eye_a, int col0, int row0);
/* [128,64] x [64,256] (+ bias[256], may be NULL) with fp16 (bf16 == 0) or bf16 operands, stages ordered by Event
 * objects (tmatmul_kernel.cpp:26-99 with isBias; docs/coding/Event.md). */
int pto_st_matmul_bias_128x64x256(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, const float *bias,
                                  int bf16);

/* [128,128] x [128,256] int8 -> int32 and [128,32] x [32,256] fp32 -> fp32 (the other operand types of TMATMUL,
 * include/pto/cpu/TMatmul.hpp:46-51; tests/cpu/st/testcase/tmatmul/gen_data.py:92-99): a row-major, b_t = b stored
 * [256][K] (column-major b); K in two halves, TMATMUL then TMATMUL_ACC.  relu != 0: stored with
 * TSTORE<..., ReluPreMode::NormalRelu, STPhase::Final> (negative results become 0). */
int pto_st_matmul_s8_128x128x256(void *stream, int32_t *out, const int8_t *a, const int8_t *b_t, int relu);
int pto_st_matmul_f32_128x32x256(void *stream, float *out, const float *a, const float *b_t, int relu);

/* MX matmul [128,256] x [256,128] -> fp32 [128,128]: a [128,256] and b_t [128][256] (column-major b) fp8 bytes in
 * format_a / format_b (0 = e4m3, 1 = e5m2; they may differ), scale_a [128,8] and scale_b_t [128][8] e8m0 bytes; K in two
 * halves, TMATMUL_MX then its accumulating form (tests/npu/a5/src/st/testcase/tmatmul_mx/tmatmul_mx_kernel.cpp).
 * scales_via_lds != 0: the scales are TLOADed into Mat tiles and TEXTRACTed from there (as the reference stages them in
 * L1) instead of being loaded from memory into scale tiles directly. */
int pto_st_matmul_mx_128x256x128(void *stream, float *out, const uint8_t *a, const uint8_t *b_t, const uint8_t *scale_a,
                                 const uint8_t *scale_b_t, int format_a, int format_b, int scales_via_lds);

/* One Vec instruction on [64,128] fp32 tiles: out = OP(a [, b | scalar | vec]).  vec is a per-row [64] operand for
 * the TROWEXPAND* ops and a per-column [128] operand for the TCOLEXPAND* ops.  op codes (PTO_VOP_*): unary
 * (cpu/TAbs.hpp, TSqrt.hpp, TRSqrt.hpp, ElementOp.h:273-350), binary incl. TPRELU and TCMP with 0/1 results
 * (ElementTileOp.h:170-238), scalar incl. TLRELU (ElementTileScalarOp.h), TSELS (scalar = select mode, TSelS.hpp),
 * row broadcasts (TRowExpand.hpp, TRowExpandOp.hpp:57-96), column broadcasts (TColExpand.hpp, TColExpandOp.hpp). */
enum {
    PTO_VOP_ABS = 0, PTO_VOP_NEG, PTO_VOP_RELU, PTO_VOP_SQRT, PTO_VOP_RSQRT, PTO_VOP_LOG, PTO_VOP_RECIP, PTO_VOP_EXP,
    PTO_VOP_ADD = 20, PTO_VOP_SUB, PTO_VOP_MUL, PTO_VOP_DIV, PTO_VOP_MAX, PTO_VOP_MIN, PTO_VOP_PRELU,
    PTO_VOP_CMP_EQ, PTO_VOP_CMP_NE, PTO_VOP_CMP_LT, PTO_VOP_CMP_LE, PTO_VOP_CMP_GT, PTO_VOP_CMP_GE, PTO_VOP_SELS,
    PTO_VOP_ADDS = 40, PTO_VOP_SUBS, PTO_VOP_MULS, PTO_VOP_DIVS, PTO_VOP_MAXS, PTO_VOP_MINS, PTO_VOP_LRELU,
    PTO_VOP_ROWEXPAND = 60, PTO_VOP_ROWEXPANDSUB, PTO_VOP_ROWEXPANDMUL, PTO_VOP_ROWEXPANDDIV, PTO_VOP_ROWEXPANDADD,
    PTO_VOP_ROWEXPANDMAX, PTO_VOP_ROWEXPANDMIN, PTO_VOP_ROWEXPANDEXPDIF,
    PTO_VOP_COLEXPAND = 80, PTO_VOP_COLEXPANDSUB, PTO_VOP_COLEXPANDMUL, PTO_VOP_COLEXPANDDIV, PTO_VOP_COLEXPANDADD,
    PTO_VOP_COLEXPANDMAX, PTO_VOP_COLEXPANDMIN, PTO_VOP_COLEXPANDEXPDIF
};
int pto_st_vec_op_f32_64x128(void *stream, float *out, const float *a, const float *b, const float *vec, float scalar, int op);
/* The arithmetic subset of the same (ABS NEG RELU, ADD SUB MUL MAX MIN, ADDS SUBS MULS MAXS MINS, the row / column
 * expand forms without the divisions) on [64,128] fp16 (dtype 0) or int32 (dtype 1) tiles; same operation codes. */
int pto_st_vec_op_typed_64x128(void *stream, void *out, const void *a, const void *b, const void *vec, float scalar, int op,
                               int dtype);
/* Bitwise, shift, remainder and three-operand Vec instructions on [64,128] tiles (pto_instr.hpp TAND TOR TXOR TSHL TSHR
 * TREM TNOT, TANDS TORS TXORS TSHLS TSHRS TREMS, TADDC TSUBC TADDSC TSUBSC; element rules cpu/ElementOp.h:145-198,
 * 305-310, 365-378, 425-470).  op: 0 AND, 1 OR, 2 XOR, 3 SHL, 4 SHR, 5 REM, 6 NOT, 7..12 the scalar forms of 0..5,
 * 13 ADDC (a + b + c), 14 SUBC (a - b + c), 15 ADDSC (a + scalar + c), 16 SUBSC (a - scalar + c).
 * dtype 1: int32 tiles, scalar_i (every op); dtype 0: fp32 tiles, scalar_f (REM, REMS and the three-operand ops).
 * a, b and c are always read. */
int pto_st_vec_bitop_64x128(void *stream, void *out, const void *a, const void *b, const void *c, float scalar_f, int scalar_i,
                            int op, int dtype);
/* Reductions over the valid region [valid_rows, valid_cols] of a [64,128] fp32 tile (row stride 128 in memory):
 * op 0 TROWMAX, 1 TROWMIN, 2 TROWSUM -> out[valid_rows]; 3 TCOLMAX, 4 TCOLMIN, 5 TCOLSUM -> out[valid_cols]
 * (cpu/TRowMax.hpp, TRowMin.hpp, TRowSum.hpp, TColMax.hpp, TColMin.hpp, TColSum.hpp). */
int pto_st_reduce_f32_64x128(void *stream, float *out, const float *a, int valid_rows, int valid_cols, int op);
/* TCMPS then TSEL on [64,128] fp32 tiles: bits[64][16] = packed (a <cmp_mode> scalar), bit c%8 of byte c/8
 * (cpu/TCmps.hpp:50-90; EQ / NE within 1e-9); sel = bit ? a : b (cpu/TSel.hpp:22-49).  cmp_mode 0..5 = EQ NE LT LE GT GE. */
int pto_st_cmps_sel_f32_64x128(void *stream, float *sel, uint8_t *bits, const float *a, const float *b, float scalar,
                               int cmp_mode);
/* TFILLPAD: out[64,128] = a inside [valid_rows, valid_cols], the pad value elsewhere; pad_kind 1 zero, 2 +inf, 3 -inf
 * (cpu/TFillPad.hpp:22-49). */
int pto_st_fillpad_f32_64x128(void *stream, float *out, const float *a, int valid_rows, int valid_cols, int pad_kind);
/* out[64,128] = scale * (relu ? max(a b, 0) : a b): fp16 matmul [64,64] x [64,128] (b_t stored [128][64]), TMOV of
 * the accumulator into a Vec tile with ReluPreMode (cpu/TMov.hpp:53-69), TMULS, TSTORE. */
/* TPARTADD (op 0), TPARTMAX (1), TPARTMIN (2) on [64,128] fp32 tiles (cpu/TPartOp.hpp:19-45): over the destination's valid
 * region, op(a, b) where both sources are valid, the valid source's element where one is, 0 where none is; out is read
 * first and keeps its elements outside the destination's valid region. */
int pto_st_tpart_f32_64x128(void *stream, float *out, const float *a, const float *b, int op, int dst_valid_rows, int dst_valid_cols,
                            int a_valid_rows, int a_valid_cols, int b_valid_rows, int b_valid_cols);
/* TSCATTER (to_memory 0; cpu/TScatter.hpp:21-44): out [64,128] is read, out[idx[i,j], j] = src[i,j] for the source's valid
 * region [valid_rows, valid_cols] (several rows to one place: the last row wins; rows outside 0..63 are dropped), the rest
 * of out keeps its values.  MSCATTER (to_memory != 0; cpu/MGatherScatter.hpp:46-69): out[idx[i,j]] = src[i,j] with out as
 * plain memory of 64 x 128 elements; THE CALLER guarantees 0 <= idx < 8192 there (distinct indices for a defined result). */
int pto_st_scatter_f32_64x128(void *stream, float *out, const float *src, const int32_t *idx, int valid_rows, int valid_cols,
                              int to_memory);
/* TGATHERB (pto_instr.hpp:1152-1158, cpu/TGatherB.hpp:21-60): out [16,128] fp32 is read; every 32-byte block (r, c) of its
 * valid region [valid_rows, valid_cols] (valid_cols % 8 == 0) becomes the 32 bytes of the [32,64] fp32 source tile's
 * row-major storage that start at byte offsets[r, c] ([16,16] uint32, any alignment); a block whose source range leaves
 * the 8192 bytes of the tile keeps its values. */
int pto_st_tgatherb_f32_16x128(void *stream, float *out, const float *src, const uint32_t *offsets, int valid_rows, int valid_cols);
/* TCI (pto_instr.hpp:808-814, cpu/TCI.hpp): out [1024] int32 is read, out[j] = start + j (descending: start - j) for
 * j < valid_cols, the rest keeps its values. */
int pto_st_tci_s32_1x1024(void *stream, int32_t *out, int32_t start, int descending, int valid_cols);
/* TSORT32 (pto_instr.hpp:786-798, cpu/TSort32.hpp) on an [8,128] tile of fp32 (dtype 0) or int32 (dtype 1) scores with
 * uint32 indices and the valid region [valid_rows, valid_cols]: out [8,256] is read, every group of 32 valid columns
 * of a row is written back as (score, index bit pattern) structures in descending order of score, equal scores in
 * ascending order of index, and the rest of out is left as it was. */
int pto_st_tsort32_8x128(void *stream, void *out, const void *src, const uint32_t *idx, int valid_rows, int valid_cols, int dtype);
/* TMRGSORT with one source (pto_instr.hpp:616-622, cpu/TMrgSort.hpp:181-230) on [1,1024] fp32 tiles: every complete
 * group of four sorted blocks of block_len elements (block_len / 2 structures) inside the first valid_cols columns is
 * merged; out is read first and keeps its other elements. */
int pto_st_tmrgsort_blocks_f32_1x1024(void *stream, float *out, const float *src, int valid_cols, int block_len);
/* TMRGSORT with 2..4 lists (pto_instr.hpp:582-614, cpu/TMrgSort.hpp:118-178): src_i [256] fp32 hold cols_i / 2 sorted
 * (score, index) structures; the merge fills the first out_cols columns of out [1024] (read first), stops early when
 * exhausted != 0 and a list runs empty, and reports in executed[4] how many structures of each list it took. */
int pto_st_tmrgsort_lists_f32(void *stream, float *out, uint32_t *executed, const float *src0, const float *src1, const float *src2,
                              const float *src3, int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted);
/* TMOV Vec -> Left / Right, Acc -> Left and TTRANS (the operand moves of the Auto-mode programs, cpu/TMov.hpp,
 * cpu/TTrans.hpp): a [64,64], b [64,128] fp16 row-major are loaded as Vec tiles and moved into operand tiles;
 * mid [64,128] = a b (fp32); out [64,64] = half(mid) b^T, with b^T made by TTRANS and half(mid) by the Acc -> Left move. */
int pto_st_matmul_vec_operands_f16_64x64x128(void *stream, float *out, float *mid, const uint16_t *a, const uint16_t *b);
/* TTRANS on fp32: out [128,64] = in [64,128] transposed. */
int pto_st_ttrans_f32_64x128(void *stream, float *out, const float *in);
int pto_st_matmul_tmov_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, int relu, float scale);

/* Two-stage pipeline through TPUSH / TPOP FIFOs (common/fifo.hpp, cpu/TPush.hpp, cpu/TPop.hpp; the hand-offs of
 * fa_performance_kernel.cpp:346-583): out[64,64] = sum_t fp16(0.25 (a b[t])) v[t], t in {0,1}.  a [64,64] fp16;
 * b_t [2][128][64] (each b[t] column-major 64 x 128); v_t [2][64][128] (each v[t] column-major 128 x 64).
 * The score tile goes accumulator -> FIFO -> Vec tile through qk_fifo (2 x 64 x 128 fp32 of global memory) or, with
 * lds_fifo != 0, through an LDS FIFO (qk_fifo unused); the probability tile goes Vec -> FIFO -> Mat tile through
 * p_fifo (2 x 64 x 128 fp16 of global memory). */
int pto_st_pushpop_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, const uint16_t *v_t,
                                 float *qk_fifo, uint16_t *p_fifo, int lds_fifo);

#ifdef __cplusplus
}
#endif
#endif /* PTO_AMD_H */
