/* Test-only entry points of libpto_st.so: single-tile PTO programs and the tuning hooks of the kernels.
 *
 * libpto_st.so is built from the sources of libpto_amd.so plus csrc/pto_optest.hip with PTO_ST_HOOKS defined.  It is what
 * the parity tests load to drive single instructions and single kernel variants through a C ABI; it is not part of the
 * product boundary (include/pto_amd.h, libpto_amd.so), and nothing in the product links or loads it.  Conventions
 * (device pointers, stream, return codes) are those of pto_amd.h. */
#ifndef PTO_AMD_ST_H
#define PTO_AMD_ST_H
#include "pto_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- tuning hooks: one kernel variant each, whatever the dispatch of the public entry point would pick -------------
 * PTO_ERR_UNSUPPORTED where the variant has no tiling for the shape, PTO_ERR_BAD_ARG for an unknown variant. */
/* the 128 x 256 / 256 x 256 block kernels on 32 x 32 x 16 MFMAs: tiling and pipeline depth by number (csrc/pto_gemm.hip) */
int pto_gemm_f16f32_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k, int variant);
/* four wavefronts, K-steps of 64, A in a ring per wave: 0 = 256 x 256 tiles, 1 = 256 x 192, 2 = 256 x 128, 3 = 192 x 256,
 * 4 = 192 x 192, 5 = 192 x 128 (csrc/pto_gemm_w4.hip) */
int pto_gemm_f16f32_w4_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k, int variant);
/* MX GEMM: variant 0 .. 3: bit 0 = quarter tiles in the last round, bit 1 = the shallower copy pipeline (csrc/pto_gemm_mx.hip);
 * fp8 formats only: 4 = the four-wave kernel with the width its estimate picks, 5 = its 256 x 192 tiles, 6 = 256 x 128
 * (csrc/pto_gemm_mxw4.hip) */
int pto_gemm_mxfp8_variant(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a,
                           const uint8_t *scale_b, int m, int n, int k, int format, int c_fp32, int variant);
/* flash attention: workgroup size, occupancy, queries per wave and MFMA shape by number (csrc/pto_fa.hip: 1 / 2 / 5 = four
 * waves at 1 / 2 / 3 workgroups per compute unit, 6 = key tiles of 32, 8 = 64 queries per wave, 10 / 20 / 21 = eight waves on
 * 32 x 32 x 16 / 16 x 16 x 32 MFMAs / the latter with fp32 output); causal != 0: the diagonal ends in the last key */
int pto_fa_fwd_f16_variant(void *stream, void *o, float *lse, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           int batch, int heads, int seq_q, int seq_kv, int head_dim, int causal, int variant);

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

/* Matmul instructions on ragged tiles: [m, k] x [k, n] (both row-major in memory) with valid m, k, n inside tiles rounded
 * up to 16 rows and 32 bytes, through TLOAD -> TFILLPAD -> TMOV / TEXTRACT -> TMATMUL / TMATMUL_ACC / TMATMUL_BIAS / TGEMV ->
 * TSTORE, as tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:26-97 and tests/npu/a2a3/src/st/testcase/tmatmul/
 * tmatmul_kernel.cpp:113-197 of the reference build them.  case_id selects element types, extents and form (the table in
 * tests/matmul_any_cases.py); the bias forms store twice the result (once through a Bias tile loaded by TMOV from L1, once
 * through one loaded by TLOAD, added together). */
int pto_st_matmul_ragged(void *stream, void *out, const void *a, const void *b, const void *bias, int case_id);

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
/* The same with a bias row [128] fp32 added: the first k half through the bias form of TMATMUL_MX (a [1, n] Bias tile;
 * pto_instr.hpp:444-451 of the reference), the second through the accumulating form.  Scales from registers. */
/* TQUANT<QuantType::MXFP8> on one Vec tile: TLOAD -> TQUANT -> TSTORE, the ND-mode program of the reference's test
 * (tests/npu/a5/src/st/testcase/tquant/tquant_kernel.cpp:27-80).  shape 0..3 = 32 x 32, 32 x 64, 64 x 128, 128 x 128 (its ND
 * cases); src [valid_rows, valid_cols] contiguous, elements outside it count as zeros.  out_fp8 [R, C] bytes, out_e8m0 and
 * out_max [R * C / 32], out_scaling [R, C] floats of which the first R * C / 32 are the groups' factors. */
int pto_st_tquant_mxfp8(void *stream, uint8_t *out_e8m0, uint8_t *out_fp8, float *out_max, float *out_scaling, const float *src,
                        int shape, int valid_rows, int valid_cols);
int pto_st_matmul_mx_bias_128x256x128(void *stream, float *out, const uint8_t *a, const uint8_t *b_t, const uint8_t *scale_a,
                                      const uint8_t *scale_b_t, const float *bias, int format_a, int format_b);

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
/* TSORT32 (pto_instr.hpp:786-798, cpu/TSort32.hpp) on an [8,128] tile of fp32 (dtype 0), int32 (1), fp16 (2) or int16 (3)
 * scores with uint32 indices and the valid region [valid_rows, valid_cols]: out [8,256] (4-byte scores) or [8,512] (2-byte
 * scores) is read, every group of 32 valid columns of a row is written back as 8-byte structures -- (score, index bit
 * pattern), or (score, 0, index & 0xffff, index >> 16) for 2-byte scores -- in descending order of score, equal scores in
 * ascending order of index, and the rest of out is left as it was. */
int pto_st_tsort32_8x128(void *stream, void *out, const void *src, const uint32_t *idx, int valid_rows, int valid_cols, int dtype);
/* TMRGSORT with one source (pto_instr.hpp:616-622, cpu/TMrgSort.hpp:181-230) on [1,1024] fp32 tiles: every complete
 * group of four sorted blocks of block_len elements (block_len / 2 structures) inside the first valid_cols columns is
 * merged; out is read first and keeps its other elements. */
int pto_st_tmrgsort_blocks_f32_1x1024(void *stream, float *out, const float *src, int valid_cols, int block_len);
/* the same on [1,2048] tiles of 2-byte elements, four to a structure with the score first (block_len / 4 structures a block):
 * dtype 0 = fp16, 1 = uint16, 2 = int16 scores (the reference's own cases use uint16: tests/cpu/st/testcase/tmrgsort/main.cpp:276-324) */
int pto_st_tmrgsort_blocks_16_1x2048(void *stream, void *out, const void *src, int valid_cols, int block_len, int dtype);
/* TMRGSORT with 2..4 lists (pto_instr.hpp:582-614, cpu/TMrgSort.hpp:118-178): src_i [256] fp32 hold cols_i / 2 sorted
 * (score, index) structures; the merge fills the first out_cols columns of out [1024] (read first), stops early when
 * exhausted != 0 and a list runs empty, and reports in executed[4] how many structures of each list it took. */
int pto_st_tmrgsort_lists_f32(void *stream, float *out, uint32_t *executed, const float *src0, const float *src1, const float *src2,
                              const float *src3, int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted);
/* the same with lists of 2-byte elements: src_i [512] hold cols_i / 4 structures, out [2048]; dtype 0 = fp16, 1 = uint16 */
int pto_st_tmrgsort_lists_16(void *stream, void *out, uint32_t *executed, const void *src0, const void *src1, const void *src2,
                             const void *src3, int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted, int dtype);
/* TMOV Vec -> Left / Right, Acc -> Left and TTRANS (the operand moves of the Auto-mode programs, cpu/TMov.hpp,
 * cpu/TTrans.hpp): a [64,64], b [64,128] fp16 row-major are loaded as Vec tiles and moved into operand tiles;
 * mid [64,128] = a b (fp32); out [64,64] = half(mid) b^T, with b^T made by TTRANS and half(mid) by the Acc -> Left move. */
int pto_st_matmul_vec_operands_f16_64x64x128(void *stream, float *out, float *mid, const uint16_t *a, const uint16_t *b);
/* TTRANS on fp32: out [128,64] = in [64,128] transposed. */
int pto_st_ttrans_f32_64x128(void *stream, float *out, const float *in);
/* TPREFETCH of an int32 [16,64] matrix into a tile, TPACK to int16 (out16) and on to int8 (out8): the low bits of every
 * element (npu/a5/TPack.hpp:21-72); print != 0: TPRINT of a [4,16] tile with a [3,10] valid region and of a [2,4] view of
 * the input, in the reference's format (npu/a2a3/TPrint.hpp:44-190), on the process's standard output. */
int pto_st_prefetch_pack_print_s32_16x64(void *stream, int16_t *out16, int8_t *out8, const int32_t *in, int print);
int pto_st_matmul_tmov_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, int relu, float scale);

/* Two-stage pipeline through TPUSH / TPOP FIFOs (common/fifo.hpp, cpu/TPush.hpp, cpu/TPop.hpp; the hand-offs of
 * fa_performance_kernel.cpp:346-583): out[64,64] = sum_t fp16(0.25 (a b[t])) v[t], t in {0,1}.  a [64,64] fp16;
 * b_t [2][128][64] (each b[t] column-major 64 x 128); v_t [2][64][128] (each v[t] column-major 128 x 64).
 * The score tile goes accumulator -> FIFO -> Vec tile through qk_fifo (2 x 64 x 128 fp32 of global memory) or, with
 * lds_fifo != 0, through an LDS FIFO (qk_fifo unused); the probability tile goes Vec -> FIFO -> Mat tile through
 * p_fifo (2 x 64 x 128 fp16 of global memory). */
int pto_st_pushpop_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, const uint16_t *v_t,
                                 float *qk_fifo, uint16_t *p_fifo, int lds_fifo);

/* The guard of TASSIGN against walking a Mat tile over a larger one by `data() + k * bytes` (pto_macro_matmul.hpp:176-177
 * of the reference does so over an L1 panel; an LDS image is swizzled row-major, a part of it is not a tile).  One
 * workgroup makes `chunks` (1 or 2) such TASSIGNs: flags[0] = 1 once it has started, flags[1] = 1 once it has reached
 * its end, which it does for one chunk only; with two it prints a "[PTO][RT] TASSIGN" line and ends at the second. */
int pto_st_mat_view_walk(void *stream, uint32_t *flags, int chunks);

#ifdef __cplusplus
}
#endif
#endif /* PTO_AMD_ST_H */
