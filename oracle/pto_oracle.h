/*
 * CPU oracle for the PTO tile compute path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference's CPU-simulation back-end
 * (cannmirror/pto-isa, include/pto/cpu/ and the flash-attention macros) for the
 * ops on the accelerated path.  It exists so that the HIP kernels can be checked
 * against the reference's arithmetic; it is never linked into or called from the
 * shipped library.  Only tests, the smoke check and the benchmark's CPU-baseline
 * leg may load it.
 *
 * Every function names the reference file:line it follows.  fp16 values are
 * carried as uint16_t bit patterns so that gcc 11 (no _Float16 on x86) builds it.
 *
 * Pinning status (what each function is checked against, besides the GPU path):
 *   po_tile_offset, po_tload, po_tstore, po_textract(mode 0), po_tmov,
 *   po_tmatmul_*, po_tcvt_f32_f16, po_tgather_*, po_mgather, po_fa_auto_f32:
 *       bit-for-bit against the compiled reference headers (oracle/_ref) and
 *       against closed forms / numpy in tests/.
 *   po_textract(mode 1, ISA sub-window): the reference CPU simulation does not
 *       implement it; pinned by brute force against the ISA definition
 *       dst[i,j] = src[r0+i, c0+j] (docs/isa/TEXTRACT.md:14-18).
 *   po_tcvt_f32_bf16: parity unpinned against the reference (its bfloat16_t
 *       aliases _Float16 with this toolchain, include/pto/common/type.hpp:259-268);
 *       pinned by the IEEE round-to-nearest-even closed form and torch's
 *       float32->bfloat16 conversion.
 *   po_fa_stream_f16: restates the manual kernel's macros, which the reference
 *       cannot run on a CPU; pinned against an fp64 dense softmax(QK^T s)V and
 *       the streaming invariants (tiling invariance, rows of P sum to S).
 */
#ifndef PTO_ORACLE_H
#define PTO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- tile layouts (include/pto/common/pto_tile.hpp:1201-1410) ---- */
enum { PO_BL_ROW = 0, PO_BL_COL = 1 };            /* BLayout  (memory.hpp:32-36) */
enum { PO_SL_NONE = 0, PO_SL_ROW = 1, PO_SL_COL = 2 }; /* SLayout (memory.hpp:38-43) */

typedef struct {
    int32_t rows, cols;       /* static tile shape */
    int32_t blayout;          /* PO_BL_* */
    int32_t slayout;          /* PO_SL_* */
    int32_t inner_rows, inner_cols;
} po_layout;

/* inner box shape rule: pto_tile.hpp:1209-1233 (512 B A/B fractal, 1024 B acc fractal) */
po_layout po_make_layout(int rows, int cols, int blayout, int slayout, int elem_bytes, int fractal_bytes);
/* element offset into linear tile storage: cpu/tile_offsets.hpp:19-60 == pto_tile.hpp:1522-1552 */
size_t po_tile_offset(const po_layout *L, size_t r, size_t c);

/* ---- data movement ---- */
/* cpu/TLoad.hpp:143-162 (+ :74-141). shape/stride are the 5-D GlobalTensor dims.
 * pad = pointer to one element used to pre-fill the tile (getPadValue, :19-40).
 * Returns 0, or -1 where the reference asserts. */
int po_tload(void *tile, const po_layout *L, int esz, const void *gm, const int64_t shape[5],
             const int64_t stride[5], int valid_row, int valid_col, const void *pad);
/* cpu/TStore.hpp:121-150 (+ :20-119) */
int po_tstore(void *gm, const int64_t shape[5], const int64_t stride[5], const void *tile, const po_layout *L,
              int esz, int valid_row, int valid_col);
/* mode 0: cpu/TExtract.hpp:17-50 (suffix window, asserts src.valid-idx==dst.valid);
 * mode 1: ISA sub-window docs/isa/TEXTRACT.md:14-18 (bounds per npu/a2a3/TExtract.hpp:537-548). */
int po_textract(void *dst, const po_layout *Ld, int dvr, int dvc, const void *src, const po_layout *Ls, int svr,
                int svc, int esz, int idx_row, int idx_col, int mode);
/* cpu/TMov.hpp:20-51; relu!=0 applies the NormalRelu clamp for fp32 (:53-70) */
int po_tmov(void *dst, const po_layout *Ld, const void *src, const po_layout *Ls, int esz, int valid_row,
            int valid_col);

/* ---- matmul: cpu/TMatmul.hpp:18-38, 73-116.  acc may be NULL (TMATMUL) or the
 * input accumulator tile (TMATMUL_ACC).  Sequential fp32 accumulation over k,
 * then acc + partial.  threads<=0 picks the online core count (cpu/parallel.hpp:41-51). */
void po_tmatmul_f16(float *dst, const float *acc, const po_layout *Lc, const uint16_t *a, const po_layout *La,
                    const uint16_t *b, const po_layout *Lb, int M, int N, int K, int threads);
void po_tmatmul_f32(float *dst, const float *acc, const po_layout *Lc, const float *a, const po_layout *La,
                    const float *b, const po_layout *Lb, int M, int N, int K, int threads);
void po_tmatmul_s8(int32_t *dst, const int32_t *acc, const po_layout *Lc, const int8_t *a, const po_layout *La,
                   const int8_t *b, const po_layout *Lb, int M, int N, int K, int threads);
/* TMATMUL_BIAS: cpu/TMatmul.hpp:98-116 (bias is a 1 x N row-major fp32 tile) */
void po_tmatmul_bias_f16(float *dst, const po_layout *Lc, const uint16_t *a, const po_layout *La, const uint16_t *b,
                         const po_layout *Lb, const float *bias, int M, int N, int K, int threads);

/* Whole-GEMM restatement of kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp:67-230:
 * C[m,n] fp32 row-major = A[m,k] fp16 row-major x B stored [n,k] fp16 (column-major k x n);
 * per base_m x base_n output block one TMATMUL (first k-step) then TMATMUL_ACC per base_k step.
 * rows [row0,row1) of C only (row1<=0 means m). */
void po_gemm_f16f32(float *C, const uint16_t *A, const uint16_t *B, int m, int n, int k, int base_k, int row0,
                    int row1, int threads);

/* MX matmul (TMATMUL_MX over a whole problem), as the reference's data generators define it
 * (tests/npu/a5/src/st/testcase/tmatmul_mx/gen_data.py:130-171, kernels/manual/a5/matmul_mxfp8_performance/scripts/gen_data.py:31-50):
 * x1[i,kk] = fp8(A[i,kk]) * 2^(SA[i,kk/32] - 127), x2[kk,j] = fp8(B[j,kk]) * 2^(SB[j,kk/32] - 127),
 * C = matmul in float64 -> float32.  A [m,k], B stored [n,k], SA [m,k/32], SB stored [n,k/32] (the generator's
 * transposed x2 / x2_scale files).  format: 0 = float8_e4m3fn, 1 = float8_e5m2 (ml_dtypes' names), 4 = float4_e2m1
 * packed two per byte, element 2i in the low nibble (pack_two_fp4, tmatmul_mx/gen_data.py:74-84; the operand then has
 * k/2 bytes per row). */
float po_fp8_e4m3fn_to_f32(uint8_t v);
uint8_t po_f32_to_fp8_e4m3fn(float x);
void po_quant_mxfp8_e4m3(uint8_t *q, uint8_t *e8m0, float *amax_out, float *scale_out, const float *src, size_t n);
float po_fp8_e5m2_to_f32(uint8_t v);
float po_fp4_e2m1_to_f32(uint8_t nibble);
void po_mx_gemm(float *C, const uint8_t *A, const uint8_t *B, const uint8_t *SA, const uint8_t *SB, int m, int n, int k,
                int format_a, int format_b, int threads);

/* Row-wise top-k as kernels/manual/a2a3/topk computes it: per row the (score, index) pairs (index = in_idx[column]) in
 * the order of the TSORT32 / TMRGSORT comparator (cpu/TSort32.hpp:32-41, 64-72: score descending, equal scores by
 * ascending index; stable), the first topk scores and indices written (golden: scripts/gen_data.py:55-64,
 * np.lexsort((idx, -row))[:topk]).  src [rows, ld] with valid_cols <= ld used per row. */
void po_topk_f32(float *out_score, uint32_t *out_index, const float *src, const uint32_t *in_idx, int rows, int valid_cols,
                 int ld, int topk);

/* ---- conversion: cpu/TCvt.hpp:65-84 ---- */
uint16_t po_f32_to_f16_rne(uint32_t bits); /* == static_cast<_Float16>(float) */
uint16_t po_f32_to_bf16_rne(uint32_t bits);
float po_f16_to_f32(uint16_t h);
void po_tcvt_f32_f16(uint16_t *dst, const float *src, size_t n);
void po_tcvt_f32_bf16(uint16_t *dst, const float *src, size_t n);
void po_tcvt_f16_f32(float *dst, const uint16_t *src, size_t n);
/* float -> int32 with a RoundMode (type.hpp:167-176), cpu/TCvt.hpp:28-63, 76-78 */
void po_tcvt_f32_s32(int32_t *dst, const float *src, size_t n, int round_mode);
/* fp32 -> fp16 round-to-nearest, ties away from zero (RoundMode::CAST_ROUND as the NPU
 * implements it, npu/a2a3/TCvt.hpp:82-111); used by the streaming flash-attention P cast. */
uint16_t po_f32_to_f16_rna(uint32_t bits);

/* ---- gather ---- */
/* index form cpu/TGather.hpp:68-100: dst[r,c] = src0.flat[idx[r,c]], out of range -> 0 */
void po_tgather_index(void *dst, const po_layout *Ld, const void *src0, const po_layout *L0, const int32_t *idx,
                      const po_layout *L1, int esz, int valid_row, int valid_col);
/* mask form cpu/TGather.hpp:102-129; pattern = MaskPattern value 1..7 (type.hpp:96-106).
 * Returns the number of elements written. */
size_t po_tgather_mask(void *dst, const po_layout *Ld, const void *src, const po_layout *Ls, int esz, int valid_row,
                       int valid_col, int pattern);
/* cpu/MGatherScatter.hpp:21-44: dst[i,j] = gm[idx[i,j]] */
void po_mgather(void *dst, const po_layout *Ld, const void *gm, const int32_t *idx, const po_layout *Li, int esz,
                int valid_row, int valid_col);
/* Row gather of config "TGATHER of int32 row indices": out[i,:] = table[idx[i],:], i.e. MGATHER with
 * idx[i,j] = idx[i]*cols + j.  Rows with idx outside [0,table_rows) are zero (TGather.hpp:78-81). */
void po_gather_rows(void *out, const void *table, const int32_t *idx, size_t n_idx, size_t table_rows, size_t cols,
                    int esz);

/* ---- fp32 vector ops on plain row-major tiles (ld = tile Cols) ---- */
void po_trowmax(float *dst, int dst_ld, const float *src, int ld, int rows, int cols);    /* cpu/TRowMax.hpp:20-59 */
void po_trowsum(float *dst, int dst_ld, const float *src, int ld, int rows, int cols);    /* cpu/TRowSum.hpp:17-39 */
void po_texp(float *dst, const float *src, int ld, int rows, int cols);                   /* cpu/TExp.hpp:22-60 (exp in double) */
void po_ttri(float *dst, int ld, int rows, int cols, int upper, int diagonal);            /* cpu/TTRI.hpp:31-76 */

/* ---- attention ---- */
/* Auto-Mode attention of tests/cpu/st/testcase/tflashattn/tflashattn_kernel.cpp:84-105:
 * fp32 q,k,v [S,D] -> out [S,D].  scores scaled before the max; exp in double. */
void po_fa_auto_f32(float *out, const float *q, const float *k, const float *v, int S, int D, int threads);

/* Streaming FA-2 forward for one head, following kernels/manual/common/flash_atten/
 * pto_macro_fa_softmax.hpp:47-215, pto_macro_fa_gu.hpp:33-56 and fa_performance_kernel.cpp:278-605:
 * fp16 q [S0,D], k,v [S1,D]; per tile_s1 key tile: X = q k^T (fp32), running max/sum with the scale
 * 1/sqrt(D) applied after the subtraction, P cast to fp16 (round_away!=0: ties away, else RNE),
 * O = O*alpha + P v, final O /= sum.  causal: keys j > q_offset+i get -3.40282e38 added on the
 * diagonal tile and later tiles are skipped.  Outputs: o fp32 [S0,D]; row_max / row_sum [S0]
 * (either may be NULL).  LSE = row_max/sqrt(D) + ln(row_sum). */
void po_fa_stream_f16(float *o, float *row_max, float *row_sum, const uint16_t *q, const uint16_t *k,
                      const uint16_t *v, int S0, int S1, int D, int tile_s1, int causal, int q_offset,
                      int round_away, int threads);

/* ResultCmp of tests/common/test_common.h:211-301: returns 1 on pass */
int po_result_cmp_f32(const float *expect, const float *actual, size_t n, float eps, double *max_diff,
                      size_t *n_bad);

int po_online_cpus(void);


/* ---- further Vec instructions (plain row-major fp32 arrays, leading dimension ld) ----
 * Parity: pinned against the compiled reference (oracle/_ref, tests/test_oracle_vec_ext.py) and against numpy
 * closed forms.  op codes are the PTO_VOP_* values of include/pto_amd.h. */
void po_vec_op(float *dst, const float *a, const float *b, const float *vec, float scalar, int op, int ld, int rows,
               int cols); /* cpu/ElementOp.h:77-535, TAbs.hpp, TSqrt.hpp, TRSqrt.hpp, TRowExpandOp.hpp:36-96, TColExpandOp.hpp, TSelS.hpp */
/* op 0 TROWMAX, 1 TROWMIN, 2 TROWSUM (dst[rows]); 3 TCOLMAX, 4 TCOLMIN, 5 TCOLSUM (dst[cols]); sequential order */
void po_reduce(float *dst, const float *a, int ld, int rows, int cols, int op); /* cpu/TRowMax.hpp, TRowMin.hpp, TRowSum.hpp, TColMax.hpp:22-35, TColMin.hpp, TColSum.hpp:22-31 */
/* packed compare with a scalar: bit c%8 of dst[r*dst_ld + c/8]; mode 0..5 = EQ NE LT LE GT GE; EQ / NE within 1e-9 */
void po_tcmps_packed(uint8_t *dst, int dst_ld, const float *a, int ld, int rows, int cols, float scalar, int mode); /* cpu/TCmps.hpp:24-90 */
/* dst = bit ? a : b, bits consumed in running order over [rows, cols], bytes along mask_valid_cols then the next mask row */
void po_tsel_packed(float *dst, const uint8_t *mask, int mask_ld, int mask_valid_cols, const float *a, const float *b,
                    int ld, int rows, int cols); /* cpu/TSel.hpp:22-49 */
/* dst[rows, cols] = a inside [vr, vc], pad elsewhere; pad_kind 1 zero, 2 +inf, 3 -inf */
void po_tfillpad(float *dst, const float *a, int ld, int rows, int cols, int vr, int vc, int pad_kind); /* cpu/TFillPad.hpp:22-49 */
/* same-shape move with optional clamp at zero */
void po_tmov_relu(float *dst, const float *src, size_t n, int relu); /* cpu/TMov.hpp:53-69 */

#ifdef __cplusplus
}
#endif
#endif
