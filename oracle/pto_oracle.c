/*
 * CPU oracle for the PTO tile compute path.  TEST INFRASTRUCTURE ONLY -- never
 * linked into the shipped library (see pto_oracle.h for the pinning status of
 * each function).  Reference = cannmirror/pto-isa; citations are file:line
 * relative to its root.
 */
#define _GNU_SOURCE
#include "pto_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ------------------------------------------------------------------ threads */
/* Row-parallel helper with the shape of cpu::parallel_for_1d
 * (include/pto/cpu/parallel.hpp:53-95): contiguous row chunks, one per thread. */
typedef void (*po_row_fn)(size_t row_begin, size_t row_end, void *ctx);
typedef struct {
    po_row_fn fn;
    void *ctx;
    size_t b, e;
} po_job;

static void *po_job_main(void *p)
{
    po_job *j = (po_job *)p;
    j->fn(j->b, j->e, j->ctx);
    return NULL;
}

int po_online_cpus(void)
{
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n > 0 ? (int)n : 1;
}

static void po_parallel_rows(size_t rows, int threads, po_row_fn fn, void *ctx)
{
    if (threads <= 0)
        threads = po_online_cpus();
    if ((size_t)threads > rows)
        threads = (int)(rows ? rows : 1);
    if (threads <= 1) {
        fn(0, rows, ctx);
        return;
    }
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    po_job *jobs = (po_job *)malloc(sizeof(po_job) * (size_t)threads);
    size_t chunk = (rows + (size_t)threads - 1) / (size_t)threads;
    int started = 0;
    for (int t = 0; t < threads; t++) {
        size_t b = (size_t)t * chunk, e = b + chunk;
        if (b >= rows)
            break;
        if (e > rows)
            e = rows;
        jobs[t].fn = fn;
        jobs[t].ctx = ctx;
        jobs[t].b = b;
        jobs[t].e = e;
        pthread_create(&tid[t], NULL, po_job_main, &jobs[t]);
        started++;
    }
    for (int t = 0; t < started; t++)
        pthread_join(tid[t], NULL);
    free(tid);
    free(jobs);
}

/* ------------------------------------------------------------------ layouts */
po_layout po_make_layout(int rows, int cols, int blayout, int slayout, int elem_bytes, int fractal_bytes)
{
    po_layout L;
    L.rows = rows;
    L.cols = cols;
    L.blayout = blayout;
    L.slayout = slayout;
    if (slayout == PO_SL_NONE) {
        L.inner_rows = 1;
        L.inner_cols = 1;
    } else if (fractal_bytes == 1024) { /* accumulator fractal: 16 x 16 */
        L.inner_rows = 16;
        L.inner_cols = 16;
    } else if (slayout == PO_SL_ROW) { /* 16 rows x 32 bytes */
        L.inner_rows = 16;
        L.inner_cols = 32 / elem_bytes;
    } else { /* 32 bytes x 16 cols */
        L.inner_rows = 32 / elem_bytes;
        L.inner_cols = 16;
    }
    return L;
}

size_t po_tile_offset(const po_layout *L, size_t r, size_t c)
{
    const size_t R = (size_t)L->rows, C = (size_t)L->cols;
    if (L->slayout == PO_SL_NONE)
        return L->blayout == PO_BL_ROW ? r * C + c : c * R + r;
    const size_t ir = (size_t)L->inner_rows, ic = (size_t)L->inner_cols;
    const size_t br = r / ir, rr = r % ir, bc = c / ic, cc = c % ic;
    if (L->blayout == PO_BL_COL && L->slayout == PO_SL_ROW) /* Nz */
        return bc * R * ic + br * ir * ic + rr * ic + cc;
    if (L->blayout == PO_BL_ROW && L->slayout == PO_SL_COL) /* Zn */
        return br * C * ir + bc * ir * ic + cc * ir + rr;
    if (L->blayout == PO_BL_ROW && L->slayout == PO_SL_ROW) /* Zz */
        return br * C * ir + bc * ir * ic + rr * ic + cc;
    return (size_t)-1; /* ColMajor + ColMajor box: the reference asserts */
}

/* ------------------------------------------------------------ data movement */
static inline void po_copy_elem(void *d, size_t di, const void *s, size_t si, int esz)
{
    memcpy((char *)d + di * (size_t)esz, (const char *)s + si * (size_t)esz, (size_t)esz);
}

static int po_gm_shape_ok(const po_layout *L, const int64_t sh[5], int vr, int vc)
{
    /* cpu/TLoad.hpp:148-149 == cpu/TStore.hpp:126-127 */
    const int row_major = L->blayout == PO_BL_ROW;
    if (row_major)
        return sh[0] * sh[1] * sh[2] * sh[3] == vr && sh[4] == vc;
    return sh[0] * sh[1] * sh[2] * sh[4] == vc && sh[3] == vr;
}

int po_tload(void *tile, const po_layout *L, int esz, const void *gm, const int64_t sh[5], const int64_t st[5],
             int valid_row, int valid_col, const void *pad)
{
    if (!po_gm_shape_ok(L, sh, valid_row, valid_col))
        return -1;
    const size_t numel = (size_t)L->rows * (size_t)L->cols;
    for (size_t i = 0; i < numel; i++) /* TLoad.hpp:151-152 */
        memcpy((char *)tile + i * (size_t)esz, pad, (size_t)esz);
    if (L->slayout != PO_SL_NONE) { /* TLoad.hpp:97-141: 2-D only */
        if (!(sh[0] == 1 && sh[1] == 1 && sh[2] == 1))
            return -1;
        for (int64_t c = 0; c < sh[4]; c++)
            for (int64_t r = 0; r < sh[3]; r++)
                po_copy_elem(tile, po_tile_offset(L, (size_t)r, (size_t)c), gm, (size_t)(r * st[3] + c * st[4]), esz);
        return 0;
    }
    /* plain: outer three dims are stacked along the tile's major axis (TLoad.hpp:42-95) */
    const int row_major = L->blayout == PO_BL_ROW;
    for (int64_t i = 0; i < sh[0]; i++)
        for (int64_t j = 0; j < sh[1]; j++)
            for (int64_t k = 0; k < sh[2]; k++) {
                const size_t slab = (size_t)((i * sh[1] + j) * sh[2] + k);
                const size_t gbase = (size_t)(i * st[0] + j * st[1] + k * st[2]);
                for (int64_t r = 0; r < sh[3]; r++)
                    for (int64_t c = 0; c < sh[4]; c++) {
                        size_t t = row_major ? (slab * (size_t)sh[3] + (size_t)r) * (size_t)L->cols + (size_t)c :
                                               (slab * (size_t)sh[4] + (size_t)c) * (size_t)L->rows + (size_t)r;
                        po_copy_elem(tile, t, gm, gbase + (size_t)(r * st[3] + c * st[4]), esz);
                    }
            }
    return 0;
}

int po_tstore(void *gm, const int64_t sh[5], const int64_t st[5], const void *tile, const po_layout *L, int esz,
              int valid_row, int valid_col)
{
    if (!po_gm_shape_ok(L, sh, valid_row, valid_col))
        return -1;
    if (L->slayout != PO_SL_NONE) { /* TStore.hpp:75-119 */
        if (!(sh[0] == 1 && sh[1] == 1 && sh[2] == 1))
            return -1;
        for (int64_t c = 0; c < sh[4]; c++)
            for (int64_t r = 0; r < sh[3]; r++)
                po_copy_elem(gm, (size_t)(r * st[3] + c * st[4]), tile, po_tile_offset(L, (size_t)r, (size_t)c), esz);
        return 0;
    }
    const int row_major = L->blayout == PO_BL_ROW; /* TStore.hpp:20-73 */
    for (int64_t i = 0; i < sh[0]; i++)
        for (int64_t j = 0; j < sh[1]; j++)
            for (int64_t k = 0; k < sh[2]; k++) {
                const size_t slab = (size_t)((i * sh[1] + j) * sh[2] + k);
                const size_t gbase = (size_t)(i * st[0] + j * st[1] + k * st[2]);
                for (int64_t r = 0; r < sh[3]; r++)
                    for (int64_t c = 0; c < sh[4]; c++) {
                        size_t t = row_major ? (slab * (size_t)sh[3] + (size_t)r) * (size_t)L->cols + (size_t)c :
                                               (slab * (size_t)sh[4] + (size_t)c) * (size_t)L->rows + (size_t)r;
                        po_copy_elem(gm, gbase + (size_t)(r * st[3] + c * st[4]), tile, t, esz);
                    }
            }
    return 0;
}

int po_textract(void *dst, const po_layout *Ld, int dvr, int dvc, const void *src, const po_layout *Ls, int svr,
                int svc, int esz, int idx_row, int idx_col, int mode)
{
    if (mode == 0) { /* TExtract.hpp:20: the CPU simulation only takes the suffix window */
        if (svr - idx_row != dvr || svc - idx_col != dvc)
            return -1;
    } else { /* a2a3/TExtract.hpp:540-543: window must lie inside the source */
        if (idx_row + dvr > Ls->rows || idx_col + dvc > Ls->cols)
            return -1;
    }
    for (int c = 0; c < dvc; c++)
        for (int r = 0; r < dvr; r++)
            po_copy_elem(dst, po_tile_offset(Ld, (size_t)r, (size_t)c), src,
                         po_tile_offset(Ls, (size_t)(r + idx_row), (size_t)(c + idx_col)), esz);
    return 0;
}

int po_tmov(void *dst, const po_layout *Ld, const void *src, const po_layout *Ls, int esz, int valid_row,
            int valid_col)
{
    for (int c = 0; c < valid_col; c++)
        for (int r = 0; r < valid_row; r++)
            po_copy_elem(dst, po_tile_offset(Ld, (size_t)r, (size_t)c), src, po_tile_offset(Ls, (size_t)r, (size_t)c),
                         esz);
    return 0;
}

/* --------------------------------------------------------------- conversion */
float po_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff, bits;
    if (e == 0) {
        if (m == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int sh = 0;
            while (!(m & 0x400)) {
                m <<= 1;
                sh++;
            }
            m &= 0x3ff;
            bits = sign | ((uint32_t)(113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 112) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16; ties_away=0: round-to-nearest-even (what static_cast<_Float16>
 * does in cpu/TCvt.hpp:79-81); ties_away=1: round-half-away (CAST_ROUND on the NPU). */
static uint16_t po_f32_to_f16_impl(uint32_t x, int ties_away)
{
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t a = x & 0x7fffffffu;
    if (a > 0x7f800000u) /* NaN: quiet it, keep the top payload bits */
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
    if (a == 0x7f800000u)
        return (uint16_t)(sign | 0x7c00u);
    const uint32_t e = a >> 23;
    uint32_t h;
    if (e >= 113) { /* normal half range or overflow */
        if (e >= 143)
            return (uint16_t)(sign | 0x7c00u);
        uint32_t v = a - (112u << 23);
        uint32_t rem = v & 0x1fffu;
        h = v >> 13;
        if (rem > 0x1000u || (rem == 0x1000u && (ties_away || (h & 1u))))
            h++;
        if (h >= 0x7c00u)
            h = 0x7c00u;
    } else if (e >= 102) { /* result is subnormal (or rounds up to the smallest normal) */
        uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e; /* 14..24 */
        uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1u);
        h = m >> shift;
        if (rem > half || (rem == half && (ties_away || (h & 1u))))
            h++;
    } else {
        h = 0;
    }
    return (uint16_t)(sign | h);
}

uint16_t po_f32_to_f16_rne(uint32_t bits) { return po_f32_to_f16_impl(bits, 0); }
uint16_t po_f32_to_f16_rna(uint32_t bits) { return po_f32_to_f16_impl(bits, 1); }

uint16_t po_f32_to_bf16_rne(uint32_t u)
{
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((u >> 16) | 0x0040u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

void po_tcvt_f32_f16(uint16_t *dst, const float *src, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        uint32_t b;
        memcpy(&b, &src[i], 4);
        dst[i] = po_f32_to_f16_rne(b);
    }
}

void po_tcvt_f32_bf16(uint16_t *dst, const float *src, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        uint32_t b;
        memcpy(&b, &src[i], 4);
        dst[i] = po_f32_to_bf16_rne(b);
    }
}

void po_tcvt_f16_f32(float *dst, const uint16_t *src, size_t n)
{
    for (size_t i = 0; i < n; i++)
        dst[i] = po_f16_to_f32(src[i]);
}

static double po_round_integral(double v, int mode)
{ /* cpu/TCvt.hpp:28-63 */
    switch (mode) {
    case 1:
        return rint(v);
    case 2:
        return round(v);
    case 3:
        return floor(v);
    case 4:
        return ceil(v);
    case 5:
        return trunc(v);
    case 6: {
        double f = floor(v), frac = v - f;
        if (frac > 0.5)
            return f + 1;
        if (frac < 0.5)
            return f;
        return (((long long)f) & 1) ? f : f + 1;
    }
    default:
        return v;
    }
}

void po_tcvt_f32_s32(int32_t *dst, const float *src, size_t n, int round_mode)
{
    for (size_t i = 0; i < n; i++)
        dst[i] = (int32_t)po_round_integral((double)src[i], round_mode);
}

/* ------------------------------------------------------------------- matmul */
typedef struct {
    void *dst;
    const void *acc;
    const po_layout *Lc, *La, *Lb;
    const void *a, *b;
    int N, K;
    const float *bias;
} po_mm_ctx;

static void po_mm_f16_rows(size_t r0, size_t r1, void *p)
{
    po_mm_ctx *c = (po_mm_ctx *)p;
    const uint16_t *a = (const uint16_t *)c->a, *b = (const uint16_t *)c->b;
    float *dst = (float *)c->dst;
    const float *acc = (const float *)c->acc;
    /* widen the row of A once; products of two halves are exact in fp32 */
    float *arow = (float *)malloc(sizeof(float) * (size_t)c->K);
    for (size_t i = r0; i < r1; i++) {
        for (int k = 0; k < c->K; k++)
            arow[k] = po_f16_to_f32(a[po_tile_offset(c->La, i, (size_t)k)]);
        for (int j = 0; j < c->N; j++) {
            float s = 0.0f;
            for (int k = 0; k < c->K; k++) {
                float prod = arow[k] * po_f16_to_f32(b[po_tile_offset(c->Lb, (size_t)k, (size_t)j)]);
                s = s + prod; /* sequential in k: cpu/TMatmul.hpp:27-32 */
            }
            size_t d = po_tile_offset(c->Lc, i, (size_t)j);
            dst[d] = acc ? acc[d] + s : s; /* cpu/TMatmul.hpp:35 */
        }
    }
    free(arow);
}

static void po_mm_f32_rows(size_t r0, size_t r1, void *p)
{
    po_mm_ctx *c = (po_mm_ctx *)p;
    const float *a = (const float *)c->a, *b = (const float *)c->b;
    float *dst = (float *)c->dst;
    const float *acc = (const float *)c->acc;
    for (size_t i = r0; i < r1; i++)
        for (int j = 0; j < c->N; j++) {
            volatile float s = 0.0f; /* volatile: keep mul and add separately rounded (no fma contraction) */
            for (int k = 0; k < c->K; k++) {
                volatile float prod =
                    a[po_tile_offset(c->La, i, (size_t)k)] * b[po_tile_offset(c->Lb, (size_t)k, (size_t)j)];
                s = s + prod;
            }
            size_t d = po_tile_offset(c->Lc, i, (size_t)j);
            dst[d] = acc ? acc[d] + s : s;
        }
}

static void po_mm_s8_rows(size_t r0, size_t r1, void *p)
{
    po_mm_ctx *c = (po_mm_ctx *)p;
    const int8_t *a = (const int8_t *)c->a, *b = (const int8_t *)c->b;
    int32_t *dst = (int32_t *)c->dst;
    const int32_t *acc = (const int32_t *)c->acc;
    for (size_t i = r0; i < r1; i++)
        for (int j = 0; j < c->N; j++) {
            int32_t s = 0;
            for (int k = 0; k < c->K; k++)
                s += (int32_t)a[po_tile_offset(c->La, i, (size_t)k)] *
                     (int32_t)b[po_tile_offset(c->Lb, (size_t)k, (size_t)j)];
            size_t d = po_tile_offset(c->Lc, i, (size_t)j);
            dst[d] = acc ? acc[d] + s : s;
        }
}

void po_tmatmul_f16(float *dst, const float *acc, const po_layout *Lc, const uint16_t *a, const po_layout *La,
                    const uint16_t *b, const po_layout *Lb, int M, int N, int K, int threads)
{
    po_mm_ctx c = {dst, acc, Lc, La, Lb, a, b, N, K, NULL};
    po_parallel_rows((size_t)M, threads, po_mm_f16_rows, &c);
}

void po_tmatmul_f32(float *dst, const float *acc, const po_layout *Lc, const float *a, const po_layout *La,
                    const float *b, const po_layout *Lb, int M, int N, int K, int threads)
{
    po_mm_ctx c = {dst, acc, Lc, La, Lb, a, b, N, K, NULL};
    po_parallel_rows((size_t)M, threads, po_mm_f32_rows, &c);
}

void po_tmatmul_s8(int32_t *dst, const int32_t *acc, const po_layout *Lc, const int8_t *a, const po_layout *La,
                   const int8_t *b, const po_layout *Lb, int M, int N, int K, int threads)
{
    po_mm_ctx c = {dst, acc, Lc, La, Lb, a, b, N, K, NULL};
    po_parallel_rows((size_t)M, threads, po_mm_s8_rows, &c);
}

void po_tmatmul_bias_f16(float *dst, const po_layout *Lc, const uint16_t *a, const po_layout *La, const uint16_t *b,
                         const po_layout *Lb, const float *bias, int M, int N, int K, int threads)
{
    po_tmatmul_f16(dst, NULL, Lc, a, La, b, Lb, M, N, K, threads);
    for (int c = 0; c < N; c++) /* cpu/TMatmul.hpp:109-115 */
        for (int r = 0; r < M; r++)
            dst[po_tile_offset(Lc, (size_t)r, (size_t)c)] += bias[c];
}

typedef struct {
    float *C;
    const uint16_t *A;
    const float *Bf; /* B widened to fp32 once, [n,k] */
    int n, k, base_k;
} po_gemm_ctx;

static void po_gemm_rows(size_t r0, size_t r1, void *p)
{
    po_gemm_ctx *g = (po_gemm_ctx *)p;
    const int k = g->k, n = g->n, bk = g->base_k;
    float *arow = (float *)malloc(sizeof(float) * (size_t)k);
    for (size_t i = r0; i < r1; i++) {
        for (int kk = 0; kk < k; kk++)
            arow[kk] = po_f16_to_f32(g->A[i * (size_t)k + (size_t)kk]);
        for (int j = 0; j < n; j++) {
            const float *brow = g->Bf + (size_t)j * (size_t)k;
            float acc = 0.0f;
            for (int k0 = 0; k0 < k; k0 += bk) { /* one TMATMUL / TMATMUL_ACC per K-step */
                float s = 0.0f;
                const int k1 = k0 + bk < k ? k0 + bk : k;
                for (int kk = k0; kk < k1; kk++) {
                    float prod = arow[kk] * brow[kk];
                    s = s + prod;
                }
                acc = k0 == 0 ? s : acc + s; /* gemm_performance_kernel.cpp:28-35 */
            }
            g->C[i * (size_t)n + (size_t)j] = acc;
        }
    }
    free(arow);
}

static void po_gemm_rows_shift(size_t r0, size_t r1, void *p);
typedef struct {
    po_gemm_ctx g;
    size_t row0;
} po_gemm_shift;

static void po_gemm_rows_shift(size_t r0, size_t r1, void *p)
{
    po_gemm_shift *s = (po_gemm_shift *)p;
    po_gemm_rows(r0 + s->row0, r1 + s->row0, &s->g);
}

void po_gemm_f16f32(float *C, const uint16_t *A, const uint16_t *B, int m, int n, int k, int base_k, int row0,
                    int row1, int threads)
{
    if (row1 <= 0 || row1 > m)
        row1 = m;
    if (row0 < 0)
        row0 = 0;
    if (base_k <= 0)
        base_k = k;
    float *Bf = (float *)malloc(sizeof(float) * (size_t)n * (size_t)k);
    po_tcvt_f16_f32(Bf, B, (size_t)n * (size_t)k);
    po_gemm_shift s = {{C, A, Bf, n, k, base_k}, (size_t)row0};
    po_parallel_rows((size_t)(row1 - row0), threads, po_gemm_rows_shift, &s);
    free(Bf);
}

/* ------------------------------------------------------------------ MX GEMM */
/* float8_e4m3fn: 1-4-3, bias 7, no infinities, S.1111.111 = NaN; float8_e5m2: 1-5-2, bias 15, IEEE-style inf / NaN */
float po_fp8_e4m3fn_to_f32(uint8_t v)
{
    const int s = v >> 7, e = (v >> 3) & 0xf, f = v & 7;
    float r;
    if (e == 0xf && f == 7)
        r = NAN;
    else if (e == 0)
        r = ldexpf((float)f, -9); /* subnormal: f/8 * 2^-6 */
    else
        r = ldexpf((float)(8 + f), e - 10);
    return s ? -r : r;
}

float po_fp8_e5m2_to_f32(uint8_t v)
{
    const int s = v >> 7, e = (v >> 2) & 0x1f, f = v & 3;
    float r;
    if (e == 0x1f)
        r = f ? NAN : INFINITY;
    else if (e == 0)
        r = ldexpf((float)f, -16); /* subnormal: f/4 * 2^-14 */
    else
        r = ldexpf((float)(4 + f), e - 17);
    return s ? -r : r;
}

/* float4_e2m1: 1-2-1, bias 1, no infinities or NaNs: 0, 0.5 (subnormal), 1, 1.5, 2, 3, 4, 6 */
float po_fp4_e2m1_to_f32(uint8_t nibble)
{
    const int s = (nibble >> 3) & 1, e = (nibble >> 1) & 3, f = nibble & 1;
    const float r = e == 0 ? 0.5f * (float)f : ldexpf((float)(2 + f), e - 2);
    return s ? -r : r;
}

typedef struct {
    float *C;
    const double *A, *B; /* dequantised operands, A [m,k], B [n,k] */
    int n, k;
} po_mx_ctx;

static void po_mx_rows(size_t r0, size_t r1, void *ctx)
{
    const po_mx_ctx *g = (const po_mx_ctx *)ctx;
    for (size_t i = r0; i < r1; i++)
        for (int j = 0; j < g->n; j++) {
            const double *a = g->A + i * (size_t)g->k, *b = g->B + (size_t)j * (size_t)g->k;
            double acc = 0.0;
            for (int kk = 0; kk < g->k; kk++)
                acc += a[kk] * b[kk];
            g->C[i * (size_t)g->n + (size_t)j] = (float)acc;
        }
}

static double *po_mx_dequant(const uint8_t *X, const uint8_t *S, int rows, int k, int format)
{
    double *out = (double *)malloc(sizeof(double) * (size_t)rows * (size_t)k);
    const int kb = k / 32;
    for (int r = 0; r < rows; r++)
        for (int kk = 0; kk < k; kk++) {
            double e;
            if (format == 4) {
                const uint8_t pair = X[((size_t)r * (size_t)k + (size_t)kk) / 2];
                e = (double)po_fp4_e2m1_to_f32((uint8_t)((kk & 1) ? pair >> 4 : pair & 15));
            } else {
                const uint8_t v = X[(size_t)r * (size_t)k + (size_t)kk];
                e = format ? (double)po_fp8_e5m2_to_f32(v) : (double)po_fp8_e4m3fn_to_f32(v);
            }
            out[(size_t)r * (size_t)k + (size_t)kk] = e * ldexp(1.0, (int)S[(size_t)r * (size_t)kb + (size_t)(kk / 32)] - 127);
        }
    return out;
}

void po_mx_gemm(float *C, const uint8_t *A, const uint8_t *B, const uint8_t *SA, const uint8_t *SB, int m, int n, int k,
                int format_a, int format_b, int threads)
{
    double *Ad = po_mx_dequant(A, SA, m, k, format_a), *Bd = po_mx_dequant(B, SB, n, k, format_b);
    po_mx_ctx c = {C, Ad, Bd, n, k};
    po_parallel_rows((size_t)m, threads, po_mx_rows, &c);
    free(Ad);
    free(Bd);
}

/* ------------------------------------------------------------------ MXFP8 quantisation */
/* fp32 -> float8_e4m3fn, round to nearest even, magnitudes above 448 (infinities included) saturate to +-448, NaN ->
 * sign | 0x7f.  (The reference converts with ROUND_R, RS_ENABLE and the saturation control bit set:
 * include/pto/npu/a5/TQuant.hpp:198, :283; its generator clips to +-448 and casts to ml_dtypes float8_e4m3fn, which
 * rounds to nearest even: tests/npu/a5/src/st/testcase/tquant/gen_data.py:27-33.) */
uint8_t po_f32_to_fp8_e4m3fn(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u)
        return (uint8_t)(sign | 0x7fu);
    if (a >= 0x43e00000u) /* 448 and above */
        return (uint8_t)(sign | 0x7eu);
    const int e = (int)(a >> 23) - 127;
    if (e < -6) { /* below the smallest normal 2^-6: multiples of 2^-9; 8 of them is that normal's code */
        float mag;
        memcpy(&mag, &a, 4);
        return (uint8_t)(sign | (uint8_t)lrintf(mag * 512.0f)); /* exact product, nearest-even under the default mode */
    }
    uint32_t m = (a >> 20) & 7u, ex = (uint32_t)(e + 7);
    const uint32_t rem = a & 0xfffffu;
    if (rem > 0x80000u || (rem == 0x80000u && (m & 1u))) {
        if (++m == 8u) {
            m = 0;
            ++ex;
        }
    }
    uint32_t code = (ex << 3) | m;
    if (code > 0x7eu)
        code = 0x7eu;
    return (uint8_t)(sign | code);
}

/* Block-scaled quantisation of fp32 to MXFP8 (e4m3 elements, one e8m0 scale per 32 consecutive elements), the rule of
 * TQUANT<QuantType::MXFP8> (include/pto/npu/a5/TQuant.hpp:128-180 ExtractB8ExponentAndScaling, :182-203
 * CalcQuantizedFP8Values) and of its generator (gen_data.py:43-57 fp32_to_fp8_element, :27-33 scale_data):
 *   amax  = largest |x| of the group, E = its biased fp32 exponent
 *   e8m0  = E - 8                          (8 = exponent of the largest e4m3 binade: 448 = 1.75 * 2^8)
 *   scale = 2^(127 - e8m0)                 (fp32 bits (254 - e8m0) << 23), q = e4m3(clip(x * scale, +-448))
 * so that amax * scale lies in [256, 512).  Outside what the generator's data reaches:
 *   E == 255 (an infinity or NaN in the group): e8m0 = 0xff as the reference stores; elements: NaN -> NaN, +-inf -> +-448,
 *       finite -> +-0 (the reference multiplies by the bit pattern 0xff read as a float, 3.6e-43);
 *   E < 8 (amax < 2^-119, all-zero groups included): e8m0 = 0 as the reference stores, scale = 2^127.  (The reference
 *       kernel's clamp constant for this case is 0x7f800000, +inf as a factor, which turns a zero group into NaNs; its
 *       generator wraps the exponent to 248 and yields zeros.  2^127 is the scale that e8m0 = 0 stands for.)
 * q [n] bytes, e8m0 [n / 32] bytes, amax / scale [n / 32] floats or NULL; n a multiple of 32. */
void po_quant_mxfp8_e4m3(uint8_t *q, uint8_t *e8m0, float *amax_out, float *scale_out, const float *src, size_t n)
{
    for (size_t g = 0; g < n / 32; ++g) {
        const float *x = src + g * 32;
        uint32_t amax = 0;
        for (int i = 0; i < 32; ++i) {
            uint32_t u;
            memcpy(&u, &x[i], 4);
            u &= 0x7fffffffu;
            if (u > amax)
                amax = u; /* as integers: a NaN is above every number */
        }
        const uint32_t E = amax >> 23;
        uint32_t scale_bits;
        uint8_t se;
        if (E == 255u) {
            se = 0xffu;
            scale_bits = 0xffu;
        } else if (E < 8u) {
            se = 0;
            scale_bits = 254u << 23;
        } else {
            se = (uint8_t)(E - 8u);
            scale_bits = (254u - (E - 8u)) << 23;
        }
        float scale, am;
        memcpy(&scale, &scale_bits, 4);
        memcpy(&am, &amax, 4);
        e8m0[g] = se;
        if (amax_out)
            amax_out[g] = am;
        if (scale_out)
            scale_out[g] = scale;
        for (int i = 0; i < 32; ++i) {
            uint32_t u;
            memcpy(&u, &x[i], 4);
            if (E == 255u) {
                const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
                const uint32_t a = u & 0x7fffffffu;
                q[g * 32 + i] = (uint8_t)(sign | (a > 0x7f800000u ? 0x7fu : a == 0x7f800000u ? 0x7eu : 0u));
            } else {
                float y = x[i] * scale; /* a power of two: exact unless it underflows, far below the smallest e4m3 */
                if (y > 448.0f)
                    y = 448.0f;
                if (y < -448.0f)
                    y = -448.0f;
                q[g * 32 + i] = po_f32_to_fp8_e4m3fn(y);
            }
        }
    }
}

/* -------------------------------------------------------------------- top-k */
typedef struct {
    float score;
    uint32_t index;
    int pos;
} po_score_index;

static int po_score_index_cmp(const void *pa, const void *pb)
{ /* cpu/TSort32.hpp:64-72; the position keeps the sort stable */
    const po_score_index *a = (const po_score_index *)pa, *b = (const po_score_index *)pb;
    if (a->score != b->score)
        return a->score > b->score ? -1 : 1;
    if (a->index != b->index)
        return a->index < b->index ? -1 : 1;
    return a->pos < b->pos ? -1 : (a->pos > b->pos ? 1 : 0);
}

void po_topk_f32(float *out_score, uint32_t *out_index, const float *src, const uint32_t *in_idx, int rows, int valid_cols,
                 int ld, int topk)
{
    po_score_index *buf = (po_score_index *)malloc(sizeof(po_score_index) * (size_t)valid_cols);
    for (int r = 0; r < rows; r++) {
        for (int c = 0; c < valid_cols; c++) {
            buf[c].score = src[(size_t)r * (size_t)ld + (size_t)c];
            buf[c].index = in_idx[c];
            buf[c].pos = c;
        }
        qsort(buf, (size_t)valid_cols, sizeof(po_score_index), po_score_index_cmp);
        for (int c = 0; c < topk; c++) {
            out_score[(size_t)r * (size_t)topk + (size_t)c] = buf[c].score;
            out_index[(size_t)r * (size_t)topk + (size_t)c] = buf[c].index;
        }
    }
    free(buf);
}

/* ------------------------------------------------------------------- gather */
void po_tgather_index(void *dst, const po_layout *Ld, const void *src0, const po_layout *L0, const int32_t *idx,
                      const po_layout *L1, int esz, int valid_row, int valid_col)
{
    const size_t numel0 = (size_t)L0->rows * (size_t)L0->cols;
    const uint32_t zero = 0;
    for (int r = 0; r < valid_row; r++)
        for (int c = 0; c < valid_col; c++) {
            const int32_t raw = idx[po_tile_offset(L1, (size_t)r, (size_t)c)];
            const size_t d = po_tile_offset(Ld, (size_t)r, (size_t)c);
            if (raw < 0 || (size_t)raw >= numel0) { /* TGather.hpp:78-81 */
                memcpy((char *)dst + d * (size_t)esz, &zero, (size_t)esz);
                continue;
            }
            const size_t flat = (size_t)raw;
            po_copy_elem(dst, d, src0, po_tile_offset(L0, flat / (size_t)L0->cols, flat % (size_t)L0->cols), esz);
        }
}

static int po_mask_select(int pattern, unsigned c)
{ /* TGather.hpp:23-45 */
    switch (pattern) {
    case 1:
        return (c % 2u) == 0;
    case 2:
        return (c % 2u) == 1;
    case 3:
        return (c % 4u) == 0;
    case 4:
        return (c % 4u) == 1;
    case 5:
        return (c % 4u) == 2;
    case 6:
        return (c % 4u) == 3;
    default:
        return 1;
    }
}

size_t po_tgather_mask(void *dst, const po_layout *Ld, const void *src, const po_layout *Ls, int esz, int valid_row,
                       int valid_col, int pattern)
{
    size_t d = po_tile_offset(Ld, 0, 0), n = 0; /* running linear index: TGather.hpp:106-115 */
    for (int r = 0; r < valid_row; r++)
        for (int c = 0; c < valid_col; c++) {
            if (!po_mask_select(pattern, (unsigned)c))
                continue;
            po_copy_elem(dst, d, src, po_tile_offset(Ls, (size_t)r, (size_t)c), esz);
            d++;
            n++;
        }
    return n;
}

void po_mgather(void *dst, const po_layout *Ld, const void *gm, const int32_t *idx, const po_layout *Li, int esz,
                int valid_row, int valid_col)
{
    for (int i = 0; i < valid_row; i++)
        for (int j = 0; j < valid_col; j++)
            po_copy_elem(dst, po_tile_offset(Ld, (size_t)i, (size_t)j), gm,
                         (size_t)idx[po_tile_offset(Li, (size_t)i, (size_t)j)], esz);
}

void po_gather_rows(void *out, const void *table, const int32_t *idx, size_t n_idx, size_t table_rows, size_t cols,
                    int esz)
{
    const size_t row_bytes = cols * (size_t)esz;
    for (size_t i = 0; i < n_idx; i++) {
        char *o = (char *)out + i * row_bytes;
        if (idx[i] < 0 || (size_t)idx[i] >= table_rows)
            memset(o, 0, row_bytes);
        else
            memcpy(o, (const char *)table + (size_t)idx[i] * row_bytes, row_bytes);
    }
}

/* --------------------------------------------------------------- vector ops */
void po_trowmax(float *dst, int dst_ld, const float *src, int ld, int rows, int cols)
{
    for (int i = 0; i < rows; i++) {
        float m = src[(size_t)i * (size_t)ld];
        for (int j = 1; j < cols; j++) {
            float v = src[(size_t)i * (size_t)ld + (size_t)j];
            m = m < v ? v : m; /* std::max(max_val, v): TRowMax.hpp:31-33 */
        }
        dst[(size_t)i * (size_t)dst_ld] = m;
    }
}

void po_trowsum(float *dst, int dst_ld, const float *src, int ld, int rows, int cols)
{
    for (int i = 0; i < rows; i++) {
        float s = 0.0f;
        for (int j = 0; j < cols; j++)
            s += src[(size_t)i * (size_t)ld + (size_t)j];
        dst[(size_t)i * (size_t)dst_ld] = s;
    }
}

void po_texp(float *dst, const float *src, int ld, int rows, int cols)
{
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++) {
            size_t x = (size_t)i * (size_t)ld + (size_t)j;
            dst[x] = (float)exp((double)src[x]); /* TExp.hpp:36 */
        }
}

void po_ttri(float *dst, int ld, int rows, int cols, int upper, int diagonal)
{
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            int one = upper ? (c >= diagonal + r) : (c < diagonal + r + 1); /* TTRI.hpp:31-63 */
            dst[(size_t)r * (size_t)ld + (size_t)c] = one ? 1.0f : 0.0f;
        }
}

/* ---------------------------------------------------------------- attention */
typedef struct {
    float *out;
    const float *q, *k, *v;
    int S, D;
} po_fa_auto_ctx;

static void po_fa_auto_rows(size_t r0, size_t r1, void *p)
{
    po_fa_auto_ctx *c = (po_fa_auto_ctx *)p;
    const int S = c->S, D = c->D;
    const float scale = 1.0f / sqrtf((float)D); /* tflashattn_kernel.cpp:60 */
    float *sc = (float *)malloc(sizeof(float) * (size_t)S);
    for (size_t i = r0; i < r1; i++) {
        for (int j = 0; j < S; j++) { /* TMATMUL (fp32, sequential k) then TMULS */
            volatile float s = 0.0f;
            for (int d = 0; d < D; d++) {
                volatile float prod = c->q[i * (size_t)D + (size_t)d] * c->k[(size_t)j * (size_t)D + (size_t)d];
                s = s + prod;
            }
            sc[j] = s * scale;
        }
        float m = sc[0];
        for (int j = 1; j < S; j++)
            m = m < sc[j] ? sc[j] : m;
        float sum = 0.0f;
        for (int j = 0; j < S; j++) {
            sc[j] = (float)exp((double)(sc[j] - m));
            sum += sc[j];
        }
        for (int j = 0; j < S; j++)
            sc[j] = sc[j] / sum;
        for (int d = 0; d < D; d++) {
            volatile float s = 0.0f;
            for (int j = 0; j < S; j++) {
                volatile float prod = sc[j] * c->v[(size_t)j * (size_t)D + (size_t)d];
                s = s + prod;
            }
            c->out[i * (size_t)D + (size_t)d] = s;
        }
    }
    free(sc);
}

void po_fa_auto_f32(float *out, const float *q, const float *k, const float *v, int S, int D, int threads)
{
    po_fa_auto_ctx c = {out, q, k, v, S, D};
    po_parallel_rows((size_t)S, threads, po_fa_auto_rows, &c);
}

typedef struct {
    float *o, *row_max, *row_sum;
    const uint16_t *q;
    const float *kf, *vf; /* K and V widened to fp32 once */
    int S0, S1, D, tile_s1, causal, q_offset, round_away;
} po_fa_ctx;

static void po_fa_stream_rows(size_t r0, size_t r1, void *p)
{
    po_fa_ctx *c = (po_fa_ctx *)p;
    const int D = c->D, T = c->tile_s1;
    /* scale = 1/sqrt(HEAD) as a float constant: pto_macro_fa_softmax.hpp:32-46 (Newton sqrt in float) */
    float guess = (float)D;
    for (int it = 0; it < 8; it++)
        guess = 0.5f * (guess + (float)D / guess);
    const float scale = 1.0f / guess;
    float *x = (float *)malloc(sizeof(float) * (size_t)T);
    float *pf = (float *)malloc(sizeof(float) * (size_t)T);
    float *ph = (float *)malloc(sizeof(float) * (size_t)T);
    float *qrow = (float *)malloc(sizeof(float) * (size_t)D);
    float *orow = (float *)malloc(sizeof(float) * (size_t)D);
    for (size_t i = r0; i < r1; i++) {
        const int qpos = c->q_offset + (int)i;
        for (int d = 0; d < D; d++) {
            qrow[d] = po_f16_to_f32(c->q[i * (size_t)D + (size_t)d]);
            orow[d] = 0.0f;
        }
        float gmax = 0.0f, gsum = 0.0f;
        int first = 1;
        /* causal: only tiles up to the one holding the diagonal (fa_performance_kernel.cpp:757-758) */
        int ntiles = (c->S1 + T - 1) / T;
        if (c->causal) {
            int lim = qpos / T + 1;
            if (lim < ntiles)
                ntiles = lim;
        }
        for (int t = 0; t < ntiles; t++) {
            const int j0 = t * T, tn = (j0 + T <= c->S1) ? T : c->S1 - j0;
            for (int j = 0; j < tn; j++) { /* compute_qk: fp16 x fp16 -> fp32, sequential over d */
                float s = 0.0f;
                const float *kr = c->kf + (size_t)(j0 + j) * (size_t)D;
                for (int d = 0; d < D; d++) {
                    float prod = qrow[d] * kr[d];
                    s = s + prod;
                }
                if (c->causal && (j0 + j) > qpos) /* triu * -3.40282e38 added: pto_macro_fa_softmax.hpp:65-80 */
                    s = s + (-3.40282e+38f);
                x[j] = s;
            }
            float lmax = x[0];
            for (int j = 1; j < tn; j++)
                lmax = lmax < x[j] ? x[j] : lmax;
            float alpha = 1.0f;
            if (first) {
                gmax = lmax;
            } else { /* pto_macro_fa_softmax.hpp:141-160 */
                float nmax = lmax < gmax ? gmax : lmax;
                alpha = (float)exp((double)((gmax - nmax) * scale));
                gmax = nmax;
            }
            float lsum = 0.0f;
            for (int j = 0; j < tn; j++) {
                pf[j] = (float)exp((double)((x[j] - gmax) * scale));
                lsum += pf[j];
                uint32_t b;
                memcpy(&b, &pf[j], 4);
                ph[j] = po_f16_to_f32(c->round_away ? po_f32_to_f16_rna(b) : po_f32_to_f16_rne(b));
            }
            gsum = first ? lsum : alpha * gsum + lsum;
            for (int d = 0; d < D; d++) { /* compute_pv + pto_macro_fa_gu */
                float s = 0.0f;
                for (int j = 0; j < tn; j++) {
                    float prod = ph[j] * c->vf[(size_t)(j0 + j) * (size_t)D + (size_t)d];
                    s = s + prod;
                }
                orow[d] = first ? s : orow[d] * alpha + s;
            }
            first = 0;
        }
        for (int d = 0; d < D; d++)
            c->o[i * (size_t)D + (size_t)d] = orow[d] / gsum;
        if (c->row_max)
            c->row_max[i] = gmax;
        if (c->row_sum)
            c->row_sum[i] = gsum;
    }
    free(x);
    free(pf);
    free(ph);
    free(qrow);
    free(orow);
}

void po_fa_stream_f16(float *o, float *row_max, float *row_sum, const uint16_t *q, const uint16_t *k,
                      const uint16_t *v, int S0, int S1, int D, int tile_s1, int causal, int q_offset,
                      int round_away, int threads)
{
    float *kf = (float *)malloc(sizeof(float) * (size_t)S1 * (size_t)D);
    float *vf = (float *)malloc(sizeof(float) * (size_t)S1 * (size_t)D);
    po_tcvt_f16_f32(kf, k, (size_t)S1 * (size_t)D);
    po_tcvt_f16_f32(vf, v, (size_t)S1 * (size_t)D);
    po_fa_ctx c = {o, row_max, row_sum, q, kf, vf, S0, S1, D, tile_s1, causal, q_offset, round_away};
    po_parallel_rows((size_t)S0, threads, po_fa_stream_rows, &c);
    free(kf);
    free(vf);
}

/* --------------------------------------------------------------- comparator */
int po_result_cmp_f32(const float *expect, const float *actual, size_t n, float eps, double *max_diff, size_t *n_bad)
{ /* tests/common/test_common.h:211-301, applied to all n elements */
    size_t bad = 0, zero = 0;
    double md = 0.0;
    for (size_t i = 0; i < n; i++) {
        float d = fabsf(expect[i] - actual[i]);
        float rel = fabsf(d / expect[i]);
        if (d > md)
            md = d;
        if (fabsf(actual[i]) <= 1e-6f && fabsf(expect[i]) > 1e-6f)
            zero++;
        if ((d > eps && rel > eps) || isnan(d))
            bad++;
    }
    if (max_diff)
        *max_diff = md;
    if (n_bad)
        *n_bad = bad;
    return bad <= (size_t)((double)n * eps) && zero <= 1000;
}

/* ------------------------------------------------- further Vec instructions */
static int po_cmp(float a, float b, int mode)
{ /* ElementOp.h:227-253; CmpMode EQ NE LT LE GT GE = 0..5 (common/type.hpp:131-139) */
    switch (mode) {
    case 0: return a == b;
    case 1: return a != b;
    case 2: return a < b;
    case 3: return a <= b;
    case 4: return a > b;
    case 5: return a >= b;
    default: return a == b;
    }
}

void po_vec_op(float *dst, const float *a, const float *b, const float *vec, float k, int op, int ld, int rows, int cols)
{
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            size_t x = (size_t)r * (size_t)ld + (size_t)c;
            float v = a[x], w = (op >= 20 && op < 40) ? b[x] : 0.0f, o;
            float rv = (op >= 60 && op < 80) ? vec[r] : 0.0f, cv = op >= 80 ? vec[c] : 0.0f;
            switch (op) {
            case 0: o = v < 0 ? -v : v; break;                          /* TAbs.hpp:24 */
            case 1: o = -v; break;                                      /* ElementOp.h:297-302 */
            case 2: o = v < 0.0f ? 0.0f : v; break;                     /* std::max(src, 0): ElementOp.h:345-350 */
            case 3: o = (float)sqrt((double)v); break;                  /* TSqrt.hpp:23 */
            case 4: o = (float)(1.0 / sqrt((double)v)); break;          /* TRSqrt.hpp:29-31 */
            case 5: o = (float)log((double)v); break;                   /* ElementOp.h:289-294 */
            case 6: o = 1.0f / v; break;                                /* TRECIP = TDIVS(dst, 1, src): pto_instr.hpp:296-304 */
            case 7: o = (float)exp((double)v); break;                   /* TExp.hpp:36 */
            case 20: o = v + w; break;
            case 21: o = v - w; break;
            case 22: o = v * w; break;
            case 23: o = v / w; break;
            case 24: o = v < w ? w : v; break;                          /* std::max */
            case 25: o = w < v ? w : v; break;                          /* std::min */
            case 26: o = v > 0.0f ? v : v * w; break;                   /* ElementOp.h:257-262 */
            case 27: case 28: case 29: case 30: case 31: case 32: o = (float)po_cmp(v, w, op - 27); break;
            case 33: o = (k == 1.0f) ? v : w; break;                    /* TSelS.hpp:20-31 */
            case 40: o = v + k; break;
            case 41: o = v - k; break;
            case 42: o = v * k; break;
            case 43: o = v / k; break;
            case 44: o = v < k ? k : v; break;
            case 45: o = k < v ? k : v; break;
            case 46: o = v > 0.0f ? v : v * k; break;                   /* ElementOp.h:503-508 */
            case 60: o = rv; break;                                     /* TRowExpand.hpp */
            case 61: o = v - rv; break;
            case 62: o = v * rv; break;
            case 63: o = v / rv; break;
            case 64: o = v + rv; break;
            case 65: o = v < rv ? rv : v; break;
            case 66: o = rv < v ? rv : v; break;
            case 67: o = (float)exp((double)(v - rv)); break;           /* ElementOp.h:265-270 */
            case 80: o = cv; break;                                     /* TColExpand.hpp:22-33 */
            case 81: o = v - cv; break;
            case 82: o = v * cv; break;
            case 83: o = v / cv; break;
            case 84: o = v + cv; break;
            case 85: o = v < cv ? cv : v; break;
            case 86: o = cv < v ? cv : v; break;
            case 87: o = (float)exp((double)(v - cv)); break;           /* TColExpandOp.hpp:75-79 */
            default: o = 0.0f; break;
            }
            dst[x] = o;
        }
}

void po_reduce(float *dst, const float *a, int ld, int rows, int cols, int op)
{
    if (op < 3) {
        for (int i = 0; i < rows; i++) {
            float acc = op == 2 ? 0.0f : a[(size_t)i * (size_t)ld];
            for (int j = (op == 2 ? 0 : 1); j < cols; j++) {
                float v = a[(size_t)i * (size_t)ld + (size_t)j];
                acc = op == 0 ? (acc < v ? v : acc) : op == 1 ? (v < acc ? v : acc) : acc + v;
            }
            dst[i] = acc;
        }
    } else {
        for (int j = 0; j < cols; j++) {
            float acc = op == 5 ? 0.0f : a[j];
            for (int i = (op == 5 ? 0 : 1); i < rows; i++) {
                float v = a[(size_t)i * (size_t)ld + (size_t)j];
                acc = op == 3 ? (v > acc ? v : acc) : op == 4 ? (v < acc ? v : acc) : acc + v; /* TColMax.hpp:27-33, TColSum.hpp:25-28 */
            }
            dst[j] = acc;
        }
    }
}

void po_tcmps_packed(uint8_t *dst, int dst_ld, const float *a, int ld, int rows, int cols, float scalar, int mode)
{
    for (int r = 0; r < rows; r++)
        for (int cb = 0; cb < cols / 8; cb++) {
            unsigned byte = 0;
            for (int bit = 0; bit < 8; bit++) {
                float v = a[(size_t)r * (size_t)ld + (size_t)(cb * 8 + bit)];
                double diff = (double)v - (double)scalar; /* TCmps.hpp:28 */
                int res;
                switch (mode) {
                case 0: res = fabs(diff) < 1e-9; break;
                case 1: res = fabs(diff) > 1e-9; break;
                case 2: res = v < scalar; break;
                case 3: res = v <= scalar; break;
                case 4: res = v > scalar; break;
                case 5: res = v >= scalar; break;
                default: res = fabs(diff) < 1e-9; break;
                }
                byte |= (unsigned)res << bit; /* TCmps.hpp:71-76 */
            }
            dst[(size_t)r * (size_t)dst_ld + (size_t)cb] = (uint8_t)byte;
        }
}

void po_tsel_packed(float *dst, const uint8_t *mask, int mask_ld, int mask_valid_cols, const float *a, const float *b, int ld,
                    int rows, int cols)
{
    /* npu/a2a3/TSel.hpp:46-57 and tsel/gen_data.py:31-47: mask row i serves row i, column j is bit j % 8 of byte j / 8.
       cpu/TSel.hpp:27-47 runs on through the mask's valid columns instead; the same thing when cols == 8 * mask_valid_cols,
       which holds for every case of the simulation's own tests. */
    (void)mask_valid_cols;
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++) {
            size_t x = (size_t)i * (size_t)ld + (size_t)j;
            unsigned sel = (mask[(size_t)i * (size_t)mask_ld + (size_t)(j >> 3)] >> (j & 7)) & 1u;
            dst[x] = sel ? a[x] : b[x];
        }
}

void po_tfillpad(float *dst, const float *a, int ld, int rows, int cols, int vr, int vc, int pad_kind)
{
    float pad = pad_kind == 2 ? INFINITY : pad_kind == 3 ? -INFINITY : 0.0f; /* TFillPad.hpp:26-38 */
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++)
            dst[(size_t)i * (size_t)ld + (size_t)j] = (i < vr && j < vc) ? a[(size_t)i * (size_t)ld + (size_t)j] : pad;
}

void po_tmov_relu(float *dst, const float *src, size_t n, int relu)
{
    for (size_t i = 0; i < n; i++)
        dst[i] = (relu && src[i] < 0.0f) ? 0.0f : src[i]; /* TMov.hpp:57-67 */
}
