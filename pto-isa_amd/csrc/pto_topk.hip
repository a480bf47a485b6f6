// Row-wise top-k for MI355X: per row, the (score, index) pairs in descending order of score, equal scores in ascending
// order of index, first k of them written as scores and as indices.
//
// Mirrors the reference kernel kernels/manual/a2a3/topk/topk_kernel.cpp:282-345 (launchTopk: TLOAD -> TSORT32 on groups of
// 32 -> TMRGSORT merges of 4 lists -> TGATHER splits scores and indices -> TSTORE) and its golden
// (scripts/gen_data.py:55-64: np.lexsort((idx, -row))[:topk]); the order is the comparator of TSORT32 / TMRGSORT
// (include/pto/cpu/TSort32.hpp:32-41: score descending, then index ascending, -0 == +0).
//
// The reference builds the order from 32-element hardware sorts and 4-way merges in its unified buffer, re-viewing one
// buffer through differently shaped tiles.  On a CDNA4 compute unit the natural form is one workgroup per row and a
// bitonic network over 64-bit keys in LDS: key = (order-preserving image of the score) << 32 | ~index, so that one
// unsigned comparison implements the comparator.  Each of the four waves owns a quarter of the row: the stages whose
// partners lie inside a quarter need no workgroup barrier (a wave's LDS operations execute in order).
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace {

constexpr int kTopkThreads = 256, kTopkWaves = 4;

// N: padded row length, a power of two in [256, 4096]
template <int N>
__global__ __launch_bounds__(kTopkThreads) void TopkRows(float *outScore, uint32_t *outIndex, const float *src, const uint32_t *inIdx,
                                                         int validCols, int ld, int topk)
{
    __shared__ uint64_t key[N];
    __shared__ uint16_t pos[N];
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const float *row = src + (size_t)blockIdx.x * (size_t)ld;
    for (int i = tid; i < N; i += kTopkThreads) {
        uint64_t kv = 0; // padding: below every real key
        if (i < validCols) {
            uint32_t b = __float_as_uint(row[i]);
            if (b == 0x80000000u)
                b = 0; // -0 and +0 compare equal
            const uint32_t ord = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
            kv = ((uint64_t)ord << 32) | (uint32_t)~inIdx[i];
        }
        key[i] = kv;
        pos[i] = (uint16_t)i;
    }
    __syncthreads();
    constexpr int kChunk = N / kTopkWaves, kPairsPerWave = kChunk / 2;
    for (int k = 2; k <= N; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            const bool crossWave = j >= kChunk;
            if (crossWave)
                __syncthreads();
            for (int u = lane; u < kPairsPerWave; u += 64) {
                const int t = wave * kPairsPerWave + u;
                const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), l = i | j;
                const uint64_t a = key[i], b = key[l];
                const bool descending = (i & k) == 0;
                if (descending ? a < b : a > b) {
                    key[i] = b;
                    key[l] = a;
                    const uint16_t pa = pos[i], pb = pos[l];
                    pos[i] = pb;
                    pos[l] = pa;
                }
            }
            if (crossWave)
                __syncthreads();
            else
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's exchanges are done before its next stage reads them
        }
    __syncthreads();
    for (int i = tid; i < topk; i += kTopkThreads) {
        const int p = pos[i];
        outScore[(size_t)blockIdx.x * (size_t)topk + i] = row[p];
        outIndex[(size_t)blockIdx.x * (size_t)topk + i] = inIdx[p];
    }
}

} // namespace

extern "C" int pto_topk_f32(void *stream, float *out_score, uint32_t *out_index, const float *src, const uint32_t *in_idx, int rows,
                            int valid_cols, int ld, int topk)
{
    if (!out_score || !out_index || !src || !in_idx || rows <= 0 || valid_cols <= 0 || topk <= 0)
        return PTO_ERR_BAD_ARG;
    if (ld < valid_cols || topk > valid_cols || valid_cols > 4096)
        return PTO_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PTO_TOPK_CASE(NN)                                                                                              \
    if (valid_cols <= NN) {                                                                                            \
        TopkRows<NN><<<dim3(rows), dim3(kTopkThreads), 0, st>>>(out_score, out_index, src, in_idx, valid_cols, ld, topk); \
        return pto_amd::check_launch();                                                                                \
    }
    PTO_TOPK_CASE(256)
    PTO_TOPK_CASE(512)
    PTO_TOPK_CASE(1024)
    PTO_TOPK_CASE(2048)
    PTO_TOPK_CASE(4096)
#undef PTO_TOPK_CASE
    return PTO_ERR_UNSUPPORTED;
}
