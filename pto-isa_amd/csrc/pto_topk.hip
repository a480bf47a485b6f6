// Row-wise top-k for MI355X: per row, the (score, index) pairs in descending order of score, equal scores in ascending
// order of index, first k of them written as scores and as indices.
//
// Mirrors the reference kernel kernels/manual/a2a3/topk/topk_kernel.cpp:282-345 (launchTopk: TLOAD -> TSORT32 on groups of
// 32 -> TMRGSORT merges of 4 lists -> TGATHER splits scores and indices -> TSTORE) and its golden
// (scripts/gen_data.py:55-64: np.lexsort((idx, -row))[:topk]); the order is the comparator of TSORT32 / TMRGSORT
// (include/pto/cpu/TSort32.hpp:32-41: score descending, then index ascending, -0 == +0).
//
// The reference builds the order from 32-element hardware sorts and 4-way merges in its unified buffer, re-viewing one
// buffer through differently shaped tiles.  On a CDNA4 compute unit the natural form is one workgroup (four waves) per
// row and a bitonic network over 64-bit keys whose unsigned order is the comparator:
//   key = (order-preserving image of the score) << 32 | low word that decides among equal scores.
// * Indices that increase with the column (the reference passes 0, 1, 2, ...): low word = ~column, and a thread keeps
//   its N/256 consecutive keys in registers.  Partners inside a thread are compared in registers, partners inside a
//   wave are fetched with lane swizzles, and only the two or three strides that cross waves go through LDS.
// * Any other index vector: low word = ~index, keys and columns in LDS, every stage a pass over LDS; each wave owns a
//   quarter of the row and the stages whose partners lie inside a quarter need no workgroup barrier.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace {

constexpr int kTopkThreads = 256, kTopkWaves = 4;

__device__ inline uint32_t ScoreOrder(uint32_t bits) { return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u); }
__device__ inline uint32_t ScoreBits(uint32_t ord) { return (ord & 0x80000000u) ? (ord & 0x7fffffffu) : ~ord; }

// value of lane ^ M of the wave, M a power of two below 64
template <int M>
__device__ inline uint32_t LaneXor(uint32_t v, int lane)
{
    // (every lane has a source lane in these three patterns, so the destination needs no initial value: mov_dpp, not
    // update_dpp with a zero that costs a move per call)
    if constexpr (M == 1)
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true); // quad_perm [1,0,3,2]
    else if constexpr (M == 2)
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true); // quad_perm [2,3,0,1]
    else if constexpr (M == 8)
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xf, 0xf, true); // row_ror:8 (rows of 16 lanes)
    else if constexpr (M < 32)
        return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (M << 10) | 0x1f); // bit mode: lane ^ M within 32 lanes
    else
        return (uint32_t)__builtin_amdgcn_ds_bpermute(((lane ^ 32) << 2), (int)v);
}
template <int M>
__device__ inline uint64_t LaneXor64(uint64_t v, int lane)
{
    return ((uint64_t)LaneXor<M>((uint32_t)(v >> 32), lane) << 32) | LaneXor<M>((uint32_t)v, lane);
}

// Compare and select on wave masks held in scalar register pairs.  (Measured on gfx950: a conditional move that takes its
// mask from VCC issues at a fifth of the rate of one that takes it from a scalar register pair, so the selects of the
// network name their masks themselves instead of leaving the choice to the compiler.)  All 64 lanes are active here.
__device__ inline uint64_t MaskLess(uint64_t a, uint64_t b)
{
    uint64_t m;
    asm("v_cmp_lt_u64_e64 %0, %1, %2" : "=s"(m) : "v"(a), "v"(b));
    return m;
}
__device__ inline uint32_t SelectWord(uint64_t mask, uint32_t ifSet, uint32_t ifClear)
{
    uint32_t r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(ifClear), "v"(ifSet), "s"(mask));
    return r;
}
__device__ inline uint64_t Select(uint64_t mask, uint64_t ifSet, uint64_t ifClear)
{
    return ((uint64_t)SelectWord(mask, (uint32_t)(ifSet >> 32), (uint32_t)(ifClear >> 32)) << 32) |
           SelectWord(mask, (uint32_t)ifSet, (uint32_t)ifClear);
}

template <int FIRST, int LAST, typename F>
__device__ inline void StaticFor(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        StaticFor<FIRST + 1, LAST>(f);
    }
}

// Bitonic sort, descending, of the 256 E keys of a workgroup; thread t holds the keys of ranks t E .. t E + E - 1.
template <int E>
__device__ inline void SortInRegisters(uint64_t (&k)[E], uint64_t *lds, int tid)
{
    constexpr int N = kTopkThreads * E, kLogN = __builtin_ctz(N), kLogE = __builtin_ctz(E);
    const int lane = tid & 63;
    // The lane predicates of the network, once: bit s of the key's rank for every run length and partner distance that
    // spans threads (as lane masks they live in scalar registers; computed per stage they were an eighth of the vector
    // instructions).
    uint64_t rankBitClear[kLogN + 1]; // wave masks
#pragma unroll
    for (int s = 0; s <= kLogN; ++s)
        rankBitClear[s] = s < kLogE ? ~0ull : __builtin_amdgcn_ballot_w64(((tid >> (s - kLogE)) & 1) == 0);
    StaticFor<1, kLogN + 1>([&](auto sizeTag) {
        constexpr int kk = 1 << decltype(sizeTag)::value; // the network sorts runs of kk keys, alternating direction
        // lanes whose run is descending (the last stage sorts the whole row downwards)
        const uint64_t descending = kk == N ? ~0ull : rankBitClear[decltype(sizeTag)::value];
        StaticFor<0, decltype(sizeTag)::value>([&](auto strideTag) {
            constexpr int j = kk >> (decltype(strideTag)::value + 1); // distance between partners
            if constexpr (j < E) {
#pragma unroll
                for (int e = 0; e < E; ++e)
                    if ((e & j) == 0) {
                        const uint64_t a = k[e], b = k[e | j];
                        const uint64_t less = MaskLess(a, b);
                        // descending runs swap where a < b, ascending ones where a >= b (equal keys are the padding:
                        // swapping them changes nothing).  Run lengths below E: the direction is a property of the
                        // register, not of the lane.
                        const uint64_t swap = kk < E ? ((e & kk) == 0 ? less : ~less) : ~(less ^ descending);
                        k[e] = Select(swap, b, a);
                        k[e | j] = Select(swap, a, b);
                    }
            } else {
                uint64_t other[E];
                if constexpr (j < 64 * E) {
#pragma unroll
                    for (int e = 0; e < E; ++e)
                        other[e] = LaneXor64<j / E>(k[e], lane);
                } else {
                    // partners are E (j / E) ranks apart: the same register of thread tid ^ (j / E).  Register e of all
                    // threads is one contiguous run of LDS, so a wave's 64 lanes touch 64 consecutive 8-byte words
                    __syncthreads(); // everyone is done reading the previous exchange
#pragma unroll
                    for (int e = 0; e < E; ++e)
                        lds[e * kTopkThreads + tid] = k[e];
                    __syncthreads();
#pragma unroll
                    for (int e = 0; e < E; ++e)
                        other[e] = lds[e * kTopkThreads + (tid ^ (j / E))];
                }
                // the lower rank of a pair keeps the larger key where the run is descending
                const uint64_t keepMax = ~(rankBitClear[__builtin_ctz(j)] ^ descending);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const uint64_t otherLarger = MaskLess(k[e], other[e]);
                    k[e] = Select(~(otherLarger ^ keepMax), other[e], k[e]);
                }
            }
        });
    });
}

// Any index vector: keys and columns in LDS, one pass over LDS per stage.
template <int N>
__device__ inline void SortInLds(uint64_t *key, uint16_t *pos, int tid)
{
    const int wave = tid / 64, lane = tid % 64;
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
}

// E: keys per thread; the row is padded to N = 256 E keys (padding keys are 0, below every real key).
template <int E>
__global__ __launch_bounds__(kTopkThreads) void TopkRows(float *outScore, uint32_t *outIndex, const float *src, const uint32_t *inIdx,
                                                         int validCols, int ld, int topk)
{
    constexpr int N = kTopkThreads * E;
    __shared__ uint64_t key[N];
    __shared__ uint16_t pos[N];
    const int tid = threadIdx.x;
    const float *row = src + (size_t)blockIdx.x * (size_t)ld;
    float *rowScore = outScore + (size_t)blockIdx.x * (size_t)topk;
    uint32_t *rowIndex = outIndex + (size_t)blockIdx.x * (size_t)topk;

    // do the indices increase with the column?  (then the column decides among equal scores, as the index would)
    bool increasing = true;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int i = tid * E + e;
        if (i + 1 < validCols)
            increasing = increasing && inIdx[i] < inIdx[i + 1];
    }
    bool inRegisters = false;
    if constexpr (E <= 8)
        inRegisters = __syncthreads_and(increasing) != 0;
    if constexpr (E <= 8) if (inRegisters) {
        uint64_t k[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int i = tid * E + e;
            k[e] = 0;
            if (i < validCols) {
                const uint32_t b = __float_as_uint(row[i]);
                const bool negZero = b == 0x80000000u; // compares equal to +0: same key, remembered below the column bits
                k[e] = ((uint64_t)ScoreOrder(negZero ? 0u : b) << 32) | ((uint32_t)(4095 - i) << 20) | (negZero ? 1u : 0u);
            }
        }
        SortInRegisters<E>(k, key, tid);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int i = tid * E + e;
            if (i < topk) {
                const uint32_t low = (uint32_t)k[e];
                rowScore[i] = __uint_as_float((low & 1u) ? 0x80000000u : ScoreBits((uint32_t)(k[e] >> 32)));
                rowIndex[i] = inIdx[4095 - (int)(low >> 20)];
            }
        }
        return;
    }
    for (int i = tid; i < N; i += kTopkThreads) {
        uint64_t kv = 0;
        if (i < validCols) {
            uint32_t b = __float_as_uint(row[i]);
            if (b == 0x80000000u)
                b = 0; // -0 and +0 compare equal
            kv = ((uint64_t)ScoreOrder(b) << 32) | (uint32_t)~inIdx[i];
        }
        key[i] = kv;
        pos[i] = (uint16_t)i;
    }
    __syncthreads();
    SortInLds<N>(key, pos, tid);
    for (int i = tid; i < topk; i += kTopkThreads) {
        const int p = pos[i];
        rowScore[i] = row[p];
        rowIndex[i] = inIdx[p];
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
#define PTO_TOPK_CASE(EE)                                                                                              \
    if (valid_cols <= kTopkThreads * EE) {                                                                             \
        TopkRows<EE><<<dim3(rows), dim3(kTopkThreads), 0, st>>>(out_score, out_index, src, in_idx, valid_cols, ld, topk); \
        return pto_amd::check_launch();                                                                                \
    }
    PTO_TOPK_CASE(1)
    PTO_TOPK_CASE(2)
    PTO_TOPK_CASE(4)
    PTO_TOPK_CASE(8)
    PTO_TOPK_CASE(16)
#undef PTO_TOPK_CASE
    return PTO_ERR_UNSUPPORTED;
}
