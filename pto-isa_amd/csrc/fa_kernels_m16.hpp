// Flash-attention forward on v_mfma_f32_16x16x32_f16 for workgroups of eight wavefronts (wave grid 1 x 8, two groups of
// four waves in opposite MFMA / softmax phases): the kernel of fa_kernels.hpp (PHASES variant) re-tiled for the MFMA shape
// that sustains the higher clock.  A wave still owns 32 queries, now as two column blocks of 16; scores are computed
// transposed (X^T = K Q^T, 16 keys x 16 queries per accumulator block), P^T in accumulator layout is the B operand of
// O^T = V^T P^T (32 keys per MFMA: two 16-key score blocks), V^T comes from the row-major V tile with transposing reads.
// Include after <pto/pto-inst.hpp> with PTO_MFMA_M 16, PTO_WAVES_M 1, PTO_WAVES_N 8.
#pragma once
#include "common.hpp"
#include <cstdlib>

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

static_assert(detail::kMfmaM == 16 && kBlockWaves == 8, "16 x 16 x 32 MFMAs, eight wavefronts");

constexpr int kBQ16 = 32 * PTO_WAVES_N; // queries per workgroup
constexpr int kBKV16 = 64;              // keys per tile
constexpr float kMaskValue16 = -3.40282e+38f; // pto_macro_fa_softmax.hpp:67

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// A lane holds one query column of a 16 x 16 block and four of its 16 key rows; the other twelve are in the lanes
// 16, 32 and 48 positions away.  Both swaps leave in (a, b) the values of the two partners in both places.
// (two distinct registers go in: a swap of a register with itself is no exchange)
AICORE inline float MaxOverRowGroups(float x)
{
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    float c = fmaxf(a, b), d = c;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(c), "+v"(d));
    return fmaxf(c, d);
}
AICORE inline float SumOverRowGroups(float x)
{
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    float c = a + b, d = c;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(c), "+v"(d));
    return c + d;
}

// LDS images.  K: the library's Mat image (256-byte rows, the 16-byte chunk c of key k at position c ^ (k % 16)); the
// fragment reads of 16 keys x 16 bytes then touch every bank once (measured: 4 clocks per ds_read_b128, 8 with the keys
// of a block permuted).  V: the same rows with the chunk position c ^ VSwz(k): a transposing read gathers keys 4g .. 4g+3
// for lane group g, the LDS serves lane groups 0-1 and 2-3 together, and the 32-byte pieces of keys 0-7 (8-15) must
// then fall into eight different 32-byte slots of the 256-byte bank line: slot = (c / 2) ^ (VSwz(k) / 2), and VSwz / 2
// runs through 0 .. 7 for k = 0 .. 7 and again for 8 .. 15 (measured: 2.3 clocks per read, 4.1 with VSwz(k) = k).
AICORE inline constexpr uint32_t VSwz(uint32_t key) { return ((key & 7u) << 1) | ((key >> 3) & 1u); }
AICORE inline constexpr uint32_t KeyOfRow16(uint32_t r) { return r; } // row r of a 16-key block of K, X^T, P^T holds key r

template <int FIRST, int LAST, typename F>
AICORE inline __attribute__((always_inline)) void StaticFor16(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        StaticFor16<FIRST + 1, LAST>(f);
    }
}

// K operand fragments: (kb, ks) = key rows 16 kb .. +15 x head-dim columns 32 ks .. +31; a lane holds 8 consecutive
// head-dim values (16 bytes) of its key.  Issued as assembly with explicit waits on the LDS counter, as in fa_kernels.hpp.
template <int D>
struct KReader16 {
    static constexpr int KS = D / 32;
    static constexpr uint32_t kRowBytes = D * (uint32_t)sizeof(half);
    uint32_t base[KS];

    AICORE inline void Init()
    {
        const uint32_t lane = (uint32_t)hw::lane();
        const uint32_t key = KeyOfRow16(lane & 15u), g = lane >> 4;
        const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)hw::lds_base();
        static_assert(detail::mat_swz<kRowBytes>(16) == detail::mat_swz<kRowBytes>(0), "the swizzle repeats every 16 keys");
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            base[ks] = ldsBase + detail::mat_chunk_off<kRowBytes>(key, g + 4u * ks);
    }
    template <uint32_t LDS_OFF, int KB_, int KS_>
    AICORE inline void Issue(f16x8 &f) const
    {
        constexpr uint32_t off = LDS_OFF + KB_ * 16u * kRowBytes;
        static_assert(off < 65536u, "the offset field of an LDS instruction has 16 bits");
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f) : "v"(base[KS_]), "n"(off));
    }
    template <int N>
    AICORE static inline void Wait(f16x8 &f)
    {
        static_assert(N >= 0 && N <= 15, "the LDS counter has 4 bits");
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f) : "n"(N));
    }
};

template <uint32_t OFF>
AICORE inline s16x4 DsReadTr16b(uint32_t addr)
{
    static_assert(OFF < 65536u, "the offset field of an LDS instruction has 16 bits");
    s16x4 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

template <int D, bool CAUSAL, bool OUT_F32>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE void FlashAttnFwdM16(__gm__ void *outO, __gm__ float *outLse, __gm__ const half *qAll,
                                                                           __gm__ const half *kAll, __gm__ const half *vAll, int heads,
                                                                           int seqQ, int seqKv, int numBH, int causalOff)
{
    constexpr int kBQ = kBQ16, kBKV = kBKV16;
    constexpr int NQ = 2;          // 16-query column blocks per wave
    constexpr int KB = kBKV / 16;  // 16-key score blocks per tile
    constexpr int KT = kBKV / 32;  // 32-key steps of the output stage per tile
    constexpr int DB = D / 16;     // 16-wide blocks of the head dimension (rows of O^T)
    constexpr int KS = D / 32;     // 32-wide steps of the head dimension (k of the score MFMAs)
    static_assert(D == 128 && DB == 8, "head dimension 128");
    using TileMatQ = Tile<TileType::Mat, half, D, kBQ, BLayout::RowMajor, D, kBQ, SLayout::ColMajor>;   // Q^T, contiguous along d
    using TileMatK = Tile<TileType::Mat, half, kBKV, D, BLayout::ColMajor, kBKV, D, SLayout::RowMajor>; // K,   contiguous along d
    using RightQ = TileRight<half, D, kBQ, D, kBQ>; // per wave: 32 queries x D as fragments [NQ][KS]
    static_assert(RightQ::Storage::NB == NQ && RightQ::Storage::KS == KS, "Q^T fragments");
    using GlobalQT = GlobalTensor<half, TileShape2D<half, D, kBQ, Layout::DN>, Stride<1, 1, 1, 1, D>, Layout::DN>;
    using GlobalKV = GlobalTensor<half, TileShape2D<half, kBKV, D, Layout::ND>, Stride<1, 1, 1, D, 1>, Layout::ND>;
    using Acc = detail::AccFrag; // 16 x 16 block: lane (column = lane % 16, g = lane / 16) holds rows 4 g .. 4 g + 3

    constexpr uint32_t kRowBytes = D * (uint32_t)sizeof(half);
    constexpr uint32_t kTileBytes = kBKV * D * sizeof(half);
    constexpr uint32_t kStageBytes = 2 * kTileBytes;
    static_assert(D * kBQ * sizeof(half) <= 2 * kStageBytes, "Q^T is staged in the K/V stages");

    // ---- which (batch*head, query tile): as in fa_kernels.hpp ----
    const int numQT = seqQ / kBQ;
    int bh, qt;
    {
        const int bid = (int)get_block_idx();
        if (numBH % 8 == 0) {
            const int xcd = bid % 8, slot = bid / 8, perXcd = numBH / 8;
            bh = xcd + 8 * (slot % perXcd);
            qt = slot / perXcd;
        } else {
            bh = bid % numBH;
            qt = bid / numBH;
        }
        if (CAUSAL)
            qt = numQT - 1 - qt;
    }
    const int q0 = qt * kBQ;
    __gm__ half *qBase = const_cast<half *>(qAll) + ((int64_t)bh * seqQ + q0) * D;
    // (the same in every lane: kept in scalar registers, so that the tile addresses of the copies are scalar arithmetic)
    __gm__ half *kBase = reinterpret_cast<half *>(const_cast<char *>(
        detail::uniform_ptr(reinterpret_cast<const char *>(kAll + (int64_t)bh * seqKv * D))));
    __gm__ half *vBase = reinterpret_cast<half *>(const_cast<char *>(
        detail::uniform_ptr(reinterpret_cast<const char *>(vAll + (int64_t)bh * seqKv * D))));
    int numTiles = seqKv / kBKV;
    if (CAUSAL) {
        const int lim = (q0 + kBQ - 1 + causalOff) / kBKV + 1;
        numTiles = lim < numTiles ? lim : numTiles;
    }

    TileMatK kMat[2];
    TileMatQ qMat;
    TASSIGN(kMat[0], 0u);
    TASSIGN(kMat[1], kStageBytes);
    TASSIGN(qMat, 0u);

    RightQ qRight;
    Acc oAcc[DB][NQ];
    float runMax[NQ], runSum[NQ]; // per lane and query block; runSum is the partial of this lane's key rows
    const int lane = hw::lane();
    const uint32_t g = (uint32_t)lane >> 4;
    const int myQuery = q0 + hw::wave_n() * 32 + (lane & 15); // query block nq: + 16 nq
    const float sLog2e = 0.08838834764831845f * 1.4426950408889634f;

    KReader16<D> kr;
    kr.Init();
    // V^T: base address of this lane's 8 bytes for head-dim block db, key step 0, read 0, tile at LDS offset 0
    uint32_t vBaseAddr[DB];
    {
        const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)hw::lds_base();
        const uint32_t i = (uint32_t)lane & 15u, key = KeyOfRow16(4u * g + (i >> 2));
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const uint32_t d0 = (uint32_t)db * 16u + 4u * (i & 3u);
            vBaseAddr[db] = ldsBase + key * kRowBytes + (((d0 >> 3) ^ VSwz(key)) << 4) + ((d0 & 7u) << 1);
        }
    }

    // ---- X^T = K Q^T: every K fragment feeds the two query blocks; 8 independent accumulator chains ----
    constexpr int kAheadK = 4, kTotalK = KB * KS, kTailHook = kTotalK - kAheadK;
    auto scoreTile = [&](Acc(&sAcc)[KB][NQ], auto stageTag, auto &&between, auto extraTag) __attribute__((always_inline)) {
        constexpr uint32_t kOff = decltype(stageTag)::value * kStageBytes;
        constexpr int kAhead = kAheadK, kExtra = decltype(extraTag)::value;
        f16x8 frag[kAhead + 1];
        StaticFor16<0, kAhead>([&](auto i) __attribute__((always_inline)) {
            constexpr int I = decltype(i)::value;
            kr.template Issue<kOff, I % KB, I / KB>(frag[I % (kAhead + 1)]);
        });
        StaticFor16<0, kTotalK>([&](auto i) __attribute__((always_inline)) {
            constexpr int I = decltype(i)::value, J = I + kAhead;
            if constexpr (J < kTotalK)
                kr.template Issue<kOff, J % KB, J / KB>(frag[J % (kAhead + 1)]);
            between(i);
            KReader16<D>::template Wait<(kTotalK - 1 - I < kAhead ? kTotalK - 1 - I : kAhead) + (I >= kTailHook ? kExtra : 0)>(
                frag[I % (kAhead + 1)]);
            constexpr int kb = I % KB, ks = I / KB;
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                if constexpr (ks == 0)
                    sAcc[kb][nq] = Acc{0.0f, 0.0f, 0.0f, 0.0f};
                sAcc[kb][nq] = detail::mfma32(frag[I % (kAhead + 1)], qRight.st.f[nq][ks], sAcc[kb][nq]); // TMATMUL_ACC, one block
                __builtin_amdgcn_sched_barrier(0);
            }
        });
    };
    // ---- streaming softmax on the accumulator blocks (one query per lane and query block) ----
    // pRight[t][nq]: P^T of key step t: k slot j <-> row 16 (2 t + j / 4) + 4 g + j % 4 of X^T
    auto softmaxTile = [&](Acc(&sAcc)[KB][NQ], int t, f16x8(&pRight)[KT][NQ], float(&alpha)[NQ], bool &anyRaise) __attribute__((always_inline)) {
        const int key0 = t * kBKV;
        if (CAUSAL && key0 + kBKV - 1 > q0 + causalOff) {
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                const int limit = myQuery + 16 * nq + causalOff;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kb * 16 + (int)KeyOfRow16(4u * g + (uint32_t)v);
                        if (key > limit)
                            sAcc[kb][nq][v] += kMaskValue16;
                    }
            }
        }
        // The running max is raised lazily and every tile but the first is tried with the running max as it stands, as in
        // fa_kernels.hpp: a lane's partial row sum of at most 2^kSlack proves that none of its P exceeds 2^kSlack, and
        // the row max of the tile is then never computed; otherwise the wave finds the row max and runs the
        // exponentials a second time.
        constexpr float kSlack = 8.0f;
        anyRaise = false;
        float locSum[NQ];
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
            alpha[nq] = 1.0f;
        bool needMax = t == 0; // wave-uniform
#pragma nounroll
        for (;;) {             // at most two rounds
            if (needMax) {
                anyRaise = t == 0;
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq) {
                    float locMax = sAcc[0][nq][0];
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            locMax = fmaxf(locMax, sAcc[kb][nq][v]);
                    locMax = MaxOverRowGroups(locMax);
                    const bool raise = t == 0 || (locMax - runMax[nq]) * sLog2e > kSlack;
                    const float newMax = raise ? locMax : runMax[nq];
                    if (t > 0)
                        anyRaise = anyRaise || __builtin_amdgcn_ballot_w64(raise) != 0;
                    alpha[nq] = (t == 0 || !raise) ? 1.0f : __builtin_amdgcn_exp2f((runMax[nq] - newMax) * sLog2e);
                    runMax[nq] = newMax;
                }
            }
            bool within = true;
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                const float negMax = -runMax[nq] * sLog2e;
                float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    f16x8 pk;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sAcc[2 * kt + j / 4][nq][j % 4], sLog2e, negMax));
                        part[j & 3] += p; // row sum over the fp32 P, as the reference does
                        pk[j] = (half)p;
                    }
                    pRight[kt][nq] = pk;
                }
                locSum[nq] = (part[0] + part[1]) + (part[2] + part[3]);
                within = within && locSum[nq] <= 256.0f; // 2^kSlack; false for a NaN
            }
            static_assert(kSlack == 8.0f, "the bound above is 2^kSlack");
            if (needMax || __builtin_amdgcn_ballot_w64(!within) == 0)
                break;
            needMax = true;
        }
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
            runSum[nq] = t == 0 ? locSum[nq] : runSum[nq] * alpha[nq] + locSum[nq];
    };
    // ---- O^T += V^T P^T.  One step = four head-dim blocks of one 32-key step: 8 transposing reads, 8 MFMAs ----
    struct VStep {
        s16x4 part[4][2];
    };
    constexpr int kStepReads = 8, kSteps = KT * 2;
    auto issueVStep = [&](auto offTag, auto stepTag, VStep &f) __attribute__((always_inline)) {
        constexpr int step = decltype(stepTag)::value, kt = step / 2, hb = step % 2;
        constexpr uint32_t off = decltype(offTag)::value + kt * 32u * kRowBytes;
        StaticFor16<0, 4>([&](auto dTag) __attribute__((always_inline)) {
            constexpr int d = decltype(dTag)::value;
            f.part[d][0] = DsReadTr16b<off>(vBaseAddr[hb * 4 + d]);
            f.part[d][1] = DsReadTr16b<off + 16u * kRowBytes>(vBaseAddr[hb * 4 + d]);
        });
    };
    auto waitVStep = [&](auto nTag, VStep &f) __attribute__((always_inline)) {
        constexpr int N = decltype(nTag)::value;
        static_assert(N >= 0 && N <= 15, "the LDS counter has 4 bits");
        asm volatile("s_waitcnt lgkmcnt(%8)"
                     : "+v"(f.part[0][0]), "+v"(f.part[0][1]), "+v"(f.part[1][0]), "+v"(f.part[1][1]), "+v"(f.part[2][0]),
                       "+v"(f.part[2][1]), "+v"(f.part[3][0]), "+v"(f.part[3][1])
                     : "n"(N));
    };
    auto outputTile = [&](auto stageTag, VStep &first, f16x8(&pRight)[KT][NQ], float(&alpha)[NQ], bool anyRaise) __attribute__((always_inline)) {
        using VOff = std::integral_constant<uint32_t, decltype(stageTag)::value * kStageBytes + kTileBytes>;
        VStep other;
        if (anyRaise) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        oAcc[db][nq][v] *= alpha[nq];
        }
        StaticFor16<0, kSteps>([&](auto stepTag) __attribute__((always_inline)) {
            constexpr int step = decltype(stepTag)::value, kt = step / 2, hb = step % 2;
            VStep &cur = (step & 1) ? other : first;
            VStep &nxt = (step & 1) ? first : other;
            if constexpr (step + 1 < kSteps) {
                issueVStep(VOff(), std::integral_constant<int, step + 1>(), nxt);
                waitVStep(std::integral_constant<int, kStepReads>(), cur);
            } else {
                waitVStep(std::integral_constant<int, 0>(), cur);
            }
            StaticFor16<0, 4>([&](auto dTag) __attribute__((always_inline)) {
                constexpr int d = decltype(dTag)::value, db = hb * 4 + d;
                const s16x8 both = {cur.part[d][0][0], cur.part[d][0][1], cur.part[d][0][2], cur.part[d][0][3],
                                    cur.part[d][1][0], cur.part[d][1][1], cur.part[d][1][2], cur.part[d][1][3]};
                const f16x8 a = __builtin_bit_cast(f16x8, both);
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq) {
                    oAcc[db][nq] = detail::mfma32(a, pRight[kt][nq], oAcc[db][nq]); // TMATMUL_ACC, one block
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
        });
    };
    // V tile (64 keys x 256 bytes) -> LDS at byte offset ldsOff with the VSwz chunk positions: two asynchronous 16-byte
    // copy instructions per wave (4 rows each, 32 rows apart: VSwz repeats every 16 rows, so one per-lane offset serves both)
    const uint32_t vLaneOff = [&]() {
        const uint32_t row = (uint32_t)hw::wave() * 4u + ((uint32_t)lane >> 4), cpos = (uint32_t)lane & 15u;
        return row * kRowBytes + ((cpos ^ VSwz(row & 15u)) << 4);
    }();
    auto loadVTile = [&](uint32_t ldsOff, __gm__ const half *tile) __attribute__((always_inline)) {
        char *lds = hw::lds_base() + ldsOff;
        const char *base = reinterpret_cast<const char *>(tile);
#pragma unroll
        for (int s0 = 0; s0 < 16; s0 += kBlockWaves) {
            const char *gp = detail::uniform_ptr(base + (int64_t)(s0 * 4) * kRowBytes) + vLaneOff;
            __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(gp), PTO_LDS_PTR(lds + (s0 + hw::wave()) * 1024), 16, 0, 0);
        }
    };
    auto keyTile = [&](__gm__ half *base, int t) {
        const int tc = t < numTiles ? t : numTiles - 1; // past the end: re-fetch the last tile (nobody reads it)
        return GlobalKV(base + (int64_t)tc * kBKV * D);
    };

#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
            oAcc[db][nq] = Acc{0.0f, 0.0f, 0.0f, 0.0f};
    {
        GlobalQT gmQ(qBase);
        TLOAD(qMat, gmQ);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        TEXTRACT(qRight, qMat, 0, 0);
        set_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1);
        wait_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1); // Q^T is in registers everywhere: the stages may be filled
        GlobalKV gmK(kBase);
        TLOAD(kMat[0], gmK);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    }

    // ---- two groups of four waves in opposite phases (the schedule of fa_kernels.hpp) ----
    const int group = hw::wave_n() >> 2;
    Acc sAcc[KB][NQ];
    f16x8 pRight[KT][NQ];
    float alpha[NQ];
    bool anyRaise = false;
    auto phaseEnd = [&]() __attribute__((always_inline)) {
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    };
    auto loadBundle = [&](int b) __attribute__((always_inline)) { // this wave's share of bundle b = {K tile b, V tile b - 1}
        TileMatK kDst;
        const uint32_t off = (uint32_t)(b & 1) * kStageBytes;
        TASSIGN(kDst, off);
        GlobalKV gmK = keyTile(kBase, b);
        TLOAD(kDst, gmK);
        const int tv = b - 1 < numTiles ? b - 1 : numTiles - 1;
        loadVTile(off + kTileBytes, vBase + (int64_t)(tv < 0 ? 0 : tv) * kBKV * D);
    };
    auto ppStep = [&](auto stageTag, int t) __attribute__((always_inline)) {
        constexpr int st = decltype(stageTag)::value;
        using VOff = std::integral_constant<uint32_t, st * kStageBytes + kTileBytes>;
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
        VStep vFirst;
        if (t < numTiles) {
            scoreTile(sAcc, stageTag, [&](auto i) __attribute__((always_inline)) {
                constexpr int I = decltype(i)::value;
                if constexpr (I == kTailHook) // at t == 0 nobody uses what these reads return
                    issueVStep(VOff(), std::integral_constant<int, 0>(), vFirst);
            }, std::integral_constant<int, kStepReads>());
        } else {
            issueVStep(VOff(), std::integral_constant<int, 0>(), vFirst);
        }
        if (t > 0)
            outputTile(stageTag, vFirst, pRight, alpha, anyRaise);
        __builtin_amdgcn_sched_barrier(0);
        phaseEnd();
        __builtin_amdgcn_sched_barrier(0);
        if (t < numTiles) {
            __builtin_amdgcn_s_setprio(0);
            loadBundle(t + 1 + group);
            softmaxTile(sAcc, t, pRight, alpha, anyRaise);
            __builtin_amdgcn_sched_barrier(0);
            phaseEnd();
        }
    };
    phaseEnd(); // K tile 0 has landed
    if (group == 1) {
        loadBundle(1);
        phaseEnd();
    }
    for (int tile = 0; tile <= numTiles; tile += 2) {
        ppStep(std::integral_constant<int, 0>(), tile);
        if (tile + 1 <= numTiles)
            ppStep(std::integral_constant<int, 1>(), tile + 1);
    }
    if (group == 0)
        phaseEnd();
    hw::wait_vm0(); // the copy issued by the last tile must not outlive the workgroup's LDS

    // ---- finish: O /= S, write O (and LSE) ----
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
        const float total = SumOverRowGroups(runSum[nq]);
        const float inv = 1.0f / total;
        const int64_t row = (int64_t)bh * seqQ + myQuery + 16 * nq;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int d = db * 16 + (int)g * 4;
            float o4[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                o4[r] = oAcc[db][nq][r] * inv;
            if constexpr (OUT_F32) {
                f32x4 v = {o4[0], o4[1], o4[2], o4[3]};
                *reinterpret_cast<f32x4 *>(static_cast<float *>(outO) + row * D + d) = v;
            } else {
                f16x4 v = {(half)o4[0], (half)o4[1], (half)o4[2], (half)o4[3]};
                *reinterpret_cast<f16x4 *>(static_cast<half *>(outO) + row * D + d) = v;
            }
        }
        if (outLse != nullptr && g == 0)
            outLse[row] = runMax[nq] * 0.08838834764831845f + __builtin_logf(total);
    }
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <int D, bool CAUSAL, bool OUT_F32>
int launch_fa_m16(hipStream_t st, void *o, float *lse, const half *q, const half *k, const half *v, int batch, int heads, int seqQ, int seqKv, int causalOff)
{
    if (seqQ % kBQ16 || seqKv % kBKV16)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 2 * 2 * kBKV16 * D * (int)sizeof(half);
    auto kernel = FlashAttnFwdM16<D, CAUSAL, OUT_F32>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int numBH = batch * heads;
    const long long blocks = (long long)numBH * (seqQ / kBQ16);
    if (blocks > 0x7fffffffLL)
        return PTO_ERR_UNSUPPORTED;
    kernel<<<dim3((unsigned)blocks), dim3(kBlockThreads), lds, st>>>(o, lse, q, k, v, heads, seqQ, seqKv, numBH, causalOff);
    return pto_amd::check_launch();
}
} // namespace
