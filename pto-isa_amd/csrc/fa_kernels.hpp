// Flash-attention forward kernel template and launcher, shared by the translation units that fix the
// wave grid (1 x 4 in pto_fa.hip, 1 x 8 in pto_fa_w8.hip).  Include after <pto/pto-inst.hpp>.
#pragma once
#include "common.hpp"
#include <cstdlib>

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kBQ1 = 32 * PTO_WAVES_N; // queries per workgroup: one 32-query block per wave
constexpr int kBKVDefault = 64; // keys per tile
constexpr float kMaskValue = -3.40282e+38f; // pto_macro_fa_softmax.hpp:67

// max of x and of the value that the lane 32 positions away holds: one cross-half register swap
// (after it `a` holds the lower half-wave's values in both halves, `b` the upper half-wave's)
AICORE inline float MaxOverHalves(float x)
{
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}
AICORE inline float SumOverHalves(float x)
{
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));

// Row r of the K operand (and so of X^T and P^T) holds key KeyOfRow(r): a permutation inside every
// group of 16 keys, chosen so that the four keys which one transposing read of V^T gathers (rows
// 4a .. 4a+3) lie in four different 64-byte bank groups of the swizzled [keys, D] LDS image:
// the XOR swizzle moves the 16-byte chunk by key % 16 for 256-byte rows (D = 128: the keys differ
// in bits 2-3) and by (key / 2) % 8 for 128-byte rows, two rows per bank line (D = 64: bits 0 and 3).
template <int D>
AICORE inline constexpr uint32_t KeyOfRow(uint32_t r)
{
    const uint32_t a = (r >> 2) & 3u, b = r & 3u;
    if (D == 128)
        return (r & ~15u) | (b << 2) | a;
    return (r & ~15u) | (b & 1u) | ((b >> 1) << 3) | (a << 1);
}

// compile-time loop: f(integral_constant<int, I>) for I = FIRST .. LAST-1
template <int FIRST, int LAST, typename F>
AICORE inline void StaticFor(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        StaticFor<FIRST + 1, LAST>(f);
    }
}

// K operand for X^T = K Q^T, one 16-wide step of the head dimension at a time: fragment (kb, ks) =
// rows kb*32 .. +31 (row r <- key KeyOfRow(r)) x d = 16 ks .. +15 of the key tile.  Issued as
// assembly, like the V^T reads below, so that the order of issue and the lookahead are what the
// source says: fragment i+kAhead is requested before the MFMA on fragment i.
template <int D>
struct KReader {
    static constexpr int KS = D / 16;
    static constexpr uint32_t kRowBytes = D * (uint32_t)sizeof(half);
    uint32_t base[KS]; // LDS byte address of this lane's 16 bytes of step ks, block 0, tile at LDS offset 0

    AICORE inline void Init()
    {
        const uint32_t lane = (uint32_t)hw::lane();
        const uint32_t key = KeyOfRow<D>(lane & 31u), khalf = lane >> 5;
        const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)hw::lds_base();
        static_assert(detail::mat_swz<kRowBytes>(32) == detail::mat_swz<kRowBytes>(0), "the swizzle repeats every 32 keys");
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            base[ks] = ldsBase + detail::mat_chunk_off<kRowBytes>(key, khalf + 2u * ks);
    }
    template <uint32_t LDS_OFF, int KB_, int KS_>
    AICORE inline void Issue(f16x8 &f) const
    {
        constexpr uint32_t off = LDS_OFF + KB_ * 32u * kRowBytes;
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

// One transposing 64-bit LDS read at byte address addr + OFF.
template <uint32_t OFF>
AICORE inline s16x4 DsReadTr16(uint32_t addr)
{
    static_assert(OFF < 65536u, "the offset field of an LDS instruction has 16 bits");
    s16x4 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

// V^T operand for O^T += V^T P^T: TEXTRACT of [32 d, 16 keys] pieces of the transposed V tile, taken
// straight from the row-major [keys, D] LDS image with transposing reads.  Key order inside every
// 16-key MFMA step matches the order in which the accumulator layout holds P^T:
// k slot j of half-wave h  <->  row 16t + 8(j/4) + 4h + j%4 of X^T, which holds key KeyOfRow(row).
//
// The reads are issued as assembly so that they carry no compiler-visible LDS dependency: before a
// compiler-generated LDS read that may alias an outstanding asynchronous copy into LDS the compiler
// waits for every outstanding copy, which would make the prefetch of the next tile synchronous.
// The workgroup barrier at the top of a tile is what orders these reads after the copy that filled
// the stage.  The matching wait on the LDS counter (LDS operations of a wave complete in order: at
// most N younger ones may still be outstanding) names the fragment registers as operands so that
// no use of them can be moved above it.
template <int D, int kBKV>
struct VTReader {
    static constexpr int DB = D / 32;
    static constexpr uint32_t kStepBytes = 16u * D * (uint32_t)sizeof(half);
    static_assert(kBKV == 32 || kBKV == 64, "key tiles of 32 or 64");
    uint32_t base[DB][2]; // LDS byte address of (block db, read u) for key step 0 of a tile at LDS offset 0

    template <typename MatT>
    AICORE inline void Init()
    {
        using Geo = detail::MatGeom<MatT>;
        static_assert(detail::mat_swz<Geo::RowBytes>(16) == detail::mat_swz<Geo::RowBytes>(0), "the swizzle repeats every 16 keys");
        const uint32_t lane = (uint32_t)hw::lane();
        const uint32_t h = lane >> 5, keyIn = (lane & 15u) >> 2;
        const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)hw::lds_base();
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint32_t d0 = (uint32_t)db * 32u + 16u * ((lane >> 4) & 1u) + 4u * (lane & 3u);
                const uint32_t key = KeyOfRow<D>(8u * u + 4u * h + keyIn);
                base[db][u] = ldsBase + detail::mat_chunk_off<Geo::RowBytes>(key, d0 >> 3) + ((d0 & 7u) << 1);
            }
    }
};

template <int D, bool CAUSAL, bool OUT_F32, int MIN_BLOCKS, int kBKV = kBKVDefault, bool PP = false, int NQ_ = 1>
__global__ __launch_bounds__(kBlockThreads, MIN_BLOCKS) AICORE void FlashAttnFwd(__gm__ void *outO, __gm__ float *outLse,
                                                                      __gm__ const half *qAll, __gm__ const half *kAll,
                                                                      __gm__ const half *vAll, int heads, int seqQ,
                                                                      int seqKv, int numBH, int causalOff)
{
    constexpr int NQ = NQ_;        // 32-query blocks per wave
    constexpr int kBQ = kBQ1 * NQ; // queries per workgroup
    constexpr int KB = kBKV / 32;  // 32-key blocks per tile
    constexpr int DB = D / 32;    // 32-wide blocks of the head dimension
    // ---- tiles ----
    using TileMatQ = Tile<TileType::Mat, half, D, kBQ, BLayout::RowMajor, D, kBQ, SLayout::ColMajor>;   // Q^T, contiguous along d
    using TileMatK = Tile<TileType::Mat, half, kBKV, D, BLayout::ColMajor, kBKV, D, SLayout::RowMajor>; // K,   contiguous along d
    using TileMatV = Tile<TileType::Mat, half, kBKV, D, BLayout::ColMajor, kBKV, D, SLayout::RowMajor>; // V,   contiguous along d
    using RightQ = TileRight<half, D, kBQ, D, kBQ>;        // per wave: 32 queries x D
    using LeftK = TileLeft<half, 32, D, 32, D>;            // 32 keys x D (every wave holds the same keys)
    using AccS = TileAcc<float, 32, kBQ, 32, kBQ>;         // X^T block: 32 keys x 32 queries per wave
    using RightP = TileRight<half, kBKV, kBQ, kBKV, kBQ>;  // P^T: kBKV keys x 32 queries per wave
    using LeftVT = TileLeft<half, 32, kBKV, 32, kBKV>;     // V^T block: 32 d x kBKV keys
    using AccO = TileAcc<float, 32, kBQ, 32, kBQ>;         // O^T block: 32 d x 32 queries per wave

    using GlobalQT = GlobalTensor<half, TileShape2D<half, D, kBQ, Layout::DN>, Stride<1, 1, 1, 1, D>, Layout::DN>;
    using GlobalKV = GlobalTensor<half, TileShape2D<half, kBKV, D, Layout::ND>, Stride<1, 1, 1, D, 1>, Layout::ND>;

    constexpr uint32_t kTileBytes = kBKV * D * sizeof(half);
    constexpr uint32_t kStageBytes = 2 * kTileBytes;
    static_assert(D * kBQ * sizeof(half) <= 2 * kStageBytes, "Q^T is staged in the K/V stages");

    // ---- which (batch*head, query tile) this workgroup owns.  Workgroups are dealt round-robin to
    // the 8 XCDs: keep a head on one XCD so that its K/V stay in that XCD's L2.  Causal: the query
    // tiles with the most keys go first.
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
    if (CAUSAL) { // tiles wholly above the diagonal are skipped (fa_performance_kernel.cpp:757-758)
        const int lastKey = q0 + kBQ - 1 + causalOff;
        const int lim = lastKey / kBKV + 1;
        numTiles = lim < numTiles ? lim : numTiles;
    }

    TileMatK kMat[2];
    TileMatV vMat[2];
    TileMatQ qMat;
    TASSIGN(kMat[0], 0u);
    TASSIGN(vMat[0], kTileBytes);
    TASSIGN(kMat[1], kStageBytes);
    TASSIGN(vMat[1], kStageBytes + kTileBytes);
    TASSIGN(qMat, 0u); // staged over both K/V stages until it has been extracted

    RightQ qRight;
    AccO oAcc[DB];
    float runMax[NQ], runSum[NQ]; // per lane and query block; runSum is the half-wave partial
    const int lane = hw::lane();
    // row of Q that this lane's column of query block 0 holds (block nb: + 32 nb)
    const int myQuery = q0 + hw::wave_n() * (32 * NQ) + (lane & 31);
    const uint32_t hHalf = (uint32_t)lane >> 5;
    // s = 1/sqrt(D) folded with log2(e): exp(s y) = exp2(s log2e y)
    const float sLog2e = (D == 128 ? 0.08838834764831845f : 0.125f) * 1.4426950408889634f;

    // ---- the three stages of one key tile ----
    // X^T = K Q^T for the key tile in LDS stage st: one MFMA per K fragment, fragments requested kAhead MFMAs ahead
    KReader<D> kr;
    kr.Init();
    // `between(i)` runs before the MFMA on fragment i (the caller issues its asynchronous copies there).
    // A scheduling barrier after every MFMA keeps the issue order exactly as written.
    // `extraTag`: number of LDS reads that between(kTotal - kAhead) issues itself (they are younger than every K read).
    constexpr int kAheadK = 4, kTailHook = KB * (D / 16) - kAheadK;
    auto scoreTile = [&](AccS(&sAcc)[KB], auto stageTag, auto &&between, auto extraTag) {
        constexpr uint32_t kOff = decltype(stageTag)::value * kStageBytes;
        constexpr int KSTEPS = D / 16, kTotal = KB * KSTEPS, kAhead = kAheadK, kExtra = decltype(extraTag)::value;
        using LeftStep = TileLeft<half, 32, 16, 32, 16>;
        using RightStep = TileRight<half, 16, kBQ, 16, kBQ>;
        f16x8 frag[kAhead + 1];
        StaticFor<0, kAhead>([&](auto i) {
            constexpr int I = decltype(i)::value;
            kr.template Issue<kOff, I % KB, I / KB>(frag[I % (kAhead + 1)]);
        });
        StaticFor<0, kTotal>([&](auto i) {
            constexpr int I = decltype(i)::value, J = I + kAhead;
            if constexpr (J < kTotal)
                kr.template Issue<kOff, J % KB, J / KB>(frag[J % (kAhead + 1)]);
            between(i);
            KReader<D>::template Wait<(kTotal - 1 - I < kAhead ? kTotal - 1 - I : kAhead) + (I >= kTailHook ? kExtra : 0)>(
                frag[I % (kAhead + 1)]);
            constexpr int kb = I % KB, ks = I / KB; // the KB accumulator chains alternate
            LeftStep a;
            RightStep b;
            a.st.f[0][0] = frag[I % (kAhead + 1)];
#pragma unroll
            for (int nb = 0; nb < NQ; ++nb)
                b.st.f[nb][0] = qRight.st.f[nb][ks];
            if constexpr (ks == 0)
                TMATMUL(sAcc[kb], a, b);
            else
                TMATMUL_ACC(sAcc[kb], sAcc[kb], a, b);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // streaming softmax on the accumulator fragments of tile t (one query per lane and query block)
    auto softmaxTile = [&](AccS(&sAcc)[KB], int t, RightP &pRight, float(&alpha)[NQ], bool &anyRaise) {
        const int key0 = t * kBKV;
        if (CAUSAL && key0 + kBKV - 1 > q0 + causalOff) { // the diagonal crosses this tile
#pragma unroll
            for (int nb = 0; nb < NQ; ++nb) {
                const int limit = myQuery + 32 * nb + causalOff; // last visible key of this lane's query
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = key0 + kb * 32 + (int)KeyOfRow<D>((v >> 2) * 8 + hHalf * 4 + (v & 3));
                        if (key > limit)
                            sAcc[kb].st.f[0][nb][v] += kMaskValue;
                    }
            }
        }
        // The running max only has to bound the scores well enough to keep exp() in range: it is raised (and O, S
        // rescaled by alpha) when a tile exceeds it by more than kSlack in the exponent, i.e. P stays below 2^kSlack.
        // O / S and max*s + ln(S) do not depend on the choice.
        // Every tile but the first is tried with the running max as it stands.  A lane's partial row sum bounds each
        // of its P from above, so a sum of at most 2^kSlack proves that no score of the tile exceeds the running max
        // by more than the slack: the max stays, nothing is rescaled, and the row max of the tile is never computed.
        // Otherwise (a larger sum, an infinity or a NaN in any lane of the wave) the wave finds the row max, raises
        // the running max where it has to, and runs the exponentials a second time.
        constexpr float kSlack = 8.0f;
        anyRaise = false;
        float locSum[NQ];
#pragma unroll
        for (int nb = 0; nb < NQ; ++nb)
            alpha[nb] = 1.0f;
        bool needMax = t == 0; // wave-uniform
#pragma nounroll
        for (;;) {             // at most two rounds
            if (needMax) {
                anyRaise = t == 0;
#pragma unroll
                for (int nb = 0; nb < NQ; ++nb) {
                    float locMax = sAcc[0].st.f[0][nb][0];
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            locMax = fmaxf(locMax, sAcc[kb].st.f[0][nb][v]);
                    locMax = MaxOverHalves(locMax);
                    const bool raise = t == 0 || (locMax - runMax[nb]) * sLog2e > kSlack;
                    const float newMax = raise ? locMax : runMax[nb];
                    if (t > 0)
                        anyRaise = anyRaise || __builtin_amdgcn_ballot_w64(raise) != 0;
                    alpha[nb] = (t == 0 || !raise) ? 1.0f : __builtin_amdgcn_exp2f((runMax[nb] - newMax) * sLog2e);
                    runMax[nb] = newMax;
                }
            }
            bool within = true;
#pragma unroll
            for (int nb = 0; nb < NQ; ++nb) {
                const float negMax = -runMax[nb] * sLog2e;
                float part[4] = {0.0f, 0.0f, 0.0f, 0.0f}; // four partial sums: no long chain of dependent additions
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int half_ = 0; half_ < 2; ++half_) {
                        f16x8 pk;
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const float p =
                                __builtin_amdgcn_exp2f(__builtin_fmaf(sAcc[kb].st.f[0][nb][half_ * 8 + j], sLog2e, negMax));
                            part[j & 3] += p; // row sum over the fp32 P, as the reference does
                            pk[j] = (half)p;
                        }
                        pRight.st.f[nb][kb * 2 + half_] = pk;
                    }
                locSum[nb] = (part[0] + part[1]) + (part[2] + part[3]);
                within = within && locSum[nb] <= 256.0f; // 2^kSlack; false for a NaN
            }
            static_assert(kSlack == 8.0f, "the bound above is 2^kSlack");
            if (needMax || __builtin_amdgcn_ballot_w64(!within) == 0)
                break;
            needMax = true;
        }
#pragma unroll
        for (int nb = 0; nb < NQ; ++nb)
            runSum[nb] = t == 0 ? locSum[nb] : runSum[nb] * alpha[nb] + locSum[nb];
    };
    using VT = VTReader<D, kBKV>;
    VT vt;
    vt.template Init<TileMatV>();
    // O^T += V^T P^T with the 16-key step as the outer loop: consecutive MFMAs go to different accumulator
    // blocks.  (An MFMA that needs the result of the one before it can only issue in the very cycle that one
    // ends; when another wave of the SIMD issues vector instructions meanwhile, every such issue slips and the
    // matrix pipe idles.  Independent MFMAs queue up behind each other and absorb the slips.)
    // One step = the V^T fragments of all DB blocks for 16 keys; the step after it is in flight.
    struct VStep {
        s16x4 part[DB][2];
    };
    constexpr int kStepReads = 2 * DB;
    auto issueVStep = [&](auto offTag, auto ksTag, VStep &f) {
        constexpr uint32_t off = decltype(offTag)::value + decltype(ksTag)::value * VT::kStepBytes;
        StaticFor<0, DB>([&](auto dbTag) {
            constexpr int db = decltype(dbTag)::value;
            f.part[db][0] = DsReadTr16<off>(vt.base[db][0]);
            f.part[db][1] = DsReadTr16<off>(vt.base[db][1]);
        });
    };
    auto waitVStep = [&](auto nTag, VStep &f) {
        constexpr int N = decltype(nTag)::value;
        static_assert(N >= 0 && N <= 15, "the LDS counter has 4 bits");
        if constexpr (DB == 4)
            asm volatile("s_waitcnt lgkmcnt(%8)"
                         : "+v"(f.part[0][0]), "+v"(f.part[0][1]), "+v"(f.part[1][0]), "+v"(f.part[1][1]), "+v"(f.part[2][0]),
                           "+v"(f.part[2][1]), "+v"(f.part[3][0]), "+v"(f.part[3][1])
                         : "n"(N));
        else
            asm volatile("s_waitcnt lgkmcnt(%4)"
                         : "+v"(f.part[0][0]), "+v"(f.part[0][1]), "+v"(f.part[1][0]), "+v"(f.part[1][1])
                         : "n"(N));
    };
    // `first` holds step 0 (requested earlier); oAcc must have been initialised (this always accumulates)
    auto outputTileWide = [&](auto stageTag, VStep &first, RightP &pRight, float(&alpha)[NQ], bool anyRaise) {
        using VOff = std::integral_constant<uint32_t, decltype(stageTag)::value * kStageBytes + kTileBytes>;
        using LeftStep = TileLeft<half, 32, 16, 32, 16>;
        using RightStep = TileRight<half, 16, kBQ, 16, kBQ>;
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        constexpr int KS = kBKV / 16;
        VStep other;
        if (anyRaise) { // wave-uniform: some lane's max was raised
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int nb = 0; nb < NQ; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        oAcc[db].st.f[0][nb][v] *= alpha[nb];
        }
        StaticFor<0, KS>([&](auto ksTag) {
            constexpr int ks = decltype(ksTag)::value;
            VStep &cur = (ks & 1) ? other : first;
            VStep &nxt = (ks & 1) ? first : other;
            if constexpr (ks + 1 < KS) {
                issueVStep(VOff(), std::integral_constant<int, ks + 1>(), nxt);
                waitVStep(std::integral_constant<int, kStepReads>(), cur);
            } else {
                waitVStep(std::integral_constant<int, 0>(), cur);
            }
            RightStep b;
#pragma unroll
            for (int nb = 0; nb < NQ; ++nb)
                b.st.f[nb][0] = pRight.st.f[nb][ks];
            StaticFor<0, DB>([&](auto dbTag) {
                constexpr int db = decltype(dbTag)::value;
                const s16x8 both = {cur.part[db][0][0], cur.part[db][0][1], cur.part[db][0][2], cur.part[db][0][3],
                                    cur.part[db][1][0], cur.part[db][1][1], cur.part[db][1][2], cur.part[db][1][3]};
                LeftStep a;
                a.st.f[0][0] = __builtin_bit_cast(f16x8, both);
                TMATMUL_ACC(oAcc[db], oAcc[db], a, b);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    auto keyTile = [&](__gm__ half *base, int t) {
        const int tc = t < numTiles ? t : numTiles - 1; // past the end: re-fetch the last tile (nobody reads it)
        return GlobalKV(base + (int64_t)tc * kBKV * D);
    };
    constexpr int kScoreFrags = KB * (D / 16); // K fragments of one tile = calls of the score stage's hook

#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int nb = 0; nb < NQ; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                oAcc[db].st.f[0][nb][v] = 0.0f;
    {
        GlobalQT gmQ(qBase);
        TLOAD(qMat, gmQ);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        TEXTRACT(qRight, qMat, 0, 0);
        set_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1);
        wait_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1); // Q^T is in registers everywhere: the stages may be filled
        GlobalKV gmK(kBase), gmV(vBase);
        TLOAD(kMat[0], gmK);
        if constexpr (!PP)
            TLOAD(vMat[0], gmV);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    }

    if constexpr (PP) {
        // ---- two groups of four waves in opposite phases ----
        // A SIMD issues one matrix or vector instruction per slot, and inside one wave an MFMA and the vector
        // instructions after it do not overlap: the softmax of one wave can only hide under the MFMAs of ANOTHER
        // wave of its SIMD.  Waves w and w+4 share a SIMD.  Time is cut into phases by workgroup barriers; in every
        // phase one group (waves 0-3 in even phases, waves 4-7 in odd ones) runs the MFMAs of O^T += V^T P^T for its
        // tile t-1 and of X^T = K Q^T for its tile t, while the other group runs the softmax of its tile and
        // issues its share of the copies for the coming phases.
        //   bundle b = {K tile b, V tile b-1} lives in stage b % 2 and is read in phases 2b (first group) and
        //   2b+1 (second group); it is copied during phases 2b-2 (second group's share) and 2b-1 (first group's),
        //   i.e. in its softmax phase of step t a wave of group g copies its share of bundle t+1+g.
        // The wave in its MFMA phase runs at raised priority.
        static_assert(kBlockWaves == 8 && NQ == 1, "two groups of four waves");
        const int group = hw::wave_n() >> 2;
        AccS sAcc[KB];
        RightP pRight;
        float alpha[NQ];
        bool anyRaise = false;
        auto phaseEnd = [&]() { // own copies landed, own LDS reads done, everyone arrived
            set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
            wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        };
        auto loadBundle = [&](int b) { // this wave's share of bundle b
            TileMatK kDst;
            TileMatV vDst;
            const uint32_t off = (uint32_t)(b & 1) * kStageBytes;
            TASSIGN(kDst, off);
            TASSIGN(vDst, off + kTileBytes);
            GlobalKV gmK = keyTile(kBase, b), gmV = keyTile(vBase, b - 1);
            TLOAD(kDst, gmK);
            TLOAD(vDst, gmV);
        };
        // Step t of a wave: MFMA phase = scores of tile t, then output of tile t-1; softmax phase = tile t.
        // The first V^T step is requested right after the last K fragment so that the output MFMAs follow the
        // score MFMAs without a gap.  The copies are issued at the start of the softmax phase, which is the
        // shorter of the two (measured: a copy instruction holds its wave for 30-100 cycles wherever it sits).
        auto ppStep = [&](auto stageTag, int t) {
            constexpr int st = decltype(stageTag)::value;
            using VOff = std::integral_constant<uint32_t, st * kStageBytes + kTileBytes>;
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(3); // the wave that feeds the matrix pipe issues first
            VStep vFirst;
            if (t < numTiles) {
                scoreTile(sAcc, stageTag, [&](auto i) {
                    constexpr int I = decltype(i)::value;
                    if constexpr (I == kTailHook) // at t == 0 nobody uses what these reads return
                        issueVStep(VOff(), std::integral_constant<int, 0>(), vFirst);
                }, std::integral_constant<int, kStepReads>());
            } else {
                issueVStep(VOff(), std::integral_constant<int, 0>(), vFirst);
            }
            if (t > 0)
                outputTileWide(stageTag, vFirst, pRight, alpha, anyRaise);
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
        if (group == 1) { // phase 0: the second group has no scores yet
            loadBundle(1);
            phaseEnd();
        }
        for (int tile = 0; tile <= numTiles; tile += 2) {
            ppStep(std::integral_constant<int, 0>(), tile);
            if (tile + 1 <= numTiles)
                ppStep(std::integral_constant<int, 1>(), tile + 1);
        }
        if (group == 0) // pairs with the barrier that ends the second group's last phase
            phaseEnd();
    } else {
    // One key tile in LDS stage st (a compile-time constant: every LDS address is an immediate).
    auto tileStep = [&](auto stageTag, int t) {
        constexpr int st = decltype(stageTag)::value;
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); // tile t has landed; everyone left tile t-1
        // The next tile is fetched while this tile's score MFMAs issue: the K copies before the second
        // MFMA, the V copies halfway.  Past the last tile the copies re-fetch it into the free stage,
        // which keeps the loop free of special cases.
        AccS sAcc[KB];
        __builtin_amdgcn_sched_barrier(0);
        scoreTile(sAcc, stageTag, [&](auto i) {
            constexpr int I = decltype(i)::value;
            if constexpr (I == 1) {
                GlobalKV gmK = keyTile(kBase, t + 1);
                TLOAD(kMat[st ^ 1], gmK);
            }
            if constexpr (I == kScoreFrags / 2 + 1) {
                GlobalKV gmV = keyTile(vBase, t + 1);
                TLOAD(vMat[st ^ 1], gmV);
                set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
            }
        }, std::integral_constant<int, 0>());
        VStep vFirst; // lands during the softmax
        issueVStep(std::integral_constant<uint32_t, st * kStageBytes + kTileBytes>(), std::integral_constant<int, 0>(), vFirst);
        RightP pRight;
        float alpha[NQ];
        bool anyRaise;
        softmaxTile(sAcc, t, pRight, alpha, anyRaise);
        outputTileWide(stageTag, vFirst, pRight, alpha, anyRaise);
    };
    for (int tile = 0; tile < numTiles; tile += 2) {
        tileStep(std::integral_constant<int, 0>(), tile);
        if (tile + 1 < numTiles)
            tileStep(std::integral_constant<int, 1>(), tile + 1);
    }
    }
    hw::wait_vm0(); // the copy issued by the last tile must not outlive the workgroup's LDS
    // ---- finish: O /= S, write O (and LSE) ----
#pragma unroll
    for (int nb = 0; nb < NQ; ++nb) {
        const float total = SumOverHalves(runSum[nb]);
        const float inv = 1.0f / total;
        const int64_t row = (int64_t)bh * seqQ + myQuery + 32 * nb;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = db * 32 + g * 8 + (int)hHalf * 4;
                float o4[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    o4[r] = oAcc[db].st.f[0][nb][g * 4 + r] * inv;
                if constexpr (OUT_F32) {
                    f32x4 v = {o4[0], o4[1], o4[2], o4[3]};
                    *reinterpret_cast<f32x4 *>(static_cast<float *>(outO) + row * D + d) = v;
                } else {
                    f16x4 v = {(half)o4[0], (half)o4[1], (half)o4[2], (half)o4[3]};
                    *reinterpret_cast<f16x4 *>(static_cast<half *>(outO) + row * D + d) = v;
                }
            }
        if (outLse != nullptr && hHalf == 0) {
            const float scale = D == 128 ? 0.08838834764831845f : 0.125f;
            outLse[row] = runMax[nb] * scale + __builtin_logf(total);
        }
    }
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <int D, bool CAUSAL, bool OUT_F32, int MIN_BLOCKS = 1, int kBKV = kBKVDefault, bool PP = false, int NQ = 1>
int launch_fa(hipStream_t st, void *o, float *lse, const half *q, const half *k, const half *v, int batch, int heads,
              int seqQ, int seqKv, int causalOff)
{
    constexpr int kBQ = kBQ1 * NQ;
    if (seqQ % kBQ || seqKv % kBKV)
        return PTO_ERR_UNSUPPORTED;
    static_assert(D * kBQ <= 4 * kBKV * D, "Q^T must fit the K/V stages it is staged in");
    constexpr int lds = 2 * 2 * kBKV * D * (int)sizeof(half);
    auto kernel = FlashAttnFwd<D, CAUSAL, OUT_F32, MIN_BLOCKS, kBKV, PP, NQ>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int numBH = batch * heads;
    const long long blocks = (long long)numBH * (seqQ / kBQ);
    if (blocks > 0x7fffffffLL)
        return PTO_ERR_UNSUPPORTED;
    kernel<<<dim3((unsigned)blocks), dim3(kBlockThreads), lds, st>>>(o, lse, q, k, v, heads, seqQ, seqKv, numBH, causalOff);
    return pto_amd::check_launch();
}
} // namespace

