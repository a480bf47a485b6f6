// GEMM tile with K-steps of 64: every row of an A / B panel is one whole 128-byte memory line per K-step.
//
// With K-steps of 32 a row segment is 64 bytes, half a line: the vector L1 fetches whole 128-byte lines from the L2, the
// 36 KiB that a K-step streams through it evict the other half before the next K-step asks for it, and every line
// crosses the L2 -> L1 path twice.  The counters of the K-32 kernel at 6144^3 read 5.98e7 L2 requests per launch for
// 3.6 GB of operand bytes (64 useful bytes per 128-byte request) and the L1 waits for L2 data in 56 % of its cycles.
//
// Two LDS stages of one K-64 step each (384 x 192 tile: 72 KiB per stage) and two sets of operand fragments, one per
// 32-wide half of a step.  The one workgroup barrier of a step sits in its middle, where the wave has read the last
// fragments of the stage: the copies of a step have a whole step (more than 2000 cycles) to land, and every fragment read
// is issued between MFMAs (with the barrier at the top of the step all eight waves would ask for 120 KiB of fragments at
// once and wait for the LDS to deliver them).
#pragma once
#include "gemm_kernels.hpp"

PTO_DEVICE_CODE_BEGIN

namespace {

template <int BM, int BN>
AICORE inline __attribute__((always_inline)) void MixTileRowsK64(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1,
                                                                 int m, int n, int k, int row0, int col0, int kLoop)
{
    constexpr int BK = 64, KS = 32, HM = BM / 2;
    using TileMatA = Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, half, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using LeftHalf = TileLeft<half, HM, KS, HM, KS>;
    using RightTile = TileRight<half, KS, BN, KS, BN>;
    using AccHalf = TileAcc<float, HM, BN, HM, BN>;
    using ShapeA = TileShape2D<half, BM, BK, Layout::ND>;
    using StrideA = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalA = GlobalTensor<half, ShapeA, StrideA, Layout::ND>;
    using ShapeB = TileShape2D<half, BK, BN, Layout::DN>;
    using StrideB = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::DN>;
    using GlobalB = GlobalTensor<half, ShapeB, StrideB, Layout::DN>;
    using ShapeC = TileShape2D<float, HM, BN, Layout::ND>;
    using StrideC = BaseShape2D<float, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<float, ShapeC, StrideC, Layout::ND>;

    constexpr uint32_t kABytes = BM * BK * sizeof(half), kBBytes = BK * BN * sizeof(half);
    constexpr uint32_t kStage = kABytes + kBBytes;
    constexpr int kLoadsPerStep = TLoadInstrs<TileMatA>() + TLoadInstrs<TileMatB>();
    constexpr int kMfmaPerHalfK = 2 * AccHalf::Storage::MB * AccHalf::Storage::NB; // both row halves, one 32-wide K half
    constexpr int kReadsPerHalfK = 2 * LeftHalf::Storage::MB + RightTile::Storage::NB;
    static_assert(LeftHalf::Storage::KS == 1 && RightTile::Storage::KS == 1, "one MFMA spans a 32-wide K half");
    // issue pattern (measured): the reads of the first half are spread over the first 6/8 of its MFMAs, the copies and
    // then the reads of the second half over its first 7/8
    constexpr int kF1 = 6, kF2 = 7;

    __gm__ half *aPanel = const_cast<half *>(src0) + (int64_t)row0 * k;
    __gm__ half *bPanel = const_cast<half *>(src1) + (int64_t)col0 * k;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);

    TileMatA aMat[2];
    TileMatB bMat[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        TASSIGN(aMat[s], s * kStage);
        TASSIGN(bMat[s], s * kStage + kABytes);
    }
    LeftHalf aUp[2], aDn[2];
    RightTile bAll[2];
    AccHalf cUp, cDn;
#pragma unroll
    for (int mb = 0; mb < AccHalf::Storage::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < AccHalf::Storage::NB; ++nb)
#pragma unroll
            for (int i = 0; i < detail::kAccElems; ++i) {
                cUp.st.f[mb][nb][i] = 0.0f;
                cDn.st.f[mb][nb][i] = 0.0f;
            }

    // Prologue: step 0 into stage 0, wait for it, then step 1 into stage 1 and the fragments of the first half of step 0.
    {
        GlobalA gmA(aPanel, ShapeA(), strideA);
        GlobalB gmB(bPanel, ShapeB(), strideB);
        TLOAD(aMat[0], gmA);
        TLOAD(bMat[0], gmB);
        hw::wait_vm0();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        GlobalA gmA1(aPanel + BK, ShapeA(), strideA);
        GlobalB gmB1(bPanel + BK, ShapeB(), strideB);
        TLOAD(aMat[1], gmA1);
        TLOAD(bMat[1], gmB1);
        TEXTRACT(bAll[0], bMat[0], 0, 0);
        TEXTRACT(aUp[0], aMat[0], 0, 0);
        TEXTRACT(aDn[0], aMat[0], HM, 0);
        __builtin_amdgcn_sched_barrier(0);
    }

    // One K-64 step on stage s (the host guarantees kLoop % 2 == 0 and kLoop >= 2), rotated by half a step so that no
    // fragment read waits behind the barrier:
    //   first half:  MFMAs on the fragments of K half 0 (read during the step before), reads of K half 1 between them;
    //   the stage is now dead for this wave: wait for this wave's copies of step it+1 (issued one step ago) and for the
    //   workgroup (stage s^1 has landed for everyone, stage s is dead for everyone), issue the copies of step it+2 into
    //   stage s;
    //   second half: MFMAs on K half 1, the copies and the reads of K half 0 of step it+1 (stage s^1) between them.
    // Past the end of K the copies re-fetch the last step and the reads fetch values nobody uses: no branches in the loop.
    auto step = [&](auto stageTag, int it) {
        constexpr int s = decltype(stageTag)::value;
        TMATMUL_ACC(cUp, cUp, aUp[0], bAll[0]);
        TMATMUL_ACC(cDn, cDn, aDn[0], bAll[0]);
        TEXTRACT(bAll[1], bMat[s], KS, 0);
        TEXTRACT(aUp[1], aMat[s], 0, KS);
        TEXTRACT(aDn[1], aMat[s], HM, KS);
        StaticFor<0, kReadsPerHalfK>([](auto iTag) {
            constexpr int i = decltype(iTag)::value;
            constexpr int budget = kMfmaPerHalfK * kF1 / 8; // the rest of the half has no read after it
            constexpr int nMfma = (i + 1) * budget / kReadsPerHalfK - i * budget / kReadsPerHalfK;
            if constexpr (nMfma > 0)
                __builtin_amdgcn_sched_group_barrier(0x008, nMfma, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        if constexpr (kMfmaPerHalfK - kMfmaPerHalfK * kF1 / 8 > 0)
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerHalfK - kMfmaPerHalfK * kF1 / 8, 0);
        __builtin_amdgcn_sched_barrier(0);
        hw::wait_lgkm0(); // the K half 1 fragments are in registers: this wave is done with stage s
        hw::wait_vm0();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int fetch = it + 2 < kLoop ? it + 2 : kLoop - 1;
        GlobalA gmA(aPanel + (int64_t)fetch * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)fetch * BK, ShapeB(), strideB);
        TLOAD(aMat[s], gmA);
        TLOAD(bMat[s], gmB);
        TMATMUL_ACC(cUp, cUp, aUp[1], bAll[1]);
        TMATMUL_ACC(cDn, cDn, aDn[1], bAll[1]);
        TEXTRACT(bAll[0], bMat[s ^ 1], 0, 0);
        TEXTRACT(aUp[0], aMat[s ^ 1], 0, 0);
        TEXTRACT(aDn[0], aMat[s ^ 1], HM, 0);
        constexpr int kSlots = kLoadsPerStep + kReadsPerHalfK;
        StaticFor<0, kSlots>([](auto iTag) {
            constexpr int i = decltype(iTag)::value;
            constexpr int budget = kMfmaPerHalfK * kF2 / 8;
            constexpr int nMfma = (i + 1) * budget / kSlots - i * budget / kSlots;
            if constexpr (nMfma > 0)
                __builtin_amdgcn_sched_group_barrier(0x008, nMfma, 0);
            if constexpr (i < kLoadsPerStep) // the copies, then the reads (the other orders spill)
                __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
            else
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        if constexpr (kMfmaPerHalfK - kMfmaPerHalfK * kF2 / 8 > 0)
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerHalfK - kMfmaPerHalfK * kF2 / 8, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    for (int it = 0; it < kLoop; it += 2) {
        step(integral_constant<int, 0>(), it);
        step(integral_constant<int, 1>(), it + 1);
    }
    hw::wait_vm0(); // the copy issued past the end of K must not outlive the workgroup's LDS
    GlobalC dstUp(out + (int64_t)row0 * n + col0, ShapeC(), StrideC(m, n));
    GlobalC dstDn(out + (int64_t)(row0 + HM) * n + col0, ShapeC(), StrideC(m, n));
    TSTORE(dstUp, cUp);
    TSTORE(dstDn, cDn);
}

// One BM x BN tile of C per workgroup, whole tiles only.
template <int BM, int BN, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32K64(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k)
{
    const int tilesM = m / BM, tilesN = n / BN;
    int tm, tn;
    TileOfId<GROUP_M>(RegroupXcd((int)get_block_idx(), tilesM * tilesN), tilesM, tilesN, tm, tn);
    MixTileRowsK64<BM, BN>(out, src0, src1, m, n, k, tm * BM, tn * BN, k / 64);
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <int BM, int BN, int GROUP_M>
int launch_gemm_k64(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    if (m % BM || n % BN || k % 128 || k < 128)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 2 * (BM * 64 + 64 * BN) * (int)sizeof(half);
    static_assert(lds <= 160 * 1024, "two K-64 stages must fit the LDS");
    auto kernel = GemmF16F32K64<BM, BN, GROUP_M>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = (m / BM) * (n / BN);
    kernel<<<dim3(tiles), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}
} // namespace
