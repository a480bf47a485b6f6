// GEMM kernels of the PTO tile path, shared by the translation units that instantiate them for
// different wave grids (PTO_WAVES_M x PTO_WAVES_N is fixed per translation unit).
#pragma once
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kXcds = 8; // MI355X: 8 accelerator dies, workgroups are dealt to them round-robin

// compile-time loop: f(integral_constant<int, I>) for I = FIRST .. LAST-1
template <int FIRST, int LAST, typename F>
AICORE inline void StaticFor(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        StaticFor<FIRST + 1, LAST>(f);
    }
}

// Workgroup id -> C tile.  Consecutive ids land on different XCDs, each with its own L2, so first
// regroup ids per XCD, then walk the tile grid in bands of GROUP_M tile rows so that the tiles
// running together on one XCD share A and B panels.
// ids [0, count) are dealt round-robin to the XCDs; give every XCD a contiguous range instead
// (XCD x gets ids x, x + 8, ...: count / 8 of them, one more for x < count % 8)
AICORE inline int RegroupXcd(int id, int count)
{
    const int xcd = id % kXcds, pos = id / kXcds, base = count / kXcds, extra = count % kXcds;
    return xcd * base + (xcd < extra ? xcd : extra) + pos;
}

// linear tile id -> (tile row, tile column), walking bands of GROUP_M tile rows column by column
template <int GROUP_M>
AICORE inline void TileOfId(int id, int tilesM, int tilesN, int &tm, int &tn)
{
    const int band = GROUP_M * tilesN;
    const int g = id / band, inBand = id % band;
    const int rowsHere = (tilesM - g * GROUP_M) < GROUP_M ? (tilesM - g * GROUP_M) : GROUP_M;
    tm = g * GROUP_M + inBand % rowsHere;
    tn = inBand / rowsHere;
}

template <int GROUP_M>
AICORE inline void TileOfBlock(int block, int tilesM, int tilesN, int &tm, int &tn)
{
    TileOfId<GROUP_M>(RegroupXcd(block, tilesM * tilesN), tilesM, tilesN, tm, tn);
}

template <int BM, int BN, int BK, int STAGES, int MIN_BLOCKS, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, MIN_BLOCKS) AICORE
    void GemmF16F32(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k)
{
    // L1 (LDS) panels: A [BM, BK] contiguous along K (Nz role), B [BK, BN] contiguous along K (Zn role)
    using TileMatA = Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, half, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using LeftTile = TileLeft<half, BM, BK, BM, BK>;
    using RightTile = TileRight<half, BK, BN, BK, BN>;
    using ResTile = TileAcc<float, BM, BN, BM, BN>;

    using ShapeA = TileShape2D<half, BM, BK, Layout::ND>;
    using StrideA = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalA = GlobalTensor<half, ShapeA, StrideA, Layout::ND>;
    using ShapeB = TileShape2D<half, BK, BN, Layout::DN>;
    using StrideB = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::DN>; // B is stored [n, k]: column-major k x n
    using GlobalB = GlobalTensor<half, ShapeB, StrideB, Layout::DN>;
    using ShapeC = TileShape2D<float, BM, BN, Layout::ND>;
    using StrideC = BaseShape2D<float, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<float, ShapeC, StrideC, Layout::ND>;

    constexpr uint32_t kABytes = BM * BK * sizeof(half), kBBytes = BK * BN * sizeof(half);
    constexpr uint32_t kStage = kABytes + kBBytes;
    // asynchronous copy instructions per wave that one K-step's two TLOADs issue
    constexpr int kLoadsPerStep = TLoadInstrs<TileMatA>() + TLoadInstrs<TileMatB>();

    int tm, tn;
    TileOfBlock<GROUP_M>((int)get_block_idx(), m / BM, n / BN, tm, tn);
    __gm__ half *aPanel = const_cast<half *>(src0) + (int64_t)tm * BM * k;
    __gm__ half *bPanel = const_cast<half *>(src1) + (int64_t)tn * BN * k;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);

    TileMatA aMat[STAGES];
    TileMatB bMat[STAGES];
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        TASSIGN(aMat[s], s * kStage);
        TASSIGN(bMat[s], s * kStage + kABytes);
    }
    LeftTile aTile;
    RightTile bTile;
    ResTile cTile;

    const int kLoop = k / BK;
    // prologue: STAGES-1 K-steps in flight
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < kLoop) {
            GlobalA gmA(aPanel + (int64_t)s * BK, ShapeA(), strideA);
            GlobalB gmB(bPanel + (int64_t)s * BK, ShapeB(), strideB);
            TLOAD(aMat[s], gmA);
            TLOAD(bMat[s], gmB);
            set_flag(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(s));
        }
    for (int kIter = 0; kIter < kLoop; kIter += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) { // unrolled over the LDS stages: stage indices are constants
            const int it = kIter + s;
            if (it < kLoop) {
                // K-step `it` has landed for every wave (the younger steps may still be in flight), and
                // every wave is done reading the stage that the next TLOAD overwrites.
                if (it + STAGES - 2 < kLoop)
                    wait_flag_pending<(STAGES - 2) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(s));
                else
                    wait_flag(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(s));
                const int nxt = it + STAGES - 1;
                if (nxt < kLoop) {
                    const int ns = (s + STAGES - 1) % STAGES;
                    GlobalA gmA(aPanel + (int64_t)nxt * BK, ShapeA(), strideA);
                    GlobalB gmB(bPanel + (int64_t)nxt * BK, ShapeB(), strideB);
                    TLOAD(aMat[ns], gmA);
                    TLOAD(bMat[ns], gmB);
                    set_flag(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(ns));
                }
                TEXTRACT(aTile, aMat[s], 0, 0);
                TEXTRACT(bTile, bMat[s], 0, 0);
                set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
                wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
                if (it == 0)
                    TMATMUL(cTile, aTile, bTile);
                else
                    TMATMUL_ACC(cTile, cTile, aTile, bTile);
                set_flag(PIPE_M, PIPE_MTE1, EVENT_ID0);
            }
        }
    }
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    GlobalC dstGlobal(out + (int64_t)tm * BM * n + (int64_t)tn * BN, ShapeC(), StrideC(m, n));
    TSTORE(dstGlobal, cTile);
}

// One wave per SIMD needs every issue slot: a wave that is stalled issuing its asynchronous copies
// (the compute unit's single vector-memory front end takes 16 cycles per 1 KiB instruction) cannot
// issue MFMAs meanwhile.  This kernel therefore (a) keeps the whole steady-state K-step in one
// straight-line region: TLOAD of stage i+STAGES-1, TMATMUL_ACC on the two 16-wide halves of stage i,
// TEXTRACT of the halves of stage i+1, and (b) tells the instruction scheduler to interleave them:
// one copy instruction per two MFMAs, then one fragment read per two MFMAs.
// C[row0 : row0+BM, col0 : col0+BN] (+)= A[row0.., kFirst*32 ..] x B[col0.., kFirst*32 ..] over kLoop K-steps of 32.
template <int BM, int BN, int STAGES>
AICORE inline __attribute__((always_inline)) void MixTile(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k,
                           int row0, int col0, int kFirst, int kLoop, bool partial)
{
    constexpr int BK = 32, KH = 16;
    using TileMatA = Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, half, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using LeftTile = TileLeft<half, BM, KH, BM, KH>;
    using RightTile = TileRight<half, KH, BN, KH, BN>;
    using ResTile = TileAcc<float, BM, BN, BM, BN>;
    using ShapeA = TileShape2D<half, BM, BK, Layout::ND>;
    using StrideA = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalA = GlobalTensor<half, ShapeA, StrideA, Layout::ND>;
    using ShapeB = TileShape2D<half, BK, BN, Layout::DN>;
    using StrideB = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::DN>;
    using GlobalB = GlobalTensor<half, ShapeB, StrideB, Layout::DN>;
    using ShapeC = TileShape2D<float, BM, BN, Layout::ND>;
    using StrideC = BaseShape2D<float, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<float, ShapeC, StrideC, Layout::ND>;

    constexpr uint32_t kABytes = BM * BK * sizeof(half), kBBytes = BK * BN * sizeof(half);
    constexpr uint32_t kStage = kABytes + kBBytes;
    constexpr int kLoadsPerStep = TLoadInstrs<TileMatA>() + TLoadInstrs<TileMatB>();
    constexpr int kMfmaPerHalf = ResTile::Storage::MB * ResTile::Storage::NB;
    constexpr int kReadsPerHalf = LeftTile::Storage::MB + RightTile::Storage::NB;
    static_assert(STAGES >= 3, "needs at least three L1 stages");

    __gm__ half *aPanel = const_cast<half *>(src0) + (int64_t)row0 * k + (int64_t)kFirst * BK;
    __gm__ half *bPanel = const_cast<half *>(src1) + (int64_t)col0 * k + (int64_t)kFirst * BK;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);

    TileMatA aMat[STAGES];
    TileMatB bMat[STAGES];
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        TASSIGN(aMat[s], s * kStage);
        TASSIGN(bMat[s], s * kStage + kABytes);
    }
    LeftTile aLo, aHi;
    RightTile bLo, bHi;
    ResTile cTile;
#pragma unroll
    for (int mb = 0; mb < ResTile::Storage::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < ResTile::Storage::NB; ++nb)
#pragma unroll
            for (int i = 0; i < detail::kAccElems; ++i)
                cTile.st.f[mb][nb][i] = 0.0f;

    // the host guarantees kLoop % STAGES == 0 and kLoop >= 2 * STAGES
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) {
        GlobalA gmA(aPanel + (int64_t)s * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)s * BK, ShapeB(), strideB);
        TLOAD(aMat[s], gmA);
        TLOAD(bMat[s], gmB);
    }
    wait_flag_pending<(STAGES - 2) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); // stage 0 is complete
    TEXTRACT(aLo, aMat[0], 0, 0);
    TEXTRACT(bLo, bMat[0], 0, 0);
    TEXTRACT(aHi, aMat[0], 0, KH);
    TEXTRACT(bHi, bMat[0], KH, 0);

    // One K-step on stage s (a compile-time constant: every LDS address is an immediate).  Past the
    // end of K the copy re-fetches the last K-step into a free stage and the fragment reads fetch
    // values nobody uses, which keeps the loop free of branches and the vmcnt bookkeeping uniform.
    auto step = [&](auto stageTag, int it) {
        constexpr int s = decltype(stageTag)::value;
        constexpr int sNext = (s + 1) % STAGES, sLoad = (s + STAGES - 1) % STAGES;
        // stage it+1 has landed for every wave; the stage that the TLOAD below overwrites was last
        // read one K-step ago, and those reads have fed MFMAs that are already issued
        hw::wait_vm<(STAGES - 3) * kLoadsPerStep>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int fetch = it + STAGES - 1 < kLoop ? it + STAGES - 1 : kLoop - 1;
        GlobalA gmA(aPanel + (int64_t)fetch * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)fetch * BK, ShapeB(), strideB);
        TLOAD(aMat[sLoad], gmA);
        TLOAD(bMat[sLoad], gmB);
        TMATMUL_ACC(cTile, cTile, aLo, bLo);
        TEXTRACT(aLo, aMat[sNext], 0, 0);
        TEXTRACT(bLo, bMat[sNext], 0, 0);
        TMATMUL_ACC(cTile, cTile, aHi, bHi);
        TEXTRACT(aHi, aMat[sNext], 0, KH);
        TEXTRACT(bHi, bMat[sNext], KH, 0);
        // issue order: 2 MFMA + 1 copy ..., then 2 MFMA + 1 fragment read ..., then the last reads
#pragma unroll
        for (int i = 0; i < kLoadsPerStep; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerHalf / kLoadsPerStep, 0);
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < kReadsPerHalf; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerHalf / kReadsPerHalf, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, kReadsPerHalf, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    for (int it = 0; it < kLoop; it += STAGES) {
        step(integral_constant<int, 0>(), it);
        step(integral_constant<int, 1>(), it + 1);
        step(integral_constant<int, 2>(), it + 2);
        if constexpr (STAGES == 4)
            step(integral_constant<int, 3>(), it + 3);
    }
    hw::wait_vm0(); // the copies issued past the end of K must not outlive the workgroup's LDS
    GlobalC dstGlobal(out + (int64_t)row0 * n + col0, ShapeC(), StrideC(m, n));
    if (partial)
        TSTORE<ResTile, GlobalC, AtomicType::AtomicAdd>(dstGlobal, cTile);
    else
        TSTORE(dstGlobal, cTile);
}

// The same K-step pipeline with the two halves of a step taken along M instead of K: the wave multiplies the
// upper half of its rows (first half), then the lower half, by the whole [32, BN] B panel of the step.  Works with
// either MFMA shape (a 16 x 16 x 32 MFMA covers the whole 32-wide K-step, so the step cannot be halved along K).
// Row halves are halves of the WORKGROUP tile: wave row wm owns rows wm*BM/4 .. of each half.
template <int BM, int BN, int STAGES>
AICORE inline __attribute__((always_inline)) void MixTileRows(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m,
                                                              int n, int k, int row0, int col0, int kLoop)
{
    constexpr int BK = 32, HM = BM / 2;
    using TileMatA = Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, half, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using LeftHalf = TileLeft<half, HM, BK, HM, BK>;
    using RightTile = TileRight<half, BK, BN, BK, BN>;
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
    constexpr int kMfmaPerHalf = AccHalf::Storage::MB * AccHalf::Storage::NB * LeftHalf::Storage::KS;
    constexpr int kReadsA = LeftHalf::Storage::MB * LeftHalf::Storage::KS, kReadsB = RightTile::Storage::NB * RightTile::Storage::KS;
    constexpr int kReads = 2 * kReadsA + kReadsB, kMfma = 2 * kMfmaPerHalf;
    // Issue pattern of a step: the copies first, kMfmaPerCopy MFMAs before each (the LDS reads may not be moved above
    // an asynchronous copy into LDS); then the fragment reads spread over the MFMAs that follow; the last kMfmaTail
    // MFMAs of the step have no read after them.
    constexpr int kMfmaPerCopy = kMfma / 4 / kLoadsPerStep > 0 ? kMfma / 4 / kLoadsPerStep : 1;
    constexpr int kMfmaTail = kMfma / 8 > 0 ? kMfma / 8 : 1;
    constexpr int kMfmaForReads = kMfma - kMfmaPerCopy * kLoadsPerStep - kMfmaTail;
    static_assert(STAGES == 4, "two fragment sets alternate with the stage index");
    static_assert(kMfmaForReads > 0, "issue pattern below");

    __gm__ half *aPanel = const_cast<half *>(src0) + (int64_t)row0 * k;
    __gm__ half *bPanel = const_cast<half *>(src1) + (int64_t)col0 * k;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);

    TileMatA aMat[STAGES];
    TileMatB bMat[STAGES];
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        TASSIGN(aMat[s], s * kStage);
        TASSIGN(bMat[s], s * kStage + kABytes);
    }
    // Two sets of operand fragments: the MFMAs of step it read set it % 2 while the fragments of step it+1 arrive in the
    // other one, every read interleaved with the MFMAs and none left for the end of the step - the wait for the LDS
    // queue that follows the barrier then finds it empty.
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

    // the host guarantees kLoop % STAGES == 0 and kLoop >= 2 * STAGES
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) {
        GlobalA gmA(aPanel + (int64_t)s * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)s * BK, ShapeB(), strideB);
        TLOAD(aMat[s], gmA);
        TLOAD(bMat[s], gmB);
    }
    wait_flag_pending<(STAGES - 2) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); // stage 0 is complete
    TEXTRACT(aUp[0], aMat[0], 0, 0);
    TEXTRACT(aDn[0], aMat[0], HM, 0);
    TEXTRACT(bAll[0], bMat[0], 0, 0);

    auto step = [&](auto stageTag, int it) {
        constexpr int s = decltype(stageTag)::value;
        constexpr int sNext = (s + 1) % STAGES, sLoad = (s + STAGES - 1) % STAGES;
        hw::wait_vm<(STAGES - 3) * kLoadsPerStep>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int fetch = it + STAGES - 1 < kLoop ? it + STAGES - 1 : kLoop - 1;
        GlobalA gmA(aPanel + (int64_t)fetch * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)fetch * BK, ShapeB(), strideB);
        TLOAD(aMat[sLoad], gmA);
        TLOAD(bMat[sLoad], gmB);
        constexpr int p = s & 1, q = p ^ 1;
        TMATMUL_ACC(cUp, cUp, aUp[p], bAll[p]);
        TMATMUL_ACC(cDn, cDn, aDn[p], bAll[p]);
        TEXTRACT(aUp[q], aMat[sNext], 0, 0);
        TEXTRACT(bAll[q], bMat[sNext], 0, 0);
        TEXTRACT(aDn[q], aMat[sNext], HM, 0);
#pragma unroll
        for (int i = 0; i < kLoadsPerStep; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerCopy, 0);
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        StaticFor<0, kReads>([](auto iTag) {
            // read i follows its share of the MFMAs: floor((i+1) N / R) - floor(i N / R)
            constexpr int i = decltype(iTag)::value;
            constexpr int n = (i + 1) * kMfmaForReads / kReads - i * kMfmaForReads / kReads;
            if constexpr (n > 0)
                __builtin_amdgcn_sched_group_barrier(0x008, n, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmaTail, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    for (int it = 0; it < kLoop; it += STAGES) {
        step(integral_constant<int, 0>(), it);
        step(integral_constant<int, 1>(), it + 1);
        step(integral_constant<int, 2>(), it + 2);
        if constexpr (STAGES == 4)
            step(integral_constant<int, 3>(), it + 3);
    }
    hw::wait_vm0(); // the copies issued past the end of K must not outlive the workgroup's LDS
    GlobalC dstUp(out + (int64_t)row0 * n + col0, ShapeC(), StrideC(m, n));
    GlobalC dstDn(out + (int64_t)(row0 + HM) * n + col0, ShapeC(), StrideC(m, n));
    TSTORE(dstUp, cUp);
    TSTORE(dstDn, cDn);
}

// Work split of the kernel below.  The first `fullTiles` workgroups (whole rounds over the compute
// units) own one BM x BN C tile each.  The tiles of the last, partial round are divided so that the
// round fills the machine: tailMode 1 = four (BM/2) x (BN/2) quarter tiles, one workgroup each;
// tailMode 2 = `splitK` K-ranges per tile whose partial products are added into a zeroed C tile
// with TSTORE<AtomicAdd> (slow: one atomic per element).
// ROWS: the halves of a K-step are taken along M (MixTileRows; needed for the 16 x 16 x 32 MFMA) instead of along K.
template <int BM, int BN, int STAGES, int GROUP_M, bool ROWS = false>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32Mix(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k,
                       int fullTiles, int tailMode, int splitK)
{
    const int tilesM = m / BM, tilesN = n / BN;
    const int block = (int)get_block_idx();
    int tm, tn;
    if (block >= fullTiles && tailMode == 1) {
        const int u = RegroupXcd(block - fullTiles, (tilesM * tilesN - fullTiles) * 4);
        TileOfId<GROUP_M>(fullTiles + u / 4, tilesM, tilesN, tm, tn);
        const int sub = u % 4;
        if constexpr (ROWS && (BN / 2) % (detail::kMfmaM * kWavesN) != 0)
            ; // this tile shape has no quarter tiles: the launcher never asks for them
        else if constexpr (ROWS)
            MixTileRows<BM / 2, BN / 2, STAGES>(out, src0, src1, m, n, k, tm * BM + (sub >> 1) * (BM / 2),
                                                tn * BN + (sub & 1) * (BN / 2), k / 32);
        else
            MixTile<BM / 2, BN / 2, STAGES>(out, src0, src1, m, n, k, tm * BM + (sub >> 1) * (BM / 2),
                                            tn * BN + (sub & 1) * (BN / 2), 0, k / 32, false);
        return;
    }
    // whole tiles and K-ranges of whole tiles share one call site, so the tile body is inlined once
    int kFirst = 0, kLoop = k / 32;
    bool partial = false;
    if (block < fullTiles) {
        TileOfId<GROUP_M>(RegroupXcd(block, fullTiles), tilesM, tilesN, tm, tn);
    } else {
        const int u = RegroupXcd(block - fullTiles, (tilesM * tilesN - fullTiles) * splitK);
        TileOfId<GROUP_M>(fullTiles + u / splitK, tilesM, tilesN, tm, tn);
        kLoop = k / 32 / splitK;
        kFirst = (u % splitK) * kLoop;
        partial = splitK > 1;
    }
    if constexpr (ROWS)
        MixTileRows<BM, BN, STAGES>(out, src0, src1, m, n, k, tm * BM, tn * BN, kLoop); // the launcher rejects K-splits
    else
        MixTile<BM, BN, STAGES>(out, src0, src1, m, n, k, tm * BM, tn * BN, kFirst, kLoop, partial);
}

// Clears the C tiles that GemmF16F32Mix accumulates into with atomic adds (tile ids >= fullTiles).
template <int BM, int BN, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE void GemmZeroTailTiles(__gm__ float *out, int m, int n, int fullTiles)
{
    using ResTile = TileAcc<float, BM, BN, BM, BN>;
    using ShapeC = TileShape2D<float, BM, BN, Layout::ND>;
    using StrideC = BaseShape2D<float, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<float, ShapeC, StrideC, Layout::ND>;
    int tm, tn;
    TileOfId<GROUP_M>(fullTiles + (int)get_block_idx(), m / BM, n / BN, tm, tn);
    ResTile zero;
#pragma unroll
    for (int mb = 0; mb < ResTile::Storage::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < ResTile::Storage::NB; ++nb)
#pragma unroll
            for (int i = 0; i < detail::kAccElems; ++i)
                zero.st.f[mb][nb][i] = 0.0f;
    GlobalC dstGlobal(out + (int64_t)tm * BM * n + (int64_t)tn * BN, ShapeC(), StrideC(m, n));
    TSTORE(dstGlobal, zero);
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <int BM, int BN, int BK, int STAGES, int MIN_BLOCKS, int GROUP_M>
int launch_gemm(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    if (m % BM || n % BN || k % BK)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM * BK + BK * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32<BM, BN, BK, STAGES, MIN_BLOCKS, GROUP_M>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int blocks = (m / BM) * (n / BN);
    kernel<<<dim3(blocks), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}
} // namespace

namespace {
// Number of K-ranges to cut the tiles of the last partial round into: the candidate that
// minimises ceil(rem * S / cus) / S, the length of that round in units of one full tile.
inline int choose_split_k(int rem, int cus, int kLoop, int stages)
{
    if (rem == 0)
        return 1;
    int best = 1;
    double bestSpan = (double)((rem + cus - 1) / cus);
    const int cand[] = {2, 3, 4, 6, 8};
    for (int s : cand) {
        if (kLoop % (s * stages) != 0 || kLoop / s < 2 * stages)
            continue;
        const double span = (double)((rem * s + cus - 1) / cus) / s;
        if (span < bestSpan - 1e-9) {
            bestSpan = span;
            best = s;
        }
    }
    return best;
}

inline int compute_units()
{
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    return cus;
}

// tailMode: 0 = whole tiles only; 1 = quarter tiles in the last partial round when they fit one round
// (the quarter tiles move twice the operand bytes per flop, so two rounds of them cost more than the
// idle compute units of a partial round); 2 = K-split with atomic adds (tuning hook only); 3 = quarter
// tiles whenever there is a partial round (tuning hook only)
template <int BM, int BN, int STAGES, int GROUP_M, bool ROWS = false>
int launch_gemm_mix(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k, int tailMode = 1)
{
    static_assert(STAGES == 3 || STAGES == 4, "three or four L1 stages");
    if (m % BM || n % BN || k % (32 * STAGES) || k / 32 < 2 * STAGES)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM * 32 + 32 * BN) * (int)sizeof(half);
    if (ROWS && tailMode == 2)
        return PTO_ERR_UNSUPPORTED;
    if (ROWS && (BN / 2) % (detail::kMfmaM * kWavesN) != 0) // no quarter tiles for this shape
        tailMode = 0;
    auto kernel = GemmF16F32Mix<BM, BN, STAGES, GROUP_M, ROWS>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = (m / BM) * (n / BN), cus = compute_units();
    int full = tiles / cus * cus;
    int splitK = 1;
    if (tailMode == 1 && (full == 0 || (tiles - full) * 4 > cus))
        tailMode = 0;
    if (tailMode == 3)
        tailMode = 1;
    if (tailMode == 2)
        splitK = choose_split_k(tiles - full, cus, k / 32, STAGES);
    if (tailMode == 0 || (tailMode == 2 && splitK == 1))
        full = tiles;
    const int tail = tiles - full;
    if (tail > 0 && tailMode == 2)
        GemmZeroTailTiles<BM, BN, GROUP_M><<<dim3(tail), dim3(kBlockThreads), 0, st>>>(c, m, n, full);
    const int units = tailMode == 1 ? tail * 4 : tail * splitK;
    kernel<<<dim3(full + units), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k, full, tailMode, splitK);
    return pto_amd::check_launch();
}

} // namespace

