// GEMM kernels of the PTO tile path, shared by the translation units that instantiate them for
// different wave grids (PTO_WAVES_M x PTO_WAVES_N is fixed per translation unit).
#pragma once
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kXcds = 8; // MI355X: 8 accelerator dies, workgroups are dealt to them round-robin

// Workgroup id -> C tile.  Consecutive ids land on different XCDs, each with its own L2, so first
// regroup ids per XCD, then walk the tile grid in bands of GROUP_M tile rows so that the tiles
// running together on one XCD share A and B panels.
template <int GROUP_M>
AICORE inline void TileOfBlock(int block, int tilesM, int tilesN, int &tm, int &tn)
{
    const int total = tilesM * tilesN;
    int id = block;
    if (total % kXcds == 0) {
        const int perXcd = total / kXcds;
        id = (block % kXcds) * perXcd + block / kXcds;
    }
    const int band = GROUP_M * tilesN;
    const int g = id / band, inBand = id % band;
    const int rowsHere = (tilesM - g * GROUP_M) < GROUP_M ? (tilesM - g * GROUP_M) : GROUP_M;
    tm = g * GROUP_M + inBand % rowsHere;
    tn = inBand / rowsHere;
}

template <int BM, int BN, int BK, int STAGES, int MIN_BLOCKS, int GROUP_M, int MODE = 0>
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
    long long tStart = 0, tLoop = 0, tEnd = 0;
    if (MODE == 4)
        tStart = clock64();
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
            auto stamp = [&](int point) {
                if (MODE == 3 && get_block_idx() == 0 && hw::tid() == 0 && it < 64)
                    reinterpret_cast<long long *>(out)[4096 + it * 8 + point] = clock64();
            };
            if (it < kLoop) {
                stamp(0);
                // K-step `it` has landed for every wave (the younger steps may still be in flight), and
                // every wave is done reading the stage that the next TLOAD overwrites.
                if (it + STAGES - 2 < kLoop)
                    wait_flag_pending<(STAGES - 2) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(s));
                else
                    wait_flag(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(s));
                stamp(1);
                const int nxt = it + STAGES - 1;
                if (MODE != 2 && nxt < kLoop) {
                    const int ns = (s + STAGES - 1) % STAGES;
                    GlobalA gmA(aPanel + (int64_t)nxt * BK, ShapeA(), strideA);
                    GlobalB gmB(bPanel + (int64_t)nxt * BK, ShapeB(), strideB);
                    TLOAD(aMat[ns], gmA);
                    TLOAD(bMat[ns], gmB);
                    set_flag(PIPE_MTE2, PIPE_MTE1, static_cast<event_t>(ns));
                }
                stamp(2);
                if (MODE != 1 || it == 0) {
                    TEXTRACT(aTile, aMat[s], 0, 0);
                    TEXTRACT(bTile, bMat[s], 0, 0);
                    if (MODE == 3) {
                        __builtin_amdgcn_sched_barrier(0);
                        stamp(3);
                        hw::wait_lgkm0();
                        stamp(4);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    set_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
                    wait_flag(PIPE_MTE1, PIPE_M, EVENT_ID0);
                    if (it == 0)
                        TMATMUL(cTile, aTile, bTile);
                    else
                        TMATMUL_ACC(cTile, cTile, aTile, bTile);
                    set_flag(PIPE_M, PIPE_MTE1, EVENT_ID0);
                    if (MODE == 3) {
                        __builtin_amdgcn_sched_barrier(0);
                        stamp(5);
                    }
                }
            }
        }
    }
    if (MODE == 3)
        return;
    if (MODE == 4) {
        __builtin_amdgcn_sched_barrier(0);
        tLoop = clock64();
    }
    set_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    wait_flag(PIPE_M, PIPE_FIX, EVENT_ID0);
    GlobalC dstGlobal(out + (int64_t)tm * BM * n + (int64_t)tn * BN, ShapeC(), StrideC(m, n));
    TSTORE(dstGlobal, cTile);
    if (MODE == 4) {
        hw::wait_vm0();
        __builtin_amdgcn_sched_barrier(0);
        tEnd = clock64();
        if (hw::tid() == 0) {
            long long *dbg = reinterpret_cast<long long *>(out + (int64_t)m * n) + get_block_idx() * 8;
            dbg[0] = tStart;
            dbg[1] = tLoop;
            dbg[2] = tEnd;
            dbg[3] = (long long)wall_clock64();
            dbg[4] = tm * 1000 + tn;
            unsigned xcc = 0;
            asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
            dbg[5] = xcc;
            unsigned hwid = 0;
            asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hwid));
            dbg[6] = hwid;
        }
    }
}

// Deeper software pipeline for one wave per SIMD (256 x 256 block, 128 x 128 per wave): the
// TEXTRACTs of K-step i+1 are issued while the TMATMULs of step i execute, so that neither the
// LDS latency nor the wait for the asynchronous TLOADs is exposed.  Each L1 stage holds BK = 32
// (two 16-wide MFMA steps); operand fragments are double-buffered per 16-wide step:
//
//   TMATMUL_ACC(step i,  k 0..15)   | wait: stage i+1 landed, barrier; TLOAD stage i+STAGES-1;
//                                   | TEXTRACT(stage i+1, k 0..15)
//   TMATMUL_ACC(step i,  k 16..31)  | TEXTRACT(stage i+1, k 16..31)
template <int BM, int BN, int STAGES, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32Deep(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k)
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
    LeftTile aLo, aHi;   // k 0..15 and k 16..31 of the current stage
    RightTile bLo, bHi;
    ResTile cTile;

    const int kLoop = k / BK;
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < kLoop) {
            GlobalA gmA(aPanel + (int64_t)s * BK, ShapeA(), strideA);
            GlobalB gmB(bPanel + (int64_t)s * BK, ShapeB(), strideB);
            TLOAD(aMat[s], gmA);
            TLOAD(bMat[s], gmB);
        }
    // stage 0 must be complete before its fragments are read
    if (STAGES - 2 < kLoop)
        wait_flag_pending<(STAGES - 2) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    else
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TEXTRACT(aLo, aMat[0], 0, 0);
    TEXTRACT(bLo, bMat[0], 0, 0);
    TEXTRACT(aHi, aMat[0], 0, KH);
    TEXTRACT(bHi, bMat[0], KH, 0);
    // zero the accumulators through one TMATMUL on zeroed... simpler: explicit clear
#pragma unroll
    for (int mb = 0; mb < ResTile::Storage::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < ResTile::Storage::NB; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                cTile.st.f[mb][nb][i] = 0.0f;

    for (int kIter = 0; kIter < kLoop; kIter += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {
            const int it = kIter + s;
            if (it < kLoop) {
                TMATMUL_ACC(cTile, cTile, aLo, bLo);
                __builtin_amdgcn_sched_barrier(0);
                const bool haveNext = it + 1 < kLoop;
                if (haveNext) {
                    // stage it+1 landed everywhere; everyone is past the reads of stage it-1
                    if (it + STAGES - 2 < kLoop)
                        wait_flag_pending<(STAGES - 3) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
                    else
                        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
                    const int nxt = it + STAGES - 1;
                    if (nxt < kLoop) {
                        const int ns = (s + STAGES - 1) % STAGES;
                        GlobalA gmA(aPanel + (int64_t)nxt * BK, ShapeA(), strideA);
                        GlobalB gmB(bPanel + (int64_t)nxt * BK, ShapeB(), strideB);
                        TLOAD(aMat[ns], gmA);
                        TLOAD(bMat[ns], gmB);
                    }
                    TEXTRACT(aLo, aMat[(s + 1) % STAGES], 0, 0);
                    TEXTRACT(bLo, bMat[(s + 1) % STAGES], 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                TMATMUL_ACC(cTile, cTile, aHi, bHi);
                __builtin_amdgcn_sched_barrier(0);
                if (haveNext) {
                    TEXTRACT(aHi, aMat[(s + 1) % STAGES], 0, KH);
                    TEXTRACT(bHi, bMat[(s + 1) % STAGES], KH, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    GlobalC dstGlobal(out + (int64_t)tm * BM * n + (int64_t)tn * BN, ShapeC(), StrideC(m, n));
    TSTORE(dstGlobal, cTile);
}

// One wave per SIMD needs every issue slot: a wave that is stalled issuing its asynchronous copies
// (the compute unit's single vector-memory front end takes 16 cycles per 1 KiB instruction) cannot
// issue MFMAs meanwhile.  This kernel therefore (a) keeps the whole steady-state K-step in one
// straight-line region: TLOAD of stage i+STAGES-1, TMATMUL_ACC on the two 16-wide halves of stage i,
// TEXTRACT of the halves of stage i+1, and (b) tells the instruction scheduler to interleave them:
// one copy instruction per two MFMAs, then one fragment read per two MFMAs.
template <int BM, int BN, int STAGES, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32Mix(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k)
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
    LeftTile aLo, aHi;
    RightTile bLo, bHi;
    ResTile cTile;
#pragma unroll
    for (int mb = 0; mb < ResTile::Storage::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < ResTile::Storage::NB; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                cTile.st.f[mb][nb][i] = 0.0f;

    const int kLoop = k / BK; // the host guarantees kLoop >= STAGES
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
    for (int it = 0; it < kLoop; it += STAGES) { // the host guarantees kLoop % STAGES == 0
        step(integral_constant<int, 0>(), it);
        step(integral_constant<int, 1>(), it + 1);
        step(integral_constant<int, 2>(), it + 2);
        if constexpr (STAGES == 4)
            step(integral_constant<int, 3>(), it + 3);
    }
    GlobalC dstGlobal(out + (int64_t)tm * BM * n + (int64_t)tn * BN, ShapeC(), StrideC(m, n));
    TSTORE(dstGlobal, cTile);
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <int BM, int BN, int BK, int STAGES, int MIN_BLOCKS, int GROUP_M, int MODE = 0>
int launch_gemm(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    if (m % BM || n % BN || k % BK)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM * BK + BK * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32<BM, BN, BK, STAGES, MIN_BLOCKS, GROUP_M, MODE>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int blocks = (m / BM) * (n / BN);
    kernel<<<dim3(blocks), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}
} // namespace

namespace {
template <int BM, int BN, int STAGES, int GROUP_M>
int launch_gemm_mix(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    static_assert(STAGES == 3 || STAGES == 4, "three or four L1 stages");
    if (m % BM || n % BN || k % (32 * STAGES) || k / 32 < 2 * STAGES)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM * 32 + 32 * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32Mix<BM, BN, STAGES, GROUP_M>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int blocks = (m / BM) * (n / BN);
    kernel<<<dim3(blocks), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}

template <int BM, int BN, int STAGES, int GROUP_M>
int launch_gemm_deep(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k)
{
    if (m % BM || n % BN || k % 32)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM * 32 + 32 * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32Deep<BM, BN, STAGES, GROUP_M>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int blocks = (m / BM) * (n / BN);
    kernel<<<dim3(blocks), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k);
    return pto_amd::check_launch();
}
} // namespace

