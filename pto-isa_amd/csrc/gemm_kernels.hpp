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
// compute units of the device that is current at the first call
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
} // namespace
