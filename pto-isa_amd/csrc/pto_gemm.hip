// fp16 x fp16 -> fp32 GEMM for MI355X written with PTO tile instructions:
//   TLOAD (HBM -> LDS, async 16-byte copies)  ->  TEXTRACT (LDS -> MFMA operand fragments)
//   ->  TMATMUL / TMATMUL_ACC (v_mfma_f32_32x32x16_f16)  ->  TSTORE (accumulators -> HBM).
//
// Same decomposition as the reference's manual kernel
// (kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp:67-230): each "core" owns
// BM x BN blocks of C, walks K in steps of BK, double-buffers the staged A / B panels and
// synchronises the stages with set_flag / wait_flag.  Differences that the hardware asks for:
// the stages are software-pipelined in program order (one instruction stream per wavefront: the
// TLOAD of step i+1 is issued before the TEXTRACT / TMATMUL of step i), one workgroup per C block
// instead of a 24-core loop nest, and an XCD-aware block -> tile map.
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

template <int BM, int BN, int BK>
__global__ __launch_bounds__(kBlockThreads) AICORE void GemmF16F32(__gm__ float *out, __gm__ const half *src0,
                                                                    __gm__ const half *src1, int m, int n, int k)
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

    int tm, tn;
    TileOfBlock<8>((int)get_block_idx(), m / BM, n / BN, tm, tn);
    __gm__ half *aPanel = const_cast<half *>(src0) + (int64_t)tm * BM * k;
    __gm__ half *bPanel = const_cast<half *>(src1) + (int64_t)tn * BN * k;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);

    TileMatA aMat[2];
    TileMatB bMat[2];
    TASSIGN(aMat[0], 0u);
    TASSIGN(bMat[0], kABytes);
    TASSIGN(aMat[1], kStage);
    TASSIGN(bMat[1], kStage + kABytes);
    LeftTile aTile;
    RightTile bTile;
    ResTile cTile;

    const int kLoop = k / BK;
    {
        GlobalA gmA(aPanel, ShapeA(), strideA);
        GlobalB gmB(bPanel, ShapeB(), strideB);
        TLOAD(aMat[0], gmA);
        TLOAD(bMat[0], gmB);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    }
    for (int kIter = 0; kIter < kLoop; kIter += 2) {
#pragma unroll
        for (int half_ = 0; half_ < 2; ++half_) { // unrolled by the two L1 stages: stage indices are constants
            const int it = kIter + half_;
            if (it < kLoop) {
                // stage `half_` has landed for every wave, and every wave is done reading the other stage
                wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
                if (it + 1 < kLoop) {
                    GlobalA gmA(aPanel + (int64_t)(it + 1) * BK, ShapeA(), strideA);
                    GlobalB gmB(bPanel + (int64_t)(it + 1) * BK, ShapeB(), strideB);
                    TLOAD(aMat[half_ ^ 1], gmA);
                    TLOAD(bMat[half_ ^ 1], gmB);
                    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
                }
                TEXTRACT(aTile, aMat[half_], 0, 0);
                TEXTRACT(bTile, bMat[half_], 0, 0);
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

extern "C" int pto_gemm_f16f32(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k)
{
    constexpr int BM = 128, BN = 256, BK = 64;
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    if (m % BM || n % BN || k % BK)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 2 * (BM * BK + BK * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32<BM, BN, BK>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int blocks = (m / BM) * (n / BN);
    kernel<<<dim3(blocks), dim3(kBlockThreads), lds, static_cast<hipStream_t>(stream)>>>(
        c, reinterpret_cast<const half *>(a), reinterpret_cast<const half *>(b), m, n, k);
    return pto_amd::check_launch();
}
