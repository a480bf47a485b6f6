// MXFP8 / MXFP4 GEMM for MI355X: C[m,n] = (A .* 2^(scaleA-127)) x (B .* 2^(scaleB-127)), fp8 (e4m3 / e5m2) or fp4
// (e2m1, two per byte) operands with one e8m0 scale per row (column) and 32-wide k block, fp32 accumulation, bf16 or
// fp32 result.
//
// Mirrors the reference kernels kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp:149-241 and
// kernels/manual/a5/matmul_mxfp4_performance/mxmatmul_performance_kernel.cpp (TLOAD of operand and scale panels ->
// TEXTRACT -> TMATMUL_MX -> TSTORE): A [m,k], B stored [n,k], scaleA [m,k/32], scaleB stored [n,k/32]
// (scripts/gen_data.py:31-66).
//
// Structure: the fp16 GEMM's K-step pipeline (workgroup tile 256 x 256, 8 waves in a 2 x 4 grid, four LDS stages of
// one 64-byte K-step filled by asynchronous copies, copies / fragment reads / MFMAs interleaved by the scheduler
// directives).  A K-step is 64 fp8 values = the same 64 bytes per row as 32 fp16 values, and one
// v_mfma_scale_f32_32x32x64_f8f6f4 (16 passes) takes the place of two v_mfma_f32_32x32x16_f16 (8 passes each), so
// bytes moved per MFMA cycle are those of the fp16 kernel at twice the flops.  The scales of 512 k (16 blocks = 16
// bytes per row) come into LDS once per eight K-steps with one 16-byte asynchronous copy instruction per wave, are
// rearranged there into the image of a Mat tile of block scales (the scales of one step of consecutive rows in
// consecutive words: a 64-lane read of words 16 bytes apart costs 6 LDS cycles instead of 2), and the two scales a lane
// needs for a K-step are read with the step's fragments (one ds_read_u8 per 32-row block); the MFMA applies them.
// fp4: a 64-byte K-step holds 128 k = two MFMAs (8 passes each) per fragment pair and four scale blocks (one ds_read_b32
// per 32-row block); a scale group is four K-steps.  Same bytes per step again, at four times the fp16 flops.
// m and n need not be multiples of the tile: the last tile row / column is moved back to end at m / n and recomputes
// what it overlaps (m, n >= 256).
#define PTO_WAVES_M 2
#define PTO_WAVES_N 4
#include "gemm_kernels.hpp"

#include <algorithm>

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kMxStepBytes = 64; // one K-step per operand row in LDS
// K-steps per scale group (16 k blocks = one 16-byte scale row): 8 steps of 64 k (8-bit) or 4 steps of 128 k (4-bit)
template <typename T>
constexpr int kMxGroupSteps = 16 / (kMxStepBytes * 8 / detail::elem_bits<T> / 32);

// One asynchronous copy instruction per wave: the 16-byte scale rows (16 k blocks = one scale group) of the workgroup's
// BM rows of A and BN columns of B -> LDS [BM + BN][16 bytes].  Instruction i covers 64 rows; wave w issues instruction
// w % ((BM + BN) / 64) (with fewer instructions than waves some waves repeat one: same data to the same place).
template <int BM, int BN>
AICORE inline void LoadScaleRows(uint32_t ldsOff, __gm__ const uint8_t *sa, __gm__ const uint8_t *sb, int64_t ld)
{
    constexpr int nA = BM / 64, nB = BN / 64;
    static_assert(BM % 64 == 0 && BN % 64 == 0 && nA + nB <= kBlockWaves, "one scale copy instruction per wave");
    int lane = hw::lane();
    // (used once per eight K-steps: keeps the address arithmetic from being hoisted into registers that live across the loop)
    asm volatile("" : "+v"(lane));
    const int inst = hw::wave() % (nA + nB);
    const bool isA = inst < nA;
    const char *base = reinterpret_cast<const char *>(isA ? sa : sb);
    const int row = (isA ? inst : inst - nA) * 64;
    const char *g = detail::uniform_ptr(base + (int64_t)row * ld) + (uint32_t)lane * (uint32_t)ld;
    __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(g), PTO_LDS_PTR(hw::lds_base() + ldsOff + inst * 1024), 16, 0, 0);
}

// [BM + BN][16 bytes] scale rows at `rawOff` -> the LDS images of a [BM, 16] left and a [16, BN] right Mat tile of block
// scales at `dstOff` and `dstOff + BM * 16` ([k block / 4][row][4 k blocks], see detail::ScaleMatGeom): one row per thread
// (with more threads than rows some rows are done twice: same data to the same place, no branch).
template <int BM, int BN>
AICORE inline void RearrangeScaleRows(uint32_t dstOff, uint32_t rawOff)
{
    static_assert(kBlockThreads % (BM + BN) == 0, "one scale row per thread");
    int t = hw::tid();
    asm volatile("" : "+v"(t)); // (as in LoadScaleRows: recompute the addresses rather than keep them in registers)
    t %= BM + BN;
    char *lds = hw::lds_base();
    const u32x4 v = *reinterpret_cast<const u32x4 *>(lds + rawOff + t * 16);
    const bool isA = t < BM;
    char *dst = lds + dstOff + (isA ? 0 : BM * 16) + (isA ? t : t - BM) * 4;
    const int major = isA ? BM : BN;
#pragma unroll
    for (int q = 0; q < 4; ++q)
        *reinterpret_cast<uint32_t *>(dst + q * major * 4) = v[q];
}

template <typename FA, typename FB, typename OutT, int BM, int BN, int STAGES, bool DEEP>
AICORE inline __attribute__((always_inline)) void MxTileRows(__gm__ OutT *out, __gm__ const FA *src0, __gm__ const FB *src1,
                                                             __gm__ const uint8_t *scale0, __gm__ const uint8_t *scale1, int m,
                                                             int n, int k, int row0, int col0)
{
    static_assert(detail::elem_bits<FA> == detail::elem_bits<FB>, "operands of one width");
    // the tile origin comes out of integer divisions, which run on the vector unit: move it (and with it every panel
    // pointer below) into scalar registers
    row0 = __builtin_amdgcn_readfirstlane(row0);
    col0 = __builtin_amdgcn_readfirstlane(col0);
    constexpr int BK = kMxStepBytes * 8 / detail::elem_bits<FA>; // k per K-step
    constexpr int kGroupSteps = kMxGroupSteps<FA>, kStepBlocks = BK / 32;
    constexpr int HM = BM / 2, KB = 16;
    using X = float8_e8m0_t;
    using TileMatA = Tile<TileType::Mat, FA, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, FB, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using TileScaleA = Tile<TileType::Mat, X, BM, KB, BLayout::RowMajor, BM, KB, SLayout::NoneBox>;
    using TileScaleB = Tile<TileType::Mat, X, KB, BN, BLayout::ColMajor, KB, BN, SLayout::NoneBox>;
    using LeftHalf = TileLeft<FA, HM, BK, HM, BK>;
    using RightTile = TileRight<FB, BK, BN, BK, BN>;
    using LeftScaleStep = TileLeftScale<X, HM, kStepBlocks>;
    using RightScaleStep = TileRightScale<X, kStepBlocks, BN>;
    using AccHalf = TileAcc<float, HM, BN, HM, BN>;
    using ShapeA = TileShape2D<FA, BM, BK, Layout::ND>;
    using StrideA = BaseShape2D<FA, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalA = GlobalTensor<FA, ShapeA, StrideA, Layout::ND>;
    using ShapeB = TileShape2D<FB, BK, BN, Layout::DN>;
    using StrideB = BaseShape2D<FB, DYNAMIC, DYNAMIC, Layout::DN>;
    using GlobalB = GlobalTensor<FB, ShapeB, StrideB, Layout::DN>;
    using ShapeC = TileShape2D<OutT, HM, BN, Layout::ND>;
    using StrideC = BaseShape2D<OutT, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<OutT, ShapeC, StrideC, Layout::ND>;

    constexpr uint32_t kABytes = BM * kMxStepBytes, kBBytes = kMxStepBytes * BN;
    constexpr uint32_t kStage = kABytes + kBBytes;
    // scale rows as copied, then two buffers of rearranged scales (the current group's and the next one's)
    constexpr uint32_t kScaleBytes = (BM + BN) * 16, kRawOff = STAGES * kStage, kScaleOff = kRawOff + kScaleBytes;
    constexpr int kLoadsPerStep = TLoadInstrs<TileMatA>() + TLoadInstrs<TileMatB>();
    constexpr int kScaleLoads = 1; // copy instructions per wave and scale group
    constexpr int kMfma = 2 * AccHalf::Storage::MB * AccHalf::Storage::NB * LeftHalf::Storage::KS;
    constexpr int kReadsA = 2 * LeftHalf::Storage::MB, kReadsB = 2 * RightTile::Storage::NB; // two ds_read_b128 per fragment
    constexpr int kReads = 2 * kReadsA + kReadsB + (2 * LeftHalf::Storage::MB + RightTile::Storage::NB); // + the scale reads
    // issue pattern of a step: the copies first, one MFMA before each; the fragment reads spread over the next MFMAs;
    // the last MFMA has no read after it
    constexpr int kMfmaCopies = kMfma >= 8 ? kLoadsPerStep : 1, kMfmaTail = 1;
    constexpr int kMfmaForReads = kMfma - kMfmaCopies - kMfmaTail;
    static_assert(STAGES == 4, "two fragment sets alternate with the stage index");
    static_assert(kMfmaForReads >= 0, "issue pattern below");

    // (operand pointers advance in bytes: one byte per 8-bit element, two 4-bit elements per byte)
    __gm__ FA *aPanel = const_cast<FA *>(src0) + (int64_t)row0 * k * detail::elem_bits<FA> / 8;
    __gm__ FB *bPanel = const_cast<FB *>(src1) + (int64_t)col0 * k * detail::elem_bits<FB> / 8;
    const int64_t ldScale = k / 32;
    __gm__ const uint8_t *saPanel = scale0 + (int64_t)row0 * ldScale;
    __gm__ const uint8_t *sbPanel = scale1 + (int64_t)col0 * ldScale;
    const StrideA strideA(m, k);
    const StrideB strideB(k, n);
    const int kLoop = k / BK, groups = kLoop / kGroupSteps;

    TileMatA aMat[STAGES];
    TileMatB bMat[STAGES];
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        TASSIGN(aMat[s], s * kStage);
        TASSIGN(bMat[s], s * kStage + kABytes);
    }
    TileScaleA aScaleMat;
    TileScaleB bScaleMat;
    TASSIGN(aScaleMat, kScaleOff);
    TASSIGN(bScaleMat, kScaleOff + BM * 16);

    // Operand fragments and their scales.  The lower row half and B have two sets: the MFMAs of step it read set it % 2
    // while the other arrives.  The upper row half, whose MFMAs come first in a step, has one (the register file of two
    // waves per SIMD does not hold a second): its reads for the next step follow its last MFMA and have half a step to land.
    LeftHalf aUp, aDn[2];
    RightTile bAll[2];
    LeftScaleStep saUp, saDn[2];
    RightScaleStep sbAll[2];
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

    // prologue: the scales of group 0, then kAhead K-steps in flight.  DEEP: a step's copies are issued STAGES steps
    // ahead, into the stage whose fragments were read one step earlier (every wave drains its LDS reads before the step's
    // barrier), instead of STAGES-1 steps ahead: they have three K-steps to land instead of two.
    constexpr int kAhead = DEEP ? STAGES : STAGES - 1;
    LoadScaleRows<BM, BN>(kRawOff, saPanel, sbPanel, ldScale);
#pragma unroll
    for (int s = 0; s < kAhead; ++s) {
        GlobalA gmA(aPanel + (int64_t)s * kMxStepBytes, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)s * kMxStepBytes, ShapeB(), strideB);
        TLOAD(aMat[s], gmA);
        TLOAD(bMat[s], gmB);
    }
    wait_flag_pending<(kAhead - 1) * kLoadsPerStep>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); // scales and stage 0 are complete
    RearrangeScaleRows<BM, BN>(kScaleOff, kRawOff);
    hw::lds_barrier();
    {   // scale rows of group 1: rearranged two steps into group 0
        const int g = 1 < groups ? 1 : groups - 1;
        LoadScaleRows<BM, BN>(kRawOff, saPanel + g * 16, sbPanel + g * 16, ldScale);
    }
    TEXTRACT(saUp, aScaleMat, 0, 0);
    TEXTRACT(saDn[0], aScaleMat, HM, 0);
    TEXTRACT(sbAll[0], bScaleMat, 0, 0);
    TEXTRACT(aUp, aMat[0], 0, 0);
    TEXTRACT(aDn[0], aMat[0], HM, 0);
    TEXTRACT(bAll[0], bMat[0], 0, 0);

    // K-step j of a scale group (compile-time: LDS stage j % 4, fragment set j % 2, scales of k blocks 2j, 2j+1 of the
    // group).  Scale buffer group % 2 holds the group's scales.  Past the end of K the copies re-fetch the last K-step /
    // scale group and the reads fetch values nobody uses.
    auto step = [&](auto jTag, int it, int group) {
        constexpr int j = decltype(jTag)::value;
        constexpr int s = j % STAGES, sNext = (s + 1) % STAGES, sLoad = (s + kAhead) % STAGES;
        // the copies of K-step it+1 have landed; only those of the kAhead-2 steps after it may still be in flight, and the
        // scale copy that follows the copies of a group's last step while that step is among them
        hw::wait_vm<(kAhead - 2) * kLoadsPerStep + (j <= kAhead - 3 ? kScaleLoads : 0)>();
        if constexpr (DEEP)
            hw::wait_lgkm0(); // this wave's reads of the stage that the copies below overwrite (issued last step) are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t otherBuf = kScaleOff + (uint32_t)((group + 1) & 1) * kScaleBytes;
        if constexpr (j == 2) {
            // The scale rows of the next group, copied during the previous group's last step (in the prologue for
            // group 1), have landed: the wait above covers every copy older than step 0's.  Into the other buffer, whose
            // scales were last read in the previous group; first read in this group's last step, a barrier later.
            static_assert(kAhead - 3 < 2 && kGroupSteps > 3, "the scale copy is older than every copy that may be in flight here");
            RearrangeScaleRows<BM, BN>(otherBuf, kRawOff);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (j == kGroupSteps - 1) { // the next step is the first of the next group
            TASSIGN(aScaleMat, otherBuf);
            TASSIGN(bScaleMat, otherBuf + BM * 16);
        }
        const int fetch = it + kAhead < kLoop ? it + kAhead : kLoop - 1;
        GlobalA gmA(aPanel + (int64_t)fetch * kMxStepBytes, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)fetch * kMxStepBytes, ShapeB(), strideB);
        TLOAD(aMat[sLoad], gmA);
        TLOAD(bMat[sLoad], gmB);
        if constexpr (j == kGroupSteps - 1) {
            // scale rows of the group after the next one (every wave rearranged the next group's earlier in this group)
            const int g = group + 2 < groups ? group + 2 : groups - 1;
            LoadScaleRows<BM, BN>(kRawOff, saPanel + g * 16, sbPanel + g * 16, ldScale);
        }
        constexpr int p = j & 1, q = p ^ 1, kbNext = kStepBlocks * ((j + 1) % kGroupSteps);
        TMATMUL_MX(cUp, cUp, aUp, saUp, bAll[p], sbAll[p]);
        TEXTRACT(aUp, aMat[sNext], 0, 0);
        TEXTRACT(saUp, aScaleMat, 0, +kbNext);
        TMATMUL_MX(cDn, cDn, aDn[p], saDn[p], bAll[p], sbAll[p]);
        TEXTRACT(bAll[q], bMat[sNext], 0, 0);
        TEXTRACT(sbAll[q], bScaleMat, +kbNext, 0);
        TEXTRACT(aDn[q], aMat[sNext], HM, 0);
        TEXTRACT(saDn[q], aScaleMat, +HM, +kbNext);
#pragma unroll
        for (int i = 0; i < kLoadsPerStep + (j == kGroupSteps - 1 ? kScaleLoads : 0); ++i) {
            if (i < kMfmaCopies)
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        StaticFor<0, kReads>([](auto iTag) {
            constexpr int i = decltype(iTag)::value;
            constexpr int cnt = (i + 1) * kMfmaForReads / kReads - i * kMfmaForReads / kReads;
            if constexpr (cnt > 0)
                __builtin_amdgcn_sched_group_barrier(0x008, cnt, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmaTail, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    static_assert(kGroupSteps % STAGES == 0, "the LDS stage of a step is a compile-time constant");
    for (int group = 0; group < groups; ++group) {
        const int it = group * kGroupSteps;
        StaticFor<0, kGroupSteps>([&](auto jTag) { step(jTag, it + decltype(jTag)::value, group); });
    }
    hw::wait_vm0(); // the copies issued past the end of K must not outlive the workgroup's LDS
    GlobalC dstUp(out + (int64_t)row0 * n + col0, ShapeC(), StrideC(m, n));
    GlobalC dstDn(out + (int64_t)(row0 + HM) * n + col0, ShapeC(), StrideC(m, n));
    TSTORE(dstUp, cUp);
    TSTORE(dstDn, cDn);
}

// The first `fullTiles` workgroups (whole rounds over the compute units) own one BM x BN C tile each; with quarter != 0
// the tiles of the last, partial round are cut into four (BM/2) x (BN/2) tiles, one workgroup each.
template <typename FA, typename FB, typename OutT, int BM, int BN, int STAGES, int GROUP_M, bool DEEP>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmMx(__gm__ OutT *out, __gm__ const FA *src0, __gm__ const FB *src1, __gm__ const uint8_t *scale0,
                __gm__ const uint8_t *scale1, int m, int n, int k, int fullTiles)
{
    const int tilesM = (m + BM - 1) / BM, tilesN = (n + BN - 1) / BN;
    const int block = (int)get_block_idx();
    int tm, tn;
    if (block >= fullTiles) { // (only when m and n are multiples of the tile)
        const int u = RegroupXcd(block - fullTiles, (tilesM * tilesN - fullTiles) * 4);
        TileOfId<GROUP_M>(fullTiles + u / 4, tilesM, tilesN, tm, tn);
        const int sub = u % 4;
        MxTileRows<FA, FB, OutT, BM / 2, BN / 2, STAGES, DEEP>(out, src0, src1, scale0, scale1, m, n, k, tm * BM + (sub >> 1) * (BM / 2),
                                                        tn * BN + (sub & 1) * (BN / 2));
        return;
    }
    TileOfId<GROUP_M>(RegroupXcd(block, fullTiles), tilesM, tilesN, tm, tn);
    // the last tile row / column ends at m / n: it recomputes the rows / columns it shares with its neighbour
    const int row0 = tm * BM + BM <= m ? tm * BM : m - BM, col0 = tn * BN + BN <= n ? tn * BN : n - BN;
    MxTileRows<FA, FB, OutT, BM, BN, STAGES, DEEP>(out, src0, src1, scale0, scale1, m, n, k, row0, col0);
}

} // namespace

PTO_DEVICE_CODE_END

namespace {

template <typename FA, typename FB, typename OutT, bool DEEP = true>
int launch_gemm_mx(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n,
                   int k, int tailMode)
{
    constexpr int BM = 256, BN = 256, STAGES = 4, GROUP_M = 4;
    if (m < BM || n < BN || k % 512) // 512 k = one 16-byte scale row in either operand width
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = STAGES * (BM + BN) * 64 + 3 * (BM + BN) * 16;
    auto kernel = GemmMx<FA, FB, OutT, BM, BN, STAGES, GROUP_M, DEEP>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN), cus = compute_units();
    int full = tiles / cus * cus;
    // quarter tiles move twice the operand bytes per flop: only when they fit one round
    if (tailMode == 0 || full == 0 || (tiles - full) * 4 > cus || m % BM || n % BN)
        full = tiles;
    kernel<<<dim3(full + (tiles - full) * 4), dim3(kBlockThreads), lds, st>>>(
        reinterpret_cast<OutT *>(c), reinterpret_cast<const FA *>(a), reinterpret_cast<const FB *>(b), sa, sb, m, n, k, full);
    return pto_amd::check_launch();
}

template <bool DEEP>
int gemm_mx_dispatch_fmt(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m,
                         int n, int k, int format, int c_fp32, int tailMode)
{
    if (format == 0)
        return c_fp32 ? launch_gemm_mx<float8_e4m3_t, float8_e4m3_t, float, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode) :
                        launch_gemm_mx<float8_e4m3_t, float8_e4m3_t, bfloat16_t, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode);
    if (format == 1)
        return c_fp32 ? launch_gemm_mx<float8_e5m2_t, float8_e5m2_t, float, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode) :
                        launch_gemm_mx<float8_e5m2_t, float8_e5m2_t, bfloat16_t, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode);
    // mixed fp8 operands (the MFMA takes a format per operand): 2 = A e4m3 x B e5m2, 3 = A e5m2 x B e4m3
    if (format == 2)
        return c_fp32 ? launch_gemm_mx<float8_e4m3_t, float8_e5m2_t, float, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode) :
                        launch_gemm_mx<float8_e4m3_t, float8_e5m2_t, bfloat16_t, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode);
    if (format == 3)
        return c_fp32 ? launch_gemm_mx<float8_e5m2_t, float8_e4m3_t, float, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode) :
                        launch_gemm_mx<float8_e5m2_t, float8_e4m3_t, bfloat16_t, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode);
    if (format == 4)
        return c_fp32 ? launch_gemm_mx<float4_e2m1x2_t, float4_e2m1x2_t, float, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode) :
                        launch_gemm_mx<float4_e2m1x2_t, float4_e2m1x2_t, bfloat16_t, DEEP>(st, c, a, b, sa, sb, m, n, k, tailMode);
    return PTO_ERR_UNSUPPORTED;
}

// variant: bit 0 = quarter tiles in the last round, bit 1 = copies issued STAGES-1 instead of STAGES steps ahead
int gemm_mx_dispatch(hipStream_t st, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *sa, const uint8_t *sb, int m, int n,
                     int k, int format, int c_fp32, int variant)
{
    return (variant & 2) ? gemm_mx_dispatch_fmt<false>(st, c, a, b, sa, sb, m, n, k, format, c_fp32, variant & 1) :
                           gemm_mx_dispatch_fmt<true>(st, c, a, b, sa, sb, m, n, k, format, c_fp32, variant & 1);
}

} // namespace

namespace {
// Two kernels: 256 x 256 tiles on eight wavefronts (this file; quarter tiles in a last partial round) and 256 x 192 /
// 256 x 128 tiles on four wavefronts (pto_gemm_mxw4.hip: the faster engine, the smaller tile).  Estimated times in
// microseconds, rounds over the compute units x (K-steps of 128 bytes x step time + fixed time) as measured in one run at
// 4096^3, 6144^3 and 8192^3 (eight against four wavefronts).  fp8: 6144^3 2240 against 2590 TFLOP/s, 8192^3 2460 against
// 2545, 4096^3 2150 against 2165.  fp4: 6144^3 3600 against 4020, 8192^3 4030 against 4090, m, k, n = 2040, 8192, 8100
// (one round of 256 x 256) 3680 against 3910.
bool mx_four_wave_is_faster(int m, int n, int k, int k_bytes, bool fp4)
{
    if (m < 256 || n < 128 || n % 4 != 0 || k % (fp4 ? 1024 : 512) != 0)
        return false;
    const int cus = compute_units(), steps = k_bytes / 128;
    const double t4 = std::min(pto_amd::mx_w4_time(m, n, k_bytes, 192, fp4), pto_amd::mx_w4_time(m, n, k_bytes, 128, fp4));
    double t8 = 1e30;
    if (n >= 256) {
        const double step = fp4 ? 1.63 : 1.5, quarter = fp4 ? 0.25 : 0.34;
        const long long tiles = (long long)((m + 255) / 256) * ((n + 255) / 256), full = tiles / cus, rest = tiles - full * cus;
        const bool quarters = rest > 0 && full > 0 && rest * 4 <= cus && m % 256 == 0 && n % 256 == 0;
        t8 = (double)full * (steps * step + 16.0) + (rest == 0 ? 0.0 : (quarters ? steps * quarter + 16.0 : steps * step + 16.0));
    }
    return t4 < t8;
}
} // namespace

extern "C" int pto_gemm_mxfp8(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a,
                              const uint8_t *scale_b, int m, int n, int k, int format, int c_fp32)
{
    if (!c || !a || !b || !scale_a || !scale_b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    if (format < 0 || format > 3)
        return PTO_ERR_UNSUPPORTED;
    if (mx_four_wave_is_faster(m, n, k, k, false))
        return pto_amd::gemm_mx_w4(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, format, c_fp32, 0);
    return gemm_mx_dispatch(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, format, c_fp32, 1);
}

extern "C" int pto_gemm_mxfp4(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a,
                              const uint8_t *scale_b, int m, int n, int k, int c_fp32)
{
    if (!c || !a || !b || !scale_a || !scale_b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    if (mx_four_wave_is_faster(m, n, k, k / 2, true))
        return pto_amd::gemm_mx_w4(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, 4, c_fp32, 0);
    return gemm_mx_dispatch(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, 4, c_fp32, 1);
}

#if defined(PTO_ST_HOOKS)
// Tuning hook (not part of the public header): variant bit 0 = quarter tiles in the last round, bit 1 = the shallower copy
// pipeline; format 0 / 1 = fp8 e4m3 / e5m2, 4 = fp4 e2m1.
extern "C" int pto_gemm_mxfp8_variant(void *stream, void *c, const uint8_t *a, const uint8_t *b, const uint8_t *scale_a,
                                      const uint8_t *scale_b, int m, int n, int k, int format, int c_fp32, int variant)
{
    if (!c || !a || !b || !scale_a || !scale_b || m <= 0 || n <= 0 || k <= 0 || variant < 0 || variant > 6)
        return PTO_ERR_BAD_ARG;
    if (variant >= 4) // the four-wave engine: 4 = width by rounds, 5 = 256 x 192 tiles, 6 = 256 x 128
        return pto_amd::gemm_mx_w4(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, format, c_fp32,
                                      variant == 4 ? 0 : (variant == 5 ? 192 : 128));
    return gemm_mx_dispatch(static_cast<hipStream_t>(stream), c, a, b, scale_a, scale_b, m, n, k, format, c_fp32, variant);
}
#endif // PTO_ST_HOOKS
