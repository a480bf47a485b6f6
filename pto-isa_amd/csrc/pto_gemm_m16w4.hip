// The 256 x 256 GEMM tile on four wavefronts (wave grid 2 x 2, one wave per SIMD, 128 x 128 of C per wave) on
// v_mfma_f32_16x16x32_f16: a third of the LDS fragment traffic of the eight-wave kernel.  With one wave per SIMD nothing
// hides a stall of that wave, so the K-step is written fragment by fragment: 64 MFMAs, and between them one asynchronous
// copy per eight MFMAs and one fragment read per three, in exactly this order.  The 256 accumulators fill the
// accumulation registers: the MFMAs are issued with the accumulator pinned there (PTO_MFMA_F16_ACC_IN_AGPRS), because
// the compiler's own placement shuttles accumulators between the two register files inside the loop.
#define PTO_WAVES_M 2
#define PTO_WAVES_N 2
#define PTO_MFMA_M 16
#define PTO_MFMA_F16_ACC_IN_AGPRS 1
#include "gemm_kernels.hpp"

PTO_DEVICE_CODE_BEGIN
namespace {

// compile-time loop whose every level is inlined whatever its size
template <int FIRST, int LAST, typename F>
__device__ __attribute__((always_inline)) inline void StaticForInl(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>());
        StaticForInl<FIRST + 1, LAST>(f);
    }
}

// One BM x BN tile of C at (row0, col0): wave (wm, wn) owns rows 32 i + 16 wm .. +15 and columns 32 j + 16 wn .. +15 of
// every 32 x 32 window (i, j), one 16 x 16 accumulator block per window.
template <int BM, int BN>
AICORE inline __attribute__((always_inline)) void FineTile(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m,
                                                           int n, int k, int row0, int col0)
{
    constexpr int BK = 32, STAGES = 4, FB = 32, NFM = BM / FB, NFN = BN / FB, NM = NFM * NFN; // FB: rows (columns) of one fragment window
    using TileMatA = Tile<TileType::Mat, half, BM, BK, BLayout::ColMajor, BM, BK, SLayout::RowMajor>;
    using TileMatB = Tile<TileType::Mat, half, BK, BN, BLayout::RowMajor, BK, BN, SLayout::ColMajor>;
    using LeftF = TileLeft<half, FB, BK, FB, BK>;
    using RightF = TileRight<half, BK, FB, BK, FB>;
    using AccF = TileAcc<float, FB, FB, FB, FB>;
    using ShapeA = TileShape2D<half, BM, BK, Layout::ND>;
    using StrideA = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalA = GlobalTensor<half, ShapeA, StrideA, Layout::ND>;
    using ShapeB = TileShape2D<half, BK, BN, Layout::DN>;
    using StrideB = BaseShape2D<half, DYNAMIC, DYNAMIC, Layout::DN>;
    using GlobalB = GlobalTensor<half, ShapeB, StrideB, Layout::DN>;
    using ShapeC = TileShape2D<float, FB, FB, Layout::ND>;
    using StrideC = BaseShape2D<float, DYNAMIC, DYNAMIC, Layout::ND>;
    using GlobalC = GlobalTensor<float, ShapeC, StrideC, Layout::ND>;
    static_assert(LeftF::Storage::MB == 1 && LeftF::Storage::KS == 1 && RightF::Storage::NB == 1 && AccF::Storage::MB == 1, "one fragment each");
    constexpr uint32_t kABytes = BM * BK * sizeof(half), kBBytes = BK * BN * sizeof(half), kStage = kABytes + kBBytes;
    constexpr int kLoadsA = TLoadInstrs<TileMatA>(), kLoadsB = TLoadInstrs<TileMatB>(), kLoads = kLoadsA + kLoadsB;
    // issue pattern of a K-step: copy c before MFMA c * kCopyEvery; fragment read r of the next step before MFMA
    // r * kReadEvery + 1 (all reads are out by three quarters of the step)
    constexpr int kReads = NFM + NFN, kReadEvery = (NM * 3 / 4) / kReads > 0 ? (NM * 3 / 4) / kReads : 1;
    static_assert(kLoads <= NM && (kReads - 1) * kReadEvery + 1 < NM, "issue pattern");

    const int kLoop = k / BK;
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
    LeftF aF[2][NFM];
    RightF bF[2][NFN];
    detail::AccFrag c[NM]; // accumulator block (i, j) at i * NFN + j
    StaticForInl<0, NM>([&](auto idxTag) __attribute__((always_inline)) {
        c[decltype(idxTag)::value] = detail::AccFrag{0.0f, 0.0f, 0.0f, 0.0f};
    });

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) {
        GlobalA gmA(aPanel + (int64_t)s * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)s * BK, ShapeB(), strideB);
        TLOAD(aMat[s], gmA);
        TLOAD(bMat[s], gmB);
    }
    wait_flag_pending<(STAGES - 2) * kLoads>(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); // stage 0 is complete
    StaticForInl<0, NFM>([&](auto iTag) __attribute__((always_inline)) {
        TEXTRACT(aF[0][decltype(iTag)::value], aMat[0], FB * decltype(iTag)::value, 0);
    });
    StaticForInl<0, NFN>([&](auto jTag) __attribute__((always_inline)) {
        TEXTRACT(bF[0][decltype(jTag)::value], bMat[0], 0, FB * decltype(jTag)::value);
    });

    auto step = [&](auto stageTag, int it) __attribute__((always_inline)) {
        constexpr int s = decltype(stageTag)::value;
        constexpr int sNext = (s + 1) % STAGES, sLoad = (s + STAGES - 1) % STAGES, p = s & 1, q = p ^ 1;
        hw::wait_vm<(STAGES - 3) * kLoads>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int fetch = it + STAGES - 1 < kLoop ? it + STAGES - 1 : kLoop - 1;
        GlobalA gmA(aPanel + (int64_t)fetch * BK, ShapeA(), strideA);
        GlobalB gmB(bPanel + (int64_t)fetch * BK, ShapeB(), strideB);
        StaticForInl<0, NM>([&](auto idxTag) __attribute__((always_inline)) {
            constexpr int idx = decltype(idxTag)::value, i = idx / NFN, j = idx % NFN;
            constexpr int cp = (idx * kLoads + NM - 1) / NM; // copy cp goes before MFMA floor(cp NM / kLoads)
            if constexpr (cp < kLoads && cp * NM / kLoads == idx) { // a copy of the operands three steps ahead
                if constexpr (cp < kLoadsA)
                    TLOAD_SLICE<cp>(aMat[sLoad], gmA);
                else
                    TLOAD_SLICE<cp - kLoadsA>(bMat[sLoad], gmB);
            }
            if constexpr (idx % kReadEvery == 1 % kReadEvery && (idx - 1) / kReadEvery < kReads && idx >= 1) {
                // a fragment read of the next step, in the order in which that step needs them: A 0, all of B, A 1 ..
                constexpr int rd = (idx - 1) / kReadEvery;
                if constexpr (rd == 0)
                    TEXTRACT(aF[q][0], aMat[sNext], 0, 0);
                else if constexpr (rd <= NFN)
                    TEXTRACT(bF[q][rd - 1], bMat[sNext], 0, FB * (rd - 1));
                else
                    TEXTRACT(aF[q][rd - NFN], aMat[sNext], FB * (rd - NFN), 0);
            }
            c[idx] = detail::mfma32(aF[p][i].st.f[0][0], bF[p][j].st.f[0][0], c[idx]); // TMATMUL_ACC on one fragment each
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using std::integral_constant;
    for (int it = 0; it < kLoop; it += STAGES) {
        step(integral_constant<int, 0>(), it);
        step(integral_constant<int, 1>(), it + 1);
        step(integral_constant<int, 2>(), it + 2);
        step(integral_constant<int, 3>(), it + 3);
    }
    hw::wait_vm0(); // the copies issued past the end of K must not outlive the workgroup's LDS
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the last MFMAs have written their accumulators
    const StrideC strideC(m, n);
    StaticForInl<0, NM>([&](auto idxTag) __attribute__((always_inline)) {
        constexpr int i = decltype(idxTag)::value / NFN, j = decltype(idxTag)::value % NFN;
        GlobalC dst(out + (int64_t)(row0 + FB * i) * n + col0 + FB * j, ShapeC(), strideC);
        AccF block;
        block.st.f[0][0] = c[i * NFN + j];
        TSTORE(dst, block);
    });
}

// The first `fullTiles` workgroups own one 256 x 256 tile each; the tiles of the last, partial round are cut into four
// 128 x 128 quarter tiles, one workgroup each, so that the round fills the machine.
template <int BM, int BN, int GROUP_M>
__global__ __launch_bounds__(kBlockThreads, 1) AICORE
    void GemmF16F32Fine(__gm__ float *out, __gm__ const half *src0, __gm__ const half *src1, int m, int n, int k, int fullTiles)
{
    const int tilesM = m / BM, tilesN = n / BN, block = (int)get_block_idx();
    int tm, tn;
    if (block < fullTiles) {
        TileOfId<GROUP_M>(RegroupXcd(block, fullTiles), tilesM, tilesN, tm, tn);
        FineTile<BM, BN>(out, src0, src1, m, n, k, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * BN));
    } else if constexpr (BM % 128 == 0 && BN % 128 == 0) {
        const int u = RegroupXcd(block - fullTiles, (tilesM * tilesN - fullTiles) * 4);
        TileOfId<GROUP_M>(fullTiles + u / 4, tilesM, tilesN, tm, tn);
        const int sub = u % 4;
        FineTile<BM / 2, BN / 2>(out, src0, src1, m, n, k, __builtin_amdgcn_readfirstlane(tm * BM + (sub >> 1) * (BM / 2)),
                                 __builtin_amdgcn_readfirstlane(tn * BN + (sub & 1) * (BN / 2)));
    }
}

} // namespace
PTO_DEVICE_CODE_END

namespace {
template <int BM, int BN>
int launch_fine(hipStream_t st, float *c, const half *a, const half *b, int m, int n, int k, bool quarterTail)
{
    if (m % BM || n % BN || k % 128 || k < 256)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 4 * (BM * 32 + 32 * BN) * (int)sizeof(half);
    auto kernel = GemmF16F32Fine<BM, BN, 4>;
    static const int attr = pto_amd::allow_lds(kernel, lds);
    if (attr != PTO_OK)
        return attr;
    const int tiles = (m / BM) * (n / BN), cus = compute_units();
    int full = tiles / cus * cus;
    // quarter tiles for the last round when they fit two rounds of their own
    if (!quarterTail || BM % 128 || BN % 128 || full == 0 || (tiles - full) * 4 > 2 * cus)
        full = tiles;
    kernel<<<dim3((unsigned)(full + (tiles - full) * 4)), dim3(kBlockThreads), lds, st>>>(c, a, b, m, n, k, full);
    return pto_amd::check_launch();
}
} // namespace

namespace pto_amd {
// 256 x 256 C tiles on four wavefronts when they fill the machine at least once; 192 x 192 tiles when those put more
// compute units to work in a single round (3072^3: 256 instead of 144 workgroups).  PTO_ERR_UNSUPPORTED: not a shape
// for this kernel (the caller falls back to the eight-wave one).
int gemm_f16f32_tile256_w4(hipStream_t st, float *c, const _Float16 *a, const _Float16 *b, int m, int n, int k)
{
    const int cus = compute_units();
    // (measured against the eight-wave kernel: +1 % at 6144^3, +5 % at 7680^3; -4 % at 4096^3 and equal at 8192^3, where
    // the tiles fill whole rounds - those stay with the eight-wave kernel)
    if (m % 256 == 0 && n % 256 == 0 && (long long)(m / 256) * (n / 256) >= cus && ((long long)(m / 256) * (n / 256)) % cus != 0)
        return launch_fine<256, 256>(st, c, a, b, m, n, k, true);
    if (m % 192 == 0 && n % 192 == 0) {
        const long long t192 = (long long)(m / 192) * (n / 192), t256 = (m % 256 || n % 256) ? 0 : (long long)(m / 256) * (n / 256);
        if (t192 <= cus && t192 > t256 && t192 * 2 >= cus)
            return launch_fine<192, 192>(st, c, a, b, m, n, k, false);
    }
    return PTO_ERR_UNSUPPORTED;
}
} // namespace pto_amd

#if defined(PTO_ST_HOOKS)
extern "C" int pto_gemm_f16f32_m16w4_variant(void *stream, float *c, const uint16_t *a, const uint16_t *b, int m, int n, int k,
                                             int variant)
{
    if (!c || !a || !b || m <= 0 || n <= 0 || k <= 0)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b);
    switch (variant) {
    case 0: return launch_fine<256, 256>(st, c, ha, hb, m, n, k, true);
    case 1: return launch_fine<256, 256>(st, c, ha, hb, m, n, k, false);
    case 2: return launch_fine<192, 256>(st, c, ha, hb, m, n, k, false);
    case 3: return launch_fine<256, 192>(st, c, ha, hb, m, n, k, false);
    case 4: return launch_fine<192, 192>(st, c, ha, hb, m, n, k, false);
    default: return PTO_ERR_BAD_ARG;
    }
}
#endif // PTO_ST_HOOKS
