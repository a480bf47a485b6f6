// Matmul instruction programs on ragged tiles: valid m, k, n inside tiles rounded up to 16 rows and 32 bytes, as the
// reference's own tests of TMOV / TMATMUL / TMATMUL_ACC / TMATMUL_BIAS / TGEMV / TSTORE build them
// (tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:26-97, tests/npu/a2a3/src/st/testcase/tmatmul/tmatmul_kernel.cpp:113-197).
// One workgroup: TLOAD the [m, k] and [k, n] matrices into L1 tiles (both row-major in memory), TMOV into Left / Right
// tiles, multiply (optionally in two k halves, the second accumulating, or with a bias row), TSTORE the valid region.
// Part of the test library only.
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int ceil_to(int v, int q) { return (v + q - 1) / q * q; }

enum class Form { Plain, Bias, SplitK, Gemv };

// MP: rows the m extent is rounded up to (16 as on the NPU, or more to reach whole MFMA blocks per wave)
// NP: likewise for n (the CPU tests' rule: 16 columns, 32 for 8-bit operands)
template <typename OutT, typename InT, int vM, int vK, int vN, Form form, int MP = 16, int NP = (sizeof(InT) == 1 ? 32 : 16)>
__global__ __launch_bounds__(kBlockThreads) AICORE void RaggedMatmul(__gm__ OutT *out, __gm__ const InT *src0, __gm__ const InT *src1,
                                                                     __gm__ const OutT *src2)
{
    constexpr int kAlign = 32 / (int)sizeof(InT);
    constexpr int M = ceil_to(vM, MP), K = ceil_to(vK, kAlign), N = ceil_to(vN, NP);
    using GmA = GlobalTensor<InT, Shape<1, 1, 1, vM, vK>, Stride<vM * vK, vM * vK, vM * vK, vK, 1>>;
    using GmB = GlobalTensor<InT, Shape<1, 1, 1, vK, vN>, Stride<vK * vN, vK * vN, vK * vN, vN, 1>>;
    using GmBias = GlobalTensor<OutT, Shape<1, 1, 1, 1, vN>, Stride<vN, vN, vN, vN, 1>>;
    using GmC = GlobalTensor<OutT, Shape<1, 1, 1, vM, vN>, Stride<vM * vN, vM * vN, vM * vN, vN, 1>>;
    using MatA = Tile<TileType::Mat, InT, M, K, BLayout::ColMajor, vM, vK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, InT, K, N, BLayout::ColMajor, vK, vN, SLayout::RowMajor, 512>;
    using MatBias = Tile<TileType::Mat, OutT, 1, N, BLayout::RowMajor, 1, vN>;
    using BiasT = Tile<TileType::Bias, OutT, 1, N, BLayout::RowMajor, 1, vN>;
    GmA gA(const_cast<InT *>(src0));
    GmB gB(const_cast<InT *>(src1));
    GmC gC(out);
    MatA aMat;
    MatB bMat;
    constexpr int kBytesA = M * K * (int)sizeof(InT), kBytesB = K * N * (int)sizeof(InT);
    TASSIGN(aMat, 0x0);
    TASSIGN(bMat, kBytesA);
    TLOAD(aMat, gA);
    TFILLPAD(aMat, aMat);
    TLOAD(bMat, gB);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    if constexpr (form == Form::SplitK) {
        // two k halves through TEXTRACT windows, the second accumulating (tmatmul_kernel.cpp:200-290 of the NPU tests)
        static_assert(K >= 2 * kAlign, "at least two 32-byte k blocks");
        constexpr int K0 = ceil_to(K / 2, kAlign), K1 = K - K0, v0 = vK < K0 ? vK : K0, v1 = vK - v0;
        TileLeft<InT, M, K0, vM, v0> a0;
        TileRight<InT, K0, N, v0, vN> b0;
        TileLeft<InT, M, K1, vM, v1> a1;
        TileRight<InT, K1, N, v1, vN> b1;
        TileAcc<OutT, M, N, vM, vN> c;
        TEXTRACT(a0, aMat, 0, 0);
        TEXTRACT(b0, bMat, 0, 0);
        TMATMUL(c, a0, b0);
        TEXTRACT(a1, aMat, 0, K0);
        TEXTRACT(b1, bMat, K0, 0);
        TMATMUL_ACC(c, c, a1, b1);
        TSTORE(gC, c);
    } else {
        TileLeft<InT, M, K, vM, vK> a;
        TileRight<InT, K, N, vK, vN> b;
        TileAcc<OutT, M, N, vM, vN> c;
        TMOV(a, aMat);
        TMOV(b, bMat);
        if constexpr (form == Form::Bias) {
            // the bias row goes through L1 into a Bias tile (NPU form), or straight from memory (CPU form): both
            GmBias gBias(const_cast<OutT *>(src2));
            MatBias biasMat;
            TASSIGN(biasMat, kBytesA + kBytesB);
            TLOAD(biasMat, gBias);
            set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID1);
            wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID1);
            BiasT bias, bias2;
            TMOV(bias, biasMat);
            TLOAD(bias2, gBias);
            TMATMUL_BIAS(c, a, b, bias);
            TileAcc<OutT, M, N, vM, vN> c2;
            TMATMUL_BIAS(c2, a, b, bias2);
            // what is stored is the sum of the two results
            TSTORE(gC, c);
            TSTORE<TileAcc<OutT, M, N, vM, vN>, GmC, AtomicType::AtomicAdd>(gC, c2);
        } else if constexpr (form == Form::Gemv) {
            TGEMV(c, a, b);
            TSTORE(gC, c);
        } else {
            TMATMUL(c, a, b);
            TSTORE(gC, c);
        }
    }
}

} // namespace

PTO_DEVICE_CODE_END

// dynamic LDS of a case: the two L1 tiles and the bias row; refused (not launched) when the kernel's static LDS, the
// staging buffers of the general matmul path, would push the workgroup past a compute unit's 160 KiB
template <typename OutT, typename InT, int vM, int vK, int vN, Form form, int MP = 16, int NP = (sizeof(InT) == 1 ? 32 : 16)>
static int launch_ragged(hipStream_t st, void *out, const void *a, const void *b, const void *bias)
{
    constexpr int kAlign = 32 / (int)sizeof(InT);
    constexpr int M = ceil_to(vM, MP), K = ceil_to(vK, kAlign), N = ceil_to(vN, NP);
    constexpr int want = (M * K + K * N) * (int)sizeof(InT) + N * (int)sizeof(OutT);
    auto kernel = RaggedMatmul<OutT, InT, vM, vK, vN, form, MP, NP>;
    hipFuncAttributes attr{};
    if (hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel)) != hipSuccess)
        return PTO_ERR_HIP;
    if ((int)attr.sharedSizeBytes + want > 160 * 1024)
        return PTO_ERR_UNSUPPORTED;
    if (form == Form::Bias && bias == nullptr)
        return PTO_ERR_BAD_ARG;
    static const int attr_rc = pto_amd::allow_lds(kernel, want);
    if (attr_rc != PTO_OK)
        return attr_rc;
    kernel<<<dim3(1), dim3(kBlockThreads), want, st>>>(static_cast<OutT *>(out), static_cast<const InT *>(a), static_cast<const InT *>(b),
                                                       static_cast<const OutT *>(bias));
    return pto_amd::check_launch();
}
#define PTO_RAGGED(...) return launch_ragged<__VA_ARGS__>(st, out, a, b, bias)

// case: see tests/matmul_any_cases.py (the table there and this switch are kept in step by a test)
extern "C" int pto_st_matmul_ragged(void *stream, void *out, const void *a, const void *b, const void *bias, int case_id)
{
    if (out == nullptr || a == nullptr || b == nullptr)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (case_id) {
    case 0: PTO_RAGGED(float, half, 40, 50, 60, Form::Plain);
    case 1: PTO_RAGGED(int32_t, int8_t, 6, 7, 8, Form::Plain);
    case 2: PTO_RAGGED(float, float, 120, 110, 50, Form::Plain);
    case 3: PTO_RAGGED(int32_t, int8_t, 8, 7, 6, Form::Bias);
    case 4: PTO_RAGGED(float, half, 16, 15, 16, Form::Bias);
    case 5: PTO_RAGGED(float, float, 127, 128, 63, Form::Bias);
    case 6: PTO_RAGGED(float, half, 31, 120, 58, Form::Plain);
    case 7: PTO_RAGGED(int32_t, int8_t, 65, 90, 89, Form::Plain);
    case 8: PTO_RAGGED(float, half, 5, 75, 11, Form::SplitK);
    case 9: PTO_RAGGED(float, half, 1, 256, 64, Form::Gemv);
    case 10: PTO_RAGGED(float, half, 1, 200, 32, Form::Gemv);
    case 11: PTO_RAGGED(float, float, 5, 75, 11, Form::Plain);
    case 12: PTO_RAGGED(float, bfloat16_t, 33, 47, 19, Form::Bias);
    // whole MFMA blocks per wave with a valid region inside: the fragment path on operands zeroed outside it
    case 13: PTO_RAGGED(float, half, 60, 50, 58, Form::Plain, 64, 64);
    case 14: PTO_RAGGED(float, half, 100, 70, 120, Form::SplitK, 64, 64);
    // Left in fragments, Right and Acc plain; and the other way round
    case 15: PTO_RAGGED(float, half, 64, 64, 16, Form::Plain, 64, 16);
    case 16: PTO_RAGGED(float, half, 20, 64, 64, Form::Bias, 16, 64);
    default: return PTO_ERR_UNSUPPORTED;
    }
}
