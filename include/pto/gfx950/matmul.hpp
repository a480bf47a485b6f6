// TMATMUL / TMATMUL_ACC / TMATMUL_BIAS for gfx950: chains of v_mfma_f32_32x32x16_{f16,bf16} (or, with
// PTO_MFMA_M 16, v_mfma_f32_16x16x32_{f16,bf16}); int8 x int8 -> int32 on v_mfma_i32_32x32x32_i8 / 16x16x64 and
// fp32 x fp32 -> fp32 on v_mfma_f32_32x32x2_f32 / 16x16x4 (the type triples of include/pto/cpu/TMatmul.hpp:46-51).
//
// Reference semantics (include/pto/cpu/TMatmul.hpp:73-116):
//   C[i,j] = (acc ? acc[i,j] : 0) + sum_k (CT)A[i,k] * (CT)B[k,j],  M,K,N = a.validRow, a.validCol, b.validCol
// Each wave owns the (Rows/PTO_WAVES_M) x (Cols/PTO_WAVES_N) sub-block of C selected by its
// position in the wave grid and holds the matching rows of A / columns of B as fragments.
// Products are exact in fp32; the order of the fp32 additions inside an MFMA differs from the
// reference's sequential k loop, which is what the 2e-3 relative tolerance covers.
#pragma once
#include "pto/common/tile.hpp"

namespace pto {
namespace detail {

// The general path for tiles that are not whole MFMA blocks per wave (pto/gfx950/matmul_any.hpp, defined after the
// memory and vector instructions it builds on).
template <typename TileT>
constexpr bool is_plain_v = is_plain_storage<typename TileT::Storage>::value;
template <typename TileT>
constexpr bool is_fully_valid_v = TileT::ValidRow == TileT::Rows && TileT::ValidCol == TileT::Cols;
template <typename TileT, typename F>
PTO_DEV void for_each_elem(TileT &t, F &&fn);
template <bool kZeroInit, typename AccT, typename LeftT, typename RightT>
PTO_DEV void mad_any(AccT &out, AccT &in, LeftT &a, RightT &b);
template <typename AccT, typename BiasT>
PTO_DEV void add_bias_any(AccT &c, BiasT &bias);
template <typename DstT, typename SrcT>
PTO_DEV void textract_any(DstT &dst, SrcT &src, uint32_t idxRow, uint32_t idxCol);
template <typename TileT, typename G>
PTO_DEV void tload_any(TileT &dst, G &src);
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu>
PTO_DEV void tstore_any(G &dst, TileT &src);
template <typename TileT>
PTO_DEV void zero_outside_valid(TileT &t);
// the conversion on the accumulator's way out (pto/gfx950/fixpipe.hpp): none but the cast, one quantisation word for the
// tile, one word per column
struct FixNone {};
struct FixScalar {
    uint64_t q;
};
struct FixVector {
    const uint64_t *table;
};
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu, typename P>
PTO_DEV void tstore_fix(G &dst, TileT &src, const P &p);
template <ReluPreMode relu, typename DstT, typename SrcT, typename P>
PTO_DEV void textract_fix(DstT &dst, SrcT &src, int idxRow, int idxCol, const P &p);
template <typename DstT, typename SrcT>
PTO_DEV void tfillpad_mat(DstT &dst, SrcT &src);

// (the accumulator type is a template parameter only so that the branch for the other MFMA shape is discarded
// instead of type-checked)
template <typename C>
PTO_DEV C mfma32(f16x8 a, f16x8 b, C c)
{
    static_assert(std::is_same_v<C, AccFrag>, "accumulator fragment of the configured MFMA shape");
#ifdef PTO_MFMA_F16_ACC_IN_AGPRS
    // The accumulator is pinned to the accumulation registers and the instruction keeps its place in the program: for
    // kernels of one wave per SIMD that use all 256 accumulation registers, where the compiler's own choice between
    // the two register files moves accumulators back and forth.  The caller leaves the wait states that the hardware
    // needs between the last MFMA and the first ordinary read of an accumulator (s_nop) to this header's user.
    if constexpr (sizeof(C) == 16) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
        return c;
    }
#endif
    if constexpr (sizeof(C) == 64)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
template <typename C>
PTO_DEV C mfma32(bf16x8 a, bf16x8 b, C c)
{
    static_assert(std::is_same_v<C, AccFrag>, "accumulator fragment of the configured MFMA shape");
    if constexpr (sizeof(C) == 64)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// one 16-byte chunk per lane of each operand: 16 int8 values, one MFMA of twice the fp16 k extent
template <typename C>
PTO_DEV C mfma32(i32x4 a, i32x4 b, C c)
{
    static_assert(std::is_same_v<C, AccFragI32>, "int32 accumulator fragment of the configured MFMA shape");
    if constexpr (sizeof(C) == 64)
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}
// 4 fp32 values per lane: four MFMAs, MFMA s takes value s of every lane's chunk
template <typename C>
PTO_DEV C mfma32(f32x4 a, f32x4 b, C c)
{
    static_assert(std::is_same_v<C, AccFrag>, "accumulator fragment of the configured MFMA shape");
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        if constexpr (sizeof(C) == 64)
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], c, 0, 0, 0);
        else
            c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], b[s], c, 0, 0, 0);
    }
    return c;
}

template <typename AccT, typename LeftT, typename RightT>
PTO_DEV constexpr void check_mad_types()
{
    using A = typename LeftT::DType;
    using B = typename RightT::DType;
    using CT = typename AccT::DType;
    static_assert(std::is_same_v<A, B> &&
                      (((std::is_same_v<A, half> || std::is_same_v<A, bfloat16_t> || std::is_same_v<A, float>) && std::is_same_v<CT, float>) ||
                       (std::is_same_v<A, int8_t> && std::is_same_v<CT, int32_t>)),
                  "[PTO][SA] TMATMUL on gfx950: fp16 / bf16 / fp32 operands -> fp32, or int8 x int8 -> int32");
    static_assert(LeftT::Loc == TileType::Left && RightT::Loc == TileType::Right && AccT::Loc == TileType::Acc,
                  "[PTO][SA] TMATMUL: operands must be Left, Right and Acc tiles");
}
template <typename AccT, typename LeftT, typename RightT>
PTO_DEV constexpr void check_mad()
{
    check_mad_types<AccT, LeftT, RightT>();
    static_assert(LeftT::Rows == AccT::Rows && LeftT::Cols == RightT::Rows && RightT::Cols == AccT::Cols,
                  "[PTO][SA] TMATMUL: inconsistent m, k, n");
}
// operands with a valid region inside the tile were zeroed outside it when they were extracted: the fragment path
// multiplies whole tiles
template <typename AccT, typename LeftT, typename RightT>
constexpr bool any_plain_v = is_plain_v<AccT> || is_plain_v<LeftT> || is_plain_v<RightT>;

template <bool kZeroInit, typename AccT, typename LeftT, typename RightT>
PTO_DEV void mad(AccT &out, const AccT &in, const LeftT &a, const RightT &b)
{
    using SA = typename AccT::Storage;
    using SL = typename LeftT::Storage;
    using CFrag = typename AccFragOf<typename AccT::DType>::type;
#pragma unroll
    for (int mb = 0; mb < SA::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < SA::NB; ++nb) {
            CFrag c;
            if constexpr (kZeroInit) {
#pragma unroll
                for (int i = 0; i < kAccElems; ++i)
                    c[i] = 0;
            } else {
                c = in.S().f[mb][nb];
            }
#pragma unroll
            for (int ks = 0; ks < SL::KS; ++ks)
                c = mfma32(a.S().f[mb][ks], b.S().f[nb][ks], c);
            out.S().f[mb][nb] = c;
        }
}

} // namespace detail

template <typename AccT, typename LeftT, typename RightT>
PTO_DEV void TMATMUL_IMPL(AccT &c, LeftT &a, RightT &b)
{
    detail::check_mad<AccT, LeftT, RightT>();
    if constexpr (detail::any_plain_v<AccT, LeftT, RightT>)
        detail::mad_any<true>(c, c, a, b);
    else
        detail::mad<true>(c, c, a, b);
}

template <typename AccT, typename LeftT, typename RightT>
PTO_DEV void TMATMUL_ACC_IMPL(AccT &cOut, AccT &cIn, LeftT &a, RightT &b)
{
    detail::check_mad<AccT, LeftT, RightT>();
    if constexpr (detail::any_plain_v<AccT, LeftT, RightT>)
        detail::mad_any<false>(cOut, cIn, a, b);
    else
        detail::mad<false>(cOut, cIn, a, b);
}

// TMATMUL_MX: C (+)= (A * scaleA) x (B * scaleB) on 8-bit MX operands, one e8m0 scale per row (column) and 32-wide
// k block; operands may also be 4-bit e2m1 pairs (reference semantics: the data generators of tests/npu/a5/src/st/testcase/tmatmul_mx and
// kernels/manual/a5/matmul_mxfp8_performance/scripts/gen_data.py:24-50: operand element x 2^(scale - 127), products
// accumulated in fp32).  v_mfma_scale_f32_32x32x64_f8f6f4 applies the scales inside the MFMA.
namespace detail {
template <typename T>
constexpr int mx_format = is_mx4_v<T> ? 4 : std::is_same_v<T, float8_e5m2_t> ? 1 : 0; // the MFMA's cbsz / blgp operand-format code

// the MFMA's operand type is eight registers whatever the format; 4-bit operands occupy the first four
PTO_DEV i32x8 mx_operand(i32x8 f) { return f; }
PTO_DEV i32x8 mx_operand(u32x4 f) { return i32x8{(int)f[0], (int)f[1], (int)f[2], (int)f[3], 0, 0, 0, 0}; }

template <bool kZeroInit, typename AccT, typename LeftT, typename LeftScaleT, typename RightT, typename RightScaleT>
PTO_DEV void mad_mx(AccT &out, const AccT &in, const LeftT &a, const LeftScaleT &sa, const RightT &b, const RightScaleT &sb)
{
    static_assert(is_mx_operand_v<typename LeftT::DType> && is_mx_operand_v<typename RightT::DType> &&
                      std::is_same_v<typename AccT::DType, float>,
                  "[PTO][SA] TMATMUL_MX on gfx950: fp8 (e4m3 / e5m2) or fp4 (e2m1) operands, fp32 accumulator");
    static_assert(LeftT::Loc == TileType::Left && RightT::Loc == TileType::Right && AccT::Loc == TileType::Acc &&
                      LeftScaleT::Loc == TileType::ScaleLeft && RightScaleT::Loc == TileType::ScaleRight,
                  "[PTO][SA] TMATMUL_MX: operands must be Left, ScaleLeft, Right, ScaleRight and Acc tiles");
    static_assert(LeftT::Rows == AccT::Rows && LeftT::Cols == RightT::Rows && RightT::Cols == AccT::Cols,
                  "[PTO][SA] TMATMUL_MX: inconsistent m, k, n");
    static_assert(LeftScaleT::Rows == LeftT::Rows && LeftScaleT::Cols * kMxBlock == LeftT::Cols &&
                      RightScaleT::Cols == RightT::Cols && RightScaleT::Rows * kMxBlock == RightT::Rows,
                  "[PTO][SA] TMATMUL_MX: one scale per row (column) and 32 k values");
    using SA = typename AccT::Storage;
    using SL = typename LeftT::Storage;
    constexpr int fa = mx_format<typename LeftT::DType>, fb = mx_format<typename RightT::DType>;
#pragma unroll
    for (int mb = 0; mb < SA::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < SA::NB; ++nb) {
            AccFrag c;
            if constexpr (kZeroInit) {
#pragma unroll
                for (int i = 0; i < kAccElems; ++i)
                    c[i] = 0.0f;
            } else {
                c = in.S().f[mb][nb];
            }
#pragma unroll
            for (int ks = 0; ks < SL::KS; ++ks) {
                // k step ks: scale byte 0 (even step) or 2 (odd step) of register ks / 2
                if (ks % 2 == 0)
                    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(mx_operand(a.S().f[mb][ks]), mx_operand(b.S().f[nb][ks]), c, fa, fb,
                                                                        0, (int)sa.S().s[mb][ks / 2], 0, (int)sb.S().s[nb][ks / 2]);
                else
                    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(mx_operand(a.S().f[mb][ks]), mx_operand(b.S().f[nb][ks]), c, fa, fb,
                                                                        2, (int)sa.S().s[mb][ks / 2], 2, (int)sb.S().s[nb][ks / 2]);
            }
            out.S().f[mb][nb] = c;
        }
}
} // namespace detail

template <typename AccT, typename LeftT, typename LeftScaleT, typename RightT, typename RightScaleT>
PTO_DEV void TMATMUL_MX_IMPL(AccT &c, LeftT &a, LeftScaleT &sa, RightT &b, RightScaleT &sb)
{
    detail::mad_mx<true>(c, c, a, sa, b, sb);
}
template <typename AccT, typename LeftT, typename LeftScaleT, typename RightT, typename RightScaleT>
PTO_DEV void TMATMUL_MX_IMPL(AccT &cOut, AccT &cIn, LeftT &a, LeftScaleT &sa, RightT &b, RightScaleT &sb)
{
    detail::mad_mx<false>(cOut, cIn, a, sa, b, sb);
}

// bias: a 1 x N fp32 row held as a Vec-distributed tile is not addressable per column from a
// wave's accumulator lanes, so the bias row is read from memory: BiasT must expose `const float *row`.
struct BiasRow {
    const float *row;
};

// the reference's form: the bias is a [1, n] Bias tile (pto_instr.hpp:504-511 of the reference, cpu/TMatmul.hpp:109-115)
template <typename AccT, typename LeftT, typename RightT, typename BiasT>
PTO_DEV void TMATMUL_BIAS_IMPL(AccT &c, LeftT &a, RightT &b, BiasT &bias)
{
    TMATMUL_IMPL(c, a, b);
    detail::add_bias_any(c, bias);
}
// the same for MX operands: the scaled product, then the bias row added to every row of the result
template <typename AccT, typename LeftT, typename LeftScaleT, typename RightT, typename RightScaleT, typename BiasT>
PTO_DEV std::enable_if_t<BiasT::Loc == TileType::Bias> TMATMUL_MX_IMPL(AccT &c, LeftT &a, LeftScaleT &sa, RightT &b, RightScaleT &sb,
                                                                     BiasT &bias)
{
    detail::mad_mx<true>(c, c, a, sa, b, sb);
    detail::add_bias_any(c, bias);
}

template <typename AccT, typename LeftT, typename RightT>
PTO_DEV void TMATMUL_BIAS_IMPL(AccT &c, LeftT &a, RightT &b, BiasRow bias)
{
    detail::check_mad<AccT, LeftT, RightT>();
    static_assert(!detail::any_plain_v<AccT, LeftT, RightT>, "[PTO][SA] TMATMUL_BIAS with a bias row in memory: fragment tiles (pass a Bias tile otherwise)");
    detail::mad<true>(c, c, a, b);
    using SA = typename AccT::Storage;
    const int col0 = hw::wave_n() * (SA::NB * detail::kMfmaM) + detail::acc_lane_col((uint32_t)hw::lane());
#pragma unroll
    for (int nb = 0; nb < SA::NB; ++nb) {
        const float bv = bias.row[col0 + nb * detail::kMfmaM]; // cpu/TMatmul.hpp:109-115: added after the product
#pragma unroll
        for (int mb = 0; mb < SA::MB; ++mb)
#pragma unroll
            for (int i = 0; i < detail::kAccElems; ++i)
                c.S().f[mb][nb][i] += bv;
    }
}

} // namespace pto
