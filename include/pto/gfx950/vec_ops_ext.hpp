// Further Vec-tile instructions for gfx950: unary math, ReLU family, compare / select, column
// reductions and broadcasts, row minimum / broadcast, TFILLPAD, and TMOV from an accumulator tile.
// Semantics follow the reference's CPU simulation (file:line at each op).  Vec tiles are distributed
// over the workgroup as in vec_ops.hpp; ops that cross lanes stage through small static LDS arrays.
#pragma once
#include "pto/gfx950/vec_ops.hpp"

#pragma clang fp contract(off) // as in vec_ops.hpp: instructions round on their own
namespace pto {

// ------------------------------------------------------------------ unary
// The CPU simulation evaluates sqrt / log / exp in double and casts (ElementOp.h:265-340, TSqrt.hpp:23,
// TRSqrt.hpp:30): the same is done here, these are not hot-loop ops.
#define PTO_DEFINE_UNARY(NAME, EXPR)                                                                    \
    template <typename DstT, typename SrcT>                                                             \
    PTO_DEV void NAME##_IMPL(DstT &dst, SrcT &src)                                                      \
    {                                                                                                   \
        using T = typename DstT::DType;                                                                 \
        using S = typename DstT::Storage;                                                               \
        detail::Conformed<DstT, SrcT> c0(src);                                                          \
        _Pragma("unroll") for (int s = 0; s < S::Slots; ++s) _Pragma("unroll") for (int i = 0; i < detail::kVecChunk; ++i) \
        {                                                                                               \
            const T a = c0.S().v[s][i];                                                                  \
            dst.S().v[s][i] = (EXPR);                                                                    \
        }                                                                                               \
    }
PTO_DEFINE_UNARY(TABS, (a < (T)0 ? -a : a))                                // TAbs.hpp:24
PTO_DEFINE_UNARY(TNEG, -a)                                                 // ElementOp.h:297-302
PTO_DEFINE_UNARY(TRELU, (a < (T)0 ? (T)0 : a))                             // ElementOp.h:345-350 (max(a, 0))
PTO_DEFINE_UNARY(TSQRT, (T)::sqrt((double)a))                      // TSqrt.hpp:23
PTO_DEFINE_UNARY(TRSQRT, (T)(1.0 / ::sqrt((double)a)))             // TRSqrt.hpp:29-31
PTO_DEFINE_UNARY(TLOG, (T)::log((double)a))                        // ElementOp.h:289-294
PTO_DEFINE_UNARY(TRECIP, (T)((T)1 / a))                                    // ElementOp.h:321-330
#undef PTO_DEFINE_UNARY

// dst = src0 > 0 ? src0 : src0 * src1  (ElementOp.h:257-262)
template <typename DstT, typename S0T, typename S1T>
PTO_DEV void TPRELU_IMPL(DstT &dst, S0T &src0, S1T &src1)
{
    using T = typename DstT::DType;
    using S = typename DstT::Storage;
    detail::Conformed<DstT, S0T> c0(src0);
    detail::Conformed<DstT, S1T> c1(src1);
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i) {
            const T a = c0.S().v[s][i], b = c1.S().v[s][i];
            dst.S().v[s][i] = a > (T)0 ? a : (T)(a * b);
        }
}
// dst = src > 0 ? src : src * k  (ElementOp.h:503-508)
template <typename DstT, typename SrcT>
PTO_DEV void TLRELU_IMPL(DstT &dst, SrcT &src, typename DstT::DType k)
{
    using T = typename DstT::DType;
    using S = typename DstT::Storage;
    detail::Conformed<DstT, SrcT> c0(src);
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i) {
            const T a = c0.S().v[s][i];
            dst.S().v[s][i] = a > (T)0 ? a : (T)(a * k);
        }
}

// ------------------------------------------------------------ compare / select
namespace detail {
template <typename T>
PTO_DEV bool cmp_exact(T a, T b, CmpMode mode)
{
    switch (mode) {
    case CmpMode::EQ: return a == b;
    case CmpMode::NE: return a != b;
    case CmpMode::LT: return a < b;
    case CmpMode::LE: return a <= b;
    case CmpMode::GT: return a > b;
    case CmpMode::GE: return a >= b;
    }
    return a == b;
}
// TCMPS compares with a tolerance for EQ / NE: |a - b| < 1e-9 in double (TCmps.hpp:28-37)
template <typename T>
PTO_DEV bool cmp_scalar(T a, T b, CmpMode mode)
{
    const double diff = (double)a - (double)b;
    const double ad = diff < 0 ? -diff : diff;
    switch (mode) {
    case CmpMode::EQ: return ad < 1e-9;
    case CmpMode::NE: return ad > 1e-9;
    case CmpMode::LT: return a < b;
    case CmpMode::GT: return a > b;
    case CmpMode::GE: return a >= b;
    case CmpMode::LE: return a <= b;
    }
    return ad < 1e-9;
}
} // namespace detail

// dst = (src0 <mode> src1) as 0 / 1 in the tiles' own type (ElementTileOp.h:178-184, ElementOp.h:227-253)
template <typename TileT>
PTO_DEV void TCMP_IMPL(TileT &dst, TileT &src0, TileT &src1, CmpMode mode)
{
    using T = typename TileT::DType;
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = detail::cmp_exact<T>(src0.S().v[s][i], src1.S().v[s][i], mode) ? (T)1 : (T)0;
}

// Packed form: bit (c % 8) of byte c / 8 of row r of dst = (src0[r,c] <mode> scalar); dst is a
// uint8 tile with the source's rows whose first Cols/8 columns receive the bytes (TCmps.hpp:50-90 with
// dst valid columns = Cols / 8, the shape its test uses).  A chunk of 8 elements is one byte.
template <typename DstT, typename SrcT, typename T>
PTO_DEV void TCMPS_IMPL(DstT &dst, SrcT &src0, T scalar, CmpMode mode)
{
    static_assert(sizeof(typename DstT::DType) == 1 && SrcT::isRowMajor && DstT::isRowMajor && SrcT::Cols % 8 == 0 &&
                      DstT::Rows == SrcT::Rows && DstT::Cols >= SrcT::Cols / 8,
                  "[PTO][SA] TCMPS: uint8 destination with the source's rows, source columns a multiple of 8");
    using S = typename SrcT::Storage;
    constexpr int kBytes = SrcT::Rows * (SrcT::Cols / 8);
    __shared__ uint8_t packed[kBytes];
    const int vr = src0.GetValidRow(), vc = src0.GetValidCol();
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        if (q < S::Chunks) {
            const int r = (q * 8) / SrcT::Cols, c0 = (q * 8) % SrcT::Cols;
            uint32_t byte = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (r < vr && c0 + i < vc && detail::cmp_scalar<typename SrcT::DType>(src0.S().v[s][i], (typename SrcT::DType)scalar, mode))
                    byte |= 1u << i;
            packed[q] = (uint8_t)byte;
        }
    }
    hw::lds_barrier();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && c < SrcT::Cols / 8)
            dst.S().v[s][i] = packed[r * (SrcT::Cols / 8) + c];
    });
    hw::lds_barrier();
}

// The NPU's tile-tile compare writes packed bits like TCMPS (npu/a2a3/TCmp.hpp; its test compares 8 elements a byte):
// bit (c % 8) of byte c / 8 of row r of the uint8 destination = (src0[r,c] <mode> src1[r,c]).
template <typename DstT, typename SrcT>
PTO_DEV void TCMP_PACKED_IMPL(DstT &dst, SrcT &src0, SrcT &src1, CmpMode mode)
{
    static_assert(sizeof(typename DstT::DType) == 1 && SrcT::isRowMajor && DstT::isRowMajor && SrcT::Cols % 8 == 0 &&
                      DstT::Rows == SrcT::Rows && DstT::Cols >= SrcT::Cols / 8,
                  "[PTO][SA] TCMP: uint8 destination with the source's rows, source columns a multiple of 8");
    using S = typename SrcT::Storage;
    constexpr int kBytes = SrcT::Rows * (SrcT::Cols / 8);
    __shared__ uint8_t packed[kBytes];
    const int vr = src0.GetValidRow(), vc = src0.GetValidCol();
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        if (q < S::Chunks) {
            const int r = (q * 8) / SrcT::Cols, c0 = (q * 8) % SrcT::Cols;
            uint32_t byte = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (r < vr && c0 + i < vc && detail::cmp_exact<typename SrcT::DType>(src0.S().v[s][i], src1.S().v[s][i], mode))
                    byte |= 1u << i;
            packed[q] = (uint8_t)byte;
        }
    }
    hw::lds_barrier();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && c < SrcT::Cols / 8)
            dst.S().v[s][i] = packed[r * (SrcT::Cols / 8) + c];
    });
    hw::lds_barrier();
}

// dst[i,j] = bit (i,j) ? src0[i,j] : src1[i,j]; row i of the mask tile holds the bits of row i, column j in byte j / 8,
// lowest bit first (npu/a2a3/TSel.hpp:46-57: one compare mask per row, read at the mask tile's row stride; its test
// generator tsel/gen_data.py:31-47).  The CPU simulation (cpu/TSel.hpp:27-47) consumes the bits in running order over
// the valid region instead; the two agree whenever the valid width is a multiple of 8 and the mask's valid width is
// exactly that many bytes, which is every case the simulation is tested on.
template <typename TileT, typename MaskT>
PTO_DEV void TSEL_IMPL(TileT &dst, MaskT &selMask, TileT &src0, TileT &src1)
{
    static_assert(sizeof(typename MaskT::DType) == 1 && TileT::isRowMajor && MaskT::isRowMajor,
                  "[PTO][SA] TSEL: row-major tiles, byte mask");
    __shared__ uint8_t bits[MaskT::Numel];
    detail::for_each_owned<MaskT>([&](int s, int i, int e) {
        if (e < MaskT::Numel)
            bits[e] = (uint8_t)selMask.S().v[s][i];
    });
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        const int r = e / TileT::Cols, c = e % TileT::Cols;
        if (e < TileT::Numel && r < vr && c < vc && r < MaskT::Rows && (c >> 3) < MaskT::Cols) {
            const uint32_t byte = bits[r * MaskT::Cols + (c >> 3)];
            dst.S().v[s][i] = ((byte >> (c & 7)) & 1u) ? src0.S().v[s][i] : src1.S().v[s][i];
        }
    });
    hw::lds_barrier();
}

// dst = selectMode == 1 ? src0 : src1 for the whole tile (TSelS.hpp:20-41)
template <typename TileT>
PTO_DEV void TSELS_IMPL(TileT &dst, TileT &src0, TileT &src1, uint8_t selectMode)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = selectMode == 1 ? src0.S().v[s][i] : src1.S().v[s][i];
}

// dst[i,j] = bit (i,j) of the mask ? src[i,j] : scalar (npu/a2a3/TSels.hpp:19-46 and its generator tsels/gen_data.py:38-45):
// row i of the mask tile, read as bytes whatever its element type, holds the bits of row i, lowest bit first.  This is the
// form the reference's front end has (pto_instr.hpp:1014-1021); the whole-tile form above is what its CPU simulation
// implements.
template <typename DstT, typename MaskT, typename SrcT>
PTO_DEV void TSELS_MASK_IMPL(DstT &dst, MaskT &mask, SrcT &src, typename SrcT::DType scalar)
{
    using T = typename DstT::DType;
    using MT = typename MaskT::DType;
    static_assert(std::is_integral_v<MT> && DstT::isRowMajor && MaskT::isRowMajor && sizeof(T) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TSELS: row-major tiles, a mask tile of integers");
    __shared__ MT bits[MaskT::Numel];
    detail::for_each_owned<MaskT>([&](int s, int i, int e) {
        if (e < MaskT::Numel)
            bits[e] = mask.S().v[s][i];
    });
    hw::lds_barrier();
    detail::Conformed<DstT, SrcT> x(src);
    constexpr int kRowBytes = MaskT::Cols * (int)sizeof(MT);
    const uint8_t *bytes = reinterpret_cast<const uint8_t *>(bits);
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < vc && r < MaskT::Rows && (c >> 3) < kRowBytes) {
            const uint32_t byte = bytes[r * kRowBytes + (c >> 3)];
            dst.S().v[s][i] = ((byte >> (c & 7)) & 1u) ? (T)x.S().v[s][i] : (T)scalar;
        }
    });
    hw::lds_barrier();
}

// ------------------------------------------------------------------ TFILLPAD
// dst = src inside the source's valid region, the destination's pad value elsewhere, over the whole
// tile (TFillPad.hpp:22-49; Max / Min pad = +/- infinity for floating types).
template <typename DstT, typename SrcT>
PTO_DEV void TFILLPAD_IMPL(DstT &dst, SrcT &src)
{
    static_assert(DstT::Rows == SrcT::Rows && DstT::Cols == SrcT::Cols && sizeof(typename DstT::DType) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TFILLPAD: same shape and element size");
    if constexpr (DstT::Loc == TileType::Mat) {
        detail::tfillpad_mat(dst, src); // an L1 tile cleared outside a ragged load (pad value Null: zero)
    } else {
        static_assert(DstT::PadVal != PadValue::Null, "[PTO][SA] TFILLPAD: the destination tile needs a pad value");
        using T = typename DstT::DType;
        const T pad = detail::pad_value<T>(DstT::PadVal);
        const int vr = src.GetValidRow(), vc = src.GetValidCol();
        detail::for_each_owned<DstT>([&](int s, int i, int e) {
            int r, c;
            detail::elem_rc<DstT>(e, r, c);
            if (e < DstT::Numel)
                dst.S().v[s][i] = (r < vr && c < vc) ? __builtin_bit_cast(T, src.S().v[s][i]) : pad;
        });
    }
}

// TFILLPAD_INPLACE: source and destination are the same buffer on the NPU; here the destination keeps the source's
// elements inside the source's valid region like TFILLPAD (npu/a2a3/TFillPad.hpp:264-271).
template <typename DstT, typename SrcT>
PTO_DEV void TFILLPAD_INPLACE_IMPL(DstT &dst, SrcT &src)
{
    TFILLPAD_IMPL(dst, src);
}
// TFILLPAD_EXPAND: the destination has at least the source's rows and columns (npu/a2a3/TFillPad.hpp:273-280)
template <typename DstT, typename SrcT>
PTO_DEV void TFILLPAD_EXPAND_IMPL(DstT &dst, SrcT &src)
{
    static_assert(DstT::Rows >= SrcT::Rows && DstT::Cols >= SrcT::Cols && sizeof(typename DstT::DType) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TFILLPAD_EXPAND: the destination is at least as large as the source, one element size");
    static_assert(DstT::PadVal != PadValue::Null, "[PTO][SA] TFILLPAD: the destination tile needs a pad value");
    using T = typename DstT::DType;
    const T pad = detail::pad_value<T>(DstT::PadVal);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    detail::Conformed<DstT, SrcT> c(src);
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        int r, col;
        detail::elem_rc<DstT>(e, r, col);
        if (e < DstT::Numel)
            dst.S().v[s][i] = (r < vr && col < vc) ? __builtin_bit_cast(T, c.S().v[s][i]) : pad;
    });
}

// TPACK: every element cut to the low bits that fit the narrower destination type: 32 -> 16, 32 -> 8, 16 -> 8 bits
// (npu/a5/TPack.hpp:21-72: a store that keeps the low half / quarter of every register element)
template <typename DstT, typename SrcT>
PTO_DEV void TPACK_IMPL(DstT &dst, SrcT &src)
{
    using T = typename DstT::DType;
    using U = typename SrcT::DType;
    static_assert(sizeof(U) > sizeof(T) && (sizeof(U) == 4 || sizeof(U) == 2) && (sizeof(T) == 2 || sizeof(T) == 1),
                  "[PTO][SA] TPACK: 32 -> 16, 32 -> 8 or 16 -> 8 bits");
    using UB = std::conditional_t<sizeof(U) == 4, uint32_t, uint16_t>;
    using TB = std::conditional_t<sizeof(T) == 2, uint16_t, uint8_t>;
    using S = typename DstT::Storage;
    detail::Conformed<DstT, SrcT> c(src);
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = __builtin_bit_cast(T, (TB)__builtin_bit_cast(UB, (U)c.S().v[s][i]));
}

// TQUANT (the a2a3 form, npu/a2a3/TQuant.hpp:26-52): src = src * scale[row] (+ offset[row]), in place as there, then
// rounded to the nearest integer (ties to even) and saturated to int8 (symmetric) or uint8 (asymmetric)
// (the a2a3 tree's enumerators keep their values, which appear in the names of its launchers' instantiations; the a5 tree
// puts MXFP8 first: npu/a5/TQuant.hpp:22-27, npu/a2a3/TQuant.hpp)
enum class QuantType { INT8_SYM, INT8_ASYM, MXFP8 };
enum class VecStoreMode { ND, NZ };                  // npu/a5/TQuant.hpp:29-33
template <QuantType quant, typename DstT, typename SrcT, typename ParaT>
PTO_DEV void TQUANT_IMPL(DstT &dst, SrcT &src, ParaT &scale, ParaT *offset = nullptr)
{
    using U = typename DstT::DType;
    static_assert(std::is_same_v<typename SrcT::DType, float>, "[PTO][SA] TQUANT: fp32 source");
    static_assert(quant == QuantType::INT8_SYM ? std::is_same_v<U, int8_t> : std::is_same_v<U, uint8_t>,
                  "[PTO][SA] TQUANT: int8 (symmetric) or uint8 (asymmetric) destination");
    TROWEXPANDMUL_IMPL(src, src, scale);
    if constexpr (quant == QuantType::INT8_ASYM)
        TROWEXPANDADD_IMPL(src, src, *offset);
    using S = typename DstT::Storage;
    detail::Conformed<DstT, SrcT> c(src);
    constexpr float lo = quant == QuantType::INT8_SYM ? -128.0f : 0.0f, hi = quant == QuantType::INT8_SYM ? 127.0f : 255.0f;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i) {
            const float t = __builtin_rintf(c.S().v[s][i]);
            dst.S().v[s][i] = (U)(int)(t < lo ? lo : t > hi ? hi : t); // a NaN compares false twice and converts to 0
        }
}

// TQUANT<QuantType::MXFP8>(dst, src, &exp, &max, &scaling), the block-scaled form (npu/a5/TQuant.hpp:262-322, ND store
// mode): every 32 consecutive elements of the fp32 source tile (row-major, Cols a multiple of 32) share one e8m0 exponent.
//   max[g]     = largest |x| of group g                                   (TQuant.hpp:35-126)
//   exp[g]     = E - 8, E the biased fp32 exponent of max[g]              (:147-151; 8 = exponent of e4m3's top binade)
//   scaling[g] = 2^(127 - exp[g]) = the float with bits (254 - exp[g]) << 23   (:153-155)
//   dst        = e4m3(clip(src * scaling[group], +-448)), round to nearest even (:182-203; the generator of the
//                reference's test clips and casts: tests/npu/a5/src/st/testcase/tquant/gen_data.py:27-33)
// Elements outside the source's valid region count as zeros.  A group with an infinity or NaN gets exp 0xff (:158-160) and
// NaN -> NaN, +-inf -> +-448, finite -> +-0; a group whose maximum is below 2^-119 gets exp 0 (:163-165 store that byte)
// and the factor 2^127 that this byte stands for (the reference multiplies by its clamp constant 0x7f800000 there).
// exp, max and scaling are linear arrays of one entry per group in their tiles' element order.  The NZ store mode (fp8 in
// the fractal layout, exponents reordered through an index tile) is not built.
namespace detail {
PTO_DEV uint8_t f32_to_e4m3_bits_sat(float y) // |y| <= 448, not NaN: the hardware conversion rounds to nearest even
{
    return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, 0.0f, 0, false) & 0xff);
}
} // namespace detail
template <QuantType quant, typename DstT, typename SrcT, typename ExpT, typename MaxT>
PTO_DEV void TQUANT_IMPL(DstT &dst, SrcT &src, ExpT *exp, MaxT *max, SrcT *scaling)
{
    static_assert(quant == QuantType::MXFP8, "[PTO][SA] TQUANT with exponent, maximum and scaling tiles is the MXFP8 form");
    static_assert(std::is_same_v<typename SrcT::DType, float> && SrcT::isRowMajor && SrcT::Cols % 32 == 0,
                  "[PTO][SA] TQUANT MXFP8: fp32 row-major source whose row length is a multiple of 32");
    static_assert(sizeof(typename DstT::DType) == 1 && DstT::Rows == SrcT::Rows && DstT::Cols == SrcT::Cols && DstT::isRowMajor,
                  "[PTO][SA] TQUANT MXFP8: one byte per element, the source's shape");
    static_assert(sizeof(typename ExpT::DType) == 1 && std::is_same_v<typename MaxT::DType, float>,
                  "[PTO][SA] TQUANT MXFP8: e8m0 bytes and fp32 maxima");
    constexpr int G = SrcT::Numel / 32;
    static_assert(ExpT::Numel >= G && MaxT::Numel >= G && G <= 8192, "[PTO][SA] TQUANT MXFP8: one entry per group of 32");
    __shared__ uint32_t groupMax[G]; // |x| as integers: a NaN is above every number
    for (int g = hw::tid(); g < G; g += kBlockThreads)
        groupMax[g] = 0;
    hw::lds_barrier();
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    detail::for_each_owned<SrcT>([&](int s, int i, int e) {
        int r, c;
        detail::elem_rc<SrcT>(e, r, c);
        if (e < SrcT::Numel && r < vr && c < vc) {
            const uint32_t a = __builtin_bit_cast(uint32_t, src.S().v[s][i]) & 0x7fffffffu;
            if (a != 0)
                atomicMax(&groupMax[e / 32], a);
        }
    });
    hw::lds_barrier();
    auto expOf = [](uint32_t a) { return (a >> 23) == 255u ? 0xffu : (a >> 23) < 8u ? 0u : (a >> 23) - 8u; };
    auto scaleOf = [&](uint32_t a) { return __builtin_bit_cast(float, (a >> 23) == 255u ? 0xffu : (254u - expOf(a)) << 23); };
    using U = typename DstT::DType;
    detail::for_each_owned<SrcT>([&](int s, int i, int e) {
        if (e >= SrcT::Numel)
            return;
        int r, c;
        detail::elem_rc<SrcT>(e, r, c);
        const float x = (r < vr && c < vc) ? src.S().v[s][i] : 0.0f;
        const uint32_t a = groupMax[e / 32], u = __builtin_bit_cast(uint32_t, x), mag = u & 0x7fffffffu;
        uint8_t code;
        if ((a >> 23) == 255u)
            code = (uint8_t)(((u >> 24) & 0x80u) | (mag > 0x7f800000u ? 0x7fu : mag == 0x7f800000u ? 0x7eu : 0u));
        else
            code = detail::f32_to_e4m3_bits_sat(__builtin_fminf(__builtin_fmaxf(x * scaleOf(a), -448.0f), 448.0f));
        dst.S().v[s][i] = __builtin_bit_cast(U, code);
    });
    using EU = typename ExpT::DType;
    detail::for_each_owned<ExpT>([&](int s, int i, int e) {
        if (e < G)
            exp->S().v[s][i] = __builtin_bit_cast(EU, (uint8_t)expOf(groupMax[e]));
    });
    detail::for_each_owned<MaxT>([&](int s, int i, int e) {
        if (e < G)
            max->S().v[s][i] = __builtin_bit_cast(float, groupMax[e]);
    });
    detail::for_each_owned<SrcT>([&](int s, int i, int e) {
        if (e < G)
            scaling->S().v[s][i] = scaleOf(groupMax[e]);
    });
    hw::lds_barrier();
}

// TDEQUANT: dst = (float(src) - offset[row]) * scale[row] over the destination's valid region, the two steps rounded
// separately; scale and offset are column 0 of their tiles (npu/a2a3/TDequant.hpp:193-202 and the generator of its test,
// tests/npu/a2a3/src/st/testcase/tdequant/gen_data.py:40-46)
template <typename DstT, typename SrcT, typename ParaT>
PTO_DEV void TDEQUANT_IMPL(DstT &dst, SrcT &src, ParaT &scale, ParaT &offset)
{
    using U = typename SrcT::DType;
    static_assert(std::is_same_v<typename DstT::DType, float> && std::is_same_v<typename ParaT::DType, float> &&
                      (std::is_same_v<U, int8_t> || std::is_same_v<U, int16_t>),
                  "[PTO][SA] TDEQUANT: int8 or int16 source, fp32 destination, scale and offset");
    __shared__ float sc[DstT::Rows], of[DstT::Rows];
    detail::stage_row_values<ParaT, DstT::Rows>(scale, sc);
    detail::stage_row_values<ParaT, DstT::Rows>(offset, of);
    hw::lds_barrier();
    detail::Conformed<DstT, SrcT> c(src);
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        int r, col;
        detail::elem_rc<DstT>(e, r, col);
        if (e < DstT::Numel && r < vr && col < vc)
            dst.S().v[s][i] = ((float)c.S().v[s][i] - of[r]) * sc[r];
    });
    hw::lds_barrier();
}

// ------------------------------------------------------- column reductions
namespace detail {
enum class Red { Max, Min, Sum, Prod };
// One value per column into a [1, Cols] tile.  A lane owns the same 8 columns in every slot (the
// number of chunks per row divides the workgroup size); its rows are g, g + G, g + 2G, ... for its
// group g of G = threads / chunks-per-row.  Per-lane partials over its rows, then the G partials of a
// column are combined in order of g.  Max / min are exact; the sum adds in this order, the CPU
// simulation in row order (TColSum.hpp:22-30).
template <Red red, typename DstT, typename SrcT>
PTO_DEV void col_reduce(DstT &dst, SrcT &src)
{
    static_assert(SrcT::isRowMajor && SrcT::Cols % kVecChunk == 0 && DstT::Rows == 1 && DstT::Cols == SrcT::Cols,
                  "[PTO][SA] column reduction: row-major source, [1, Cols] destination");
    constexpr int CPR = SrcT::Cols / kVecChunk;
    static_assert(CPR <= kBlockThreads && kBlockThreads % CPR == 0, "[PTO][SA] column reduction: chunks per row must divide the workgroup size");
    constexpr int G = kBlockThreads / CPR;
    using S = typename SrcT::Storage;
    using A = float;
    __shared__ A part[G][SrcT::Cols];
    const int vr = src.GetValidRow();
    const int g = hw::tid() / CPR, c0 = (hw::tid() % CPR) * kVecChunk;
    A acc[kVecChunk];
    bool any = false;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int r = s * G + g;
        if (r < vr && r < SrcT::Rows) {
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i) {
                const A v = (A)src.S().v[s][i];
                if (!any)
                    acc[i] = v;
                else if (red == Red::Max)
                    acc[i] = acc[i] < v ? v : acc[i];
                else if (red == Red::Min)
                    acc[i] = v < acc[i] ? v : acc[i];
                else if (red == Red::Prod)
                    acc[i] *= v;
                else
                    acc[i] += v;
            }
            any = true;
        }
    }
    __shared__ int has[G];
    if (hw::tid() % CPR == 0)
        has[g] = any ? 1 : 0;
    if (any) {
#pragma unroll
        for (int i = 0; i < kVecChunk; ++i)
            part[g][c0 + i] = acc[i];
    }
    hw::lds_barrier();
    const int vc = src.GetValidCol();
    for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < DstT::Numel && e < vc && vr > 0) {
            A a = part[0][e];
            for (int k = 1; k < G; ++k)
                if (has[k]) {
                    const A v = part[k][e];
                    a = red == Red::Max ? (a < v ? v : a) : red == Red::Min ? (v < a ? v : a) : red == Red::Prod ? a * v : a + v;
                }
            dst.S().v[s][i] = (typename DstT::DType)a;
        }
    });
    hw::lds_barrier();
}

enum class ColOp { Copy, Sub, Mul, Div, Add, Max, Min, ExpDif };
// dst[i,j] = src0[i,j] <op> src1[0,j]  (TColExpand.hpp:22-33, TColExpandOp.hpp)
template <ColOp op, typename DstT, typename ColT>
PTO_DEV void col_expand(DstT &dst, DstT &src0, ColT &src1)
{
    // the per-column operand is row 0 of its tile (a [1, Cols] tile, or a taller one of which one row is valid:
    // tests/npu/a2a3/src/st/testcase/tcolexpand/tcolexpand_kernel.cpp:27-30)
    static_assert(DstT::isRowMajor && ColT::isRowMajor && ColT::Cols == DstT::Cols, "[PTO][SA] column broadcast: a row-major source of the destination's width");
    using T = typename DstT::DType;
    __shared__ typename ColT::DType colv[DstT::Cols];
    for_each_owned<ColT>([&](int s, int i, int e) {
        if (e < ColT::Cols)
            colv[e] = src1.S().v[s][i];
    });
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < vc) {
            const T a = src0.S().v[s][i], b = (T)colv[c];
            T o;
            if constexpr (op == ColOp::Copy)
                o = b;
            else if constexpr (op == ColOp::Sub)
                o = a - b;
            else if constexpr (op == ColOp::Mul)
                o = a * b;
            else if constexpr (op == ColOp::Div)
                o = a / b;
            else if constexpr (op == ColOp::Add)
                o = a + b;
            else if constexpr (op == ColOp::Max)
                o = a < b ? b : a;
            else if constexpr (op == ColOp::ExpDif)
                o = (T)::exp((double)(T)(a - b)); // ElementOp.h:265-270, as TROWEXPANDEXPDIF
            else
                o = b < a ? b : a;
            dst.S().v[s][i] = o;
        }
    });
    hw::lds_barrier();
}
} // namespace detail

template <typename DstT, typename SrcT>
PTO_DEV void TCOLMAX_IMPL(DstT &dst, SrcT &src) { detail::col_reduce<detail::Red::Max>(dst, src); } // TColMax.hpp:22-35
template <typename DstT, typename SrcT>
PTO_DEV void TCOLMIN_IMPL(DstT &dst, SrcT &src) { detail::col_reduce<detail::Red::Min>(dst, src); } // TColMin.hpp
template <typename DstT, typename SrcT>
PTO_DEV void TCOLSUM_IMPL(DstT &dst, SrcT &src) { detail::col_reduce<detail::Red::Sum>(dst, src); } // TColSum.hpp:22-31
template <typename DstT, typename SrcT, typename TmpT>
PTO_DEV void TCOLSUM_IMPL(DstT &dst, SrcT &src, TmpT &, bool) { detail::col_reduce<detail::Red::Sum>(dst, src); }
template <typename DstT, typename SrcT>
PTO_DEV void TCOLPROD_IMPL(DstT &dst, SrcT &src) { detail::col_reduce<detail::Red::Prod>(dst, src); } // npu/a2a3/TColProd.hpp

template <typename DstT, typename ColT>
PTO_DEV void TCOLEXPAND_IMPL(DstT &dst, ColT &src) { detail::col_expand<detail::ColOp::Copy>(dst, dst, src); }
#define PTO_DEFINE_COLEXPAND(NAME, OP)                                \
    template <typename DstT, typename ColT>                           \
    PTO_DEV void NAME##_IMPL(DstT &dst, DstT &src0, ColT &src1)       \
    {                                                                 \
        detail::col_expand<detail::ColOp::OP>(dst, src0, src1);       \
    }
PTO_DEFINE_COLEXPAND(TCOLEXPANDSUB, Sub)
PTO_DEFINE_COLEXPAND(TCOLEXPANDMUL, Mul)
PTO_DEFINE_COLEXPAND(TCOLEXPANDDIV, Div)
PTO_DEFINE_COLEXPAND(TCOLEXPANDADD, Add)
PTO_DEFINE_COLEXPAND(TCOLEXPANDMAX, Max)
PTO_DEFINE_COLEXPAND(TCOLEXPANDMIN, Min)
PTO_DEFINE_COLEXPAND(TCOLEXPANDEXPDIF, ExpDif) // TColExpandOp.hpp:75-79
#undef PTO_DEFINE_COLEXPAND

// ------------------------------------------------ more row reductions / broadcasts
// row minimum (TRowMin.hpp:22-58); exact
template <typename DstT, typename SrcT, typename TmpT>
PTO_DEV void TROWMIN_IMPL(DstT &dst, SrcT &src, TmpT &)
{
    detail::row_reduce<2>(dst, src);
}
// product of the valid columns of every row (npu/a2a3/TRowProd.hpp; the reference's generator: prod(axis=1))
template <typename DstT, typename SrcT, typename TmpT>
PTO_DEV void TROWPROD_IMPL(DstT &dst, SrcT &src, TmpT &)
{
    detail::row_reduce<3>(dst, src);
}

// dst[i,j] = src[i]  (TRowExpand.hpp)
template <typename DstT, typename RowT>
PTO_DEV void TROWEXPAND_IMPL(DstT &dst, RowT &src)
{
    static_assert(DstT::isRowMajor, "[PTO][SA] TROWEXPAND: row-major destination");
    __shared__ typename RowT::DType rowv[DstT::Rows];
    detail::stage_row_values<RowT, DstT::Rows>(src, rowv);
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < vc)
            dst.S().v[s][i] = (typename DstT::DType)rowv[r];
    });
    hw::lds_barrier();
}
// LDS staging arrays of the moves that redistribute a tile over the workgroup (Acc -> Vec, Vec / Acc -> Left / Right,
// TTRANS): one array per power-of-two size class, shared by every move of that class in a kernel.
namespace detail {
constexpr int stage_bytes(int n)
{
    int b = 1024;
    while (b < n)
        b *= 2;
    return b;
}
// staging arrays are shared by all moves of a size class
template <int Bytes>
PTO_DEV char *stage_buffer()
{
    __shared__ __attribute__((aligned(16))) char buf[Bytes];
    return buf;
}
// a Vec tile's elements in row-major order, as they lie in a buffer of the reference
template <typename TileT>
PTO_DEV void stage_tile_rows_raw(TileT &t, void *lds)
{
    static_assert(TileT::isRowMajor, "row-major tile");
    using T = typename TileT::DType;
    T *p = static_cast<T *>(lds);
    for_each_owned<TileT>([&](int s, int i, int e) {
        if (e < TileT::Numel)
            p[e] = t.S().v[s][i];
    });
}
} // namespace detail

// ------------------------------------------------------- TMOV Acc -> Vec
// Same-shape copy of an accumulator tile into a Vec tile, optionally clamped at zero
// (TMov.hpp:20-69).  The accumulator's per-wave MFMA layout is redistributed through LDS.
template <ReluPreMode relu = ReluPreMode::NoRelu, typename DstT, typename AccT>
PTO_DEV void TMOV_ACC2VEC_IMPL(DstT &dst, AccT &src)
{
    static_assert(AccT::Loc == TileType::Acc && DstT::Loc == TileType::Vec && DstT::isRowMajor && DstT::Rows == AccT::Rows &&
                      DstT::Cols == AccT::Cols && sizeof(typename DstT::DType) == 4 && sizeof(typename AccT::DType) == 4,
                  "[PTO][SA] TMOV Acc->Vec: row-major fp32 Vec tile of the accumulator's shape");
    using S = typename AccT::Storage;
    using T = typename DstT::DType;
    T *stage = reinterpret_cast<T *>(detail::stage_buffer<detail::stage_bytes(AccT::Rows * AccT::Cols * (int)sizeof(T))>());
    const uint32_t lane = (uint32_t)hw::lane();
    const int rbase = hw::wave_m() * (S::MB * detail::kMfmaM) + detail::acc_lane_row(lane);
    const int cbase = hw::wave_n() * (S::NB * detail::kMfmaM) + detail::acc_lane_col(lane);
#pragma unroll
    for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
            for (int v = 0; v < detail::kAccElems; ++v) {
                const int r = rbase + mb * detail::kMfmaM + detail::acc_elem_row(v), c = cbase + nb * detail::kMfmaM;
                stage[r * AccT::Cols + c] = (T)src.S().f[mb][nb][v];
            }
    hw::lds_barrier();
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < vc) {
            T v = stage[e];
            if (relu == ReluPreMode::NormalRelu && v < (T)0)
                v = (T)0;
            dst.S().v[s][i] = v;
        }
    });
    hw::lds_barrier();
}

// ------------------------------------- TMOV Vec / Acc -> Left / Right, TTRANS
// Same-shape moves from a register tile that the whole workgroup holds (Vec) or that the waves hold as MFMA
// results (Acc) into the per-wave operand fragments of TMATMUL, and the transpose of a Vec tile (the reference's
// Auto-mode programs chain matmuls this way: demos/cpu/mla_attention_demo/mla_attention_demo.cpp:300-395; element
// rules cpu/TMov.hpp, cpu/TTrans.hpp).  All of them redistribute through an LDS staging array that holds the
// destination's element type: k-contiguous per row for a Left destination, per column for a Right destination, so
// that a fragment is one 16-byte read.
namespace detail {
// every element (r, c) of a Vec or Acc tile -> stage[index(r, c)]
template <typename T, typename SrcT, typename IndexF>
PTO_DEV void stage_write(SrcT &src, T *stage, IndexF &&index)
{
    if constexpr (SrcT::Loc == TileType::Acc) {
        using S = typename SrcT::Storage;
        const uint32_t lane = (uint32_t)hw::lane();
        const int rbase = hw::wave_m() * (S::MB * kMfmaM) + acc_lane_row(lane);
        const int cbase = hw::wave_n() * (S::NB * kMfmaM) + acc_lane_col(lane);
#pragma unroll
        for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
                for (int v = 0; v < kAccElems; ++v)
                    stage[index(rbase + mb * kMfmaM + acc_elem_row(v), cbase + nb * kMfmaM)] = (T)src.S().f[mb][nb][v];
    } else {
        static_assert(SrcT::Loc == TileType::Vec, "[PTO][SA] TMOV / TTRANS: Vec or Acc source");
        for_each_owned<SrcT>([&](int s, int i, int e) {
            if (e < SrcT::Numel) {
                int r, c;
                elem_rc<SrcT>(e, r, c);
                stage[index(r, c)] = (T)src.S().v[s][i];
            }
        });
    }
}
} // namespace detail

template <typename DstT, typename SrcT>
PTO_DEV void TMOV_TO_OPERAND_IMPL(DstT &dst, SrcT &src)
{
    static_assert((DstT::Loc == TileType::Left || DstT::Loc == TileType::Right) && DstT::Rows == SrcT::Rows && DstT::Cols == SrcT::Cols,
                  "[PTO][SA] TMOV to a matmul operand: Left or Right destination of the source's shape");
    using T = typename DstT::DType;
    static_assert(!detail::is_mx_operand_v<T>, "[PTO][SA] TMOV to a matmul operand: fp16, bf16, int8 or fp32 elements");
    using S = typename DstT::Storage;
    using Frag = typename detail::FragOf<T>::type;
    constexpr bool left = DstT::Loc == TileType::Left;
    constexpr int K = left ? DstT::Cols : DstT::Rows; // extent along k; a row (column) of the operand is K contiguous elements
    constexpr int kChunkElems = 16 / (int)sizeof(T), kStepChunks = kWaveSize / detail::kMfmaM;
    T *stage = reinterpret_cast<T *>(detail::stage_buffer<detail::stage_bytes(DstT::Numel * (int)sizeof(T))>());
    detail::stage_write<T>(src, stage, [&](int r, int c) { return left ? r * K + c : c * K + r; });
    hw::lds_barrier();
    const uint32_t lane = (uint32_t)hw::lane();
    const int major = (int)detail::frag_lane_major(lane), kgroup = (int)detail::frag_lane_kgroup(lane);
    if constexpr (left) {
        const int row0 = hw::wave_m() * (S::MB * detail::kMfmaM) + major;
#pragma unroll
        for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
            for (int ks = 0; ks < S::KS; ++ks)
                dst.S().f[mb][ks] =
                    *reinterpret_cast<const Frag *>(stage + (row0 + mb * detail::kMfmaM) * K + (kgroup + ks * kStepChunks) * kChunkElems);
    } else {
        const int col0 = hw::wave_n() * (S::NB * detail::kMfmaM) + major;
#pragma unroll
        for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
            for (int ks = 0; ks < S::KS; ++ks)
                dst.S().f[nb][ks] =
                    *reinterpret_cast<const Frag *>(stage + (col0 + nb * detail::kMfmaM) * K + (kgroup + ks * kStepChunks) * kChunkElems);
    }
    hw::lds_barrier();
}

// dst[c][r] = src[r][c] (cpu/TTrans.hpp); the scratch tile of the reference's form is not needed
template <typename DstT, typename SrcT>
PTO_DEV void TTRANS_IMPL(DstT &dst, SrcT &src)
{
    // The destination holds the transpose in its top left corner; its own extents may be larger (the NPU's tests round
    // its row length up to 32 bytes: tests/npu/a2a3/src/st/testcase/ttrans/ttrans_kernel.cpp:31-35).  What lies outside
    // the transpose of the source tile is left as it is.
    static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec && DstT::Rows >= SrcT::Cols && DstT::Cols >= SrcT::Rows &&
                      sizeof(typename DstT::DType) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TTRANS: Vec tiles, a destination that holds the transposed shape, same element size");
    using T = typename DstT::DType;
    T *stage = reinterpret_cast<T *>(detail::stage_buffer<detail::stage_bytes(SrcT::Numel * (int)sizeof(T))>());
    detail::stage_write<T>(src, stage, [&](int r, int c) { return c * SrcT::Rows + r; }); // row-major image of the transpose
    hw::lds_barrier();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < DstT::Numel) {
            int r, c;
            detail::elem_rc<DstT>(e, r, c);
            if (r < SrcT::Cols && c < SrcT::Rows)
                dst.S().v[s][i] = stage[r * SrcT::Rows + c];
        }
    });
    hw::lds_barrier();
}

// ------------------------------------------------ bitwise, shift, remainder and three-operand forms
// (cpu/ElementOp.h:145-198, 305-310, 365-378, 425-470; ElementTileOp.h:108-166, 203, 287; ElementTileScalarOp.h:113-):
// integer tiles for the bitwise and shift ops; TREM is `%` on integers and fmod (evaluated in double) on floats, a
// zero divisor is the caller's error as in the reference; TADDC = a + b + c, TSUBC = a - b + c.
namespace detail {
// bitwise instructions on floating-point tiles work on the bit patterns (the NPU's vand / vor take any 16- or 32-bit type:
// the reference's tand test has an fp16 case)
template <typename T>
using BitsOf = std::conditional_t<sizeof(T) == 1, uint8_t, std::conditional_t<sizeof(T) == 2, uint16_t, uint32_t>>;
template <typename T, typename F>
PTO_DEV T bitwise(T a, T b, F f)
{
    if constexpr (std::is_integral_v<T>)
        return (T)f(a, b);
    else
        return __builtin_bit_cast(T, (BitsOf<T>)f(__builtin_bit_cast(BitsOf<T>, a), __builtin_bit_cast(BitsOf<T>, b)));
}
template <typename T>
PTO_DEV T elem_rem(T a, T b)
{
    if constexpr (std::is_integral_v<T>)
        return (T)(a % b);
    else
        return (T)::fmod((double)a, (double)b);
}
// TREM / TREMS exist in two meanings in the reference.  The CPU simulation takes C's % and fmod (cpu/ElementOp.h:145-156):
// the result has the sign of the dividend; that is elem_rem above and the default here, as for every instruction.  The
// NPU computes a - floor(a / b) b in the tile's own floating-point type, integer tiles through a conversion to that type
// and back by rounding (npu/a2a3/TRem.hpp:17-95, TRemS.hpp:17-56, and np.remainder in the generators of its tests): the
// result has the sign of the divisor.  A translation unit that defines PTO_TREM_FLOOR_FORM gets the NPU's meaning.
template <typename T>
PTO_DEV T elem_rem_floor(T a, T b)
{
    if constexpr (std::is_integral_v<T>) {
        using F = std::conditional_t<sizeof(T) == 2, half, float>;
        const F r = elem_rem_floor<F>((F)a, (F)b);
        return (T)__builtin_rintf((float)r);
    } else {
        const T q = (T)(a / b);
        const T f = (T)__builtin_floorf((float)q);
        const T p = (T)(f * b);
        return (T)(a - p);
    }
}
template <typename T>
PTO_DEV T elem_trem(T a, T b)
{
#if defined(PTO_TREM_FLOOR_FORM)
    return elem_rem_floor<T>(a, b);
#else
    return elem_rem<T>(a, b);
#endif
}
} // namespace detail

#define PTO_DEFINE_BINARY_EXT(NAME, INT_ONLY, EXPR)                                                     \
    template <typename DstT, typename S0T, typename S1T>                                                \
    PTO_DEV void NAME##_IMPL(DstT &dst, S0T &src0, S1T &src1)                                           \
    {                                                                                                   \
        using T = typename DstT::DType;                                                                 \
        static_assert(!(INT_ONLY) || std::is_integral_v<T>, "[PTO][SA] " #NAME ": integer tiles");      \
        using S = typename DstT::Storage;                                                               \
        detail::Conformed<DstT, S0T> c0(src0);                                                          \
        detail::Conformed<DstT, S1T> c1(src1);                                                          \
        _Pragma("unroll") for (int s = 0; s < S::Slots; ++s) _Pragma("unroll") for (int i = 0; i < detail::kVecChunk; ++i) \
        {                                                                                               \
            const T a = c0.S().v[s][i], b = c1.S().v[s][i];                                               \
            dst.S().v[s][i] = (T)(EXPR);                                                                 \
        }                                                                                               \
    }
PTO_DEFINE_BINARY_EXT(TAND, false, detail::bitwise(a, b, [](auto x, auto y) { return x & y; }))
PTO_DEFINE_BINARY_EXT(TOR, false, detail::bitwise(a, b, [](auto x, auto y) { return x | y; }))
PTO_DEFINE_BINARY_EXT(TXOR, false, detail::bitwise(a, b, [](auto x, auto y) { return x ^ y; }))
PTO_DEFINE_BINARY_EXT(TSHL, true, a << b)
PTO_DEFINE_BINARY_EXT(TSHR, true, a >> b)
PTO_DEFINE_BINARY_EXT(TREM, false, detail::elem_trem<T>(a, b))
PTO_DEFINE_BINARY_EXT(TFMOD, false, detail::elem_rem<T>(a, b)) // C fmod / integer %: the sign of the dividend (tfmod/gen_data.py:32)
#undef PTO_DEFINE_BINARY_EXT

#define PTO_DEFINE_SCALAR_EXT(NAME, INT_ONLY, EXPR)                                                     \
    template <typename DstT, typename SrcT>                                                             \
    PTO_DEV void NAME##_IMPL(DstT &dst, SrcT &src, typename DstT::DType k)                              \
    {                                                                                                   \
        using T = typename DstT::DType;                                                                 \
        static_assert(!(INT_ONLY) || std::is_integral_v<T>, "[PTO][SA] " #NAME ": integer tiles");      \
        using S = typename DstT::Storage;                                                               \
        detail::Conformed<DstT, SrcT> c0(src);                                                          \
        _Pragma("unroll") for (int s = 0; s < S::Slots; ++s) _Pragma("unroll") for (int i = 0; i < detail::kVecChunk; ++i) \
        {                                                                                               \
            const T a = c0.S().v[s][i];                                                                  \
            dst.S().v[s][i] = (T)(EXPR);                                                                 \
        }                                                                                               \
    }
PTO_DEFINE_SCALAR_EXT(TANDS, false, detail::bitwise(a, (T)k, [](auto x, auto y) { return x & y; }))
PTO_DEFINE_SCALAR_EXT(TORS, false, detail::bitwise(a, (T)k, [](auto x, auto y) { return x | y; }))
PTO_DEFINE_SCALAR_EXT(TXORS, false, detail::bitwise(a, (T)k, [](auto x, auto y) { return x ^ y; }))
PTO_DEFINE_SCALAR_EXT(TSHLS, true, a << k)
PTO_DEFINE_SCALAR_EXT(TSHRS, true, a >> k)
PTO_DEFINE_SCALAR_EXT(TREMS, false, detail::elem_trem<T>(a, k))
PTO_DEFINE_SCALAR_EXT(TFMODS, false, detail::elem_rem<T>(a, k))
#undef PTO_DEFINE_SCALAR_EXT

template <typename DstT, typename SrcT>
PTO_DEV void TNOT_IMPL(DstT &dst, SrcT &src)
{
    static_assert(detail::same_dist<DstT, SrcT> && std::is_integral_v<typename DstT::DType>, "[PTO][SA] TNOT: integer Vec tiles of equal size");
    using S = typename DstT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = (typename DstT::DType)~src.S().v[s][i];
}

// dst = src0 +/- src1 + src2; the scalar forms take the scalar as the second operand
template <bool kSub, typename TileT>
PTO_DEV void vec_addc(TileT &dst, TileT &src0, TileT &src1, TileT &src2)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i) {
            const auto a = src0.S().v[s][i], b = src1.S().v[s][i], c = src2.S().v[s][i];
            dst.S().v[s][i] = kSub ? a - b + c : a + b + c;
        }
}
template <typename TileT>
PTO_DEV void TADDC_IMPL(TileT &dst, TileT &src0, TileT &src1, TileT &src2) { vec_addc<false>(dst, src0, src1, src2); }
template <typename TileT>
PTO_DEV void TSUBC_IMPL(TileT &dst, TileT &src0, TileT &src1, TileT &src2) { vec_addc<true>(dst, src0, src1, src2); }
template <bool kSub, typename TileT>
PTO_DEV void vec_addsc(TileT &dst, TileT &src0, typename TileT::DType k, TileT &src1)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i) {
            const auto a = src0.S().v[s][i], c = src1.S().v[s][i];
            dst.S().v[s][i] = kSub ? a - k + c : a + k + c;
        }
}
template <typename TileT>
PTO_DEV void TADDSC_IMPL(TileT &dst, TileT &src0, typename TileT::DType k, TileT &src1) { vec_addsc<false>(dst, src0, k, src1); }
template <typename TileT>
PTO_DEV void TSUBSC_IMPL(TileT &dst, TileT &src0, typename TileT::DType k, TileT &src1) { vec_addsc<true>(dst, src0, k, src1); }

// ------------------------------------------------------ TPARTADD / TPARTMAX / TPARTMIN
// Elementwise over the destination's valid region where the sources' valid regions may be smaller (cpu/TPartOp.hpp:19-45):
// both sources valid -> op(src0, src1); one valid -> that source's element; none -> 0.
namespace detail {
template <int KIND, typename DstT, typename S0T, typename S1T> // KIND: 0 add, 1 max, 2 min, 3 mul
PTO_DEV void part_op(DstT &dst, S0T &src0, S1T &src1)
{
    using T = typename DstT::DType;
    // sources of another static shape than the destination (the NPU's tests give each operand the tile of its own valid
    // region: tests/npu/a2a3/src/st/testcase/tpartadd/tpartadd_kernel.cpp:26-28) are paired with it by (row, column)
    static_assert(DstT::Loc == TileType::Vec && S0T::Loc == TileType::Vec && S1T::Loc == TileType::Vec, "[PTO][SA] TPART*: Vec tiles");
    static_assert(std::is_same_v<typename S0T::DType, T> && std::is_same_v<typename S1T::DType, T>, "[PTO][SA] TPART*: one element type");
    const int dvr = dst.GetValidRow(), dvc = dst.GetValidCol(), avr = src0.GetValidRow(), avc = src0.GetValidCol(),
              bvr = src1.GetValidRow(), bvc = src1.GetValidCol();
    Conformed<DstT, S0T> x0(src0);
    Conformed<DstT, S1T> x1(src1);
    for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < DstT::Numel) {
            int r, c;
            elem_rc<DstT>(e, r, c);
            if (r < dvr && c < dvc) {
                const bool in0 = r < avr && c < avc, in1 = r < bvr && c < bvc;
                const T a = x0.S().v[s][i], b = x1.S().v[s][i];
                const T both = KIND == 0 ? (T)(a + b) : KIND == 1 ? (a < b ? b : a) : KIND == 2 ? (b < a ? b : a) : (T)(a * b);
                dst.S().v[s][i] = in0 && in1 ? both : in0 ? a : in1 ? b : (T)0;
            }
        }
    });
}
} // namespace detail
template <typename DstT, typename S0T, typename S1T>
PTO_DEV void TPARTADD_IMPL(DstT &dst, S0T &src0, S1T &src1) { detail::part_op<0>(dst, src0, src1); }
template <typename DstT, typename S0T, typename S1T>
PTO_DEV void TPARTMAX_IMPL(DstT &dst, S0T &src0, S1T &src1) { detail::part_op<1>(dst, src0, src1); }
template <typename DstT, typename S0T, typename S1T>
PTO_DEV void TPARTMIN_IMPL(DstT &dst, S0T &src0, S1T &src1) { detail::part_op<2>(dst, src0, src1); }
template <typename DstT, typename S0T, typename S1T>
PTO_DEV void TPARTMUL_IMPL(DstT &dst, S0T &src0, S1T &src1) { detail::part_op<3>(dst, src0, src1); }

// ------------------------------------------------------------ TCI, TSCATTER, MSCATTER
// TCI (cpu/TCI.hpp:16-35): dst[0, j] = start + j (descending: start - j) over the valid columns of a one-row tile.
template <typename TileT, typename T, int descending>
PTO_DEV void TCI_IMPL(TileT &dst, T start)
{
    static_assert(TileT::Loc == TileType::Vec && TileT::Rows == 1 && std::is_same_v<typename TileT::DType, T>,
                  "[PTO][SA] TCI: one-row Vec tile of the start value's type");
    const int vc = dst.GetValidCol();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        if (e < vc)
            dst.S().v[s][i] = descending == 1 ? (T)(start - (T)e) : (T)(start + (T)e);
    });
}

// TSCATTER (cpu/TScatter.hpp:21-44): dst[indexes[i, j], j] = src[i, j] over the source's valid region.  The reference
// walks the rows in order, so where several rows send an element to the same place the last one wins: the winner is
// found with an atomic maximum over the source row numbers in LDS.  Rows outside the tile are dropped (the reference
// writes out of bounds there).
template <typename TileT, typename IdxT>
PTO_DEV void TSCATTER_IMPL(TileT &dst, TileT &src, IdxT &indexes)
{
    using T = typename TileT::DType;
    static_assert(TileT::Loc == TileType::Vec && IdxT::Loc == TileType::Vec && TileT::isRowMajor && IdxT::isRowMajor &&
                      std::is_integral_v<typename IdxT::DType> && IdxT::Rows == TileT::Rows && IdxT::Cols == TileT::Cols,
                  "[PTO][SA] TSCATTER: row-major Vec tiles, integer index tile of the same shape");
    constexpr int N = TileT::Numel;
    int *owner = reinterpret_cast<int *>(detail::stage_buffer<detail::stage_bytes((4 + (int)sizeof(T)) * N)>());
    T *value = reinterpret_cast<T *>(owner + N);
    for (int e = hw::tid(); e < N; e += kBlockThreads)
        owner[e] = -1;
    hw::lds_barrier();
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        const int r = e / TileT::Cols, c = e % TileT::Cols;
        const uint32_t row = (uint32_t)indexes.S().v[s][i];
        if (e < N && r < vr && c < vc && row < (uint32_t)TileT::Rows)
            atomicMax(&owner[row * TileT::Cols + c], r);
    });
    hw::lds_barrier();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        const int r = e / TileT::Cols, c = e % TileT::Cols;
        const uint32_t row = (uint32_t)indexes.S().v[s][i];
        if (e < N && r < vr && c < vc && row < (uint32_t)TileT::Rows && owner[row * TileT::Cols + c] == r)
            value[row * TileT::Cols + c] = src.S().v[s][i];
    });
    hw::lds_barrier();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        if (e < N && owner[e] >= 0)
            dst.S().v[s][i] = value[e];
    });
    hw::lds_barrier();
}

// TSCATTER as the NPU implementation defines it (npu/a2a3/TScatter.hpp:17-36): the index tile holds element numbers of the
// destination's storage, dst[indexes[i, j]] = src[i, j] over the index tile's valid region, walked in row-major order (the
// last writer of an element wins: found with an atomic maximum over i * cols + j).  The index tile may have another shape
// than the source.  Translation units choose this form with PTO_TSCATTER_FLAT_INDEX; the default is the CPU simulation's
// row-index form above.
template <typename DstT, typename SrcT, typename IdxT>
PTO_DEV void TSCATTER_FLAT_IMPL(DstT &dst, SrcT &src, IdxT &indexes)
{
    using T = typename DstT::DType;
    static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec && IdxT::Loc == TileType::Vec && DstT::isRowMajor && SrcT::isRowMajor &&
                      IdxT::isRowMajor && std::is_same_v<T, typename SrcT::DType> && std::is_integral_v<typename IdxT::DType>,
                  "[PTO][SA] TSCATTER: row-major Vec tiles, destination and source of one type, integer indices");
    constexpr int N = DstT::Numel;
    int *owner = reinterpret_cast<int *>(detail::stage_buffer<detail::stage_bytes((4 + (int)sizeof(T)) * N)>());
    T *value = reinterpret_cast<T *>(owner + N);
    for (int e = hw::tid(); e < N; e += kBlockThreads)
        owner[e] = -1;
    detail::Conformed<IdxT, SrcT> c(src); // src (i, j) in the lane that holds index (i, j)
    hw::lds_barrier();
    const int vr = indexes.GetValidRow(), vc = indexes.GetValidCol();
    detail::for_each_owned<IdxT>([&](int s, int i, int e) {
        const int r = e / IdxT::Cols, col = e % IdxT::Cols;
        const uint32_t to = (uint32_t)(int)indexes.S().v[s][i];
        if (e < IdxT::Numel && r < vr && col < vc && to < (uint32_t)N)
            atomicMax(&owner[to], e);
    });
    hw::lds_barrier();
    detail::for_each_owned<IdxT>([&](int s, int i, int e) {
        const int r = e / IdxT::Cols, col = e % IdxT::Cols;
        const uint32_t to = (uint32_t)(int)indexes.S().v[s][i];
        if (e < IdxT::Numel && r < vr && col < vc && to < (uint32_t)N && owner[to] == e)
            value[to] = c.S().v[s][i];
    });
    hw::lds_barrier();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < N && owner[e] >= 0)
            dst.S().v[s][i] = value[e];
    });
    hw::lds_barrier();
}

// MSCATTER (cpu/MGatherScatter.hpp:46-69): memory[indexes[i, j]] = src[i, j] over the source's valid region, the dual of
// MGATHER.  Elements sent to the same address: the reference keeps the last in row-major order, here one of them
// arrives last - callers that need the reference's result pass distinct indices.
template <typename G, typename SrcT, typename IdxT>
PTO_DEV void MSCATTER_IMPL(G &dst, SrcT &src, IdxT &indexes)
{
    static_assert(sizeof(typename SrcT::DType) == sizeof(typename G::DType), "[PTO][SA] MSCATTER: element sizes differ");
    static_assert(SrcT::Numel == IdxT::Numel && SrcT::isRowMajor == IdxT::isRowMajor && std::is_integral_v<typename IdxT::DType>,
                  "[PTO][SA] MSCATTER: source and integer index tiles of the same shape");
    using T = typename SrcT::DType;
    T *gm = reinterpret_cast<T *>(dst.data());
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    detail::for_each_owned<SrcT>([&](int s, int i, int e) {
        int r, c;
        detail::elem_rc<SrcT>(e, r, c);
        if (e < SrcT::Numel && r < vr && c < vc)
            gm[(size_t)indexes.S().v[s][i]] = src.S().v[s][i];
    });
}

// ---------------------------------------------------------------------- TGATHERB
// Block gather (cpu/TGatherB.hpp:21-60): for every row r and every 32-byte block c of the destination's valid region,
// dst block (r, c) = the 32 bytes of the source tile's storage that start at byte offset[r, c]; blocks whose source range
// does not lie inside the source tile are left as they are.
template <typename DstT, typename SrcT, typename OffT>
PTO_DEV void TGATHERB_IMPL(DstT &dst, SrcT &src, OffT &offset)
{
    using T = typename DstT::DType;
    static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec && OffT::Loc == TileType::Vec && DstT::isRowMajor && SrcT::isRowMajor &&
                      OffT::isRowMajor,
                  "[PTO][SA] TGATHERB: row-major Vec tiles");
    static_assert(sizeof(typename SrcT::DType) == sizeof(T) && sizeof(typename OffT::DType) == 4 && OffT::Rows == DstT::Rows,
                  "[PTO][SA] TGATHERB: one element size, 32-bit offsets, one offset row per destination row");
    constexpr int kSrcBytes = SrcT::Numel * (int)sizeof(T), kOffs = OffT::Numel, kPerBlock = 32 / (int)sizeof(T);
    char *bytes = detail::stage_buffer<detail::stage_bytes(kSrcBytes + 4 + 4 * kOffs)>();
    uint32_t *offs = reinterpret_cast<uint32_t *>(bytes + (kSrcBytes + 3) / 4 * 4);
    detail::stage_tile_rows_raw(src, bytes);
    detail::stage_tile_rows_raw(offset, offs);
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols, cb = c / kPerBlock;
        if (e < DstT::Numel && r < vr && (cb + 1) * kPerBlock <= vc && cb < OffT::Cols) {
            const uint32_t off = offs[r * OffT::Cols + cb];
            if (off <= (uint32_t)kSrcBytes - 32u) {
                T v;
                __builtin_memcpy(&v, bytes + off + (uint32_t)(c % kPerBlock) * sizeof(T), sizeof(T)); // any byte alignment
                dst.S().v[s][i] = v;
            }
        }
    });
    hw::lds_barrier();
}

} // namespace pto
#pragma clang fp contract(fast)
