// Vec-tile instructions for gfx950: TCVT, TGATHER (index and mask forms), MGATHER, elementwise
// and row-broadcast arithmetic, row reductions, TTRI, TRESHAPE.
//
// A Vec tile is spread over the workgroup's lanes in chunks of 8 consecutive elements of its
// linear order (common/tile.hpp), so every elementwise instruction between tiles of equal shape
// is lane-local VALU work.  Row reductions combine the chunks of a row with wavefront shuffles where a
// row lies inside one wavefront; the other instructions that move data across lanes (row broadcasts,
// gathers) stage through a small statically allocated LDS buffer sized by the tile.
//
// Reference semantics: include/pto/cpu/TCvt.hpp:65-92, TGather.hpp:58-129, MGatherScatter.hpp:21-44,
// TRowMax.hpp:20-59, TRowSum.hpp:17-63, TRowExpandOp.hpp:37-96, TExp.hpp:22-60, TBinSOps.hpp,
// TAdd/TSub/TMul/TMax.hpp, TTRI.hpp:31-76, TReshape.hpp.
#pragma once
#include "pto/common/global_tensor.hpp"
#include "pto/common/tile.hpp"

// Every tile instruction rounds on its own, as the reference's do: a multiplication in one instruction and an addition in
// the next (TMUL then TADD, the two halves of TQUANT) must not be contracted into one fused multiply-add once both are
// inlined into a kernel.  Contraction is switched off for the instruction bodies of this header and back to hipcc's
// default for device code at its end.
#pragma clang fp contract(off)
namespace pto {
namespace detail {

// ---- conversions -----------------------------------------------------------------------
// fp32 -> fp16, round-to-nearest-even: v_cvt_f16_f32 under the default rounding mode.  NaNs are
// canonicalised in software to sign | 0x7e00 | top 9 payload bits, the result of
// static_cast<_Float16>(float) on the host, so that the conversion is bit-exact everywhere.
PTO_DEV uint16_t f32_to_f16_bits_rne(float x)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const _Float16 h = static_cast<_Float16>(x);
    uint16_t hb = __builtin_bit_cast(uint16_t, h);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        hb = (uint16_t)(((u >> 16) & 0x8000u) | 0x7e00u | ((u >> 13) & 0x1ffu));
    return hb;
}

// fp32 -> fp16 with an explicit rounding rule, in integer arithmetic (RoundMode values 2..6).
PTO_DEV uint16_t f32_to_f16_bits_mode(float x, RoundMode mode)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const uint32_t sign = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u)
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
    if (a == 0x7f800000u)
        return (uint16_t)(sign | 0x7c00u);
    const uint32_t e = a >> 23;
    uint32_t h, rem, half_ulp;
    if (e >= 143u) { // beyond the largest finite half
        const bool toInf = mode == RoundMode::CAST_ROUND || mode == RoundMode::CAST_RINT ||
                           (mode == RoundMode::CAST_CEIL && !sign) || (mode == RoundMode::CAST_FLOOR && sign);
        return (uint16_t)(sign | (toInf ? 0x7c00u : 0x7bffu));
    }
    if (e >= 113u) {
        const uint32_t v = a - (112u << 23);
        h = v >> 13;
        rem = v & 0x1fffu;
        half_ulp = 0x1000u;
    } else if (e >= 102u) {
        const uint32_t m = (a & 0x7fffffu) | 0x800000u, shift = 126u - e;
        h = m >> shift;
        rem = m & ((1u << shift) - 1u);
        half_ulp = 1u << (shift - 1u);
    } else {
        h = 0;
        rem = a ? 1u : 0u; // something below half an ulp of the smallest subnormal
        half_ulp = 2u;
    }
    bool up = false;
    switch (mode) {
    case RoundMode::CAST_ROUND: up = rem >= half_ulp; break;
    case RoundMode::CAST_FLOOR: up = sign && rem; break;
    case RoundMode::CAST_CEIL: up = !sign && rem; break;
    case RoundMode::CAST_TRUNC: up = false; break;
    case RoundMode::CAST_ODD: return (uint16_t)(sign | (h | (rem ? 1u : 0u)));
    default: up = rem > half_ulp || (rem == half_ulp && (h & 1u)); break;
    }
    h += up ? 1u : 0u;
    if (h > 0x7c00u)
        h = 0x7c00u;
    return (uint16_t)(sign | h);
}

// fp32 -> bf16 round-to-nearest-even, integer closed form; NaN -> quiet NaN keeping the top payload bits.
PTO_DEV uint16_t f32_to_bf16_bits_rne(float x)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u) ? ((u >> 16) | 0x0040u) : r);
}

PTO_DEV float round_integral(float v, RoundMode mode)
{ // cpu/TCvt.hpp:28-63
    switch (mode) {
    case RoundMode::CAST_RINT: return __builtin_rintf(v);
    case RoundMode::CAST_ROUND: return __builtin_roundf(v);
    case RoundMode::CAST_FLOOR: return __builtin_floorf(v);
    case RoundMode::CAST_CEIL: return __builtin_ceilf(v);
    case RoundMode::CAST_TRUNC: return __builtin_truncf(v);
    case RoundMode::CAST_ODD: {
        const float f = __builtin_floorf(v), frac = v - f;
        if (frac > 0.5f)
            return f + 1.0f;
        if (frac < 0.5f)
            return f;
        return (((long long)f) & 1) ? f : f + 1.0f;
    }
    default: return v;
    }
}

template <typename D, typename S>
PTO_DEV D convert(S v, RoundMode mode)
{
    if constexpr (std::is_same_v<S, float> && std::is_same_v<D, half>) {
        const uint16_t b = mode == RoundMode::CAST_RINT || mode == RoundMode::CAST_NONE ? f32_to_f16_bits_rne(v) :
                                                                                            f32_to_f16_bits_mode(v, mode);
        return __builtin_bit_cast(half, b);
    } else if constexpr (std::is_same_v<S, float> && std::is_same_v<D, bfloat16_t>) {
        return __builtin_bit_cast(bfloat16_t, f32_to_bf16_bits_rne(v));
    } else if constexpr ((std::is_same_v<S, float> || std::is_same_v<S, half>)&&std::is_integral_v<D>) {
        return static_cast<D>(round_integral(static_cast<float>(v), mode));
    } else {
        return static_cast<D>(v);
    }
}

// linear element index -> (row, col) of a tile
template <typename TileT>
PTO_DEV void elem_rc(int e, int &r, int &c)
{
    if constexpr (TileT::isRowMajor) {
        r = e / TileT::Cols;
        c = e % TileT::Cols;
    } else {
        c = e / TileT::Rows;
        r = e % TileT::Rows;
    }
}
template <typename TileT>
PTO_DEV int elem_index(int r, int c)
{
    return TileT::isRowMajor ? r * TileT::Cols + c : c * TileT::Rows + r;
}

// visit every element this lane owns: fn(slot, i, linear element index)
template <typename TileT, typename F>
PTO_DEV void for_each_owned(F &&fn)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
#pragma unroll
        for (int i = 0; i < kVecChunk; ++i)
            fn(s, i, q * kVecChunk + i);
    }
}

template <typename A, typename B>
constexpr bool same_dist = A::Numel == B::Numel && A::Loc == TileType::Vec && B::Loc == TileType::Vec;

// An elementwise instruction pairs the elements of its operands by (row, column) over the valid region.  Operands with
// the destination's number of elements pair up lane by lane as they are.  A Vec operand of another static shape (the
// reference's per-instruction tests give source and destination tiles different widths, e.g. 32 x 128 and 32 x 112 with
// a 32 x 111 valid region: tests/npu/a2a3/src/st/testcase/tadds) is first brought into the destination's distribution
// through LDS: Conformed<DstT, SrcT>(src).S() then holds src's element (r, c) where dst keeps its (r, c).
template <int Bytes>
PTO_DEV char *conform_buffer()
{
    __shared__ __attribute__((aligned(16))) char buf[Bytes];
    return buf;
}
template <typename DstT, typename SrcT, bool kAsIs = same_dist<DstT, SrcT>>
struct Conformed {
    SrcT &t;
    PTO_DEV explicit Conformed(SrcT &src) : t(src) {}
    PTO_DEV auto &S() { return t.S(); }
};
template <typename DstT, typename SrcT>
struct Conformed<DstT, SrcT, false> {
    using T = typename SrcT::DType;
    using Storage = ::pto::detail::TileStorage<TileType::Vec, T, DstT::Rows, DstT::Cols>;
    Storage st;
    PTO_DEV explicit Conformed(SrcT &src)
    {
        static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec, "[PTO][SA] elementwise instruction: Vec tiles");
        constexpr int kBytes = (int)sizeof(T) * DstT::Numel;
        T *lds = reinterpret_cast<T *>(conform_buffer<(kBytes + 1023) / 1024 * 1024>());
        for_each_owned<SrcT>([&](int s, int i, int e) {
            if (e < SrcT::Numel) {
                int r, c;
                elem_rc<SrcT>(e, r, c);
                if (r < DstT::Rows && c < DstT::Cols)
                    lds[r * DstT::Cols + c] = src.S().v[s][i];
            }
        });
        hw::lds_barrier();
        for_each_owned<DstT>([&](int s, int i, int e) {
            if (e < DstT::Numel) {
                int r, c;
                elem_rc<DstT>(e, r, c);
                st.v[s][i] = (r < SrcT::Rows && c < SrcT::Cols) ? lds[r * DstT::Cols + c] : T{};
            }
        });
        hw::lds_barrier();
    }
    PTO_DEV Storage &S() { return st; }
};

// one value per row (a [R,1] / [1,R] / first-column tile) -> LDS array of R floats, visible to all lanes
template <typename RowT, int R>
PTO_DEV void stage_row_values(RowT &t, typename RowT::DType *lds)
{
    for_each_owned<RowT>([&](int s, int i, int e) {
        if (e < RowT::Numel) {
            int r, c;
            elem_rc<RowT>(e, r, c);
            // the per-row scalar is element (r,0) of a column tile or (0,r) of a row tile (TRowExpandOp.hpp:20-33)
            if (RowT::Cols == 1 || (RowT::Rows != 1 && c == 0)) {
                if (c == 0 && r < R)
                    lds[r] = t.S().v[s][i];
            } else if (RowT::Rows == 1 && c < R) {
                lds[c] = t.S().v[s][i];
            }
        }
    });
}

} // namespace detail

// --------------------------------------------------------------------- TCVT
template <typename DstT, typename SrcT>
PTO_DEV void TCVT_IMPL(DstT &dst, SrcT &src, RoundMode mode)
{
    static_assert(detail::same_dist<DstT, SrcT>, "[PTO][SA] TCVT: Vec tiles with the same number of elements");
    using S = typename SrcT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = detail::convert<typename DstT::DType>(src.S().v[s][i], mode);
}
template <typename DstT, typename SrcT>
PTO_DEV void TCVT_IMPL(DstT &dst, SrcT &src, RoundMode mode, SaturationMode)
{
    TCVT_IMPL(dst, src, mode);
}

// ------------------------------------------------------------- elementwise
#define PTO_DEFINE_BINARY(NAME, EXPR)                                                                   \
    template <typename DstT, typename S0T, typename S1T>                                                \
    PTO_DEV void NAME##_IMPL(DstT &dst, S0T &src0, S1T &src1)                                           \
    {                                                                                                   \
        using T = typename DstT::DType;                                                                 \
        using S = typename DstT::Storage;                                                               \
        detail::Conformed<DstT, S0T> c0(src0);                                                          \
        detail::Conformed<DstT, S1T> c1(src1);                                                          \
        _Pragma("unroll") for (int s = 0; s < S::Slots; ++s) _Pragma("unroll") for (int i = 0; i < detail::kVecChunk; ++i) \
        {                                                                                               \
            const T a = c0.S().v[s][i], b = c1.S().v[s][i];                                               \
            dst.S().v[s][i] = (EXPR);                                                                    \
        }                                                                                               \
    }
PTO_DEFINE_BINARY(TADD, a + b)
PTO_DEFINE_BINARY(TSUB, a - b)
PTO_DEFINE_BINARY(TMUL, a *b)
PTO_DEFINE_BINARY(TDIV, a / b)
PTO_DEFINE_BINARY(TMAX, (a < b ? b : a))
PTO_DEFINE_BINARY(TMIN, (b < a ? b : a))
#undef PTO_DEFINE_BINARY

#define PTO_DEFINE_SCALAR(NAME, EXPR)                                                                   \
    template <typename DstT, typename SrcT>                                                             \
    PTO_DEV void NAME##_IMPL(DstT &dst, SrcT &src, typename DstT::DType k)                              \
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
PTO_DEFINE_SCALAR(TMULS, a *k)
PTO_DEFINE_SCALAR(TADDS, a + k)
PTO_DEFINE_SCALAR(TSUBS, a - k)
PTO_DEFINE_SCALAR(TDIVS, a / k)
PTO_DEFINE_SCALAR(TDIVS_SCALAR_FIRST, k / a)
PTO_DEFINE_SCALAR(TMAXS, (a < k ? k : a))
PTO_DEFINE_SCALAR(TMINS, (k < a ? k : a))
#undef PTO_DEFINE_SCALAR

template <typename TileT>
PTO_DEV void TEXP_IMPL(TileT &dst, TileT &src)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = (typename TileT::DType)::exp((double)src.S().v[s][i]); // evaluated in double: TExp.hpp:36
}

template <typename TileT>
PTO_DEV void TEXPANDS_IMPL(TileT &dst, typename TileT::DType k)
{
    using S = typename TileT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = k;
}

// same storage, new logical shape: both tiles have the same element count and so the same
// lane distribution of their linear order
template <typename DstT, typename SrcT>
PTO_DEV void TRESHAPE_IMPL(DstT &dst, SrcT &src)
{
    // a [R, 1] column-major tile and a [1, R] row-major tile store the same sequence: vectors may change their major order
    constexpr bool vectors = (DstT::Rows == 1 || DstT::Cols == 1) && (SrcT::Rows == 1 || SrcT::Cols == 1) &&
                             (DstT::isRowMajor ? DstT::Rows == 1 : DstT::Cols == 1) && (SrcT::isRowMajor ? SrcT::Rows == 1 : SrcT::Cols == 1);
    static_assert(detail::same_dist<DstT, SrcT> && sizeof(typename DstT::DType) == sizeof(typename SrcT::DType) &&
                      (DstT::isRowMajor == SrcT::isRowMajor || vectors),
                  "[PTO][SA] TRESHAPE: same element count, element size and major order");
    using S = typename SrcT::Storage;
#pragma unroll
    for (int s = 0; s < S::Slots; ++s)
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = __builtin_bit_cast(typename DstT::DType, src.S().v[s][i]);
}

// upper (1) / lower (0) triangular 0/1 mask: TTRI.hpp:31-63
template <typename TileT, int isUpperOrLower>
PTO_DEV void TTRI_IMPL(TileT &dst, int diagonal)
{
    static_assert(TileT::isRowMajor, "[PTO][SA] TTRI: row-major tiles");
    using T = typename TileT::DType;
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<TileT>([&](int s, int i, int e) {
        const int r = e / TileT::Cols, c = e % TileT::Cols;
        if (r < vr && c < vc) {
            const bool one = isUpperOrLower ? (c >= diagonal + r) : (c < diagonal + r + 1);
            dst.S().v[s][i] = one ? (T)1 : (T)0;
        }
    });
}

// --------------------------------------------------------- row reductions
namespace detail {
// KIND: 0 sum, 1 maximum, 2 minimum, 3 product
template <int KIND, typename DstT, typename SrcT>
PTO_DEV void row_reduce(DstT &dst, SrcT &src)
{
    static_assert(SrcT::isRowMajor && SrcT::Loc == TileType::Vec && DstT::Loc == TileType::Vec,
                  "[PTO][SA] row reduction: row-major Vec source");
    static_assert(SrcT::Cols % kVecChunk == 0, "[PTO][SA] row reduction: cols must be a multiple of 8");
    // (the destination may have another row count than the source, e.g. a [8, 1] column for one valid row of a [1, 8]
    // source: tests/npu/a2a3/src/st/testcase/trowprod/trowprod_kernel.cpp:30-31; the valid rows must fit both)
    using A = float;
    using S = typename SrcT::Storage;
    constexpr int CPR = SrcT::Cols / kVecChunk; // chunks per row
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    // A row of at most 64 chunks whose count is a power of two lies in consecutive lanes of one wavefront: the lanes
    // combine their chunks' partial results with a butterfly of wavefront shuffles (every lane of the row ends with the
    // row's result), and one value per row goes through LDS to the lane that holds element (r, 0) of the destination.
    if constexpr (CPR <= kWaveSize && (CPR & (CPR - 1)) == 0) {
        __shared__ A rowval[SrcT::Rows];
        auto op = [](A a, A b) { return KIND == 1 ? (a < b ? b : a) : KIND == 2 ? (b < a ? b : a) : KIND == 3 ? a * b : a + b; };
#pragma unroll
        for (int s = 0; s < S::Slots; ++s) {
            const int q = s * kBlockThreads + hw::tid();
            const int c0 = (q % CPR) * kVecChunk;
            A acc = KIND == 1 ? -__builtin_huge_valf() : KIND == 2 ? __builtin_huge_valf() : KIND == 3 ? 1.0f : 0.0f;
            if (q < S::Chunks) {
#pragma unroll
                for (int i = 0; i < kVecChunk; ++i)
                    if (c0 + i < vc)
                        acc = op(acc, (A)src.S().v[s][i]);
            }
#pragma unroll
            for (int off = CPR / 2; off >= 1; off >>= 1)
                acc = op(acc, __shfl_xor(acc, off, kWaveSize));
            if (q < S::Chunks && q % CPR == 0)
                rowval[q / CPR] = acc;
        }
        hw::lds_barrier();
        for_each_owned<DstT>([&](int s, int i, int e) {
            if (e < DstT::Numel) {
                int r, c;
                elem_rc<DstT>(e, r, c);
                if (c == 0 && r < vr && r < SrcT::Rows)
                    dst.S().v[s][i] = (typename DstT::DType)rowval[r];
            }
        });
        hw::lds_barrier();
        return;
    }
    __shared__ A part[S::Chunks];
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        if (q < S::Chunks) {
            const int c0 = (q % CPR) * kVecChunk;
            A acc = KIND == 1 ? -__builtin_huge_valf() : KIND == 2 ? __builtin_huge_valf() : KIND == 3 ? 1.0f : 0.0f;
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i)
                if (c0 + i < vc) {
                    const A v = (A)src.S().v[s][i];
                    acc = KIND == 1 ? (acc < v ? v : acc) : KIND == 2 ? (v < acc ? v : acc) : KIND == 3 ? acc * v : acc + v;
                }
            part[q] = acc;
        }
    }
    hw::lds_barrier();
    for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < DstT::Numel) {
            int r, c;
            elem_rc<DstT>(e, r, c);
            if (c == 0 && r < vr && r < SrcT::Rows) {
                A acc = part[r * CPR];
                for (int j = 1; j < CPR; ++j) {
                    const A v = part[r * CPR + j];
                    acc = KIND == 1 ? (acc < v ? v : acc) : KIND == 2 ? (v < acc ? v : acc) : KIND == 3 ? acc * v : acc + v;
                }
                dst.S().v[s][i] = (typename DstT::DType)acc;
            }
        }
    });
    hw::lds_barrier();
}

enum class RowOp { Sub, Mul, Div, Add, Max, Min, ExpDif };

// The per-row operand of a row-broadcast instruction: a [R,1] column (or [1,R] row) tile with one value per row, or, on
// the NPU, a row-major [R, 32 / sizeof(T)] tile whose row r is applied to every 32-byte block of row r of the other
// operand: value (r, c % width) (npu/a2a3/TRowExpandSub.hpp:59-77 and its test generator, trowexpandadd/gen_data.py:24-34).
// A destination that is itself 32 bytes wide makes that form the elementwise operation.
template <typename RowT, typename DstT>
inline constexpr int kRowOperandWidth =
    (RowT::isRowMajor && RowT::Rows > 1 && RowT::Cols * (int)sizeof(typename RowT::DType) == 32) ? RowT::Cols : 1;
template <typename T, typename DstT>
inline constexpr bool kIsRowOperand = !(T::Rows == DstT::Rows && T::Cols == DstT::Cols);

// dst = mat (op) row, or row (op) mat when kRowFirst (the instruction computes src0 (op) src1 in argument order; either
// of them may be the per-row operand: TRowExpandSub.hpp:63-77)
template <RowOp op, bool kRowFirst, typename DstT, typename MatT, typename RowT>
PTO_DEV void row_expand(DstT &dst, MatT &mat, RowT &row)
{
    static_assert(DstT::isRowMajor && same_dist<DstT, MatT> && MatT::Cols == DstT::Cols, "[PTO][SA] row broadcast: row-major Vec tiles of one shape");
    using T = typename DstT::DType;
    constexpr int K = kRowOperandWidth<RowT, DstT>;
    __shared__ typename RowT::DType rowv[DstT::Rows * K];
    if constexpr (K == 1) {
        stage_row_values<RowT, DstT::Rows>(row, rowv);
    } else {
        for_each_owned<RowT>([&](int s, int i, int e) {
            if (e < RowT::Numel && e < DstT::Rows * K)
                rowv[e] = row.S().v[s][i];
        });
    }
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < vc) {
            const T m = mat.S().v[s][i], v = (T)rowv[r * K + (K == 1 ? 0 : c % K)];
            const T a = kRowFirst ? v : m, b = kRowFirst ? m : v;
            T o;
            if constexpr (op == RowOp::Sub)
                o = a - b;
            else if constexpr (op == RowOp::Mul)
                o = a * b;
            else if constexpr (op == RowOp::Div)
                o = a / b;
            else if constexpr (op == RowOp::Add)
                o = a + b;
            else if constexpr (op == RowOp::Max)
                o = a < b ? b : a;
            else if constexpr (op == RowOp::Min)
                o = b < a ? b : a;
            else
                o = (T)::exp((double)(T)(a - b)); // exp evaluated in double (cpu/TRowExpandOp.hpp:93-96, ElementOp.h:265-270)
            dst.S().v[s][i] = o;
        }
    });
    hw::lds_barrier();
}
template <RowOp op, typename DstT, typename A, typename B>
PTO_DEV void row_expand_any(DstT &dst, A &src0, B &src1)
{
    // as the reference decides it (npu/a2a3/TRowExpandAdd.hpp:48-66): a first operand of the destination's shape is the
    // matrix, whatever the second looks like (a full-size column-major tile may carry the per-row values in its first
    // column: demos/cpu/mla_attention_demo); only otherwise is the first operand the per-row one
    if constexpr (!kIsRowOperand<A, DstT>)
        row_expand<op, false>(dst, src0, src1);
    else
        row_expand<op, true>(dst, src1, src0);
}
} // namespace detail

template <typename DstT, typename SrcT, typename TmpT>
PTO_DEV void TROWMAX_IMPL(DstT &dst, SrcT &src, TmpT &)
{
    detail::row_reduce<1>(dst, src);
}
template <typename DstT, typename SrcT, typename TmpT>
PTO_DEV void TROWSUM_IMPL(DstT &dst, SrcT &src, TmpT &)
{
    detail::row_reduce<0>(dst, src);
}
#define PTO_DEFINE_ROWEXPAND(NAME, OP)                                \
    template <typename DstT, typename A, typename B>                  \
    PTO_DEV void NAME##_IMPL(DstT &dst, A &src0, B &src1)             \
    {                                                                 \
        detail::row_expand_any<detail::RowOp::OP>(dst, src0, src1);   \
    }
PTO_DEFINE_ROWEXPAND(TROWEXPANDSUB, Sub)
PTO_DEFINE_ROWEXPAND(TROWEXPANDMUL, Mul)
PTO_DEFINE_ROWEXPAND(TROWEXPANDDIV, Div)
PTO_DEFINE_ROWEXPAND(TROWEXPANDADD, Add)
PTO_DEFINE_ROWEXPAND(TROWEXPANDMAX, Max)
PTO_DEFINE_ROWEXPAND(TROWEXPANDMIN, Min)
PTO_DEFINE_ROWEXPAND(TROWEXPANDEXPDIF, ExpDif)
#undef PTO_DEFINE_ROWEXPAND

// ------------------------------------------------------------------ TGATHER
// index form: dst[r,c] = src0.flat[idx[r,c]]; out-of-range or negative indices give 0
// (cpu/TGather.hpp:68-89).  src0 is staged in LDS, then every lane reads its own elements.
template <typename DstT, typename Src0T, typename IdxT>
PTO_DEV void TGATHER_IMPL(DstT &dst, Src0T &src0, IdxT &idx)
{
    using T = typename DstT::DType;
    static_assert(sizeof(T) == 2 || sizeof(T) == 4, "[PTO][SA] TGATHER: 16- or 32-bit elements");
    static_assert(sizeof(typename IdxT::DType) == 4, "[PTO][SA] TGATHER: 32-bit indices");
    static_assert(std::is_same_v<T, typename Src0T::DType>, "[PTO][SA] TGATHER: dst and src0 types differ");
    static_assert(DstT::Numel == IdxT::Numel && DstT::isRowMajor == IdxT::isRowMajor,
                  "[PTO][SA] TGATHER: dst and index tiles must have the same shape");
    static_assert(Src0T::Numel * sizeof(T) <= 128 * 1024, "[PTO][SA] TGATHER: source tile must fit 128 KiB of LDS");
    __shared__ T stage[Src0T::Numel]; // in (row, col) row-major order
    detail::for_each_owned<Src0T>([&](int s, int i, int e) {
        if (e < Src0T::Numel) {
            int r, c;
            detail::elem_rc<Src0T>(e, r, c);
            stage[r * Src0T::Cols + c] = src0.S().v[s][i];
        }
    });
    hw::lds_barrier();
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        int r, c;
        detail::elem_rc<DstT>(e, r, c);
        if (e < DstT::Numel && r < vr && c < vc) {
            const int32_t raw = (int32_t)idx.S().v[s][i];
            const bool ok = raw >= 0 && raw < Src0T::Numel;
            dst.S().v[s][i] = ok ? stage[raw] : (T)0;
        }
    });
    hw::lds_barrier();
}

// mask form: the selected columns of every valid row, packed in row-major running order
// (cpu/TGather.hpp:102-129).  Staged through LDS because the packed position differs from the source's.
template <typename DstT, typename SrcT, MaskPattern pattern>
PTO_DEV void TGATHER_IMPL(DstT &dst, SrcT &src)
{
    using T = typename SrcT::DType;
    static_assert(DstT::isRowMajor && SrcT::isRowMajor, "[PTO][SA] TGATHER(mask): row-major tiles");
    static_assert(sizeof(typename DstT::DType) == sizeof(T), "[PTO][SA] TGATHER(mask): element sizes differ");
    constexpr int p = (int)pattern;
    constexpr int div = p == 7 ? 1 : (p <= 2 ? 2 : 4);
    constexpr int phase = p == 7 ? 0 : (p <= 2 ? p - 1 : p - 3);
    __shared__ T stage[DstT::Numel];
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const int perRow = (vc - phase + div - 1) / div; // selected columns per row
    detail::for_each_owned<SrcT>([&](int s, int i, int e) {
        const int r = e / SrcT::Cols, c = e % SrcT::Cols;
        if (e < SrcT::Numel && r < vr && c < vc && (c % div) == phase) {
            const int pos = r * perRow + c / div;
            if (pos < DstT::Numel)
                stage[pos] = src.S().v[s][i];
        }
    });
    hw::lds_barrier();
    const int total = vr * perRow;
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < DstT::Numel && e < total)
            dst.S().v[s][i] = __builtin_bit_cast(typename DstT::DType, stage[e]);
    });
    hw::lds_barrier();
}

// ------------------------------------------------------------------ MGATHER
// dst[i,j] = gm[idx[i,j]] (cpu/MGatherScatter.hpp:21-44): one global load per element.
template <typename DstT, typename G, typename IdxT>
PTO_DEV void MGATHER_IMPL(DstT &dst, G &src, IdxT &idx)
{
    static_assert(sizeof(typename DstT::DType) == sizeof(typename G::DType), "[PTO][SA] MGATHER: element sizes differ");
    static_assert(DstT::Numel == IdxT::Numel && DstT::isRowMajor == IdxT::isRowMajor,
                  "[PTO][SA] MGATHER: dst and index tiles must have the same shape");
    using T = typename DstT::DType;
    const T *gm = reinterpret_cast<const T *>(src.data());
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        int r, c;
        detail::elem_rc<DstT>(e, r, c);
        if (e < DstT::Numel && r < vr && c < vc)
            dst.S().v[s][i] = gm[(size_t)idx.S().v[s][i]];
    });
}

// Row form of MGATHER: dst[i,:] = table[rowIdx[i], :], i.e. MGATHER with idx[i,j] = rowIdx[i]*Cols + j,
// done with 16-byte loads.  rowIdx is a [Rows,1] int32 tile; rows whose index lies outside
// [0, tableRows) are zero-filled (the out-of-range rule of TGATHER, cpu/TGather.hpp:78-81).
template <typename DstT, typename G, typename IdxT>
PTO_DEV void MGATHER_ROWS_IMPL(DstT &dst, G &table, IdxT &rowIdx, int tableRows)
{
    using T = typename DstT::DType;
    using S = typename DstT::Storage;
    static_assert(DstT::isRowMajor && DstT::Cols % detail::kVecChunk == 0, "[PTO][SA] MGATHER rows: row-major, cols % 8 == 0");
    static_assert(IdxT::Rows == DstT::Rows && sizeof(typename IdxT::DType) == 4, "[PTO][SA] MGATHER rows: [Rows,1] int32 indices");
    __shared__ int32_t rows[DstT::Rows];
    detail::stage_row_values<IdxT, DstT::Rows>(rowIdx, rows);
    hw::lds_barrier();
    const T *gm = reinterpret_cast<const T *>(table.data());
    const int64_t ld = table.GetStride(3);
    typedef T VT __attribute__((ext_vector_type(detail::kVecChunk), aligned(sizeof(T))));
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        const int e0 = q * detail::kVecChunk;
        const int r = e0 / DstT::Cols, c0 = e0 % DstT::Cols;
        VT v = {};
        if (q < S::Chunks && r < vr && c0 + detail::kVecChunk <= vc) {
            const int32_t ri = rows[r];
            if (ri >= 0 && ri < tableRows)
                v = *reinterpret_cast<const VT *>(gm + (int64_t)ri * ld + c0);
        }
#pragma unroll
        for (int i = 0; i < detail::kVecChunk; ++i)
            dst.S().v[s][i] = v[i];
    }
    hw::lds_barrier();
}

} // namespace pto
#pragma clang fp contract(fast)
