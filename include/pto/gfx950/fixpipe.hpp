// The accumulator's way out with a conversion on it (the reference's "fix pipe"): Acc -> Mat (TMOV, TEXTRACT, TINSERT)
// and Acc -> GM (TSTORE), each plain (fp32 -> fp16 / bf16 / fp32, int32 -> int32), with a clamp at zero, with one
// quantisation word for the whole tile (`preQuantScalar`) or with one word per column held in a Scaling tile (the _FP
// forms).  Reference: include/pto/common/pto_instr.hpp:196-236, 625-660, 716-752, 881-915; npu/a2a3/TMov.hpp:88-240,
// TExtract.hpp:457-625, TInsert.hpp:19-100, TStore.hpp.
//
// The quantisation word (the layout the reference's tests build and decode: tests/npu/a2a3/src/st/testcase/
// tmov_acc2mat/gen_data.py:27-100, tmov_acc2mat_kernel.cpp:270-283):
//   bits 31..13  the scale M1: sign, 8 exponent bits, 10 mantissa bits = a float with its low 13 bits dropped
//   bits 35..32  n: int32 -> int16 shifts right by n + 1
//   bits 45..37  offset, added after the scaled value has been rounded and clamped to 9 bits (8-bit results)
//   bit  46      the 8-bit result is signed
//   8-bit result:  clamp(round-half-even(x * M1), -256, 255) + offset, clamped to int8 or uint8
//   fp16 / bf16:   x * M1 converted with round-to-nearest-even (fp16 clamped to +-65504)
//   int16:         clamp(x >> (n + 1), -32768, 32767)
//
// On gfx950 these are ordinary vector instructions on the registers that hold the accumulator; a Mat destination is
// written element by element into its LDS image, a Scaling tile is an offset into a small LDS table of its own (the
// reference's FB buffer), filled by TMOV from a Mat tile.
#pragma once
#include "pto/gfx950/matmul_any.hpp"

#pragma clang fp contract(off) // as in vec_ops.hpp: instructions round on their own
namespace pto {
namespace detail {

constexpr uint32_t kFbBytes = 4096; // 512 quantisation words
PTO_DEV char *fb_base()
{
    __shared__ __attribute__((aligned(16))) char fb[kFbBytes];
    return fb;
}

PTO_DEV float quant_scale(uint64_t q) { return __builtin_bit_cast(float, (uint32_t)q & 0xFFFFE000u); }

template <typename D, typename S>
PTO_DEV D fix_quant(S x, uint64_t q)
{
    if constexpr (std::is_same_v<D, int16_t>) {
        static_assert(std::is_same_v<S, int32_t>, "[PTO][SA] fix pipe: int16 results come from int32 accumulators");
        int32_t t = x >> (int)(((q >> 32) & 0xFu) + 1u);
        t = t < -32768 ? -32768 : t > 32767 ? 32767 : t;
        return (int16_t)t;
    } else {
        const float y = (float)x * quant_scale(q);
        if constexpr (sizeof(D) == 1) {
            float t = __builtin_rintf(y); // round half to even
            t = t < -256.0f ? -256.0f : t > 255.0f ? 255.0f : t;
            int v = (int)t + (int)((q >> 37) & 0x1FFu);
            if ((q >> 46) & 1u)
                v = v < -128 ? -128 : v > 127 ? 127 : v;
            else
                v = v < 0 ? 0 : v > 255 ? 255 : v;
            return (D)v;
        } else if constexpr (std::is_same_v<D, half>) {
            const float c = y < -65504.0f ? -65504.0f : y > 65504.0f ? 65504.0f : y;
            return (half)c;
        } else {
            return store_cast<D>(y);
        }
    }
}

template <ReluPreMode relu, typename D, typename S, typename P>
PTO_DEV D fix_apply(S x, int col, const P &p)
{
    if constexpr (relu == ReluPreMode::NormalRelu)
        x = x < 0 ? 0 : x; // scales are positive: before or after the conversion is the same
    if constexpr (std::is_same_v<P, FixNone>)
        return store_cast<D>(x);
    else if constexpr (std::is_same_v<P, FixScalar>)
        return fix_quant<D>(x, p.q);
    else
        return fix_quant<D>(x, p.table[col]);
}

template <typename D, typename S, typename P>
constexpr void check_fix_types()
{
    static_assert(std::is_same_v<S, float> || std::is_same_v<S, int32_t>, "[PTO][SA] fix pipe: fp32 or int32 accumulator");
    if constexpr (std::is_same_v<P, FixNone>)
        static_assert(std::is_same_v<S, float> ? (std::is_same_v<D, float> || std::is_same_v<D, half> || std::is_same_v<D, bfloat16_t>) :
                                                 std::is_same_v<D, int32_t>,
                      "[PTO][SA] fix pipe without a quantisation word: fp32 -> fp32 / fp16 / bf16, int32 -> int32");
    else
        static_assert(sizeof(D) == 1 || std::is_same_v<D, half> || std::is_same_v<D, bfloat16_t> || (std::is_same_v<D, int16_t> && std::is_same_v<S, int32_t>),
                      "[PTO][SA] fix pipe with a quantisation word: 8-bit, fp16, bf16 results, int16 from int32");
}

// elements [srcRow0, +rows) x [srcCol0, +cols) of the accumulator into the Mat tile at (dstRow0, dstCol0)
template <ReluPreMode relu, typename DstT, typename SrcT, typename P>
PTO_DEV void acc_to_mat(DstT &dst, SrcT &src, int srcRow0, int srcCol0, int dstRow0, int dstCol0, int rows, int cols, const P &p)
{
    static_assert(DstT::Loc == TileType::Mat && SrcT::Loc == TileType::Acc, "[PTO][SA] fix pipe: Acc -> Mat");
    using D = typename DstT::DType;
    using S = typename SrcT::DType;
    check_fix_types<D, S, P>();
    using Geo = MatGeom<DstT>;
    char *lds = hw::lds_base() + dst.st.lds;
    // the destination may lie where an operand of the matmul lay, which other waves may still be reading; and what is
    // written here is read by other waves next (a TSTORE or TEXTRACT of the Mat tile)
    hw::lds_barrier();
    for_each_elem(src, [&](int r, int c, S v, bool owner) {
        const int rr = r - srcRow0, cc = c - srcCol0;
        if (owner && rr >= 0 && cc >= 0 && rr < rows && cc < cols && dstRow0 + rr < DstT::Rows && dstCol0 + cc < DstT::Cols)
            *reinterpret_cast<D *>(lds + Geo::elem_off((uint32_t)(dstRow0 + rr), (uint32_t)(dstCol0 + cc))) = fix_apply<relu, D>(v, c, p);
        return v;
    });
    hw::lds_barrier();
}

// columns the fix pipe moves for `valid` valid ones: whole 32-byte blocks of the destination type
template <typename D>
PTO_DEV int fix_cols(int valid)
{
    constexpr int c0 = 32 / (int)sizeof(D);
    return (valid + c0 - 1) / c0 * c0;
}

template <typename FpT>
PTO_DEV FixVector fix_vector(FpT &fp)
{
    static_assert(FpT::Loc == TileType::Scaling && sizeof(typename FpT::DType) == 8, "[PTO][SA] fix pipe: the quantisation words come in a Scaling tile of 64-bit elements");
    return FixVector{reinterpret_cast<const uint64_t *>(fb_base() + fp.st.fb)};
}

template <ReluPreMode relu, typename DstT, typename SrcT, typename P>
PTO_DEV void tmov_fix(DstT &dst, SrcT &src, const P &p)
{ // every row of the source, the valid columns in whole blocks (npu/a2a3/TMov.hpp:101-102)
    acc_to_mat<relu>(dst, src, 0, 0, 0, 0, SrcT::Rows, fix_cols<typename DstT::DType>(src.GetValidCol()), p);
}
template <ReluPreMode relu, typename DstT, typename SrcT, typename P>
PTO_DEV void textract_fix(DstT &dst, SrcT &src, int idxRow, int idxCol, const P &p)
{ // the destination's valid rows and columns, taken from (idxRow, idxCol) of the source (TExtract.hpp:471-472)
    acc_to_mat<relu>(dst, src, idxRow, idxCol, 0, 0, dst.GetValidRow(), fix_cols<typename DstT::DType>(dst.GetValidCol()), p);
}
template <ReluPreMode relu, typename DstT, typename SrcT, typename P>
PTO_DEV void tinsert_fix(DstT &dst, SrcT &src, int idxRow, int idxCol, const P &p)
{ // the source goes to (idxRow, idxCol) of the destination; the rest of the destination stays (TInsert.hpp:19-37)
    acc_to_mat<relu>(dst, src, 0, 0, idxRow, idxCol, SrcT::Rows, fix_cols<typename DstT::DType>(src.GetValidCol()), p);
}

// Acc -> GM through the conversion, into ND, DN or NZ memory
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu, typename P>
PTO_DEV void tstore_fix(G &dst, TileT &src, const P &p)
{
    using S = typename TileT::DType;
    using D = typename G::DType;
    check_fix_types<D, S, P>();
    D *gm = reinterpret_cast<D *>(dst.data());
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    for_each_elem(src, [&](int r, int c, S x, bool) {
        if (r < vr && c < vc) {
            D *ptr = gm + gm_elem_offset(dst, r, c);
            const D y = fix_apply<relu, D>(x, c, p);
            if constexpr (atomic == AtomicType::AtomicAdd)
                atomic_add(ptr, y);
            else
                *ptr = y;
        }
        return x;
    });
}

} // namespace detail

// Mat -> Scaling: the words of a [1, n] Mat tile into the table (npu/a2a3/TMov.hpp: the Mat -> Scaling pair)
template <typename DstT, typename SrcT>
PTO_DEV void TMOV_MAT2SCALING_IMPL(DstT &dst, SrcT &src)
{
    static_assert(DstT::Loc == TileType::Scaling && SrcT::Loc == TileType::Mat && sizeof(typename DstT::DType) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TMOV: Mat -> Scaling of one element type");
    static_assert(DstT::Rows == 1 && SrcT::Rows == 1 && DstT::Cols <= SrcT::Cols, "[PTO][SA] TMOV: [1, n] tiles");
    using T = typename DstT::DType;
    const char *lds = hw::lds_base() + src.st.lds;
    T *table = reinterpret_cast<T *>(detail::fb_base() + dst.st.fb);
    hw::wait_vm0(); // the asynchronous copies of the TLOAD that filled the Mat tile
    hw::lds_barrier();
    for (int c = hw::tid(); c < DstT::Cols; c += kBlockThreads)
        if (dst.st.fb + (uint32_t)(c + 1) * sizeof(T) <= detail::kFbBytes)
            table[c] = *reinterpret_cast<const T *>(lds + detail::MatGeom<SrcT>::elem_off(0, (uint32_t)c));
    hw::lds_barrier();
}

} // namespace pto
#pragma clang fp contract(fast)
