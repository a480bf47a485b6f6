// Front end of the PTO tile instructions: every instruction waits on the events passed after its
// operands, runs its gfx950 implementation and returns a RecordEvent
// (the calling convention of the reference's include/pto/common/pto_instr.hpp:20-1511).
#pragma once
#include "pto/common/event.hpp"
#include "pto/gfx950/matmul.hpp"
#include "pto/gfx950/mem_ops.hpp"
#include "pto/gfx950/vec_ops.hpp"
#include "pto/gfx950/vec_ops_ext.hpp"
#include "pto/gfx950/fifo_ops.hpp"
#include "pto/gfx950/sort_ops.hpp"
#include "pto/gfx950/matmul_any.hpp"
#include "pto/gfx950/fixpipe.hpp"
#include "pto/gfx950/debug_ops.hpp"

namespace pto {

template <typename... Ev>
PTO_INST void TSYNC(Ev &... ev)
{
    WaitAllEvents(ev...);
}
template <Op OpCode>
PTO_INST void TSYNC()
{
    pipe_barrier(OpPipe(OpCode));
}

template <typename T, typename AddrType>
PTO_INST void TASSIGN(T &obj, AddrType addr)
{
    TASSIGN_IMPL(obj, addr);
}
template <std::size_t Addr, typename T>
PTO_INST std::enable_if_t<is_tile_data_v<T>> TASSIGN(T &obj)
{
    if constexpr (T::Loc == TileType::Mat) {
        static_assert(Addr % 16 == 0, "[PTO][SA] TASSIGN: Mat tiles are 16-byte aligned in LDS");
        static_assert(Addr + detail::mat_tile_bytes<T>() <= detail::kLdsBytes, "[PTO][SA] TASSIGN: tile exceeds the 160 KiB LDS of a CU");
    }
    TASSIGN_IMPL(obj, Addr);
}

namespace detail {
// Vec tiles in memory (PTO_VEC_TILES_IN_MEMORY): an instruction loads the valid region of every Vec tile among its
// operands from the unified buffer into the tile's registers (UbFetch), runs on the registers, and writes the valid
// region of its destination, the first operand, back (UbCommit), after which the stores are drained and the workgroup
// meets at a barrier: the next instruction, in any wave, sees the result.  Other translation units: nothing.
template <typename T>
PTO_DEV void UbFetchOne(T &t)
{
    if constexpr (is_tile_data_v<T>) {
        static_assert(!(T::inMemory && T::isBoxedLayout), "[PTO][SA] Vec tiles in memory: plain row-major or column-major tiles");
        UbFetchTile(t);
    }
}
template <typename... Ts>
PTO_DEV void UbFetch(Ts &... ts)
{
    (UbFetchOne(ts), ...);
}
PTO_DEV void UbFetch() {}
template <typename T, typename... Rest>
PTO_DEV void UbCommit(T &dst, Rest &...)
{
    if constexpr (is_tile_data_v<T>)
        UbCommitTile(dst);
}
} // namespace detail

#define PTO_FRONT(NAME, TPARAMS, PARAMS, ARGS)          \
    template <TPARAMS, typename... Ev>                  \
    PTO_INST RecordEvent NAME(PARAMS, Ev &... ev)       \
    {                                                   \
        TSYNC(ev...);                                   \
        detail::UbFetch ARGS;                           \
        NAME##_IMPL ARGS;                               \
        detail::UbCommit ARGS;                          \
        return {};                                      \
    }
#define PTO_C ,

template <typename TileT, typename G, typename... Ev>
PTO_INST RecordEvent TLOAD(TileT &dst, G &src, Ev &... ev)
{
    TSYNC(ev...);
    TLOAD_IMPL(dst, src);
    if constexpr (is_tile_data_v<TileT>)
        detail::UbCommitLoaded(dst);
    return {};
}
PTO_FRONT(TEXTRACT, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C uint16_t idxRow PTO_C uint16_t idxCol,
          (dst, src, idxRow, idxCol))
PTO_FRONT(TMATMUL, typename C PTO_C typename A PTO_C typename B, C &c PTO_C A &a PTO_C B &b, (c, a, b))
PTO_FRONT(TMATMUL_ACC, typename C PTO_C typename A PTO_C typename B, C &cOut PTO_C C &cIn PTO_C A &a PTO_C B &b,
          (cOut, cIn, a, b))
PTO_FRONT(TMATMUL_BIAS, typename C PTO_C typename A PTO_C typename B, C &c PTO_C A &a PTO_C B &b PTO_C BiasRow bias,
          (c, a, b, bias))
// TMATMUL_BIAS with the bias in a [1, n] Bias tile, and the TGEMV forms: a matmul whose left operand has one valid row
// (pto_instr.hpp:504-571 of the reference)
template <typename C, typename A, typename B, typename Bias, typename... Ev,
          std::enable_if_t<Bias::Loc == TileType::Bias, int> = 0>
PTO_INST RecordEvent TMATMUL_BIAS(C &c, A &a, B &b, Bias &bias, Ev &... ev)
{
    TSYNC(ev...);
    TMATMUL_BIAS_IMPL(c, a, b, bias);
    detail::UbCommit(c);
    return {};
}
template <typename C, typename A, typename B, typename... Ev>
PTO_INST RecordEvent TGEMV(C &c, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    TGEMV_IMPL(c, a, b);
    detail::UbCommit(c);
    return {};
}
template <typename C, typename A, typename B, typename... Ev>
PTO_INST RecordEvent TGEMV_ACC(C &cOut, C &cIn, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(cIn);
    TGEMV_ACC_IMPL(cOut, cIn, a, b);
    detail::UbCommit(cOut);
    return {};
}
template <typename C, typename A, typename B, typename Bias, typename... Ev,
          std::enable_if_t<Bias::Loc == TileType::Bias, int> = 0>
PTO_INST RecordEvent TGEMV_BIAS(C &c, A &a, B &b, Bias &bias, Ev &... ev)
{
    TSYNC(ev...);
    TGEMV_BIAS_IMPL(c, a, b, bias);
    detail::UbCommit(c);
    return {};
}
PTO_FRONT(TCVT, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C RoundMode mode, (dst, src, mode))
PTO_FRONT(TGATHER, typename D PTO_C typename S0 PTO_C typename I, D &dst PTO_C S0 &src0 PTO_C I &idx, (dst, src0, idx))
PTO_FRONT(MGATHER, typename D PTO_C typename G PTO_C typename I, D &dst PTO_C G &src PTO_C I &idx, (dst, src, idx))
PTO_FRONT(MGATHER_ROWS, typename D PTO_C typename G PTO_C typename I, D &dst PTO_C G &table PTO_C I &rowIdx PTO_C int tableRows,
          (dst, table, rowIdx, tableRows))
PTO_FRONT(TADD, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TSUB, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TMUL, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TDIV, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TMAX, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TMIN, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TMULS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TADDS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TSUBS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TDIVS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TMAXS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TMINS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TEXP, typename T, T &dst PTO_C T &src, (dst, src))
PTO_FRONT(TEXPANDS, typename T, T &dst PTO_C typename T::DType k, (dst, k))
PTO_FRONT(TROWMAX, typename D PTO_C typename S PTO_C typename T, D &dst PTO_C S &src PTO_C T &tmp, (dst, src, tmp))
PTO_FRONT(TROWPROD, typename D PTO_C typename S PTO_C typename T, D &dst PTO_C S &src PTO_C T &tmp, (dst, src, tmp))
PTO_FRONT(TROWSUM, typename D PTO_C typename S PTO_C typename T, D &dst PTO_C S &src PTO_C T &tmp, (dst, src, tmp))
PTO_FRONT(TROWEXPANDSUB, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDMUL, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDDIV, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDADD, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDMAX, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDMIN, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPANDEXPDIF, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &src0 PTO_C B &src1, (dst, src0, src1))
PTO_FRONT(TROWEXPAND, typename D PTO_C typename R, D &dst PTO_C R &src, (dst, src))
PTO_FRONT(TROWMIN, typename D PTO_C typename S PTO_C typename T, D &dst PTO_C S &src PTO_C T &tmp, (dst, src, tmp))
PTO_FRONT(TCOLMAX, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TCOLPROD, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TCOLMIN, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TCOLSUM, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TCOLEXPAND, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TCOLEXPANDSUB, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDMUL, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDDIV, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDADD, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDMAX, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDMIN, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TCOLEXPANDEXPDIF, typename D PTO_C typename R, D &dst PTO_C D &src0 PTO_C R &src1, (dst, src0, src1))
PTO_FRONT(TABS, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TNEG, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TRELU, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TSQRT, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TRSQRT, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TLOG, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TRECIP, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
template <typename D, typename A, typename B, typename... Ev>
PTO_INST std::enable_if_t<(... && is_wait_event<Ev>::value), RecordEvent> TPRELU(D &dst, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, a, b);
    TPRELU_IMPL(dst, a, b);
    detail::UbCommit(dst);
    return {};
}
// bitwise / shift / remainder / three-operand forms (pto_instr.hpp:72-86, 246-333, 1137, 1215-1300, 1418 of the reference;
// the forms that take a scratch tile accept and ignore it)
PTO_FRONT(TAND, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TOR, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TSHL, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TSHR, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TREM, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TFMOD, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TNOT, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TGATHERB, typename D PTO_C typename S PTO_C typename O, D &dst PTO_C S &src PTO_C O &offset, (dst, src, offset))
#if defined(PTO_TSCATTER_FLAT_INDEX)
// the NPU implementation's TSCATTER: indices are element numbers of the destination (npu/a2a3/TScatter.hpp:17-36)
template <typename D, typename S, typename I, typename... Ev>
PTO_INST RecordEvent TSCATTER(D &dst, S &src, I &indexes, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src, indexes);
    TSCATTER_FLAT_IMPL(dst, src, indexes);
    detail::UbCommit(dst);
    return {};
}
#else
PTO_FRONT(TSCATTER, typename D PTO_C typename I, D &dst PTO_C D &src PTO_C I &indexes, (dst, src, indexes))
#endif
PTO_FRONT(MSCATTER, typename G PTO_C typename S PTO_C typename I, G &dst PTO_C S &src PTO_C I &indexes, (dst, src, indexes))
PTO_FRONT(TPARTADD, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TPARTMAX, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TPARTMIN, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TPARTMUL, typename D PTO_C typename A PTO_C typename B, D &dst PTO_C A &a PTO_C B &b, (dst, a, b))
PTO_FRONT(TANDS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TORS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TSHLS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TSHRS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TREMS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TFMODS, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TADDC, typename T, T &dst PTO_C T &a PTO_C T &b PTO_C T &c, (dst, a, b, c))
PTO_FRONT(TSUBC, typename T, T &dst PTO_C T &a PTO_C T &b PTO_C T &c, (dst, a, b, c))
PTO_FRONT(TADDSC, typename T, T &dst PTO_C T &a PTO_C typename T::DType k PTO_C T &b, (dst, a, k, b))
PTO_FRONT(TSUBSC, typename T, T &dst PTO_C T &a PTO_C typename T::DType k PTO_C T &b, (dst, a, k, b))
template <typename D, typename A, typename B, typename Tmp, typename... Ev>
PTO_INST std::enable_if_t<is_tile_data_v<Tmp>, RecordEvent> TXOR(D &dst, A &a, B &b, Tmp &, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, a, b);
    TXOR_IMPL(dst, a, b);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename S, typename Tmp, typename... Ev>
PTO_INST std::enable_if_t<is_tile_data_v<Tmp>, RecordEvent> TXORS(D &dst, S &src, typename S::DType k, Tmp &, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TXORS_IMPL(dst, src, k);
    detail::UbCommit(dst);
    return {};
}
PTO_FRONT(TLRELU, typename D PTO_C typename S, D &dst PTO_C S &src PTO_C typename D::DType k, (dst, src, k))
PTO_FRONT(TCMP, typename T, T &dst PTO_C T &src0 PTO_C T &src1 PTO_C CmpMode mode, (dst, src0, src1, mode))
PTO_FRONT(TCMPS, typename D PTO_C typename S PTO_C typename T, D &dst PTO_C S &src0 PTO_C T src1 PTO_C CmpMode mode,
          (dst, src0, src1, mode))
PTO_FRONT(TSEL, typename T PTO_C typename M, T &dst PTO_C M &selMask PTO_C T &src0 PTO_C T &src1, (dst, selMask, src0, src1))
// TSELS has two meanings in the reference.  Its front end (pto_instr.hpp:1014-1021) and the NPU take (dst, mask, src, scalar):
// a tile of integers as bit mask.  Its CPU simulation implements (dst, src0, src1, selectMode) on three tiles of one type,
// the whole of src0 or of src1.  A second operand that is a tile of integers is a mask; three floating-point tiles of one
// type are the whole-tile form.
template <typename T, typename... Ev, std::enable_if_t<!std::is_integral_v<typename T::DType>, int> = 0>
PTO_INST RecordEvent TSELS(T &dst, T &src0, T &src1, uint8_t selectMode, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src0, src1, selectMode);
    TSELS_IMPL(dst, src0, src1, selectMode);
    detail::UbCommit(dst, src0, src1, selectMode);
    return {};
}
template <typename D, typename M, typename S, typename... Ev, std::enable_if_t<std::is_integral_v<typename M::DType>, int> = 0>
PTO_INST RecordEvent TSELS(D &dst, M &mask, S &src, typename S::DType scalar, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(mask, src);
    TSELS_MASK_IMPL(dst, mask, src, scalar);
    detail::UbCommit(dst);
    return {};
}
PTO_FRONT(TFILLPAD, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TFILLPAD_INPLACE, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TFILLPAD_EXPAND, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
PTO_FRONT(TPACK, typename D PTO_C typename S, D &dst PTO_C S &src, (dst, src))
// TPREFETCH (pto_instr.hpp:135-140 of the reference; cpu/TPrefetch.hpp copies the region into the tile): a TLOAD here
PTO_FRONT(TPREFETCH, typename TileT PTO_C typename G, TileT &dst PTO_C G &src, (dst, src))
// TQUANT, the block-scaled MXFP8 form (pto_instr.hpp:1481-1490 of the reference): exponent, maximum and scaling tiles by address
template <auto quant, typename D, typename S, typename E, typename M, typename... Ev>
PTO_INST RecordEvent TQUANT(D &dst, S &src, E *exp, M *max, S *scaling, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TQUANT_IMPL<quant>(dst, src, exp, max, scaling);
    detail::UbCommit(dst);
    detail::UbCommit(*exp);
    detail::UbCommit(*max);
    detail::UbCommit(*scaling);
    return {};
}
// TQUANT, the row-scale form (pto_instr.hpp:1503-1510 of the reference)
template <auto quant, typename D, typename S, typename P, typename... Ev>
PTO_INST RecordEvent TQUANT(D &dst, S &src, P &scale, P *offset = nullptr, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src, scale);
    if (offset != nullptr)
        detail::UbFetch(*offset);
    TQUANT_IMPL<quant>(dst, src, scale, offset);
    detail::UbCommit(dst);
    detail::UbCommit(src);
    return {};
}
// TDEQUANT (pto_instr.hpp:1407-1415 of the reference)
template <typename D, typename S, typename P, typename... Ev>
PTO_INST RecordEvent TDEQUANT(D &dst, S &src, P &scale, P &offset, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src, scale, offset);
    TDEQUANT_IMPL(dst, src, scale, offset);
    detail::UbCommit(dst);
    return {};
}
// TGEMV_MX (pto_instr.hpp:341-398 of the reference): TMATMUL_MX on a left operand with one valid row
template <typename C, typename A, typename SA, typename B, typename SB, typename... Ev>
PTO_INST std::enable_if_t<A::Loc == TileType::Left, RecordEvent> TGEMV_MX(C &c, A &a, SA &sa, B &b, SB &sb, Ev &... ev)
{
    return TMATMUL_MX(c, a, sa, b, sb, ev...);
}
template <typename C, typename A, typename SA, typename B, typename SB, typename... Ev>
PTO_INST std::enable_if_t<A::Loc == TileType::Left, RecordEvent> TGEMV_MX(C &cOut, C &cIn, A &a, SA &sa, B &b, SB &sb, Ev &... ev)
{
    return TMATMUL_MX(cOut, cIn, a, sa, b, sb, ev...);
}
// TPRINT (pto_instr.hpp:316-322 of the reference): a Vec tile or a GlobalTensor written to the host's stdout
template <typename T, typename... Ev>
PTO_INST RecordEvent TPRINT(T &src, Ev &... ev)
{
    TSYNC(ev...);
    if constexpr (is_tile_data_v<T>)
        detail::UbFetch(src);
    TPRINT_IMPL(src);
    return {};
}
PTO_FRONT(TPUSH, typename P PTO_C typename T PTO_C typename F, P &prod PTO_C T &tile PTO_C F &fifo, (prod, tile, fifo))
PTO_FRONT(TPOP, typename P PTO_C typename T PTO_C typename F, P &cons PTO_C T &tile PTO_C F &fifo, (cons, tile, fifo))
#undef PTO_FRONT
#undef PTO_C
// the forms that name the pipe (pto_instr.hpp:1442-1471 of the reference)
template <typename TileData, typename Pipe, typename... Ev, std::enable_if_t<is_tile_data_v<TileData>, int> = 0>
PTO_INST RecordEvent TPUSH(TileData &tile, Pipe &pipe, Ev &... ev)
{
    TSYNC(ev...);
    TPUSH_IMPL(tile, pipe);
    return {};
}
template <typename TileData, typename Pipe, typename... Ev, std::enable_if_t<is_tile_data_v<TileData>, int> = 0>
PTO_INST RecordEvent TPOP(TileData &tile, Pipe &pipe, Ev &... ev)
{
    TSYNC(ev...);
    TPOP_IMPL(tile, pipe);
    return {};
}
template <typename Pipe, typename... Ev>
PTO_INST RecordEvent TFREE(Pipe &pipe, Ev &... ev)
{
    TSYNC(ev...);
    TFREE_IMPL(pipe);
    return {};
}

// TRESHAPE (pto_instr.hpp:998 of the reference): the same storage under another shape.  Register tiles: a copy of the
// registers (both shapes have the same distribution).  Vec tiles in memory: dst becomes a VIEW of src's storage, as on a
// machine where the tile is an address (the reference's softmax stage writes a [R,1] tile through its [1,R] view).
template <typename D, typename S, typename... Ev>
PTO_INST RecordEvent TRESHAPE(D &dst, S &src, Ev &... ev)
{
    TSYNC(ev...);
#if defined(PTO_VEC_TILES_IN_MEMORY)
    if constexpr (D::inMemory && S::inMemory) {
        static_assert(D::Numel * sizeof(typename D::DType) == S::Numel * sizeof(typename S::DType), "[PTO][SA] TRESHAPE: same storage size");
        if (src.mem_ != nullptr) {
            dst.mem_ = reinterpret_cast<typename D::DType *>(src.mem_);
            return {};
        }
    }
#endif
    TRESHAPE_IMPL(dst, src);
    return {};
}

// TMOV (pto_instr.hpp:881-940): Mat -> Left / Right, register tile copies, and accumulator -> Vec with an
// optional clamp at zero; the split mode over Vec cores is an Ascend hint
template <typename D, typename S, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TMOV(D &dst, S &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    if constexpr (S::Loc == TileType::Acc && D::Loc == TileType::Vec)
        TMOV_ACC2VEC_IMPL<relu>(dst, src);
    else if constexpr (S::Loc == TileType::Acc && D::Loc == TileType::Mat)
        detail::tmov_fix<relu>(dst, src, detail::FixNone{});
    else if constexpr (S::Loc == TileType::Mat && D::Loc == TileType::Scaling)
        TMOV_MAT2SCALING_IMPL(dst, src);
    else if constexpr ((S::Loc == TileType::Acc || S::Loc == TileType::Vec) && (D::Loc == TileType::Left || D::Loc == TileType::Right))
        TMOV_TO_OPERAND_IMPL(dst, src); // the chained matmuls of the Auto-mode programs
    else
        TMOV_IMPL(dst, src);
    detail::UbCommit(dst);
    return {};
}
// TTRANS (pto_instr.hpp:1032 of the reference): the scratch tile is accepted and ignored
template <typename D, typename S, typename Tmp, typename... Ev>
PTO_INST RecordEvent TTRANS(D &dst, S &src, Tmp &, Ev &... ev)
{
    TSYNC(ev...);
    TTRANS_IMPL(dst, src);
    return {};
}
template <typename D, typename S, AccToVecMode mode, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TMOV(D &dst, S &src, Ev &... ev)
{
    TSYNC(ev...);
    TMOV_ACC2VEC_IMPL<relu>(dst, src);
    return {};
}

// The accumulator's way out with a conversion (pto/gfx950/fixpipe.hpp): one quantisation word for the tile, or one per
// column in a Scaling tile (pto_instr.hpp:196-236, 625-660, 716-752, 893-915 of the reference)
template <typename D, typename S, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TMOV(D &dst, S &src, uint64_t preQuantScalar, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tmov_fix<relu>(dst, src, detail::FixScalar{preQuantScalar});
    return {};
}
template <typename D, typename S, typename Fp, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TMOV_FP(D &dst, S &src, Fp &fp, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tmov_fix<relu>(dst, src, detail::fix_vector(fp));
    return {};
}
template <typename D, typename S, ReluPreMode relu, typename... Ev>
PTO_INST RecordEvent TEXTRACT(D &dst, S &src, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::textract_fix<relu>(dst, src, idxRow, idxCol, detail::FixNone{});
    return {};
}
template <typename D, typename S, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TEXTRACT(D &dst, S &src, uint64_t preQuantScalar, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::textract_fix<relu>(dst, src, idxRow, idxCol, detail::FixScalar{preQuantScalar});
    return {};
}
template <typename D, typename S, typename Fp, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TEXTRACT_FP(D &dst, S &src, Fp &fp, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::textract_fix<relu>(dst, src, idxRow, idxCol, detail::fix_vector(fp));
    return {};
}
template <typename D, typename S, typename... Ev>
PTO_INST RecordEvent TINSERT(D &dst, S &src, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tinsert_fix<ReluPreMode::NoRelu>(dst, src, idxRow, idxCol, detail::FixNone{});
    return {};
}
template <typename D, typename S, ReluPreMode relu, typename... Ev>
PTO_INST RecordEvent TINSERT(D &dst, S &src, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tinsert_fix<relu>(dst, src, idxRow, idxCol, detail::FixNone{});
    return {};
}
template <typename D, typename S, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TINSERT(D &dst, S &src, uint64_t preQuantScalar, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tinsert_fix<relu>(dst, src, idxRow, idxCol, detail::FixScalar{preQuantScalar});
    return {};
}
template <typename D, typename S, typename Fp, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TINSERT_FP(D &dst, S &src, Fp &fp, uint16_t idxRow, uint16_t idxCol, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tinsert_fix<relu>(dst, src, idxRow, idxCol, detail::fix_vector(fp));
    return {};
}
template <typename TileT, typename G, AtomicType atomic = AtomicType::AtomicNone, ReluPreMode relu = ReluPreMode::NoRelu, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, uint64_t preQuantScalar, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tstore_fix<TileT, G, atomic, relu>(dst, src, detail::FixScalar{preQuantScalar});
    return {};
}
template <STPhase Phase, typename TileT, typename G, AtomicType atomic = AtomicType::AtomicNone, ReluPreMode relu = ReluPreMode::NoRelu,
          typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, uint64_t preQuantScalar, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tstore_fix<TileT, G, atomic, relu>(dst, src, detail::FixScalar{preQuantScalar});
    return {};
}
template <typename TileT, typename G, typename Fp, AtomicType atomic = AtomicType::AtomicNone, ReluPreMode relu = ReluPreMode::NoRelu,
          typename... Ev>
PTO_INST RecordEvent TSTORE_FP(G &dst, TileT &src, Fp &fp, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    detail::tstore_fix<TileT, G, atomic, relu>(dst, src, detail::fix_vector(fp));
    return {};
}

// TCI (pto_instr.hpp:808-814 of the reference)
template <typename TileT, typename T, int descending, typename... Ev>
PTO_INST RecordEvent TCI(TileT &dst, T start, Ev &... ev)
{
    TSYNC(ev...);
    TCI_IMPL<TileT, T, descending>(dst, start);
    return {};
}

// TSORT32 (pto_instr.hpp:786-798 of the reference; it takes no events) and TMRGSORT (pto_instr.hpp:582-622).  Both leave
// parts of the destination as they were, so the destination is fetched as well where Vec tiles live in memory; the
// sources may alias it (the reference's top-k kernel merges in place, topk_kernel.cpp:77-82): every operand is in
// registers before the instruction runs.
template <typename D, typename S, typename I>
PTO_INST RecordEvent TSORT32(D &dst, S &src, I &idx)
{
    detail::UbFetch(dst, src, idx);
    TSORT32_IMPL(dst, src, idx);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename S, typename I, typename Tmp>
PTO_INST RecordEvent TSORT32(D &dst, S &src, I &idx, Tmp &tmp)
{
    detail::UbFetch(dst, src, idx);
    TSORT32_IMPL(dst, src, idx, tmp);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename Tmp, typename S0, typename S1, typename S2, typename S3, bool exhausted, typename... Ev>
PTO_INST RecordEvent TMRGSORT(D &dst, MrgSortExecutedNumList &executed, Tmp &tmp, S0 &src0, S1 &src1, S2 &src2, S3 &src3, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src0, src1, src2, src3);
    TMRGSORT_IMPL<D, Tmp, S0, S1, S2, S3, exhausted>(dst, executed, tmp, src0, src1, src2, src3);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename Tmp, typename S0, typename S1, typename S2, bool exhausted, typename... Ev>
PTO_INST RecordEvent TMRGSORT(D &dst, MrgSortExecutedNumList &executed, Tmp &tmp, S0 &src0, S1 &src1, S2 &src2, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src0, src1, src2);
    TMRGSORT_IMPL<D, Tmp, S0, S1, S2, exhausted>(dst, executed, tmp, src0, src1, src2);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename Tmp, typename S0, typename S1, bool exhausted, typename... Ev>
PTO_INST RecordEvent TMRGSORT(D &dst, MrgSortExecutedNumList &executed, Tmp &tmp, S0 &src0, S1 &src1, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src0, src1);
    TMRGSORT_IMPL<D, Tmp, S0, S1, exhausted>(dst, executed, tmp, src0, src1);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename S, typename... Ev>
PTO_INST RecordEvent TMRGSORT(D &dst, S &src, uint32_t blockLen, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TMRGSORT_IMPL(dst, src, blockLen);
    detail::UbCommit(dst);
    return {};
}

// TPRELU with a scratch tile (pto_instr.hpp:306-313 of the reference): accepted and ignored
template <typename D, typename A, typename B, typename Tmp, typename... Ev>
PTO_INST std::enable_if_t<is_tile_data_v<Tmp>, RecordEvent> TPRELU(D &dst, A &a, B &b, Tmp &, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, a, b);
    TPRELU_IMPL(dst, a, b);
    detail::UbCommit(dst);
    return {};
}
// TCMP with a uint8 destination: packed bits, the NPU's form (the CPU simulation's writes 0 / 1 in the sources' type)
template <typename D, typename S, typename... Ev>
PTO_INST std::enable_if_t<!std::is_same_v<D, S> && sizeof(typename D::DType) == 1, RecordEvent> TCMP(D &dst, S &src0, S &src1, CmpMode mode,
                                                                                                     Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src0, src1);
    TCMP_PACKED_IMPL(dst, src0, src1, mode);
    detail::UbCommit(dst);
    return {};
}
// TDIVS(dst, scalar, src) = scalar / src (pto_instr.hpp:1176-1182 of the reference)
template <typename D, typename S, typename... Ev>
PTO_INST std::enable_if_t<is_tile_data_v<S>, RecordEvent> TDIVS(D &dst, typename D::DType k, S &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TDIVS_SCALAR_FIRST_IMPL(dst, src, k);
    detail::UbCommit(dst);
    return {};
}
// TCOLSUM with a scratch tile and the choice of a pairwise order (pto_instr.hpp:966-972): both accepted and ignored
template <typename D, typename S, typename Tmp, typename... Ev>
PTO_INST RecordEvent TCOLSUM(D &dst, S &src, Tmp &tmp, bool isBinary, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TCOLSUM_IMPL(dst, src, tmp, isBinary);
    detail::UbCommit(dst);
    return {};
}

// forms whose template arguments come first
template <typename TileT, typename G, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, AtomicType::AtomicNone>(dst, src);
    return {};
}
template <STPhase Phase, typename TileT, typename G, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{ // the unit-flag phase is an Ascend fix-pipe hint; a store is a store here
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, AtomicType::AtomicNone>(dst, src);
    return {};
}
template <typename TileT, typename G, AtomicType atomic, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, atomic>(dst, src);
    return {};
}
// (pto_instr.hpp:183-207 of the reference: atomic type + unit-flag phase, atomic type + ReLU, all three)
template <typename TileT, typename G, AtomicType atomic, STPhase Phase, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, atomic>(dst, src);
    return {};
}
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, atomic, relu>(dst, src);
    return {};
}
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu, STPhase Phase, typename... Ev>
PTO_INST RecordEvent TSTORE(G &dst, TileT &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(src);
    TSTORE_IMPL<TileT, G, atomic, relu>(dst, src);
    return {};
}
// the form without indices; index arguments that are lvalues (`TEXTRACT(dst, src, row, col)` with int variables) must
// not be taken for events
template <typename D, typename S, typename... Ev, std::enable_if_t<(is_wait_event<Ev>::value && ...), int> = 0>
PTO_INST RecordEvent TEXTRACT(D &dst, S &src, Ev &... ev)
{
    TSYNC(ev...);
    TEXTRACT_IMPL(dst, src, 0, 0);
    return {};
}
template <AccPhase Phase, typename C, typename A, typename B, typename... Ev>
PTO_INST RecordEvent TMATMUL(C &c, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    TMATMUL_IMPL(c, a, b);
    detail::UbCommit(c);
    return {};
}
template <AccPhase Phase, typename C, typename A, typename B, typename... Ev>
PTO_INST RecordEvent TMATMUL_ACC(C &cOut, C &cIn, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(cIn);
    TMATMUL_ACC_IMPL(cOut, cIn, a, b);
    detail::UbCommit(cOut);
    return {};
}
template <AccPhase Phase = AccPhase::Unspecified, typename C, typename A, typename B, typename... Ev>
PTO_INST std::enable_if_t<A::Loc == TileType::Left, RecordEvent> TMATMUL_ACC(C &c, A &a, B &b, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(c);
    TMATMUL_ACC_IMPL(c, c, a, b);
    detail::UbCommit(c);
    return {};
}
// TMATMUL_MX(c, a, aScale, b, bScale) and the accumulating form (cOut, cIn, a, aScale, b, bScale)  (pto_instr.hpp:403-440)
template <typename C, typename A, typename AS, typename B, typename BS, typename... Ev>
PTO_INST std::enable_if_t<A::Loc == TileType::Left, RecordEvent> TMATMUL_MX(C &c, A &a, AS &aScale, B &b, BS &bScale, Ev &... ev)
{
    TSYNC(ev...);
    TMATMUL_MX_IMPL(c, a, aScale, b, bScale);
    return {};
}
template <typename C, typename A, typename AS, typename B, typename BS, typename... Ev>
PTO_INST std::enable_if_t<A::Loc == TileType::Left, RecordEvent> TMATMUL_MX(C &cOut, C &cIn, A &a, AS &aScale, B &b, BS &bScale,
                                                                             Ev &... ev)
{
    TSYNC(ev...);
    TMATMUL_MX_IMPL(cOut, cIn, a, aScale, b, bScale);
    return {};
}
// TMATMUL_MX with a [1, n] Bias tile: c = a x b + bias  (pto_instr.hpp:444-451 of the reference)
template <typename C, typename A, typename AS, typename B, typename BS, typename Bias, typename... Ev,
          std::enable_if_t<A::Loc == TileType::Left && Bias::Loc == TileType::Bias, int> = 0>
PTO_INST RecordEvent TMATMUL_MX(C &c, A &a, AS &aScale, B &b, BS &bScale, Bias &bias, Ev &... ev)
{
    TSYNC(ev...);
    TMATMUL_MX_IMPL(c, a, aScale, b, bScale, bias);
    return {};
}
template <typename D, typename S, typename... Ev>
PTO_INST RecordEvent TCVT(D &dst, S &src, RoundMode mode, SaturationMode sat, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TCVT_IMPL(dst, src, mode, sat);
    detail::UbCommit(dst);
    return {};
}
template <typename D, typename S, MaskPattern pattern, typename... Ev>
PTO_INST RecordEvent TGATHER(D &dst, S &src, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst, src);
    TGATHER_IMPL<D, S, pattern>(dst, src);
    detail::UbCommit(dst);
    return {};
}
template <typename TileT, int isUpperOrLower, typename... Ev>
PTO_INST RecordEvent TTRI(TileT &dst, int diagonal, Ev &... ev)
{
    TSYNC(ev...);
    detail::UbFetch(dst);
    TTRI_IMPL<TileT, isUpperOrLower>(dst, diagonal);
    detail::UbCommit(dst);
    return {};
}

} // namespace pto
