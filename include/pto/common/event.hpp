// Events of the PTO API: every tile instruction returns a RecordEvent and accepts trailing
// events to wait on (reference: include/pto/common/event.hpp:19-140, npu/a2a3/TSync.hpp:137-226).
// On gfx950 an Event between two pipes reduces to the wait_flag rule of that pipe pair.
#pragma once
#include <type_traits>
#include <utility>
#include "pto/gfx950/platform.hpp"

namespace pto {

// Instruction names as event end points: the reference's list and order (include/pto/common/event.hpp:19-105), then the
// names this library adds (TEXTRACT without a location pair, the accumulating matmul forms).
enum class Op : uint16_t {
    TLOAD, TSTORE_VEC, SCALAR, TRESHAPE, VECTOR,
    TADD, TADDS, TSUB, TMUL, TMULS, TDIV, TDIVS, TMIN, TMINS, TMAX, TAND, TOR, TSEL, TSHL, TSHR, TEXP, TSELS, TSQRT, TRSQRT,
    TEXPANDS, TPARTADD, TPARTMUL, TPARTMAX, TPARTMIN, TCMPS, TMRGSORT, TSORT32, TCI, TGATHER, TGATHERB, TCVT,
    TROWSUM, TROWPROD, TROWMAX, TROWMIN, TROWEXPAND, TCOLSUM, TCOLPROD, TCOLMAX, TCOLMIN, TTRANS, TTRI,
    TREM, TFMOD, TREMS, TFMODS, TSUBS, TMAXS, TLRELU, TPRELU,
    TMOV_V2V, TMOV_V2M, TEXTRACT_V2M, TMOV_M2B, TMOV_M2L, TMOV_M2R, TMOV_M2S, TMOV_A2V, TMOV_A2M, TSTORE_ACC, TSTORE_MAT,
    TMATMUL, TGEMV, TMATMUL_MX, TEXTRACT_M2LR, TANDS, TORS, TSHLS, TSHRS, TXOR, TXORS, TEXTRACT_A2M, TINSERT_A2M,
    TIMG2COL, TSETFMATRIX, TSET_IMG2COL_RPT, TSET_IMG2COL_PADDING, TDEQUANT,
    OP_COUNT,
    TEXTRACT, TMATMUL_ACC, TMATMUL_BIAS
};

// Pipe an Op runs on, in the reference's model (npu/a2a3/TSync.hpp:26-109).
PTO_HD constexpr pipe_t OpPipe(Op op)
{
    switch (op) {
    case Op::TLOAD: return PIPE_MTE2;
    case Op::TSTORE_VEC:
    case Op::TSTORE_MAT: return PIPE_MTE3;
    case Op::SCALAR:
    case Op::TRESHAPE:
    case Op::TCI:
    case Op::TSETFMATRIX:
    case Op::TSET_IMG2COL_RPT:
    case Op::TSET_IMG2COL_PADDING: return PIPE_S;
    case Op::TMOV_M2B:
    case Op::TMOV_M2L:
    case Op::TMOV_M2R:
    case Op::TEXTRACT_M2LR:
    case Op::TIMG2COL:
    case Op::TEXTRACT: return PIPE_MTE1;
    case Op::TMATMUL:
    case Op::TGEMV:
    case Op::TMATMUL_MX:
    case Op::TMATMUL_ACC:
    case Op::TMATMUL_BIAS: return PIPE_M;
    case Op::TMOV_V2M:
    case Op::TEXTRACT_V2M:
    case Op::TMOV_M2S:
    case Op::TMOV_A2V:
    case Op::TMOV_A2M:
    case Op::TSTORE_ACC:
    case Op::TEXTRACT_A2M:
    case Op::TINSERT_A2M: return PIPE_FIX;
    default: return PIPE_V;
    }
}

struct RecordEvent {};

template <Op SrcOp, Op DstOp, bool AutoToken = true, event_t EventID = EVENT_ID0>
struct Event {
    static constexpr pipe_t srcPipe = OpPipe(SrcOp);
    static constexpr pipe_t dstPipe = OpPipe(DstOp);
    PTO_DEV Event &Init() { return *this; }
    PTO_DEV Event &Record()
    {
        set_flag(srcPipe, dstPipe, EventID);
        return *this;
    }
    PTO_DEV Event &Wait()
    {
        wait_flag(srcPipe, dstPipe, EventID);
        return *this;
    }
    PTO_DEV Event &operator=(RecordEvent) { return Record(); }
};

// true for the types an instruction may take after its operands: anything with a Wait() member (event.hpp:136-140 of the
// reference waits on each of them)
template <typename T, typename = void>
struct is_wait_event : std::false_type {};
template <typename T>
struct is_wait_event<T, std::void_t<decltype(std::declval<T &>().Wait())>> : std::true_type {};

template <typename... WaitEvents>
PTO_DEV void WaitAllEvents(WaitEvents &... events)
{
    (events.Wait(), ...);
}

// set_flag + wait_flag on event 0 of a pipe pair (event.hpp:142-152 of the reference)
template <pipe_t SrcPipe, pipe_t DstPipe>
PTO_DEV void PtoSetWaitFlag()
{
    set_flag(SrcPipe, DstPipe, EVENT_ID0);
    wait_flag(SrcPipe, DstPipe, EVENT_ID0);
}

} // namespace pto
