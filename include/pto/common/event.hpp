// Events of the PTO API: every tile instruction returns a RecordEvent and accepts trailing
// events to wait on (reference: include/pto/common/event.hpp:19-140, npu/a2a3/TSync.hpp:137-226).
// On gfx950 an Event between two pipes reduces to the wait_flag rule of that pipe pair.
#pragma once
#include <type_traits>
#include <utility>
#include "pto/gfx950/platform.hpp"

namespace pto {

enum class Op : uint16_t {
    TLOAD, TSTORE_VEC, TSTORE_ACC, TMOV_M2L, TMOV_M2R, TMOV_A2V, TMOV_V2M, TEXTRACT, TMATMUL, TMATMUL_ACC, TMATMUL_BIAS,
    VECTOR, SCALAR, OP_COUNT
};

// Pipe an Op runs on, in the reference's model (npu/a2a3/TSync.hpp:26-109).
PTO_HD constexpr pipe_t OpPipe(Op op)
{
    switch (op) {
    case Op::TLOAD: return PIPE_MTE2;
    case Op::TSTORE_VEC: return PIPE_MTE3;
    case Op::TSTORE_ACC: return PIPE_FIX;
    case Op::TMOV_M2L:
    case Op::TMOV_M2R:
    case Op::TEXTRACT: return PIPE_MTE1;
    case Op::TMATMUL:
    case Op::TMATMUL_ACC:
    case Op::TMATMUL_BIAS: return PIPE_M;
    case Op::TMOV_A2V: return PIPE_FIX;
    case Op::TMOV_V2M: return PIPE_MTE3;
    case Op::SCALAR: return PIPE_S;
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

} // namespace pto
