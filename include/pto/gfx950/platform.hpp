// gfx950 (MI355X / CDNA4) platform layer of the PTO tile API.
//
// Takes the place of the reference's platform shim (include/pto/common/cpu_stub.hpp:29-90 for the
// CPU simulation, the CCE compiler builtins on Ascend): memory-space qualifiers, pipe and event
// names, set_flag / wait_flag / pipe_barrier, block indices.
//
// Execution model.  One PTO "core" is one HIP workgroup of PTO_WAVES_M x PTO_WAVES_N wavefronts
// (64 lanes each).  A tile instruction is executed cooperatively by the whole workgroup:
//   Mat tiles           live in LDS (the role of L1),
//   Left / Right / Acc  are per-wave MFMA operand / accumulator fragments in VGPRs / AGPRs (L0A/L0B/L0C),
//   Vec tiles           are distributed over the workgroup's lanes in VGPRs (UB).
// Ascend pipes become the hardware counters of one instruction stream:
//   MTE2 (GM->L1)  = asynchronous global->LDS loads, tracked by vmcnt
//   MTE1 (L1->L0)  = ds_read, tracked by lgkmcnt (the compiler inserts those waits)
//   M, V, FIX      = MFMA / VALU / global stores on registers: ordered by data dependences
// so a wait_flag only has to do something where LDS contents cross wavefronts.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <type_traits>

#define PTO_HD __host__ __device__ __forceinline__
#define PTO_DEV __device__ __forceinline__
#define PTO_INST PTO_DEV
#define PTO_INTERNAL PTO_DEV

// Qualifiers of the Ascend dialect that kernel sources carry; all memory is reached through
// generic pointers here.
#define AICORE
#define __aicore__
#define __gm__
#define __ubuf__
#define __cbuf__
#define __ca__
#define __cb__
#define __cc__
#define __fbuf__
#define __in__
#define __out__
#define __tf__

#ifndef PTO_WAVES_M
#define PTO_WAVES_M 2
#endif
#ifndef PTO_WAVES_N
#define PTO_WAVES_N 2
#endif
// Output block of the MFMA behind TMATMUL: 32 (v_mfma_f32_32x32x16) or 16 (v_mfma_f32_16x16x32).  Same flops per
// cycle; the 16-wide form moves half the accumulator registers per flop and sustains a higher clock under the
// chip's power limit (measured on pure MFMA loops: 1.87 GHz against 1.70 GHz).
#ifndef PTO_MFMA_M
#define PTO_MFMA_M 32
#endif

namespace pto {
constexpr int kWaveSize = 64;
constexpr int kWavesM = PTO_WAVES_M;
constexpr int kWavesN = PTO_WAVES_N;
constexpr int kBlockWaves = kWavesM * kWavesN;
constexpr int kBlockThreads = kBlockWaves * kWaveSize;

namespace hw {
PTO_DEV int lane() { return static_cast<int>(threadIdx.x) & (kWaveSize - 1); }
// wave index as a scalar (SGPR) value
PTO_DEV int wave() { return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6); }
PTO_DEV int wave_m() { return wave() / kWavesN; }
PTO_DEV int wave_n() { return wave() % kWavesN; }
PTO_DEV int tid() { return static_cast<int>(threadIdx.x); }

// Base of the workgroup's dynamic LDS allocation: address 0 of the "L1" space that TASSIGN names.
PTO_DEV char *lds_base()
{
    extern __shared__ __attribute__((aligned(16))) char pto_dynamic_lds[];
    return pto_dynamic_lds;
}

PTO_DEV void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// wait until at most N of this wave's vector-memory instructions are still outstanding (N <= 63)
template <int N>
PTO_DEV void wait_vm()
{
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
PTO_DEV void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// Workgroup barrier that orders LDS traffic only; outstanding global loads keep flying.
PTO_DEV void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
} // namespace hw

namespace host {
constexpr unsigned kCuLdsBytes = 160 * 1024;
// Dynamic LDS size for the launch of `kernel`: `want`, less whatever would push the workgroup's total past the
// compute unit's 160 KiB.  The kernel's `__shared__` variables (staging buffers of tile instructions, per-wave slots
// of function-local statics) are part of that total, and a dispatch that asks for more aborts the queue.
inline unsigned LaunchLds(const void *kernel, unsigned want)
{
    hipFuncAttributes attr{};
    if (hipFuncGetAttributes(&attr, kernel) != hipSuccess)
        return want;
    const unsigned fixed = static_cast<unsigned>(attr.sharedSizeBytes);
    if (fixed >= kCuLdsBytes)
        return 0;
    return want + fixed > kCuLdsBytes ? kCuLdsBytes - fixed : want;
}
} // namespace host
} // namespace pto

// ---- pipes and events (global names, as kernel sources use them unqualified) ----
enum pipe_t : int { PIPE_S = 0, PIPE_V, PIPE_M, PIPE_MTE1, PIPE_MTE2, PIPE_MTE3, PIPE_ALL, PIPE_FIX };
enum event_t : int { EVENT_ID0 = 0, EVENT_ID1, EVENT_ID2, EVENT_ID3, EVENT_ID4, EVENT_ID5, EVENT_ID6, EVENT_ID7 };
constexpr int EVENT_ID_MAX = 8;

// set_flag records "everything issued so far on `src`"; in one instruction stream that is implicit.
PTO_DEV void set_flag(pipe_t, pipe_t, event_t) {}

// wait_flag(src, dst): later `dst` work may start once earlier `src` work is complete.
// The forms that order memory across wavefronts (src MTE2; dst MTE2 after MTE1 / V / MTE3 / FIX) contain a workgroup
// barrier: every wave of the workgroup must reach them, so they may not sit under wave-divergent control flow.
PTO_DEV void wait_flag(pipe_t src, pipe_t dst, event_t)
{
    if (src == PIPE_MTE2) {
        // global->LDS copies of every wave must have landed before anyone reads the tile
        pto::hw::wait_vm0();
        pto::hw::lds_barrier();
    } else if (dst == PIPE_MTE2 && (src == PIPE_MTE3 || src == PIPE_FIX)) {
        // a tile that TSTORE wrote to global memory (from a Vec tile: MTE3, from an Acc tile: FIX) is loaded back, possibly
        // by another wave of the workgroup (the reference's global-memory FIFO / workspace pattern): the stores of every
        // wave must have completed and be visible to the workgroup before any wave's load
        pto::hw::wait_vm0();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        pto::hw::lds_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    } else if (dst == PIPE_MTE2 && (src == PIPE_MTE1 || src == PIPE_V)) {
        // every wave must be done reading an LDS tile before a load overwrites it
        pto::hw::lds_barrier();
    } else if (src == PIPE_MTE3 && dst != PIPE_S) {
        pto::hw::wait_vm0();
    }
    // MTE1->M, M->MTE1, M->FIX, FIX->M, V<->M ...: register dependences, nothing to do
}

// kernel sources also pass the event id as a plain integer (pto_macro_matmul.hpp:173: a uint64_t ping-pong index)
template <typename I, std::enable_if_t<std::is_integral<I>::value, int> = 0>
PTO_DEV void set_flag(pipe_t s, pipe_t d, I id)
{
    set_flag(s, d, static_cast<event_t>(id));
}
template <typename I, std::enable_if_t<std::is_integral<I>::value, int> = 0>
PTO_DEV void wait_flag(pipe_t s, pipe_t d, I id)
{
    wait_flag(s, d, static_cast<event_t>(id));
}

// Pipelined form of wait_flag(PIPE_MTE2, PIPE_MTE1, id) for software pipelines that keep several
// TLOADs in flight: returns once all but the `Pending` most recently issued asynchronous copy
// instructions of every wave have landed in LDS (vmcnt retires in order).  Pending is a count of
// wave instructions; pto::TLoadInstrs<Tile>() gives the number one TLOAD issues.
template <int Pending>
PTO_DEV void wait_flag_pending(pipe_t, pipe_t, event_t)
{
    pto::hw::wait_vm<Pending>();
    pto::hw::lds_barrier();
}

PTO_DEV void pipe_barrier(pipe_t p)
{
    if (p == PIPE_ALL) {
        pto::hw::wait_vm0();
        pto::hw::lds_barrier();
    } else if (p == PIPE_MTE2 || p == PIPE_MTE3) {
        pto::hw::wait_vm0();
    }
}

PTO_DEV int64_t get_block_idx() { return static_cast<int64_t>(blockIdx.x); }
PTO_DEV int64_t get_block_num() { return static_cast<int64_t>(gridDim.x); }
PTO_DEV int64_t get_subblockid() { return 0; }
// Address of the scale buffer that belongs to an L0A / L0B address (include/pto/npu/a5/utils.hpp:82-87).  Scale tiles are
// register tiles here and TASSIGN on them binds nothing: any value will do.
template <typename T>
PTO_DEV uint64_t GetScaleAddr(T *) { return 0; }
PTO_DEV int64_t get_subblockdim() { return 1; }
PTO_DEV int64_t get_coreid() { return static_cast<int64_t>(blockIdx.x); }
PTO_DEV int64_t get_sys_cnt() { return static_cast<int64_t>(wall_clock64()); }

// ---- cache maintenance of the Ascend scalar core (the preamble of the reference's tfillpad / tload test kernels:
// tests/npu/a2a3/src/st/testcase/tfillpad/tfillpad_kernel.cpp:124-139): a data barrier, an instruction-cache preload and
// its status.  A wave's own stores are visible to its later loads, and there is no instruction cache to warm by hand.
enum dsb_mode_t { DSB_ALL = 0, DSB_DDR, DSB_UB };
PTO_DEV void dsb(dsb_mode_t) { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup"); }
PTO_DEV void preload(const void *, int64_t) {}
PTO_DEV int64_t get_icache_prl_st() { return 0; }

// ---- cross-core flags of the Cube / Vec kernels (fa_performance_kernel.cpp:617, TPush.hpp:140-160 of the reference) ----
// On Ascend a Cube core and its Vec cores are separate instruction streams that signal each other through FFTS flags.
// Here one workgroup runs both roles in program order, so the producer's code has always run before the consumer's: what
// is left of a signal is "my global-memory stores are complete and visible to the workgroup", of a wait "the workgroup
// has got this far".  Both are reached by every wave (kernel control flow around them is uniform).
PTO_DEV void set_ffts_base_addr(uint64_t) {}
PTO_DEV void ffts_cross_core_sync(pipe_t, uint64_t)
{
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
}
PTO_DEV void wait_flag_dev(int64_t)
{
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// ---- function-local `static` variables of a core (pto_macro_matmul.hpp:58-65, fa_performance_kernel.cpp:263-275) ----
// On Ascend such a variable is private to the core and keeps its value between calls for the length of the kernel.  A GPU
// function cannot hold a `static` in a register; port_ascend_source.py rewrites `static T name = init;` inside device
// functions into PTO_CORE_STATIC(T, name, init, number): `name` becomes a reference to one of 32 eight-byte slots in LDS, private
// to the wave (every wave runs the same scalar program, so each keeps its own copy and no barrier is needed), initialised
// on first use after PTO_KERNEL_PROLOGUE(), which the script puts at the top of every kernel.  Instantiations of one
// template share the slot of the declaration.
namespace pto {
namespace detail {
struct CoreStaticArea {
    uint64_t slot[kBlockWaves][32];
    uint32_t inited[kBlockWaves];
};
PTO_DEV CoreStaticArea &core_static_area()
{
    __shared__ CoreStaticArea area;
    return area;
}
template <typename T, int ID>
PTO_DEV T &core_static(T init)
{
    static_assert(sizeof(T) <= 8 && ID >= 0 && ID < 32, "[PTO][SA] PTO_CORE_STATIC: up to 32 variables of up to 8 bytes");
    CoreStaticArea &a = core_static_area();
    const int w = hw::wave();
    T *p = reinterpret_cast<T *>(&a.slot[w][ID]);
    if (!((a.inited[w] >> ID) & 1u)) {
        *p = init;
        a.inited[w] |= 1u << ID;
    }
    return *p;
}
} // namespace detail
} // namespace pto
#define PTO_KERNEL_PROLOGUE() (pto::detail::core_static_area().inited[pto::hw::wave()] = 0u)
// ID: the variable's number in its translation unit (0 .. 31), which port_ascend_source.py counts itself
#define PTO_CORE_STATIC(T, NAME, INIT, ID) T &NAME = pto::detail::core_static<T, ID>(INIT)
