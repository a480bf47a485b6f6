// The unified buffer of translation units that keep their Vec tiles in memory (PTO_VEC_TILES_IN_MEMORY, see
// pto/common/tile.hpp): PTO_UB_BYTES of global memory per workgroup, the address space that TASSIGN of a Vec tile names
// (the reference's kernels place their Vec tiles at byte offsets of the 192 KiB unified buffer of a vector core:
// fa_performance_kernel.cpp:215-262).
//
// The arena is one device allocation, `blocks * PTO_UB_BYTES` bytes, made by pto::host::PrepareUnifiedBuffer before a
// launch (port_ascend_source.py puts the call in front of every launch statement); the kernels of the translation unit
// find it through a device variable.  Launches of one translation unit that overlap in time share the arena: keep them on
// one stream.  Host threads may call concurrently (one lock around the bookkeeping); when the arena has to grow, the
// whole device is synchronised before the old one is freed, whichever streams still use it.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <mutex>

#ifndef PTO_UB_BYTES
#define PTO_UB_BYTES (512 * 1024)
#endif
// Acc tiles that were given an address keep their image in the upper part of the same arena: address a of the
// accumulator memory is byte PTO_ACC_ARENA_OFFSET + a of the workgroup's unified buffer
#ifndef PTO_ACC_ARENA_OFFSET
#define PTO_ACC_ARENA_OFFSET (256 * 1024)
#endif

namespace pto {
namespace detail {
// one copy per translation unit: set by PrepareUnifiedBuffer of the same translation unit
static __device__ char *g_ub_arena;

__device__ __forceinline__ char *ub_base()
{
    return g_ub_arena + (size_t)blockIdx.x * (size_t)PTO_UB_BYTES;
}
} // namespace detail

namespace host {
// Makes sure that the arena holds `blocks` unified buffers and that the kernels of this translation unit see it.
// Returns hipSuccess or the first HIP error.  The arena only grows and is kept until the process ends.
inline hipError_t PrepareUnifiedBuffer(unsigned blocks, hipStream_t stream)
{
    static std::mutex lock;
    static char *arena = nullptr;
    static size_t capacity = 0;
    const std::lock_guard<std::mutex> guard(lock);
    const size_t need = (size_t)blocks * (size_t)PTO_UB_BYTES;
    hipError_t e = hipSuccess;
    if (need > capacity) {
        if (arena) {
            e = hipDeviceSynchronize();
            if (e == hipSuccess)
                e = hipFree(arena);
            if (e != hipSuccess)
                return e;
            arena = nullptr;
            capacity = 0;
        }
        e = hipMalloc(reinterpret_cast<void **>(&arena), need);
        if (e != hipSuccess)
            return e;
        capacity = need;
        e = hipMemsetAsync(arena, 0, need, stream);
        if (e != hipSuccess)
            return e;
    }
    return hipMemcpyToSymbolAsync(HIP_SYMBOL(detail::g_ub_arena), &arena, sizeof(arena), 0, hipMemcpyHostToDevice, stream);
}
// For launch configurations: `kernel<<<LaunchBlocks(blocks, stream), threads, lds, stream>>>(...)` prepares the unified
// buffer for `blocks` workgroups and hands `blocks` on.  A failure shows as the launch's own error (0 blocks).
inline unsigned LaunchBlocks(unsigned blocks, hipStream_t stream)
{
    return PrepareUnifiedBuffer(blocks, stream) == hipSuccess ? blocks : 0u;
}
} // namespace host
} // namespace pto
