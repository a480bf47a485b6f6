// TCVT and gather kernels for MI355X, written with PTO tile instructions.  Both are pure
// streaming work (bound by HBM bandwidth): every workgroup moves one Vec tile
//   TLOAD (16-byte coalesced loads into registers) -> TCVT / MGATHER -> TSTORE (16-byte stores).
// Test kernels of the same shape in the reference: tests/cpu/st/testcase/tcvt/tcvt_kernel.cpp:18-52,
// tests/cpu/st/testcase/tgather/tgather_kernel.cpp, tests/cpu/st/testcase/mgather/.
// The outputs of these kernels are written once and not read again by them: non-temporal stores keep them from pushing
// the data still to be read out of the caches (measured: conversion +2.6 %, row gather +12 %; non-temporal loads of the
// conversion's input +1.3 % alone, nothing on top of the stores, and -6 % for the gather, whose table is re-read).
#define PTO_VEC_STREAM_NT 2
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kCvtTile = 8192; // elements per workgroup: 4 chunks of 8 per lane

template <typename D, bool kTail>
__global__ __launch_bounds__(kBlockThreads) AICORE void CvtF32(__gm__ D *dst, __gm__ const float *src, size_t n,
                                                               size_t firstTile, int mode)
{
    const size_t tile = firstTile + get_block_idx();
    const size_t base = tile * (size_t)kCvtTile;
    using Shape1 = Shape<1, 1, 1, 1, DYNAMIC>;
    using Stride1 = Stride<1, 1, 1, DYNAMIC, 1>;
    using GSrc = GlobalTensor<float, Shape1, Stride1>;
    using GDst = GlobalTensor<D, Shape1, Stride1>;
    constexpr int VC = kTail ? DYNAMIC : kCvtTile;
    using TileSrc = Tile<TileType::Vec, float, 1, kCvtTile, BLayout::RowMajor, 1, VC>;
    using TileDst = Tile<TileType::Vec, D, 1, kCvtTile, BLayout::RowMajor, 1, VC>;
    const int valid = kTail ? (int)(n - base) : kCvtTile;
    auto mk = [&](auto tag) {
        using T = decltype(tag);
        if constexpr (kTail)
            return T((size_t)valid);
        else
            return T();
    };
    TileSrc srcTile = mk(TileSrc());
    TileDst dstTile = mk(TileDst());
    GSrc srcGlobal(const_cast<float *>(src) + base, Shape1(valid), Stride1(valid));
    GDst dstGlobal(dst + base, Shape1(valid), Stride1(valid));
    TLOAD(srcTile, srcGlobal);
    set_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    TCVT(dstTile, srcTile, static_cast<RoundMode>(mode));
    set_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    wait_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    TSTORE(dstGlobal, dstTile);
}

// Whole tiles in the default rounding mode take a streaming form of the same conversion below the tile instructions:
// a lane loads 16 bytes and stores 8, so that every load instruction of a wave covers 1 KiB of consecutive addresses and
// every store 512 bytes (a Vec tile gives a lane eight consecutive elements, i.e. two loads 32 bytes apart per lane and
// half-used lines per instruction), all eight loads of a lane are in flight before the first conversion, and there is
// no barrier; the stores are non-temporal (measured with inputs and outputs that no cache holds: 6.5 against 6.2 TB/s
// with plain stores).  Same element function as TCVT (detail::convert), so the results are the same bits.
template <typename D>
__global__ __launch_bounds__(kBlockThreads) void CvtF32Stream(D *dst, const float *src, size_t firstTile)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    constexpr int kPerStep = kBlockThreads * 4, kSteps = kCvtTile / kPerStep;
    static_assert(kCvtTile % kPerStep == 0 && sizeof(D) == 2, "whole steps of 16-bit results");
    const size_t base = (firstTile + blockIdx.x) * (size_t)kCvtTile + 4 * threadIdx.x;
    f32x4 x[kSteps];
#pragma unroll
    for (int i = 0; i < kSteps; ++i)
        x[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + base + (size_t)i * kPerStep));
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        u16x4 y;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            y[j] = __builtin_bit_cast(uint16_t, ::pto::detail::convert<D, float>(x[i][j], RoundMode::CAST_RINT));
        __builtin_nontemporal_store(y, reinterpret_cast<u16x4 *>(dst + base + (size_t)i * kPerStep));
    }
}

constexpr int kGatherRows = 32, kGatherCols = 256; // one Vec tile: 8192 elements

template <typename T, bool kTailCols>
__global__ __launch_bounds__(kBlockThreads) AICORE void GatherRows(__gm__ T *out, __gm__ const T *table,
                                                                   __gm__ const int32_t *idx, int nIdx, int tableRows,
                                                                   int cols, int colBlocks)
{
    const int rb = (int)(get_block_idx() / colBlocks), cb = (int)(get_block_idx() % colBlocks);
    const int row0 = rb * kGatherRows, col0 = cb * kGatherCols;
    const int vRows = nIdx - row0 < kGatherRows ? nIdx - row0 : kGatherRows;
    const int vCols = cols - col0 < kGatherCols ? cols - col0 : kGatherCols;
    using IdxTile = Tile<TileType::Vec, int32_t, kGatherRows, 1, BLayout::ColMajor, DYNAMIC, 1>;
    using DstTile = Tile<TileType::Vec, T, kGatherRows, kGatherCols, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    using GIdx = GlobalTensor<int32_t, Shape<1, 1, 1, DYNAMIC, 1>, Stride<1, 1, 1, 1, DYNAMIC>, Layout::DN>;
    using GTab = GlobalTensor<T, Shape<1, 1, 1, DYNAMIC, DYNAMIC>, Stride<1, 1, 1, DYNAMIC, 1>>;
    IdxTile idxTile((size_t)vRows);
    DstTile dstTile((size_t)vRows, (size_t)vCols);
    GIdx idxGlobal(const_cast<int32_t *>(idx) + row0, Shape<1, 1, 1, DYNAMIC, 1>(vRows), Stride<1, 1, 1, 1, DYNAMIC>(vRows));
    GTab tableGlobal(const_cast<T *>(table) + col0, Shape<1, 1, 1, DYNAMIC, DYNAMIC>(tableRows, vCols),
                     Stride<1, 1, 1, DYNAMIC, 1>(cols));
    GTab outGlobal(out + (int64_t)row0 * cols + col0, Shape<1, 1, 1, DYNAMIC, DYNAMIC>(vRows, vCols),
                   Stride<1, 1, 1, DYNAMIC, 1>(cols));
    TLOAD(idxTile, idxGlobal);
    MGATHER_ROWS(dstTile, tableGlobal, idxTile, tableRows);
    set_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    wait_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    TSTORE(outGlobal, dstTile);
}

// One-tile TGATHER (index form), the half 16x1024 -> 16x128 case of the reference's tgather test.
__global__ __launch_bounds__(kBlockThreads) AICORE void TGatherIndex16x1024(__gm__ half *dst, __gm__ const half *src0,
                                                                            __gm__ const int32_t *idx)
{
    using Src0Tile = Tile<TileType::Vec, half, 16, 1024, BLayout::RowMajor>;
    using IdxTile = Tile<TileType::Vec, int32_t, 16, 128, BLayout::RowMajor>;
    using DstTile = Tile<TileType::Vec, half, 16, 128, BLayout::RowMajor>;
    using G0 = GlobalTensor<half, Shape<1, 1, 1, 16, 1024>, Stride<16384, 16384, 16384, 1024, 1>>;
    using GI = GlobalTensor<int32_t, Shape<1, 1, 1, 16, 128>, Stride<2048, 2048, 2048, 128, 1>>;
    using GD = GlobalTensor<half, Shape<1, 1, 1, 16, 128>, Stride<2048, 2048, 2048, 128, 1>>;
    Src0Tile s0;
    IdxTile ti;
    DstTile td;
    G0 g0(const_cast<half *>(src0));
    GI gi(const_cast<int32_t *>(idx));
    GD gd(dst);
    TLOAD(s0, g0);
    TLOAD(ti, gi);
    TGATHER(td, s0, ti);
    TSTORE(gd, td);
}

} // namespace

PTO_DEVICE_CODE_END

namespace {
template <typename D>
int launch_cvt(void *stream, D *dst, const float *src, size_t n, int mode)
{
    if (!dst || !src)
        return n == 0 ? PTO_OK : PTO_ERR_BAD_ARG;
    if (mode < PTO_CAST_RINT || mode > PTO_CAST_ODD)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t full = n / kCvtTile, tail = n % kCvtTile;
    // (the streaming kernel for buffers aligned to its accesses: 16-byte loads, 8-byte stores)
    const bool aligned = reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 8 == 0;
    // the grid's x extent is limited to 2^31-1 blocks; stay far below it per launch
    constexpr size_t kMaxBlocks = 1u << 30;
    for (size_t t0 = 0; t0 < full; t0 += kMaxBlocks) {
        const size_t nb = full - t0 < kMaxBlocks ? full - t0 : kMaxBlocks;
        if (mode == PTO_CAST_RINT && aligned)
            CvtF32Stream<D><<<dim3((unsigned)nb), dim3(kBlockThreads), 0, st>>>(dst, src, t0);
        else
            CvtF32<D, false><<<dim3((unsigned)nb), dim3(kBlockThreads), 0, st>>>(dst, src, n, t0, mode);
    }
    if (tail)
        CvtF32<D, true><<<dim3(1), dim3(kBlockThreads), 0, st>>>(dst, src, n, full, mode);
    return pto_amd::check_launch();
}
} // namespace

extern "C" int pto_tcvt_f32_f16(void *stream, uint16_t *dst, const float *src, size_t n, int round_mode)
{
    return launch_cvt(stream, reinterpret_cast<half *>(dst), src, n, round_mode);
}

extern "C" int pto_tcvt_f32_bf16(void *stream, uint16_t *dst, const float *src, size_t n, int round_mode)
{
    if (round_mode != PTO_CAST_RINT)
        return PTO_ERR_UNSUPPORTED;
    return launch_cvt(stream, reinterpret_cast<bfloat16_t *>(dst), src, n, round_mode);
}

extern "C" int pto_gather_rows(void *stream, void *out, const void *table, const int32_t *idx, size_t n_idx,
                               size_t table_rows, size_t cols, int elem_bytes)
{
    if (n_idx == 0 || cols == 0)
        return PTO_OK;
    if (!out || !table || !idx || table_rows == 0)
        return PTO_ERR_BAD_ARG;
    if (elem_bytes != 2 && elem_bytes != 4)
        return PTO_ERR_BAD_ARG;
    if (cols % 8 || n_idx > 0x7fffffffu || table_rows > 0x7fffffffu || cols > 0x7fffffffu)
        return PTO_ERR_UNSUPPORTED;
    const size_t rowBlocks = (n_idx + kGatherRows - 1) / kGatherRows, colBlocks = (cols + kGatherCols - 1) / kGatherCols;
    if (rowBlocks * colBlocks > 0x7fffffffu)
        return PTO_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)(rowBlocks * colBlocks)), block(kBlockThreads);
    if (elem_bytes == 2)
        GatherRows<uint16_t, true><<<grid, block, 0, st>>>(static_cast<uint16_t *>(out), static_cast<const uint16_t *>(table),
                                                           idx, (int)n_idx, (int)table_rows, (int)cols, (int)colBlocks);
    else
        GatherRows<uint32_t, true><<<grid, block, 0, st>>>(static_cast<uint32_t *>(out), static_cast<const uint32_t *>(table),
                                                           idx, (int)n_idx, (int)table_rows, (int)cols, (int)colBlocks);
    return pto_amd::check_launch();
}

extern "C" int pto_tgather_index_f16_16x1024_16x128(void *stream, uint16_t *dst, const uint16_t *src0, const int32_t *idx)
{
    if (!dst || !src0 || !idx)
        return PTO_ERR_BAD_ARG;
    TGatherIndex16x1024<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<half *>(dst), reinterpret_cast<const half *>(src0), idx);
    return pto_amd::check_launch();
}
