// TPUSH / TPOP: tile hand-off through a ring of slots (reference: include/pto/common/fifo.hpp:18-84,
// include/pto/cpu/TPush.hpp:19-141, TPop.hpp:19-52, npu/a2a3/TPush.hpp:60-260).
//
// On Ascend the producer and the consumer are different cores (Cube and Vec) that exchange tiles through
// a global-memory FIFO and cross-core flags.  A CDNA4 workgroup does both kinds of work itself, so here the
// producer and the consumer are the SAME workgroup at two points of its program:
//   TPUSH(prod, tile, fifo)  stores the tile into slot prod.tile_id % Depth and advances the producer,
//   TPOP(cons, tile, fifo)   waits until that store is visible to the whole workgroup, loads the slot into
//                            `tile` (which may have another location or distribution than the pushed tile:
//                            Acc -> Vec, Vec -> Mat ...) and advances the consumer.
// FIFOType::GM_FIFO keeps the slots in global memory (drop-in for the reference's FIFOs: slot i is a dense
// row-major [Rows, Cols] image at fifoBase + i * Numel).  FIFOType::VEC_FIFO / MAT_FIFO keep them in LDS
// (byte offset into the workgroup's dynamic LDS), the native form of the hand-off: nothing leaves the CU.
// Depth bounds how many pushed tiles may be outstanding; as both ends run in program order, an overrun is a
// programming error of the kernel, not a run-time wait.
#pragma once
#include "pto/gfx950/mem_ops.hpp"
#include "pto/gfx950/vec_ops.hpp"

namespace pto {

enum class FIFOType : uint8_t { GM_FIFO = 0, VEC_FIFO = 1, MAT_FIFO = 2 };
enum class VecCubeRatio : uint8_t { V1C1_VEC0 = 0, V1C1_VEC1 = 1, V2C1_VECS = 2 };

template <typename DataType, FIFOType FifoType, int Depth, int Period>
struct DataFIFO {
    static constexpr int fifoDepth = Depth;
    static constexpr int fifoPeriod = Period;
    static constexpr FIFOType fifoType = FifoType;
    using DType = DataType;
    DataType *fifoBase = nullptr; // GM_FIFO: global pointer
    uint32_t ldsBase = 0;         // VEC_FIFO / MAT_FIFO: byte offset into the dynamic LDS
    PTO_HD DataFIFO(DataType *ptr) : fifoBase(ptr) {}
    PTO_HD DataFIFO(uint32_t ldsOffset, int) : ldsBase(ldsOffset) {}
    PTO_HD DataType *getBasePtr() { return fifoBase; }
};

enum class TSyncOpType : uint8_t { TSTORE_C2GM, TSTORE_V2GM, TMOV_C2UB, TINSERT_V2L1, TLOAD, TSTORE_C2GM_UFON = TSTORE_C2GM, TSTORE_C2GM_UFOFF = TSTORE_C2GM };

template <uint16_t FlagID, typename DataFifoT, TSyncOpType ProducerOp, TSyncOpType ConsumerOp>
struct TFIFOSync {
    static_assert(ConsumerOp == TSyncOpType::TLOAD, "[PTO][SA] TFIFOSync: the consumer operation is TLOAD");
    static constexpr int fifoSize = DataFifoT::fifoDepth;
    static constexpr int syncPeriod = DataFifoT::fifoPeriod;
    struct Producer {
        int tile_id = 0;
        PTO_HD void set_tile_id(int t, int) { tile_id = t; }
        PTO_HD int get_tile_id() const { return tile_id; }
        PTO_HD void allocate() {} // the slot is free: the consumer ran earlier in program order
        PTO_HD void record() { tile_id = (tile_id + 1) % fifoSize; }
    };
    struct Consumer {
        int tile_id = 0;
        PTO_HD void set_tile_id(int t, int) { tile_id = t; }
        PTO_HD int get_tile_id() const { return tile_id; }
        // the pushed data become visible to every wave of the workgroup: outstanding stores drain, then a barrier
        PTO_DEV void wait()
        {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        PTO_HD void free() { tile_id = (tile_id + 1) % fifoSize; }
    };
};

namespace detail {
// dense row-major [Rows, Cols] image of a register tile in LDS at byte offset `off`
template <typename TileT, typename T>
PTO_DEV void lds_image_store(uint32_t off, TileT &tile)
{
    T *img = reinterpret_cast<T *>(hw::lds_base() + off);
    if constexpr (TileT::Loc == TileType::Acc) {
        using S = typename TileT::Storage;
        const uint32_t lane = (uint32_t)hw::lane();
        const int rbase = hw::wave_m() * (S::MB * kMfmaM) + acc_lane_row(lane);
        const int cbase = hw::wave_n() * (S::NB * kMfmaM) + acc_lane_col(lane);
#pragma unroll
        for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
                for (int v = 0; v < kAccElems; ++v) {
                    const int r = rbase + mb * kMfmaM + acc_elem_row(v), c = cbase + nb * kMfmaM;
                    img[r * TileT::Cols + c] = store_cast<T>(tile.S().f[mb][nb][v]);
                }
    } else {
        static_assert(TileT::Loc == TileType::Vec && TileT::isRowMajor, "[PTO][SA] TPUSH to an LDS FIFO: Acc or row-major Vec tile");
        for_each_owned<TileT>([&](int s, int i, int e) {
            if (e < TileT::Numel)
                img[e] = (T)tile.S().v[s][i];
        });
    }
}
template <typename TileT, typename T>
PTO_DEV void lds_image_load(TileT &tile, uint32_t off)
{
    static_assert(TileT::Loc == TileType::Vec && TileT::isRowMajor, "[PTO][SA] TPOP from an LDS FIFO: row-major Vec tile");
    const T *img = reinterpret_cast<const T *>(hw::lds_base() + off);
    for_each_owned<TileT>([&](int s, int i, int e) {
        if (e < TileT::Numel)
            tile.S().v[s][i] = (typename TileT::DType)img[e];
    });
}
} // namespace detail

template <typename PipeProd, typename TileData, typename DataFifoT>
PTO_DEV void TPUSH_IMPL(PipeProd &prod, TileData &tile, DataFifoT &fifo)
{
    using T = typename DataFifoT::DType;
    prod.allocate();
    const int slot = prod.get_tile_id() % DataFifoT::fifoDepth;
    if constexpr (DataFifoT::fifoType == FIFOType::GM_FIFO) {
        using G = GlobalTensor<T, Shape<1, 1, 1, TileData::Rows, TileData::Cols>,
                               Stride<TileData::Numel, TileData::Numel, TileData::Numel, TileData::Cols, 1>>;
        G gt(fifo.getBasePtr() + (size_t)TileData::Numel * slot);
        TSTORE_IMPL<TileData, G, AtomicType::AtomicNone>(gt, tile);
    } else {
        detail::lds_image_store<TileData, T>(fifo.ldsBase + (uint32_t)(slot * TileData::Numel * sizeof(T)), tile);
    }
    prod.record();
}

template <typename PipeCons, typename TileData, typename DataFifoT>
PTO_DEV void TPOP_IMPL(PipeCons &cons, TileData &tile, DataFifoT &fifo)
{
    using T = typename DataFifoT::DType;
    cons.wait();
    const int slot = cons.get_tile_id() % DataFifoT::fifoDepth;
    if constexpr (DataFifoT::fifoType == FIFOType::GM_FIFO) {
        using G = GlobalTensor<T, Shape<1, 1, 1, TileData::Rows, TileData::Cols>,
                               Stride<TileData::Numel, TileData::Numel, TileData::Numel, TileData::Cols, 1>>;
        G gt(fifo.getBasePtr() + (size_t)TileData::Numel * slot);
        TLOAD_IMPL(tile, gt);
        if constexpr (TileData::Loc == TileType::Mat) { // the asynchronous copy has landed for every wave
            set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID7);
            wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID7);
        }
    } else {
        detail::lds_image_load<TileData, T>(tile, fifo.ldsBase + (uint32_t)(slot * TileData::Numel * sizeof(T)));
        hw::lds_barrier(); // the slot may be pushed again
    }
    cons.free();
}

} // namespace pto
