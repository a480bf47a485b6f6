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

namespace detail {
// stores of every wave complete and visible to the workgroup, then a barrier
PTO_DEV void UbSyncPoint()
{
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
// Vec tiles kept in memory (PTO_VEC_TILES_IN_MEMORY): registers <- unified buffer, unified buffer <- registers + sync
template <typename TileT>
PTO_DEV void UbFetchTile(TileT &t)
{
#if defined(PTO_VEC_TILES_IN_MEMORY)
    if constexpr (TileT::inMemory) {
        if (t.mem_ != nullptr) {
            const typename TileT::DType *p = t.mem_;
            const int vr = t.GetValidRow(), vc = t.GetValidCol();
            for_each_owned<TileT>([&](int s, int i, int e) {
                int r, c;
                elem_rc<TileT>(e, r, c);
                if (e < TileT::Numel && r < vr && c < vc)
                    t.S().v[s][i] = p[e];
            });
        }
    } else if constexpr (TileT::accInMemory) { // the whole [Rows, Cols] image, row-major
        if (t.mem_ != nullptr) {
            using T = typename TileT::DType;
            const T *p = t.mem_;
            for_each_elem(t, [&](int r, int c, T, bool) { return p[r * TileT::Cols + c]; });
        }
    }
#else
    (void)t;
#endif
}
// after a TLOAD: the valid region and, as the NPU's copy into the unified buffer does, the pad value up to the end of the
// last 32-byte block of every valid row (column, for a column-major tile): what another tile object at the same address
// then finds there (tests/npu/a2a3/src/st/testcase/tload/tload_kernel.cpp:121-150 stores through such a second tile)
template <typename TileT>
PTO_DEV void UbCommitLoaded(TileT &t)
{
#if defined(PTO_VEC_TILES_IN_MEMORY)
    if constexpr (TileT::inMemory) {
        if (t.mem_ != nullptr) {
            typename TileT::DType *p = t.mem_;
            constexpr int kBlock = 32 / (int)sizeof(typename TileT::DType) > 0 ? 32 / (int)sizeof(typename TileT::DType) : 1;
            const int vr = t.GetValidRow(), vc = t.GetValidCol();
            const int pr = TileT::isRowMajor ? vr : (vr + kBlock - 1) / kBlock * kBlock, pc = TileT::isRowMajor ? (vc + kBlock - 1) / kBlock * kBlock : vc;
            for_each_owned<TileT>([&](int s, int i, int e) {
                int r, c;
                elem_rc<TileT>(e, r, c);
                if (e < TileT::Numel && r < pr && c < pc)
                    p[e] = t.S().v[s][i];
            });
        }
        UbSyncPoint();
    }
#else
    (void)t;
#endif
}
template <typename TileT>
PTO_DEV void UbCommitTile(TileT &t)
{
#if defined(PTO_VEC_TILES_IN_MEMORY)
    if constexpr (TileT::inMemory) {
        if (t.mem_ != nullptr) {
            typename TileT::DType *p = t.mem_;
            const int vr = t.GetValidRow(), vc = t.GetValidCol();
            for_each_owned<TileT>([&](int s, int i, int e) {
                int r, c;
                elem_rc<TileT>(e, r, c);
                if (e < TileT::Numel && r < vr && c < vc)
                    p[e] = t.S().v[s][i];
            });
        }
        UbSyncPoint();
    } else if constexpr (TileT::accInMemory) {
        if (t.mem_ != nullptr) {
            using T = typename TileT::DType;
            T *p = t.mem_;
            for_each_elem(t, [&](int r, int c, T v, bool owner) {
                if (owner)
                    p[r * TileT::Cols + c] = v;
                return v;
            });
            UbSyncPoint();
        }
    }
#else
    (void)t;
#endif
}
} // namespace detail

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

// ---------------------------------------------------------------------------------------------------------------
// TPipe: the struct form of the hand-off (npu/a2a3/TPush.hpp:60-335 of the reference): one type names the FIFO, its
// producer and its consumer; the kernel sets tile ids, entry offsets and the allocate / record / wait / free switches on
// the two ends and calls TPUSH(prod, tile, fifo) / TPOP(cons, tile, fifo) (fa_performance_kernel.cpp:339-345, 401-407).
// The slot layout in global memory is the reference's, so a workspace sized by its host code fits:
//   Acc  -> FIFO  slot = tile_id % Depth, kTileFactor = ConsCols / ProdCols sub-tiles per slot, each a dense row-major
//                 [ProdRows, ProdCols] image at slot * kTileFactor * ProdRows * ProdCols + entryOffset bytes;
//   FIFO -> Vec   the consumer tile [ConsRows, ConsCols] gathers its column blocks from the kTileFactor sub-tile images;
//   Vec  -> FIFO  the producer tile [ProdRows, ProdCols] scatters its column blocks of ConsCols columns into dense
//                 [ConsRows, ConsCols] images (rows at entryOffset);
//   FIFO -> Mat   TLOAD of the dense [ConsRows, ConsCols] image.
// Cross-core flags: record() = this workgroup's stores are complete and visible + barrier; wait() = the same barrier;
// allocate() / free() = nothing (the consumer ran earlier in program order).
template <uint8_t FlagID, FIFOType FiFoType, uint8_t FiFoDepth, uint8_t FiFoSyncT, typename TileDataProd, typename TileDataCons,
          TSyncOpType ProducerOp, TSyncOpType ConsumerOp, VecCubeRatio VCRatio = VecCubeRatio::V2C1_VECS>
struct TPipe {
    static_assert(ConsumerOp == TSyncOpType::TLOAD, "[PTO][SA] TPipe: the consumer operation is TLOAD");
    static_assert(FiFoType == FIFOType::GM_FIFO, "[PTO][SA] TPipe: global-memory FIFOs (the LDS FIFOs use TFIFOSync)");
    using DataFiFo = DataFIFO<typename TileDataCons::DType, FiFoType, FiFoDepth, FiFoSyncT>;
    static constexpr bool is_c2v = TileDataProd::Loc == TileType::Acc;
    static constexpr bool is_v2c = TileDataProd::Loc == TileType::Vec;

    struct Producer {
        static constexpr bool isTPipeEnd = true;
        int tile_id = -1, sub_tile_id = -1, entryOffset = 0;
        bool isAllocate = false, isRecord = false;
        PTO_HD void setTileId(int t, int sub) { tile_id = t; sub_tile_id = sub; }
        PTO_HD int getTileId() const { return tile_id; }
        PTO_HD int getSubTileId() const { return sub_tile_id; }
        PTO_HD void setAllocateStatus(bool v) { isAllocate = v; }
        PTO_HD bool getAllocateStatus() const { return isAllocate; }
        PTO_HD void setRecordStatus(bool v) { isRecord = v; }
        PTO_HD bool getRecordStatus() const { return isRecord; }
        PTO_HD void setEntryOffset(int off) { entryOffset = off; }
        PTO_DEV void allocate() const {}
        PTO_DEV void record() const { detail::UbSyncPoint(); }
        PTO_DEV void push(DataFiFo &fifo, TileDataProd &tile)
        {
            using T = typename TileDataProd::DType;
            constexpr int ProdM = TileDataProd::Rows, ProdN = TileDataProd::Cols, ConsM = TileDataCons::Rows, ConsN = TileDataCons::Cols;
            const uint32_t slot = (uint32_t)(tile_id % DataFiFo::fifoDepth);
            if constexpr (TileDataProd::Loc == TileType::Acc) {
                constexpr int kTileFactor = ConsN / ProdN;
                const size_t entryBase = (size_t)slot * kTileFactor * ProdM * ProdN * sizeof(T);
                using G = GlobalTensor<T, Shape<1, 1, 1, ProdM, ProdN>, Stride<1, 1, 1, ProdN, 1>>;
                G gt(reinterpret_cast<T *>(reinterpret_cast<char *>(fifo.fifoBase) + entryBase + entryOffset));
                TSTORE_IMPL<TileDataProd, G, AtomicType::AtomicNone>(gt, tile);
            } else {
                static_assert(TileDataProd::Loc == TileType::Vec && TileDataProd::isRowMajor, "[PTO][SA] TPUSH: Acc or row-major Vec tile");
                static_assert(ProdN % ConsN == 0, "[PTO][SA] TPUSH: the producer tile is a whole number of consumer tiles wide");
                constexpr int kTileFactor = ProdN / ConsN;
                const size_t entryBase = (size_t)slot * kTileFactor * ConsM * ConsN * sizeof(T);
                T *dst = reinterpret_cast<T *>(reinterpret_cast<char *>(fifo.fifoBase) + entryBase + entryOffset);
                detail::UbFetchTile(tile);
                detail::for_each_owned<TileDataProd>([&](int s, int i, int e) {
                    if (e < TileDataProd::Numel) {
                        const int r = e / ProdN, c = e % ProdN;
                        dst[(size_t)(c / ConsN) * ConsM * ConsN + (size_t)r * ConsN + c % ConsN] = tile.S().v[s][i];
                    }
                });
            }
        }
    };

    struct Consumer {
        static constexpr bool isTPipeEnd = true;
        int tile_id = -1, sub_tile_id = -1, entryOffset = 0;
        bool isWait = false, isFree = false;
        PTO_HD void setTileId(int t, int sub) { tile_id = t; sub_tile_id = sub; }
        PTO_HD int getTileId() const { return tile_id; }
        PTO_HD int getSubTileId() const { return sub_tile_id; }
        PTO_HD void setEntryOffset(int off) { entryOffset = off; }
        PTO_HD void setWaitStatus(bool v) { isWait = v; }
        PTO_HD bool getWaitStatus() const { return isWait; }
        PTO_HD void setFreeStatus(bool v) { isFree = v; }
        PTO_HD bool getFreeStatus() const { return isFree; }
        PTO_DEV void wait() const { detail::UbSyncPoint(); }
        PTO_DEV void free() const {}
        PTO_DEV void pop(DataFiFo &fifo, TileDataCons &tile)
        {
            using T = typename TileDataCons::DType;
            constexpr int ProdM = TileDataProd::Rows, ProdN = TileDataProd::Cols, ConsM = TileDataCons::Rows, ConsN = TileDataCons::Cols;
            const uint32_t slot = (uint32_t)(tile_id % DataFiFo::fifoDepth);
            if constexpr (TileDataCons::Loc == TileType::Vec) {
                static_assert(TileDataCons::isRowMajor && ConsN % ProdN == 0, "[PTO][SA] TPOP: row-major Vec tile, a whole number of producer tiles wide");
                constexpr int kTileFactor = ConsN / ProdN;
                const size_t entryBase = (size_t)slot * kTileFactor * ProdM * ProdN * sizeof(T);
                const T *src = reinterpret_cast<const T *>(reinterpret_cast<const char *>(fifo.fifoBase) + entryBase + entryOffset);
                detail::for_each_owned<TileDataCons>([&](int s, int i, int e) {
                    if (e < TileDataCons::Numel) {
                        const int r = e / ConsN, c = e % ConsN;
                        tile.S().v[s][i] = src[(size_t)(c / ProdN) * ProdM * ProdN + (size_t)r * ProdN + c % ProdN];
                    }
                });
                detail::UbCommitTile(tile);
            } else {
                static_assert(TileDataCons::Loc == TileType::Mat, "[PTO][SA] TPOP: Vec or Mat tile");
                const size_t entryBase = (size_t)slot * ConsM * ProdN * sizeof(T);
                using G = GlobalTensor<T, Shape<1, 1, 1, ConsM, ConsN>, Stride<1, 1, 1, ConsN, 1>>;
                G gt(reinterpret_cast<T *>(reinterpret_cast<char *>(fifo.fifoBase) + entryBase + entryOffset));
                TLOAD_IMPL(tile, gt); // asynchronous: the kernel orders it with set_flag / wait_flag(PIPE_MTE2, PIPE_MTE1)
            }
        }
    };

    DataFiFo fifo;
    Producer prod;
    Consumer cons;
    PTO_HD explicit TPipe(typename TileDataCons::DType *fifoBase) : fifo(fifoBase), prod(), cons() {}
};

namespace detail {
template <typename T, typename = void>
struct is_tpipe_end : std::false_type {};
template <typename T>
struct is_tpipe_end<T, std::enable_if_t<T::isTPipeEnd>> : std::true_type {};
} // namespace detail

template <typename PipeProd, typename TileData, typename DataFifoT>
PTO_DEV void TPUSH_IMPL(PipeProd &prod, TileData &tile, DataFifoT &fifo)
{
    using T = typename DataFifoT::DType;
    if constexpr (detail::is_tpipe_end<PipeProd>::value) { // TPush.hpp:356-374: allocate, store, record, each as switched on
        if (prod.getAllocateStatus())
            prod.allocate();
        prod.push(fifo, tile);
        if (prod.getRecordStatus())
            prod.record();
        return;
    } else {
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
}
template <typename TileData, typename Pipe>
PTO_DEV void TPUSH_IMPL(TileData &tile, Pipe &pipe)
{
    TPUSH_IMPL(pipe.prod, tile, pipe.fifo);
}

template <typename PipeCons, typename TileData, typename DataFifoT>
PTO_DEV void TPOP_IMPL(PipeCons &cons, TileData &tile, DataFifoT &fifo)
{
    using T = typename DataFifoT::DType;
    if constexpr (detail::is_tpipe_end<PipeCons>::value) { // TPop.hpp:26-58: wait, load, free, each as switched on
        if (cons.getWaitStatus())
            cons.wait();
        cons.pop(fifo, tile);
        if (cons.getFreeStatus())
            cons.free();
        return;
    } else {
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
}
template <typename TileData, typename Pipe>
PTO_DEV void TPOP_IMPL(TileData &tile, Pipe &pipe)
{
    TPOP_IMPL(pipe.cons, tile, pipe.fifo);
}
// TFREE (pto_instr.hpp:1465-1471 of the reference): release the slot that the consumer holds
template <typename Pipe>
PTO_DEV void TFREE_IMPL(Pipe &pipe)
{
    pipe.cons.free();
}

} // namespace pto
