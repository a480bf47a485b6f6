// TASSIGN / TLOAD / TSTORE / TEXTRACT / TMOV for gfx950.
//
// Reference semantics: include/pto/cpu/TLoad.hpp:143-162, TStore.hpp:121-150, TExtract.hpp:17-50
// (window form per docs/isa/TEXTRACT.md:14-18), TMov.hpp:20-51, TAssign.hpp:17-29.  A tile's
// logical content tile(r,c) <-> gm[r*stride3 + c*stride4] is what is preserved; the physical
// placement is the one described in common/tile.hpp.
//
// Mat tile LDS image.  Let `major` index the non-contiguous logical dimension and k the
// contiguous one (k = column for an Nz tile, row for a Zn tile), RowBytes = extent_k * sizeof(T) (extent_k / 2 for 4-bit elements).
// Element (major, k) lives at   major*RowBytes + ((chunk ^ swz(major)) << 4) + (k*sizeof(T) & 15),
// chunk = k*sizeof(T) >> 4.  swz() spreads consecutive `major` values at the same logical chunk over the
// 16-byte bank groups so that the ds_read_b128 fragment reads are conflict free (checked with the LDS
// bank-conflict counter and with read-rate probes), and the 1 KiB-contiguous write pattern of
// global_load_lds_dwordx4 is conflict free by construction.
#pragma once
#include "pto/common/global_tensor.hpp"
#include "pto/common/tile.hpp"

namespace pto {
namespace detail {

constexpr bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

template <int RowBytes>
PTO_DEV constexpr uint32_t mat_swz(uint32_t major)
{
    constexpr int cpr = RowBytes / 16;
    if constexpr (!is_pow2(cpr) || cpr < 2) {
        return 0;
    } else {
        // rows per swizzle step.  64-byte rows: the 16 lanes that a ds_read_b128 serves together read 16 consecutive rows
        // at one logical chunk; rows 4 apart share their banks, so the chunk position has to differ among them: a step
        // of 4 rows for the 32-row blocks of the 32 x 32 MFMAs, of 2 rows for the 16-row blocks of the 16 x 16 ones
        // (where 16 lanes are 16 rows x 1 chunk but the next 16 lanes the same rows at the next chunk).  The LDS
        // bank-conflict counter reads 0 for either pairing and about one conflict cycle per read cycle for the other.
        constexpr int div = cpr >= 16 ? 1 : (cpr == 4 ? (kMfmaM == 32 ? 4 : 2) : 16 / cpr);
        constexpr int mod = cpr >= 16 ? 16 : cpr;
        return (major / div) % mod;
    }
}

template <int RowBytes>
PTO_DEV constexpr uint32_t mat_chunk_off(uint32_t major, uint32_t chunk)
{
    return major * RowBytes + ((chunk ^ mat_swz<RowBytes>(major)) << 4);
}

// geometry of a Mat tile's LDS image
template <typename TileT>
struct MatGeom {
    using T = typename TileT::DType;
    static constexpr bool colsK = TileT::colsContiguous;
    static constexpr int Major = colsK ? TileT::Rows : TileT::Cols;
    static constexpr int KExt = colsK ? TileT::Cols : TileT::Rows;
    static constexpr int RowBytes = KExt * elem_bits<T> / 8;
    static constexpr int ChunksPerRow = RowBytes / 16;
    static constexpr int Bytes = Major * RowBytes;
    static_assert(RowBytes % 16 == 0, "[PTO][SA] Mat tile: contiguous extent must be a multiple of 16 bytes");
    // byte offset of logical element (r, c)
    PTO_DEV static uint32_t elem_off(uint32_t r, uint32_t c)
    {
        const uint32_t major = colsK ? r : c, k = colsK ? c : r;
        const uint32_t kb = k * elem_bits<T> / 8;
        return mat_chunk_off<RowBytes>(major, kb >> 4) + (kb & 15u);
    }
};

#define PTO_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define PTO_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// index of the outer (stacked) slab and the in-slab row for a 5-D GlobalTensor whose first four
// dims are stacked along the tile's rows (TLoad.hpp:74-95)
template <typename G>
PTO_DEV int64_t gm_row_offset(const G &g, int64_t r)
{
    const int64_t s3 = g.GetShape(3), s2 = g.GetShape(2), s1 = g.GetShape(1);
    const int64_t rr = r % s3;
    int64_t slab = r / s3;
    const int64_t k = slab % s2;
    slab /= s2;
    const int64_t j = slab % s1, i = slab / s1;
    return i * g.GetStride(0) + j * g.GetStride(1) + k * g.GetStride(2) + rr * g.GetStride(3);
}

// Offset of logical element (r, c) of a 2-D tile in a 5-D GlobalTensor (TLoad.hpp:74-131 of the CPU simulation, the NZ
// descriptors of npu/a2a3/TLoad.hpp): ND stacks the four outer dimensions along the rows, DN (column-major tiles) along
// the columns, both with the innermost of them fastest; NZ is [col blocks 0][col blocks 1][row blocks][rows in a block]
// [columns in a block]: row = i2 s3 + i3, column = (i0 s1 + i1) s4 + i4.
template <typename G>
PTO_DEV int64_t gm_elem_offset(const G &g, int64_t r, int64_t c)
{
    const int64_t s1 = g.GetShape(1), s2 = g.GetShape(2), s3 = g.GetShape(3), s4 = g.GetShape(4);
    int64_t i0, i1, i2, i3, i4;
    if constexpr (G::layout == Layout::NZ) {
        i2 = r / s3, i3 = r % s3, i4 = c % s4;
        const int64_t b = c / s4;
        i1 = b % s1, i0 = b / s1;
    } else if constexpr (G::layout == Layout::DN) {
        i3 = r, i4 = c % s4;
        int64_t b = c / s4;
        i2 = b % s2, b /= s2;
        i1 = b % s1, i0 = b / s1;
    } else {
        i4 = c, i3 = r % s3;
        int64_t b = r / s3;
        i2 = b % s2, b /= s2;
        i1 = b % s1, i0 = b / s1;
    }
    return i0 * g.GetStride(0) + i1 * g.GetStride(1) + i2 * g.GetStride(2) + i3 * g.GetStride(3) + i4 * g.GetStride(4);
}

template <typename T>
PTO_DEV T pad_value(PadValue p)
{
    if (p == PadValue::Max) {
        if constexpr (std::is_integral_v<T>)
            return (T)(~(T)0 ^ (std::is_signed_v<T> ? (T)((T)1 << (sizeof(T) * 8 - 1)) : (T)0));
        else
            return (T)__builtin_huge_valf();
    }
    if (p == PadValue::Min) {
        if constexpr (std::is_integral_v<T>)
            return std::is_signed_v<T> ? (T)((T)1 << (sizeof(T) * 8 - 1)) : (T)0;
        else
            return (T)(-__builtin_huge_valf());
    }
    return (T)0;
}

} // namespace detail

// ------------------------------------------------------------------ TASSIGN
// Mat tiles: `addr` is a byte offset into the workgroup's dynamic LDS (the L1 address space), or a pointer obtained from
// a Mat tile's data() (pto_macro_matmul.hpp:176-177 rebinds a tile to `data() + bytes`): a generic pointer into LDS has
// the shared aperture in its upper half, its lower half is the LDS address.
// Register tiles have no address: the call is accepted and ignored, as in the CPU simulation
// (cpu/TAssign.hpp:20-21).  GlobalTensor: rebinding the base pointer.
#if defined(PTO_VEC_TILES_IN_MEMORY)
} // namespace pto
#include "pto/gfx950/ub_mode.hpp"
namespace pto {
#endif
namespace detail {
constexpr uint32_t kLdsBytes = 160 * 1024; // LDS of one gfx950 compute unit
// bytes of a Mat tile's LDS image (a Mat tile of block scales is stored one byte per scale)
template <typename TileT>
constexpr uint32_t mat_tile_bytes()
{
    if constexpr (std::is_same_v<typename TileT::DType, float8_e8m0_t>)
        return TileT::Rows * TileT::Cols;
    else
        return MatGeom<TileT>::Bytes;
}
// A call that survives optimisation stops the build: a TASSIGN whose address the compiler knows lies beyond the LDS
// (the reference checks its compile-time form the same way, tassign_check.hpp:18-30).
#if defined(__HIP_DEVICE_COMPILE__)
__device__ void tassign_beyond_lds() __attribute__((error("[PTO][SA] TASSIGN: the Mat tile ends beyond the 160 KiB LDS of a compute unit")));
__device__ void tassign_beyond_ub() __attribute__((error("[PTO][SA] TASSIGN: the Vec tile ends beyond the part of the workgroup's unified buffer that Vec tiles may use")));
__device__ void tassign_moves_mat_view() __attribute__((error("[PTO][SA] TASSIGN: a Mat tile that has an address is moved by a pointer taken from data(): the LDS image of a tile is not the L1 layout, a part of it is not a tile")));
#endif
} // namespace detail
template <typename T, typename AddrType>
PTO_DEV void TASSIGN_IMPL(T &obj, AddrType addr)
{
    if constexpr (is_global_data_v<T>) {
        obj.SetAddr(reinterpret_cast<typename T::DType *>(addr));
    } else if constexpr (T::Loc == TileType::Mat) {
        const uint64_t a = (uint64_t)(uintptr_t)addr;
        // a literal L1 byte offset, or a value made from a Mat tile's data() (tag in the upper half, offset in the lower)
        const uint32_t off = (uint32_t)a;
#if defined(PTO_TASSIGN_BEYOND_LDS_ENDS_KERNEL)
        // For translation units that hold many kernels of which a few need more L1 than a compute unit has LDS (the
        // reference's per-instruction test sources): such a kernel ends at the TASSIGN, every wave alike, having done
        // nothing, instead of stopping the build of the others.
        if (off + detail::mat_tile_bytes<T>() > detail::kLdsBytes)
            __builtin_amdgcn_endpgm();
#elif defined(__HIP_DEVICE_COMPILE__)
        if (__builtin_constant_p(off) && off + detail::mat_tile_bytes<T>() > detail::kLdsBytes)
            detail::tassign_beyond_lds();
#endif
#if defined(_DEBUG) || defined(PTO_DEBUG)
        if (off + detail::mat_tile_bytes<T>() > detail::kLdsBytes)
            __builtin_trap(); // the run-time form of the reference's PTO_ASSERT (debug builds only)
#endif
        // A tile that already has an address, moved by an address computed from a tile's data(): the reference's stage
        // macros walk a large L1 tile in chunks this way (pto_macro_matmul.hpp:176-177: data() + k * Cube_K * Cube_M).  The
        // LDS image of a Mat tile is swizzled row-major, not Nz: a chunk of it is not the image of a smaller tile, so the
        // second and later chunks would read another part of the data.  Stops the build where the compiler knows both
        // addresses; otherwise the kernel reports it and ends (every wave makes the same call).
        if ((a >> 32) != 0 && obj.st.bound && off != obj.st.lds) {
#if defined(__HIP_DEVICE_COMPILE__)
            if (__builtin_constant_p(off) && __builtin_constant_p(obj.st.lds))
                detail::tassign_moves_mat_view();
#endif
            if (hw::tid() == 0)
                printf("[PTO][RT] TASSIGN: a Mat tile at LDS offset %u is moved to %u by a pointer taken from data(); a part of a "
                       "tile's LDS image is not a tile (block %d)\n", obj.st.lds, off, (int)blockIdx.x);
            __builtin_amdgcn_endpgm();
        }
        obj.st.lds = off;
        obj.st.bound = true;
    } else if constexpr (T::Loc == TileType::Scaling) {
        obj.st.fb = (uint32_t)(uintptr_t)addr; // offset into the table of quantisation words
    } else {
#if defined(PTO_VEC_TILES_IN_MEMORY)
        if constexpr (T::inMemory) {
            // a byte offset into the workgroup's unified buffer, or a pointer obtained from another Vec tile's data()
            const uint64_t a = (uint64_t)(uintptr_t)addr;
            // offset form: the tile has to end inside this workgroup's buffer, and below the accumulator images when
            // those live in its upper part
#if defined(PTO_ACC_TILES_IN_MEMORY)
            constexpr uint64_t vecLimit = PTO_ACC_ARENA_OFFSET;
#else
            constexpr uint64_t vecLimit = PTO_UB_BYTES;
#endif
            constexpr uint64_t bytes = (uint64_t)T::Numel * sizeof(typename T::DType);
            if (a < (uint64_t)PTO_UB_BYTES && a + bytes > vecLimit) {
#if defined(__HIP_DEVICE_COMPILE__)
                if (__builtin_constant_p(a))
                    detail::tassign_beyond_ub();
#endif
#if defined(_DEBUG) || defined(PTO_DEBUG)
                __builtin_trap();
#endif
            }
            obj.mem_ = a < (uint64_t)PTO_UB_BYTES ? reinterpret_cast<typename T::DType *>(detail::ub_base() + a) :
                                                   reinterpret_cast<typename T::DType *>((uintptr_t)a);
            return;
        } else if constexpr (T::accInMemory) {
            const uint64_t a = (uint64_t)(uintptr_t)addr;
            obj.mem_ = a + sizeof(typename T::DType) * T::Numel <= (uint64_t)(PTO_UB_BYTES - PTO_ACC_ARENA_OFFSET) ?
                           reinterpret_cast<typename T::DType *>(detail::ub_base() + PTO_ACC_ARENA_OFFSET + a) :
                           nullptr; // beyond the arena: the tile stays in registers only
            return;
        }
#endif
        (void)obj;
        (void)addr;
    }
}

// -------------------------------------------------------------------- TLOAD
namespace detail {

// Tells the compiler that p is the same in every lane (it then lives in scalar registers and the
// access can use the scalar-base + 32-bit lane offset addressing form).
PTO_DEV const char *uniform_ptr(const char *p)
{
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char *>((uintptr_t)(((uint64_t)hi << 32) | lo));
}

// GM -> LDS Mat tile.  Fast path: the tile's contiguous dimension is the unit-stride one in
// memory, the valid region is the whole tile: 16-byte asynchronous global->LDS copies, 1 KiB of
// LDS per wave instruction; the swizzle is applied on the global-address side.
// SLICE >= 0: only the SLICE-th group of kBlockWaves copy instructions (one per wave).
template <int SLICE = -1, typename TileT, typename G>
PTO_DEV void tload_mat(TileT &dst, G &src)
{
    using T = typename TileT::DType;
    using Geo = MatGeom<TileT>;
    char *lds = hw::lds_base() + dst.st.lds;
    const T *gm = reinterpret_cast<const T *>(src.data());
    const int64_t st_r = src.GetStride(3), st_c = src.GetStride(4);
    constexpr bool fullValid = TileT::ValidRow == TileT::Rows && TileT::ValidCol == TileT::Cols;
    constexpr bool staticUnit = Geo::colsK ? (G::staticStride[4] == 1) : (G::staticStride[3] == 1);
    if constexpr (fullValid && staticUnit) {
        const int64_t ld = (Geo::colsK ? st_r : st_c) * elem_bits<T> / 8; // bytes between consecutive rows (columns) in memory
        constexpr int total = Geo::Major * Geo::ChunksPerRow; // 16-byte chunks
        constexpr int perWaveInst = kWaveSize;
        constexpr int nInst = cdiv(total, perWaveInst);
        const int lane = hw::lane(), wave = hw::wave();
        constexpr int cpr = Geo::ChunksPerRow;
        // rows that one wave instruction covers, when a row is at most one instruction long
        constexpr int rpi = (cpr <= kWaveSize && kWaveSize % cpr == 0) ? kWaveSize / cpr : 0;
        if constexpr (rpi > 0 && (rpi * kBlockWaves) % 16 == 0 && total % perWaveInst == 0 && (nInst % kBlockWaves == 0 || SLICE < 0) &&
                      (nInst % kBlockWaves == 0 || nInst > kBlockWaves)) {
            // The swizzle repeats every 16 rows and the instructions of one wave are a multiple of 16
            // rows apart: every instruction of this wave uses the same per-lane byte offset (32 bits: a
            // tile spans less than 4 GiB of memory) on top of a wave-uniform base, which the loop
            // around the TLOAD only has to advance with scalar arithmetic.
            const uint32_t major0 = (uint32_t)wave * rpi + (uint32_t)lane / cpr, cpos = (uint32_t)lane % cpr;
            const uint32_t chunk = cpos ^ mat_swz<Geo::RowBytes>(major0);
            const uint32_t laneOff = major0 * (uint32_t)ld + chunk * 16;
            const char *base = reinterpret_cast<const char *>(gm);
            constexpr int first = SLICE < 0 ? 0 : SLICE * kBlockWaves, last = SLICE < 0 ? nInst : first + kBlockWaves;
            static_assert(last <= nInst, "[PTO][SA] TLOAD slice: the tile has fewer copy instructions");
#pragma unroll
            for (int s0 = first; s0 < last; s0 += kBlockWaves) {
                // When the last round of instructions is not full, the waves past its end repeat their instruction
                // of the round before (same data to the same place): every wave then issues TLoadInstrs<TileT>()
                // copies, which keeps the vmcnt bookkeeping of software pipelines uniform and the code branch-free.
                const int s0e = (nInst % kBlockWaves != 0 && s0 + wave >= nInst) ? s0 - kBlockWaves : s0;
                const char *g = uniform_ptr(base + (int64_t)(s0e * rpi) * ld) + laneOff;
                __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(g), PTO_LDS_PTR(lds + (s0e + wave) * (perWaveInst * 16)), 16, 0, 0);
            }
        } else {
            static_assert(SLICE < 0, "[PTO][SA] TLOAD slice: this tile geometry has no per-wave slices");
#pragma unroll
            for (int s0 = 0; s0 < nInst; s0 += kBlockWaves) {
                const int s = s0 + wave;
                const uint32_t q = (uint32_t)(s * perWaveInst + lane);
                constexpr bool evenInst = nInst % kBlockWaves == 0, evenTotal = total % perWaveInst == 0;
                if ((evenInst || s < nInst) && (evenTotal || q < (uint32_t)total)) {
                    const uint32_t major = q / Geo::ChunksPerRow, cpos = q % Geo::ChunksPerRow;
                    const uint32_t chunk = cpos ^ mat_swz<Geo::RowBytes>(major);
                    const char *g = reinterpret_cast<const char *>(gm) + (int64_t)major * ld + chunk * 16;
                    __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(g), PTO_LDS_PTR(lds + s * (perWaveInst * 16)), 16, 0, 0);
                }
            }
        }
    } else {
        static_assert(SLICE < 0, "[PTO][SA] TLOAD slice: only for fully valid, unit-stride Mat tiles");
        const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
        if constexpr (staticUnit && TileT::PadVal == PadValue::Null && G::layout != Layout::NZ) {
            // Run-time valid extents with whole rows of the contiguous dimension (the last row / column block of a matrix
            // that the tiles do not divide): the same 16-byte copies; rows past the valid ones repeat the last valid row
            // (memory past it may not exist, and what a tile holds outside its valid region is unspecified).
            const int vMajor = Geo::colsK ? vr : vc, vMinor = Geo::colsK ? vc : vr;
            const bool plain2d = src.GetShape(0) * src.GetShape(1) * src.GetShape(2) == 1; // (no stacked outer dimensions)
            if (plain2d && vMinor == (Geo::colsK ? TileT::Cols : TileT::Rows) && vMajor > 0) {
                const int64_t ld = (Geo::colsK ? st_r : st_c) * elem_bits<T> / 8;
                constexpr int total = Geo::Major * Geo::ChunksPerRow, nInst = cdiv(total, kWaveSize);
                const int lane = hw::lane(), wave = hw::wave();
#pragma unroll
                for (int s0 = 0; s0 < nInst; s0 += kBlockWaves) {
                    const int s = s0 + wave;
                    const uint32_t q = (uint32_t)(s * kWaveSize + lane);
                    constexpr bool evenInst = nInst % kBlockWaves == 0, evenTotal = total % kWaveSize == 0;
                    if ((evenInst || s < nInst) && (evenTotal || q < (uint32_t)total)) {
                        const uint32_t major = q / Geo::ChunksPerRow, cpos = q % Geo::ChunksPerRow;
                        const uint32_t chunk = cpos ^ mat_swz<Geo::RowBytes>(major);
                        const uint32_t from = major < (uint32_t)vMajor ? major : (uint32_t)vMajor - 1u;
                        const char *g = reinterpret_cast<const char *>(gm) + (int64_t)from * ld + chunk * 16;
                        __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(g), PTO_LDS_PTR(lds + s * (kWaveSize * 16)), 16, 0, 0);
                    }
                }
                return;
            }
        }
        if constexpr (elem_bits<T> < 8) {
            // (4-bit elements have no address of their own)
            if (hw::tid() == 0)
                printf("[PTO][RT] TLOAD of 4-bit elements into a Mat tile: whole rows of the contiguous dimension only\n");
            __builtin_amdgcn_endpgm();
        } else {
        // general path: element by element, pad outside the valid region (TLoad.hpp:151-152)
        const T pad = pad_value<T>(TileT::PadVal);
        const bool stacked = src.GetShape(0) * src.GetShape(1) * src.GetShape(2) != 1;
        for (int e = hw::tid(); e < TileT::Numel; e += kBlockThreads) {
            const int r = e / TileT::Cols, c = e % TileT::Cols;
            T v = pad;
            if (r < vr && c < vc) // views with stacked outer dimensions and NZ memory: by the 5-D rule; else rows and columns
                v = (G::layout == Layout::NZ || stacked) ? gm[gm_elem_offset(src, r, c)] : gm[(int64_t)r * st_r + (int64_t)c * st_c];
            *reinterpret_cast<T *>(lds + Geo::elem_off(r, c)) = v;
        }
        }
    }
}

// GM -> Vec register tile.  Chunk q of 8 consecutive elements (in the tile's BLayout order).
// PTO_VEC_STREAM_NT (per translation unit): bit 0 = non-temporal 16-byte loads, bit 1 = non-temporal 16-byte stores of Vec
// tiles, for kernels that stream data they do not touch again.
template <typename TileT, typename G>
PTO_DEV void tload_vec(TileT &dst, G &src)
{
    using T = typename TileT::DType;
    using S = typename TileT::Storage;
    // (a box layout of a Vec tile names the order of its elements in Ascend's unified buffer; the register distribution
    // holds logical elements, and only the NZ layout of the memory side shows in the addresses)
    static_assert(TileT::SFractal == SLayout::NoneBox || !kVecTilesInMemory, "[PTO][SA] boxed Vec tiles: register tiles only");
    const T *gm = reinterpret_cast<const T *>(src.data());
    constexpr int Minor = TileT::isRowMajor ? TileT::Cols : TileT::Rows; // contiguous extent of the tile
    const int vMajor = TileT::isRowMajor ? dst.GetValidRow() : dst.GetValidCol();
    const int vMinor = TileT::isRowMajor ? dst.GetValidCol() : dst.GetValidRow();
    const int64_t stMinor = TileT::isRowMajor ? src.GetStride(4) : src.GetStride(3);
    const bool stacked = src.GetShape(0) * src.GetShape(1) * src.GetShape(2) != 1;
    const T pad = pad_value<T>(TileT::PadVal);
    constexpr bool vecOK = Minor % kVecChunk == 0 && (kVecChunk * sizeof(T)) % 16 == 0 || Minor % kVecChunk == 0;
    // NZ memory, or outer dimensions stacked along the columns of a column-major tile: element by element
    if (G::layout == Layout::NZ || (!TileT::isRowMajor && stacked)) {
        const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
#pragma unroll
        for (int s = 0; s < S::Slots; ++s)
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i) {
                const int e = (s * kBlockThreads + hw::tid()) * kVecChunk + i;
                const int r = TileT::isRowMajor ? e / TileT::Cols : e % TileT::Rows, c = TileT::isRowMajor ? e % TileT::Cols : e / TileT::Rows;
                dst.S().v[s][i] = (e < TileT::Numel && r < vr && c < vc) ? gm[gm_elem_offset(src, r, c)] : pad;
            }
        return;
    }
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        const int e0 = q * kVecChunk;
        if (S::Chunks % kBlockThreads != 0 && q >= S::Chunks) {
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i)
                dst.S().v[s][i] = pad;
            continue;
        }
        const int major = e0 / Minor, minor0 = e0 % Minor;
        int64_t base;
        if (TileT::isRowMajor)
            base = stacked ? gm_row_offset(src, major) : (int64_t)major * src.GetStride(3);
        else
            base = (int64_t)major * src.GetStride(4);
        if (vecOK && stMinor == 1 && major < vMajor && minor0 + kVecChunk <= vMinor) {
            // 8 contiguous elements: one or two 16-byte loads
            // element-aligned only: rows of a strided view need not start on a 16-byte boundary
            typedef T VT __attribute__((ext_vector_type(kVecChunk), aligned(sizeof(T))));
#if defined(PTO_VEC_STREAM_NT) && (PTO_VEC_STREAM_NT & 1)
            VT v = __builtin_nontemporal_load(reinterpret_cast<const VT *>(gm + base + minor0));
#else
            VT v = *reinterpret_cast<const VT *>(gm + base + minor0);
#endif
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i)
                dst.S().v[s][i] = v[i];
        } else {
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i) {
                const int e = e0 + i;
                const int mj = e / Minor, mn = e % Minor;
                T v = pad;
                if (e < TileT::Numel && mj < vMajor && mn < vMinor) {
                    int64_t b = TileT::isRowMajor ? (stacked ? gm_row_offset(src, mj) : (int64_t)mj * src.GetStride(3)) :
                                                    (int64_t)mj * src.GetStride(4);
                    v = gm[b + (int64_t)mn * stMinor];
                }
                dst.S().v[s][i] = v;
            }
        }
    }
}

} // namespace detail

// Number of asynchronous global->LDS copy instructions that one TLOAD of a fully valid Mat tile
// issues per wave (what wait_flag_pending counts).
// One slice of a Mat tile's TLOAD: the SLICE-th of TLoadInstrs<TileT>() asynchronous copy instructions
// of every wave (TLOAD == all slices).  Lets a kernel spread the copies of a tile over its
// instruction stream, and lets the waves of a workgroup issue theirs at different points, so that
// they do not queue up behind each other at the compute unit's one vector-memory address unit.
template <int SLICE, typename TileT, typename G>
PTO_DEV void TLOAD_SLICE(TileT &dst, G &src)
{
    static_assert(TileT::Loc == TileType::Mat, "[PTO][SA] TLOAD_SLICE: destination must be a Mat tile");
    detail::tload_mat<SLICE>(dst, src);
}

namespace detail {
template <typename TileT>
constexpr bool is_scale_mat_v = TileT::Loc == TileType::Mat && std::is_same_v<typename TileT::DType, float8_e8m0_t>;

// GM -> Mat tile of block scales ([rows, k blocks] row-major for a left operand, [k blocks, columns] column-major for a
// right one; k blocks contiguous in memory; plain or boxed tile types alike).  LDS image: [k block / 4][row (column)][4 k blocks], so that the scales
// of one k step of 32 consecutive rows are 32 consecutive words (fragment reads without bank conflicts).  One 4-byte
// asynchronous copy instruction per 64 rows and 4 k blocks.
template <typename TileT>
struct ScaleMatGeom {
    static constexpr bool left = TileT::isRowMajor;
    static constexpr int Major = left ? TileT::Rows : TileT::Cols, KB = left ? TileT::Cols : TileT::Rows;
    // The box layout of the tile type (the reference keeps its scale panels as zZ / nN boxes of 32 bytes in L1:
    // mxmatmul_performance_kernel.cpp:314-317) names a physical arrangement that this image replaces; only the logical
    // (row, k block) contract is kept.
    static_assert(KB % 4 == 0 && Major % kWaveSize == 0, "[PTO][SA] Mat tile of block scales: multiples of 64 rows (columns) and of 4 k blocks");
    static constexpr int nInst = (Major / kWaveSize) * (KB / 4);
    PTO_DEV static uint32_t off(uint32_t major, uint32_t kb) { return ((kb / 4) * Major + major) * 4 + kb % 4; }
};
template <typename TileT, typename G>
PTO_DEV void tload_scale_mat(TileT &dst, G &src)
{
    using Geo = ScaleMatGeom<TileT>;
    static_assert(Geo::left ? G::staticStride[4] == 1 : G::staticStride[3] == 1, "[PTO][SA] TLOAD of block scales: k blocks must be contiguous");
    // (run-time valid extents: every k block of the tile, any number of rows / columns; those past the valid ones repeat the
    // last valid one, as for operand tiles)
    const int vMajor = Geo::left ? dst.GetValidRow() : dst.GetValidCol();
    char *lds = hw::lds_base() + dst.st.lds;
    const char *gm = reinterpret_cast<const char *>(src.data());
    const int64_t ld = Geo::left ? src.GetStride(3) : src.GetStride(4);
    const int lane = hw::lane(), wave = hw::wave();
    static_assert(Geo::nInst % kBlockWaves == 0 || Geo::nInst > kBlockWaves, "[PTO][SA] TLOAD: fewer copy instructions than waves");
#pragma unroll
    for (int s0 = 0; s0 < Geo::nInst; s0 += kBlockWaves) {
        // (waves past the end of an incomplete last round repeat their previous instruction, as for operand tiles)
        const int s = ((Geo::nInst % kBlockWaves != 0 && s0 + wave >= Geo::nInst) ? s0 - kBlockWaves : s0) + wave;
        const int q = s / (Geo::Major / kWaveSize), g = s % (Geo::Major / kWaveSize);
        const char *p;
        if constexpr (TileT::ValidRow != TileT::Rows || TileT::ValidCol != TileT::Cols) {
            const int major = g * kWaveSize + lane;
            p = gm + (int64_t)(major < vMajor ? major : vMajor - 1) * ld + 4 * q;
        } else {
            p = uniform_ptr(gm + (int64_t)(g * kWaveSize) * ld + 4 * q) + (uint32_t)lane * (uint32_t)ld;
        }
        __builtin_amdgcn_global_load_lds(PTO_GLOBAL_PTR(p), PTO_LDS_PTR(lds + s * (kWaveSize * 4)), 4, 0, 0);
    }
}

// GM -> block-scale register tile (the reference stages scales in L1 and TEXTRACTs them; a scale tile here is a few
// registers per lane, so it is loaded straight from memory: one 4-byte load per four k blocks and 32-row block).
// The k-block index must be the unit-stride dimension and the tile's first k block 4-byte aligned in memory.
template <typename TileT, typename G>
PTO_DEV void tload_scale(TileT &dst, G &src)
{
    using S = typename TileT::Storage;
    constexpr bool left = TileT::Loc == TileType::ScaleLeft;
    static_assert(left ? G::staticStride[4] == 1 : G::staticStride[3] == 1, "[PTO][SA] TLOAD of a scale tile: k blocks must be contiguous");
    const char *gm = reinterpret_cast<const char *>(src.data());
    const int64_t ld = left ? src.GetStride(3) : src.GetStride(4);
    const uint32_t lane = (uint32_t)hw::lane();
    const uint32_t shift = (lane / kMxM) * 8;
    constexpr int blocks = S::Blocks;
    const uint32_t major0 = (uint32_t)(left ? hw::wave_m() : hw::wave_n()) * (blocks * kMxM) + lane % kMxM;
#pragma unroll
    for (int b = 0; b < blocks; ++b) {
        const char *p = gm + (int64_t)(major0 + b * kMxM) * ld;
        if constexpr (S::KB == 2) {
            dst.S().s[b][0] = (uint32_t)*reinterpret_cast<const uint16_t *>(p) >> shift;
        } else if constexpr (S::Regs % 4 == 0) {
#pragma unroll
            for (int r = 0; r < S::Regs; r += 4) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(p + 4 * r);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    dst.S().s[b][r + i] = v[i] >> shift;
            }
        } else {
#pragma unroll
            for (int r = 0; r < S::Regs; ++r)
                dst.S().s[b][r] = *reinterpret_cast<const uint32_t *>(p + 4 * r) >> shift;
        }
    }
}
} // namespace detail

template <typename TileT>
constexpr int TLoadInstrs()
{
    if constexpr (detail::is_scale_mat_v<TileT>) {
        return detail::cdiv(detail::ScaleMatGeom<TileT>::nInst, kBlockWaves);
    } else {
        using Geo = detail::MatGeom<TileT>;
        return detail::cdiv(detail::cdiv(Geo::Major * Geo::ChunksPerRow, kWaveSize), kBlockWaves);
    }
}
template <typename TileT, typename G>
PTO_DEV void TLOAD_IMPL(TileT &dst, G &src)
{
    static_assert(sizeof(typename TileT::DType) == sizeof(typename G::DType), "[PTO][SA] TLOAD: element sizes differ");
    if constexpr (detail::is_scale_mat_v<TileT>)
        detail::tload_scale_mat(dst, src);
    else if constexpr (TileT::Loc == TileType::Mat)
        detail::tload_mat(dst, src);
    else if constexpr (TileT::Loc == TileType::Vec)
        detail::tload_vec(dst, src);
    else if constexpr (TileT::Loc == TileType::ScaleLeft || TileT::Loc == TileType::ScaleRight)
        detail::tload_scale(dst, src);
    else if constexpr (TileT::Loc == TileType::Bias)
        detail::tload_any(dst, src);
    else
        static_assert(TileT::Loc == TileType::Mat, "[PTO][SA] TLOAD: destination must be a Mat or Vec tile");
}

// TPREFETCH: the region ends up in the tile (cpu/TPrefetch.hpp:18-41), as after a TLOAD
template <typename TileT, typename G>
PTO_DEV void TPREFETCH_IMPL(TileT &dst, G &src)
{
    TLOAD_IMPL(dst, src);
}

// ----------------------------------------------------------------- TEXTRACT
// dst[i,j] = src[idxRow+i, idxCol+j].  Mat -> Left / Right: one ds_read_b128 per row block and k step, in the
// MFMA operand layout (lane l: row/col l % kMfmaM, the 16-byte chunk l / kMfmaM of the step: 8 fp16 / bf16, 16 int8 or
// 4 fp32 values).  The k offset must be a multiple of 16 bytes.
namespace detail {
// Mat -> Left / Right of an MX operand.  8-bit: two ds_read_b128 per 32-row block and 64-wide k step (lane l: row
// l % 32, bytes 16 (l / 32) .. +15 and 32 + 16 (l / 32) .. +15 of the step).  4-bit: one ds_read_b128 (bytes
// 16 (l / 32) .. +15 of the step's 32).  The k offset must be a multiple of 64.
template <typename DstT, typename SrcT>
PTO_DEV void textract_mx(DstT &dst, SrcT &src, uint32_t idxRow, uint32_t idxCol)
{
    using Geo = MatGeom<SrcT>;
    using S = typename DstT::Storage;
    constexpr bool left = DstT::Loc == TileType::Left;
    static_assert(left ? Geo::colsK : !Geo::colsK, "[PTO][SA] TEXTRACT: the source must be contiguous along k");
    const char *lds = hw::lds_base() + src.st.lds;
    const uint32_t lane = (uint32_t)hw::lane();
    constexpr int blocks = S::Blocks;
    const uint32_t major0 = (left ? idxRow : idxCol) + (uint32_t)(left ? hw::wave_m() : hw::wave_n()) * (blocks * kMxM) + lane % kMxM;
    using T = typename DstT::DType;
    const uint32_t chunk0 = (((left ? idxCol : idxRow) * elem_bits<T> / 8) >> 4) + lane / kMxM;
#pragma unroll
    for (int b = 0; b < blocks; ++b)
#pragma unroll
        for (int ks = 0; ks < S::KS; ++ks) {
            if constexpr (is_mx4_v<T>) {
                dst.S().f[b][ks] = *reinterpret_cast<const u32x4 *>(lds + mat_chunk_off<Geo::RowBytes>(major0 + b * kMxM, chunk0 + ks * 2));
            } else {
                const u32x4 lo = *reinterpret_cast<const u32x4 *>(lds + mat_chunk_off<Geo::RowBytes>(major0 + b * kMxM, chunk0 + ks * 4));
                const u32x4 hi = *reinterpret_cast<const u32x4 *>(lds + mat_chunk_off<Geo::RowBytes>(major0 + b * kMxM, chunk0 + ks * 4 + 2));
                dst.S().f[b][ks] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            }
        }
}

// Mat tile of scales in LDS (image [k block / 4][row][4 k blocks], see tload_scale_mat) -> scale register tile:
// k blocks [kb, kb + dst.KB) of rows [idx, idx + extent); kb a multiple of 4 (of 2 for a tile of one k step: one
// ds_read_u8 per 32-row block, lanes 32-63 read the step's second block)
template <typename DstT, typename SrcT>
PTO_DEV void textract_scale_mat(DstT &dst, SrcT &src, uint32_t idxMajor, uint32_t kb)
{
    using Geo = ScaleMatGeom<SrcT>;
    using D = typename DstT::Storage;
    constexpr bool left = DstT::Loc == TileType::ScaleLeft;
    static_assert(is_scale_mat_v<SrcT> && left == Geo::left, "[PTO][SA] TEXTRACT of scales: from a Mat tile of block scales of the same side");
    const char *lds = hw::lds_base() + src.st.lds;
    const uint32_t lane = (uint32_t)hw::lane();
    const uint32_t shift = (lane / kMxM) * 8;
    constexpr int blocks = D::Blocks;
    const uint32_t major0 = idxMajor + (uint32_t)(left ? hw::wave_m() : hw::wave_n()) * (blocks * kMxM) + lane % kMxM;
#pragma unroll
    for (int b = 0; b < blocks; ++b) {
        const char *p = lds + Geo::off(major0 + b * kMxM, kb);
        if constexpr (D::KB == 2) {
            dst.S().s[b][0] = *reinterpret_cast<const uint8_t *>(p + lane / kMxM);
        } else {
#pragma unroll
            for (int r = 0; r < D::Regs; ++r)
                dst.S().s[b][r] = *reinterpret_cast<const uint32_t *>(p + r * (Geo::Major * 4)) >> shift;
        }
    }
}

// scale tile -> scale tile window (registers only): k blocks [kb, kb + dst.KB) of the source; kb a multiple of 2,
// and of 4 unless the destination holds a single k step (2 blocks)
template <typename DstT, typename SrcT>
PTO_DEV void textract_scale(DstT &dst, const SrcT &src, uint32_t kb)
{
    using D = typename DstT::Storage;
    using S = typename SrcT::Storage;
    constexpr bool left = DstT::Loc == TileType::ScaleLeft;
    static_assert(left ? DstT::Rows == SrcT::Rows : DstT::Cols == SrcT::Cols, "[PTO][SA] TEXTRACT of scales: windows along k only");
    constexpr int blocks = D::Blocks;
#pragma unroll
    for (int b = 0; b < blocks; ++b) {
        if constexpr (D::KB == 2) {
            dst.S().s[b][0] = src.S().s[b][kb / 4] >> ((kb % 4) * 8);
        } else {
#pragma unroll
            for (int r = 0; r < D::Regs; ++r)
                dst.S().s[b][r] = src.S().s[b][kb / 4 + r];
        }
    }
}
} // namespace detail

template <typename DstT, typename SrcT>
PTO_DEV void textract_frag(DstT &dst, SrcT &src, uint32_t idxRow, uint32_t idxCol)
{
    static_assert(SrcT::Loc == TileType::Mat, "[PTO][SA] TEXTRACT: source must be a Mat tile");
    static_assert(sizeof(typename DstT::DType) == sizeof(typename SrcT::DType), "[PTO][SA] TEXTRACT: dtype mismatch");
    using Geo = detail::MatGeom<SrcT>;
    using Frag = typename detail::FragOf<typename DstT::DType>::type;
    const char *lds = hw::lds_base() + src.st.lds;
    const uint32_t lane = (uint32_t)hw::lane();
    const uint32_t l32 = detail::frag_lane_major(lane), khalf = detail::frag_lane_kgroup(lane);
    using ElemT = typename DstT::DType;
    constexpr uint32_t kStepChunks = kWaveSize / detail::kMfmaM; // 16-byte chunks per fragment (one per lane group)
    constexpr uint32_t kChunkElems = 16 / sizeof(ElemT);
    if constexpr (DstT::Loc == TileType::Left) {
        using S = typename DstT::Storage;
        const uint32_t row0 = idxRow + (uint32_t)hw::wave_m() * (S::MB * detail::kMfmaM) + l32;
        if constexpr (Geo::colsK) {
            const uint32_t chunk0 = idxCol / kChunkElems + khalf;
#pragma unroll
            for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
                for (int ks = 0; ks < S::KS; ++ks)
                    dst.S().f[mb][ks] = *reinterpret_cast<const Frag *>(
                        lds + detail::mat_chunk_off<Geo::RowBytes>(row0 + mb * detail::kMfmaM, chunk0 + ks * kStepChunks));
        } else {
            // the source is contiguous along its rows (an A operand stored transposed): element-wise gather, the slow path
            // that keeps every layout pair of the reference's TEXTRACT legal (a2a3/TExtract.hpp:537-548)
#pragma unroll
            for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
                for (int ks = 0; ks < S::KS; ++ks) {
                    ElemT tmp[kChunkElems];
#pragma unroll
                    for (uint32_t j = 0; j < kChunkElems; ++j)
                        tmp[j] = *reinterpret_cast<const ElemT *>(
                            lds + Geo::elem_off(row0 + mb * detail::kMfmaM, idxCol + (khalf + ks * kStepChunks) * kChunkElems + j));
                    __builtin_memcpy(&dst.S().f[mb][ks], tmp, 16);
                }
        }
    } else if constexpr (DstT::Loc == TileType::Right) {
        using S = typename DstT::Storage;
        const uint32_t col0 = idxCol + (uint32_t)hw::wave_n() * (S::NB * detail::kMfmaM) + l32;
        if constexpr (!Geo::colsK) {
            const uint32_t chunk0 = idxRow / kChunkElems + khalf;
#pragma unroll
            for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
                for (int ks = 0; ks < S::KS; ++ks)
                    dst.S().f[nb][ks] = *reinterpret_cast<const Frag *>(
                        lds + detail::mat_chunk_off<Geo::RowBytes>(col0 + nb * detail::kMfmaM, chunk0 + ks * kStepChunks));
        } else {
            // the source is contiguous along its columns (a B operand [k, n] stored row-major, the V tile of the
            // reference's attention kernel: fa_performance_kernel.cpp:676-677): element-wise gather, the slow path
#pragma unroll
            for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
                for (int ks = 0; ks < S::KS; ++ks) {
                    ElemT tmp[kChunkElems];
#pragma unroll
                    for (uint32_t j = 0; j < kChunkElems; ++j)
                        tmp[j] = *reinterpret_cast<const ElemT *>(
                            lds + Geo::elem_off(idxRow + (khalf + ks * kStepChunks) * kChunkElems + j, col0 + nb * detail::kMfmaM));
                    __builtin_memcpy(&dst.S().f[nb][ks], tmp, 16);
                }
        }
    } else {
        static_assert(DstT::Loc == TileType::Left, "[PTO][SA] TEXTRACT: destination must be a Left or Right tile");
    }
}

template <typename DstT, typename SrcT>
PTO_DEV void TEXTRACT_IMPL(DstT &dst, SrcT &src, uint32_t idxRow = 0, uint32_t idxCol = 0)
{
    if constexpr (SrcT::Loc == TileType::Acc && DstT::Loc == TileType::Mat) {
        detail::textract_fix<ReluPreMode::NoRelu>(dst, src, (int)idxRow, (int)idxCol, detail::FixNone{}); // pto/gfx950/fixpipe.hpp
        return;
    } else if constexpr (DstT::Loc == TileType::ScaleLeft || DstT::Loc == TileType::ScaleRight) {
        constexpr bool left = DstT::Loc == TileType::ScaleLeft;
        if constexpr (SrcT::Loc == TileType::Mat) {
            detail::textract_scale_mat(dst, src, left ? idxRow : idxCol, left ? idxCol : idxRow);
        } else {
            static_assert(SrcT::Loc == DstT::Loc, "[PTO][SA] TEXTRACT of scales: from a Mat tile or a scale tile of the same kind");
            detail::textract_scale(dst, src, left ? idxCol : idxRow);
        }
        return;
    } else if constexpr (detail::is_mx_operand_v<typename DstT::DType>) {
        static_assert(SrcT::Loc == TileType::Mat && std::is_same_v<typename SrcT::DType, typename DstT::DType>,
                      "[PTO][SA] TEXTRACT: Mat source of the same element type");
        detail::textract_mx(dst, src, idxRow, idxCol);
        return;
    } else if constexpr (detail::is_plain_v<DstT>) {
        detail::textract_any(dst, src, idxRow, idxCol);
    } else {
        textract_frag(dst, src, idxRow, idxCol);
        if constexpr (!detail::is_fully_valid_v<DstT>)
            detail::zero_outside_valid(dst); // TMATMUL multiplies whole fragments
    }
}

// --------------------------------------------------------------------- TMOV
// Same-shape move between locations.  Mat -> Left/Right is TEXTRACT at (0,0); register tiles of
// the same location and shape copy their fragments.
template <typename DstT, typename SrcT>
PTO_DEV void TMOV_IMPL(DstT &dst, SrcT &src)
{
    if constexpr (SrcT::Loc == TileType::Mat && (DstT::Loc == TileType::Left || DstT::Loc == TileType::Right)) {
        TEXTRACT_IMPL(dst, src, 0, 0);
    } else if constexpr (SrcT::Loc == TileType::Mat && DstT::Loc == TileType::Bias) {
        detail::textract_any(dst, src, 0, 0); // L1 -> bias table (npu/a2a3/TMov.hpp: the Mat -> Bias pair)
    } else if constexpr (SrcT::Loc == DstT::Loc && SrcT::Rows == DstT::Rows && SrcT::Cols == DstT::Cols &&
                         std::is_same_v<typename SrcT::DType, typename DstT::DType> && SrcT::Loc != TileType::Mat) {
        dst.st = src.st;
    } else {
        static_assert(SrcT::Loc == TileType::Mat && DstT::Loc == TileType::Left,
                      "[PTO][SA] TMOV: this location pair is not available on gfx950");
    }
}

// ------------------------------------------------------------------- TSTORE
namespace detail {

template <typename D, typename S>
PTO_DEV D store_cast(S v)
{
    if constexpr (std::is_same_v<D, S>)
        return v;
    else
        return static_cast<D>(v); // fp32 -> fp16 / bf16: hardware round-to-nearest-even
}

// *p += v for any element type: 32-bit types with the hardware's atomic, narrower ones with a compare-and-swap loop on
// the aligned 32-bit word that holds them (the reference's fix pipe accumulates into fp16, bf16 and 8-bit results too:
// tests/npu/a2a3/src/st/testcase/tstore_acc2gm)
template <typename D>
PTO_DEV void atomic_add(D *p, D v)
{
    if constexpr (std::is_same_v<D, float> || std::is_same_v<D, int32_t> || std::is_same_v<D, uint32_t>) {
        atomicAdd(p, v);
    } else {
        static_assert(sizeof(D) < 4, "[PTO][SA] atomic add: 8-, 16- or 32-bit elements");
        using Bits = std::conditional_t<sizeof(D) == 2, uint16_t, uint8_t>;
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        unsigned int *word = reinterpret_cast<unsigned int *>(a & ~(uintptr_t)3);
        const unsigned shift = (unsigned)(a & 3) * 8;
        const unsigned int mask = (unsigned int)(Bits)~(Bits)0 << shift;
        unsigned int seen = *word, want;
        do {
            const D cur = __builtin_bit_cast(D, (Bits)((seen & mask) >> shift));
            const D sum = (D)(cur + v);
            want = (seen & ~mask) | ((unsigned int)__builtin_bit_cast(Bits, sum) << shift);
            const unsigned int prev = atomicCAS(word, seen, want);
            if (prev == seen)
                break;
            seen = prev;
        } while (true);
    }
}

// Acc fragments -> GM.  MFMA result layout: lane l, register v holds row acc_elem_row(v) + acc_lane_row(l),
// column l % kMfmaM of the block (32 x 32: row 8*(v/4) + 4*(l/32) + v%4).
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu = ReluPreMode::NoRelu>
PTO_DEV void tstore_acc(G &dst, TileT &src)
{
    using S = typename TileT::Storage;
    using GT = typename G::DType;
    GT *gm = reinterpret_cast<GT *>(dst.data());
    const int64_t st_r = dst.GetStride(3), st_c = dst.GetStride(4);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const uint32_t lane = (uint32_t)hw::lane();
    const int rbase = hw::wave_m() * (S::MB * kMfmaM) + acc_lane_row(lane);
    const int cbase = hw::wave_n() * (S::NB * kMfmaM) + acc_lane_col(lane);
    constexpr bool full = TileT::ValidRow == TileT::Rows && TileT::ValidCol == TileT::Cols;
#pragma unroll
    for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < S::NB; ++nb) {
            const int c = cbase + nb * kMfmaM;
#pragma unroll
            for (int v = 0; v < kAccElems; ++v) {
                const int r = rbase + mb * kMfmaM + acc_elem_row(v);
                if (full || (r < vr && c < vc)) {
                    GT *p = gm + (int64_t)r * st_r + (int64_t)c * st_c;
                    auto x = src.S().f[mb][nb][v];
                    if constexpr (relu == ReluPreMode::NormalRelu)
                        x = x < 0 ? 0 : x; // before the conversion, as the fix pipe does (a2a3/TStore.hpp:328)
                    if constexpr (atomic == AtomicType::AtomicAdd)
                        atomic_add(p, store_cast<GT>(x));
                    else
                        *p = store_cast<GT>(x);
                }
            }
        }
}

template <typename TileT, typename G>
PTO_DEV void tstore_vec(G &dst, TileT &src)
{
    using T = typename TileT::DType;
    using S = typename TileT::Storage;
    T *gm = reinterpret_cast<T *>(dst.data());
    constexpr int Minor = TileT::isRowMajor ? TileT::Cols : TileT::Rows;
    const int vMajor = TileT::isRowMajor ? src.GetValidRow() : src.GetValidCol();
    const int vMinor = TileT::isRowMajor ? src.GetValidCol() : src.GetValidRow();
    const int64_t stMinor = TileT::isRowMajor ? dst.GetStride(4) : dst.GetStride(3);
    const bool stacked = dst.GetShape(0) * dst.GetShape(1) * dst.GetShape(2) != 1;
    if (G::layout == Layout::NZ || (!TileT::isRowMajor && stacked)) { // as in tload_vec
        const int vr = src.GetValidRow(), vc = src.GetValidCol();
#pragma unroll
        for (int s = 0; s < S::Slots; ++s)
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i) {
                const int e = (s * kBlockThreads + hw::tid()) * kVecChunk + i;
                const int r = TileT::isRowMajor ? e / TileT::Cols : e % TileT::Rows, c = TileT::isRowMajor ? e % TileT::Cols : e / TileT::Rows;
                if (e < TileT::Numel && r < vr && c < vc)
                    gm[gm_elem_offset(dst, r, c)] = src.S().v[s][i];
            }
        return;
    }
#pragma unroll
    for (int s = 0; s < S::Slots; ++s) {
        const int q = s * kBlockThreads + hw::tid();
        if (S::Chunks % kBlockThreads != 0 && q >= S::Chunks)
            continue;
        const int e0 = q * kVecChunk;
        const int major = e0 / Minor, minor0 = e0 % Minor;
        int64_t base;
        if (TileT::isRowMajor)
            base = stacked ? gm_row_offset(dst, major) : (int64_t)major * dst.GetStride(3);
        else
            base = (int64_t)major * dst.GetStride(4);
        if (Minor % kVecChunk == 0 && stMinor == 1 && major < vMajor && minor0 + kVecChunk <= vMinor) {
            typedef T VT __attribute__((ext_vector_type(kVecChunk), aligned(sizeof(T))));
            VT v;
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i)
                v[i] = src.S().v[s][i];
#if defined(PTO_VEC_STREAM_NT) && (PTO_VEC_STREAM_NT & 2)
            __builtin_nontemporal_store(v, reinterpret_cast<VT *>(gm + base + minor0));
#else
            *reinterpret_cast<VT *>(gm + base + minor0) = v;
#endif
        } else {
#pragma unroll
            for (int i = 0; i < kVecChunk; ++i) {
                const int e = e0 + i;
                const int mj = e / Minor, mn = e % Minor;
                if (e < TileT::Numel && mj < vMajor && mn < vMinor) {
                    int64_t b = TileT::isRowMajor ? (stacked ? gm_row_offset(dst, mj) : (int64_t)mj * dst.GetStride(3)) :
                                                    (int64_t)mj * dst.GetStride(4);
                    gm[b + (int64_t)mn * stMinor] = src.S().v[s][i];
                }
            }
        }
    }
}

// LDS Mat tile -> GM, element by element (not on any hot path)
template <typename TileT, typename G>
PTO_DEV void tstore_mat(G &dst, TileT &src)
{
    using T = typename TileT::DType;
    using Geo = MatGeom<TileT>;
    const char *lds = hw::lds_base() + src.st.lds;
    T *gm = reinterpret_cast<T *>(dst.data());
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const bool stacked = dst.GetShape(0) * dst.GetShape(1) * dst.GetShape(2) != 1;
    for (int e = hw::tid(); e < TileT::Numel; e += kBlockThreads) {
        const int r = e / TileT::Cols, c = e % TileT::Cols;
        if (r < vr && c < vc)
            gm[(G::layout == Layout::NZ || stacked) ? gm_elem_offset(dst, r, c) : (int64_t)r * dst.GetStride(3) + (int64_t)c * dst.GetStride(4)] =
                *reinterpret_cast<const T *>(lds + Geo::elem_off(r, c));
    }
}

} // namespace detail

template <typename TileT, typename G, AtomicType atomic = AtomicType::AtomicNone, ReluPreMode relu = ReluPreMode::NoRelu>
PTO_DEV void TSTORE_IMPL(G &dst, TileT &src)
{
    static_assert(relu == ReluPreMode::NoRelu || TileT::Loc == TileType::Acc, "[PTO][SA] TSTORE: ReLU applies to Acc tiles");
    if constexpr (TileT::Loc == TileType::Acc && G::layout == Layout::NZ) {
        detail::tstore_fix<TileT, G, atomic, relu>(dst, src, detail::FixNone{}); // pto/gfx950/fixpipe.hpp
    } else if constexpr (TileT::Loc == TileType::Acc && detail::is_plain_v<TileT>) {
        detail::tstore_any<TileT, G, atomic, relu>(dst, src);
    } else if constexpr (TileT::Loc == TileType::Acc) {
        detail::tstore_acc<TileT, G, atomic, relu>(dst, src);
    } else if constexpr (TileT::Loc == TileType::Vec) {
        static_assert(sizeof(typename TileT::DType) == sizeof(typename G::DType), "[PTO][SA] TSTORE: element sizes differ");
        detail::tstore_vec(dst, src);
    } else if constexpr (TileT::Loc == TileType::Mat) {
        detail::tstore_mat(dst, src);
    } else {
        static_assert(TileT::Loc == TileType::Acc, "[PTO][SA] TSTORE: source must be an Acc, Vec or Mat tile");
    }
}

} // namespace pto
