// pto::Tile for gfx950: the reference's template signature and static members
// (include/pto/common/pto_tile.hpp:1201-1410, aliases :1412-1463) over storage that is native to
// CDNA4 instead of Ascend's L1/L0/UB buffers:
//
//   TileType::Mat    a handle (byte offset, set by TASSIGN) to an LDS-resident tile.  Physical layout:
//                    the contraction dimension is contiguous (columns for an Nz tile, rows for a Zn
//                    tile) and 16-byte chunks are XOR-swizzled so that the ds_read_b128 fragment
//                    loads of TEXTRACT are bank-conflict free.  BLayout/SLayout only select which
//                    logical dimension is the contiguous one.
//   Left/Right       per-wave MFMA operand fragments in VGPRs: [row block][k step] x 8 halves; a block is
//                    PTO_MFMA_M rows, a k step 512 / PTO_MFMA_M columns (32 x 16 or 16 x 32).
//   Acc              per-wave MFMA accumulator fragments: [row block][col block] x (16 or 4) floats.
//   Vec              register tile spread over the workgroup in chunks of 8 consecutive elements of
//                    the tile's linear (BLayout) order: chunk q -> thread q % kBlockThreads, slot q / kBlockThreads.
//
// Copies.  A PTO tile object is a handle, and kernel sources written for Ascend pass tiles by value
// (gemm_performance_kernel.cpp:28 `MatmulAcc(OutTile cTile, ...)`).  A Mat tile copies its LDS offset.  A register
// tile has no address; copying one is a compile error unless the translation unit defines PTO_TILE_COPY_WRITEBACK
// before the include.  Then a COPY takes the registers' values and remembers the tile it was copied from, and hands its
// values back when it goes out of scope: `f(TileAcc c)` updates the caller's accumulator as it does on a machine where
// the tile is an address.  Limits of that mode: the original must outlive its copies, and while a copy is alive the
// original and the copy are not views of each other.  After inlining the transfers are register renames.  (The mode is
// opt-in because a class with a destructor keeps arrays of tiles in memory until late in the optimiser, which costs
// the tuned kernels a few registers.)
//
// Vec tiles in memory.  Kernel sources written for Ascend also treat a Vec tile as an address in the unified buffer: they
// TASSIGN a tile to `other.data() + offset` to get a view of a few rows or columns of another tile, re-view a [R,1] tile
// as [1,R] with TRESHAPE and expect a write through one view to show in the other, and pass tiles by value
// (pto_macro_fa_softmax.hpp:141-215, fa_performance_kernel.cpp:504-515).  A translation unit that defines
// PTO_VEC_TILES_IN_MEMORY before the include gets exactly that: a Vec tile is a handle to `Rows * Cols` elements in the
// reference's storage order inside a per-workgroup unified buffer in global memory (pto/gfx950/ub_mode.hpp); every
// instruction loads its Vec operands from there into the register distribution described above, runs, and writes its
// destination back, followed by a workgroup barrier.  It is the compatibility mode for unmodified sources, several
// times slower than register-resident Vec tiles, which stay the default.
#pragma once
#include "pto/common/types.hpp"
#include "pto/gfx950/platform.hpp"

namespace pto {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

namespace detail {

#if defined(PTO_TILE_COPY_WRITEBACK)
constexpr bool kTileCopyWriteback = true;
#else
constexpr bool kTileCopyWriteback = false;
#endif
#if defined(PTO_VEC_TILES_IN_MEMORY)
constexpr bool kVecTilesInMemory = true;
#else
constexpr bool kVecTilesInMemory = false;
#endif
#if defined(PTO_ACC_TILES_IN_MEMORY)
#if !defined(PTO_VEC_TILES_IN_MEMORY)
#error "PTO_ACC_TILES_IN_MEMORY needs PTO_VEC_TILES_IN_MEMORY (the accumulator images live in the same per-workgroup arena)"
#endif
constexpr bool kAccTilesInMemory = true;
#else
constexpr bool kAccTilesInMemory = false;
#endif

static_assert(PTO_MFMA_M == 32 || PTO_MFMA_M == 16, "v_mfma_f32_32x32x16 or v_mfma_f32_16x16x32");
constexpr int kMfmaM = PTO_MFMA_M;                     // the MFMA's output block is kMfmaM x kMfmaM
constexpr int kMfmaK = 512 / kMfmaM;                   // k extent of one MFMA
constexpr int kAccElems = kMfmaM * kMfmaM / kWaveSize; // accumulator values per lane and block
constexpr int kVecChunk = 8;
typedef float AccFrag __attribute__((ext_vector_type(kAccElems)));
typedef int AccFragI32 __attribute__((ext_vector_type(kAccElems)));
template <typename T>
struct AccFragOf {
    using type = AccFrag;
};
template <>
struct AccFragOf<int32_t> {
    using type = AccFragI32;
};

// Operand layout (both shapes): lane l holds row (column) l % kMfmaM of the block and the eight k values
// 8 * (l / kMfmaM) .. +7 of the step.  Result layout: lane l holds column l % kMfmaM and, in register v,
// row acc_elem_row(v) + acc_lane_row(l) of the block.
PTO_DEV uint32_t frag_lane_major(uint32_t lane) { return lane % kMfmaM; }
PTO_DEV uint32_t frag_lane_kgroup(uint32_t lane) { return lane / kMfmaM; }
PTO_DEV int acc_lane_col(uint32_t lane) { return (int)(lane % kMfmaM); }
PTO_DEV int acc_lane_row(uint32_t lane) { return (int)(lane / kMfmaM) * 4; }
constexpr int acc_elem_row(int v) { return (v >> 2) * (4 * (kWaveSize / kMfmaM)) + (v & 3); }

template <typename T>
struct FragOf {
    using type = u32x4;
};
template <>
struct FragOf<_Float16> {
    using type = f16x8;
};
template <>
struct FragOf<__bf16> {
    using type = bf16x8;
};
template <>
struct FragOf<int8_t> {
    using type = i32x4;
};
template <>
struct FragOf<float> {
    using type = f32x4;
};
// Operand element types of the plain (unscaled) MFMAs.  Whatever the type, a lane holds 16 bytes of its row per
// fragment: 8 fp16 / bf16, 16 int8 or 4 fp32 values; the lanes of a row cover 64 / PTO_MFMA_M such chunks, which is the
// k extent of one fragment (fp16: one MFMA; int8: one MFMA of twice the k; fp32: four MFMAs, MFMA s taking value s of
// every lane's chunk - the same assignment of k to MFMAs on both operands, so the sum over k is unchanged).
template <typename T>
constexpr bool is_mfma_operand_v = std::is_same_v<T, _Float16> || std::is_same_v<T, __bf16> || std::is_same_v<T, int8_t> ||
                                   std::is_same_v<T, float>;
template <typename T>
constexpr int kFragK = (16 / (int)sizeof(T)) * (kWaveSize / kMfmaM);

constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }

struct Empty {};

template <TileType Loc, typename T, int Rows, int Cols>
struct TileStorage { // unsupported locations: no storage
    Empty none;
};

template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Mat, T, Rows, Cols> {
    uint32_t lds = 0;   // byte offset into the workgroup's dynamic LDS ("L1" address 0 = its first byte)
    bool bound = false; // a TASSIGN has given the tile its address
};

template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Scaling, T, Rows, Cols> {
    uint32_t fb = 0; // byte offset into the table of quantisation words (pto/gfx950/fixpipe.hpp)
};

// 8-bit MX operands (v_mfma_scale_f32_32x32x64_f8f6f4): a fragment is 32 rows x 64 k; lane l holds row l % 32 and the
// bytes k = 16 (l / 32) .. +15 (first four registers) and k = 32 + 16 (l / 32) .. +15 (last four).
template <typename T>
constexpr bool is_mx8_v = std::is_same_v<T, float8_e4m3_t> || std::is_same_v<T, float8_e5m2_t>;
template <typename T>
constexpr bool is_mx4_v = std::is_same_v<T, float4_e2m1x2_t>;
template <typename T>
constexpr bool is_mx_operand_v = is_mx8_v<T> || is_mx4_v<T>;
// bits per logical element (extents of 4-bit types count elements, their storage type holds two)
template <typename T>
constexpr int elem_bits = is_mx4_v<T> ? 4 : 8 * (int)sizeof(T);
constexpr int kMxM = 32, kMxK = 64, kMxBlock = 32;
// upper half of the value that data() of a Mat tile returns (the lower half is the tile's L1 byte offset)
constexpr uint64_t kMatHandleTag = 0x4D41540000000000ull; // "MAT"

template <int Rows, int Cols>
struct TileStorage<TileType::Left, float8_e4m3_t, Rows, Cols> {
    static_assert(kMfmaM == kMxM, "MX operand tiles need PTO_MFMA_M 32 (accumulator layout of the 32 x 32 MFMA)");
    static_assert(Rows % (kMxM * kWavesM) == 0 && Cols % kMxK == 0, "MX Left tile: multiples of 32 x PTO_WAVES_M rows, 64 columns");
    static constexpr int MB = Rows / (kMxM * kWavesM), Blocks = MB;
    static constexpr int KS = Cols / kMxK;
    i32x8 f[MB][KS];
};
template <int Rows, int Cols>
struct TileStorage<TileType::Left, float8_e5m2_t, Rows, Cols> : TileStorage<TileType::Left, float8_e4m3_t, Rows, Cols> {};
template <int Rows, int Cols>
struct TileStorage<TileType::Right, float8_e4m3_t, Rows, Cols> {
    static_assert(kMfmaM == kMxM, "MX operand tiles need PTO_MFMA_M 32 (accumulator layout of the 32 x 32 MFMA)");
    static_assert(Cols % (kMxM * kWavesN) == 0 && Rows % kMxK == 0, "MX Right tile: multiples of 32 x PTO_WAVES_N columns, 64 rows");
    static constexpr int NB = Cols / (kMxM * kWavesN), Blocks = NB;
    static constexpr int KS = Rows / kMxK;
    i32x8 f[NB][KS];
};
template <int Rows, int Cols>
struct TileStorage<TileType::Right, float8_e5m2_t, Rows, Cols> : TileStorage<TileType::Right, float8_e4m3_t, Rows, Cols> {};

// 4-bit MX operands: a fragment is 32 rows x 64 k = 32 bytes per row; lane l holds row l % 32 and the 16 bytes
// k = 32 (l / 32) .. +31 (four registers).
template <int Rows, int Cols>
struct TileStorage<TileType::Left, float4_e2m1x2_t, Rows, Cols> {
    static_assert(kMfmaM == kMxM, "MX operand tiles need PTO_MFMA_M 32 (accumulator layout of the 32 x 32 MFMA)");
    static_assert(Rows % (kMxM * kWavesM) == 0 && Cols % kMxK == 0, "MX Left tile: multiples of 32 x PTO_WAVES_M rows, 64 columns");
    static constexpr int MB = Rows / (kMxM * kWavesM), Blocks = MB;
    static constexpr int KS = Cols / kMxK;
    u32x4 f[MB][KS];
};
template <int Rows, int Cols>
struct TileStorage<TileType::Right, float4_e2m1x2_t, Rows, Cols> {
    static_assert(kMfmaM == kMxM, "MX operand tiles need PTO_MFMA_M 32 (accumulator layout of the 32 x 32 MFMA)");
    static_assert(Cols % (kMxM * kWavesN) == 0 && Rows % kMxK == 0, "MX Right tile: multiples of 32 x PTO_WAVES_N columns, 64 rows");
    static constexpr int NB = Cols / (kMxM * kWavesN), Blocks = NB;
    static constexpr int KS = Rows / kMxK;
    u32x4 f[NB][KS];
};

// Block scales of an MX operand tile: one e8m0 value per row (column) and 32-wide k block, KB blocks per row.
// Per 32-row block of its part of the operand a wave holds the scales of the lane's row, four k blocks to a
// register, each register shifted right by 8 bits in lanes 32-63: the MFMA of 64-wide k step s takes the scale of
// k block 2 s (lanes 0-31) / 2 s + 1 (lanes 32-63), which then is byte 0 (s even) or byte 2 (s odd) of register s / 2.
template <typename T, int Rows, int Cols>
struct TileStorage<TileType::ScaleLeft, T, Rows, Cols> {
    static_assert(sizeof(T) == 1 && Cols % 2 == 0 && (Cols == 2 || Cols % 4 == 0) && Rows % (kMxM * kWavesM) == 0,
                  "scale tile: 2 or a multiple of 4 k blocks per row");
    static constexpr int MB = Rows / (kMxM * kWavesM), Blocks = MB;
    static constexpr int KB = Cols, Regs = (Cols + 3) / 4;
    uint32_t s[MB][Regs];
};
template <typename T, int Rows, int Cols>
struct TileStorage<TileType::ScaleRight, T, Rows, Cols> {
    static_assert(sizeof(T) == 1 && Rows % 2 == 0 && (Rows == 2 || Rows % 4 == 0) && Cols % (kMxM * kWavesN) == 0,
                  "scale tile: 2 or a multiple of 4 k blocks per column");
    static constexpr int NB = Cols / (kMxM * kWavesN), Blocks = NB;
    static constexpr int KB = Rows, Regs = (Rows + 3) / 4;
    uint32_t s[NB][Regs];
};

template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Vec, T, Rows, Cols> {
    static constexpr int Chunks = cdiv(Rows * Cols, kVecChunk);
    static constexpr int Slots = cdiv(Chunks, kBlockThreads);
    T v[Slots][kVecChunk];
};

// Left / Right / Acc tiles whose extents are whole MFMA blocks per wave are fragments (below).  Any other extent (the
// reference's own matmul tests use 48 x 64, 16 x 16, 32 x 128 ... tiles with run-time or static valid regions inside:
// tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:28-45) gets the element distribution of a Vec tile, and the
// instructions on such a tile take the general path of pto/gfx950/matmul_any.hpp: correct for every shape, far from the
// speed of the fragment path.  Bias tiles always have it.
template <typename T, int Rows, int Cols>
struct PlainStorage : TileStorage<TileType::Vec, T, Rows, Cols> {
    static constexpr bool kPlain = true;
};
template <typename S, typename = void>
struct is_plain_storage : std::false_type {};
template <typename S>
struct is_plain_storage<S, std::void_t<decltype(S::kPlain)>> : std::true_type {};

template <typename T, int Rows, int Cols>
constexpr bool kLeftFragShaped = is_mfma_operand_v<T> && Rows % (kMfmaM * kWavesM) == 0 && Cols % kFragK<T> == 0;
template <typename T, int Rows, int Cols>
constexpr bool kRightFragShaped = is_mfma_operand_v<T> && Cols % (kMfmaM * kWavesN) == 0 && Rows % kFragK<T> == 0;
template <typename T, int Rows, int Cols>
constexpr bool kAccFragShaped = (std::is_same_v<T, float> || std::is_same_v<T, int32_t>) && Rows % (kMfmaM * kWavesM) == 0 &&
                                Cols % (kMfmaM * kWavesN) == 0;

template <typename T, int Rows, int Cols>
struct LeftFragStorage {
    static constexpr int MB = Rows / (kMfmaM * kWavesM);
    static constexpr int KS = Cols / kFragK<T>;
    typename FragOf<T>::type f[MB][KS];
};
template <typename T, int Rows, int Cols>
struct RightFragStorage {
    static constexpr int NB = Cols / (kMfmaM * kWavesN);
    static constexpr int KS = Rows / kFragK<T>;
    typename FragOf<T>::type f[NB][KS];
};
template <typename T, int Rows, int Cols>
struct AccFragStorage {
    static constexpr int MB = Rows / (kMfmaM * kWavesM);
    static constexpr int NB = Cols / (kMfmaM * kWavesN);
    typename AccFragOf<T>::type f[MB][NB];
};

template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Left, T, Rows, Cols>
    : std::conditional_t<kLeftFragShaped<T, Rows, Cols>, LeftFragStorage<T, Rows, Cols>, PlainStorage<T, Rows, Cols>> {
    static_assert(std::is_arithmetic_v<T> || is_mfma_operand_v<T>, "Left tiles: fp16, bf16, int8 or fp32 operands (fp8 / fp4 for TMATMUL_MX)");
};
template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Right, T, Rows, Cols>
    : std::conditional_t<kRightFragShaped<T, Rows, Cols>, RightFragStorage<T, Rows, Cols>, PlainStorage<T, Rows, Cols>> {
    static_assert(std::is_arithmetic_v<T> || is_mfma_operand_v<T>, "Right tiles: fp16, bf16, int8 or fp32 operands (fp8 / fp4 for TMATMUL_MX)");
};
template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Acc, T, Rows, Cols>
    : std::conditional_t<kAccFragShaped<T, Rows, Cols>, AccFragStorage<T, Rows, Cols>, PlainStorage<T, Rows, Cols>> {
    static_assert(std::is_same_v<T, float> || std::is_same_v<T, int32_t>, "Acc tiles: fp32 or int32 accumulators");
};
template <typename T, int Rows, int Cols>
struct TileStorage<TileType::Bias, T, Rows, Cols> : PlainStorage<T, Rows, Cols> {};

} // namespace detail

template <TileType Loc_, typename Element_, const int Rows_, const int Cols_, const BLayout BFractal_ = BLayout::RowMajor,
          const int RowValid_ = Rows_, const int ColValid_ = Cols_, const SLayout SFractal_ = SLayout::NoneBox,
          const int SFractalSize_ = TileConfig::fractalABSize, const PadValue PadVal_ = PadValue::Null,
          const CompactMode Compact_ = CompactMode::Null>
struct Tile {
    using DType = Element_;
    static constexpr TileType Loc = Loc_;
    static constexpr int Rows = Rows_;
    static constexpr int Cols = Cols_;
    static constexpr int ValidRow = RowValid_;
    static constexpr int ValidCol = ColValid_;
    static constexpr BLayout BFractal = BFractal_;
    static constexpr SLayout SFractal = SFractal_;
    static constexpr int SFractalSize = SFractalSize_;
    static constexpr PadValue PadVal = PadVal_;
    static constexpr CompactMode Compact = Compact_;
    static constexpr int Numel = Rows * Cols;
    static constexpr bool isRowMajor = BFractal_ == BLayout::RowMajor;
    static constexpr int RowStride = isRowMajor ? Cols : 1;
    static constexpr int ColStride = isRowMajor ? 1 : Rows;
    static constexpr bool isBoxedLayout = SFractal_ != SLayout::NoneBox;
    static constexpr bool isInnerRowMajor = SFractal_ == SLayout::RowMajor;
    static constexpr bool isInnerColMajor = SFractal_ == SLayout::ColMajor;
    // box geometry of the reference layouts (16 x 32 B, 32 B x 16, or 16 x 16 for the 1 KiB accumulator box)
    static constexpr int InnerRows =
        SFractalSize_ == TileConfig::fractalCSize ?
            TileConfig::fixedRowSize :
            (isBoxedLayout ? (isInnerRowMajor ? TileConfig::fixedRowSize : TileConfig::alignedSize / (int)sizeof(DType)) : 1);
    static constexpr int InnerCols =
        SFractalSize_ == TileConfig::fractalCSize ?
            TileConfig::fixedColSize :
            (isBoxedLayout ? (isInnerRowMajor ? TileConfig::alignedSize / (int)sizeof(DType) : TileConfig::fixedColSize) : 1);
    static constexpr int InnerNumel = InnerRows * InnerCols;

    static_assert(Rows > 0 && Cols > 0 && ValidRow <= Rows && ValidCol <= Cols, "[PTO][SA] invalid tile extents");
    static_assert(Loc_ == TileType::Vec || Rows_ == 1 || Rows % InnerRows == 0,
                  "[PTO][SA] tile rows must be a multiple of the inner box rows");
    static_assert(Cols % InnerCols == 0, "[PTO][SA] tile cols must be a multiple of the inner box cols");
    // (scale tiles are register tiles of a few bytes per row; a Mat tile of block scales holds multiples of 4 per row)
    static_assert(isBoxedLayout || Loc_ == TileType::ScaleLeft || Loc_ == TileType::ScaleRight ||
                      (isRowMajor ? (Cols * sizeof(DType)) : (Rows * sizeof(DType))) %
                              (Loc_ == TileType::Mat && std::is_same_v<DType, float8_e8m0_t> ? 4 : TileConfig::alignedSize) == 0,
                  "[PTO][SA] unboxed tiles need a 32-byte aligned contiguous extent");

    // The logical dimension that is contiguous in a Mat tile's LDS image: columns unless the tile
    // is a Zn (row-major boxes, column-major inside) or plain column-major tile.
    static constexpr bool colsContiguous = isBoxedLayout ? isInnerRowMajor : isRowMajor;

    using Storage = detail::TileStorage<Loc_, Element_, Rows_, Cols_>;
    Storage st;
    int RowMaskInternal = RowValid_;
    int ColMaskInternal = ColValid_;
    Tile *origin_ = nullptr; // register tiles: set in a copy, the tile it was copied from (values go back on destruction)
    // the object itself is an address: Mat tiles, and Vec tiles of a translation unit that keeps them in memory
    static constexpr bool inMemory = Loc_ == TileType::Vec && detail::kVecTilesInMemory;
    // With PTO_ACC_TILES_IN_MEMORY as well, an Acc tile that was given an address is an address too: every instruction that writes
    // it stores its [Rows, Cols] image (row-major) there and every instruction that reads it loads it from there, so that
    // another Acc tile object TASSIGNed to the same address sees the accumulator (the reference's test kernels multiply
    // in one function and declare the tile again in the next: tests/npu/a2a3/src/st/testcase/tmov_acc2mat).  The values
    // still live in registers in between; the object is not a handle.
    static constexpr bool accInMemory = Loc_ == TileType::Acc && detail::kAccTilesInMemory;
    static constexpr bool isHandle = Loc_ == TileType::Mat || inMemory;
#if defined(PTO_VEC_TILES_IN_MEMORY)
    DType *mem_ = nullptr; // Vec tiles: element 0 of the tile in the unified buffer (nullptr: not assigned, registers only)
#endif

    PTO_HD Tile() {}
    PTO_HD Tile(const Tile &o) : RowMaskInternal(o.RowMaskInternal), ColMaskInternal(o.ColMaskInternal) { Bind(o); }
    PTO_HD Tile &operator=(const Tile &o)
    {
        RowMaskInternal = o.RowMaskInternal;
        ColMaskInternal = o.ColMaskInternal;
        Bind(o);
        return *this;
    }
    // `tile = TileT(validRows, validCols)`: a temporary that no TASSIGN has given an address (and whose registers hold
    // nothing yet) brings its valid extents only; the tile stays where it is.  (The reference's kernels re-shape their
    // TASSIGNed tiles this way per block: mxmatmul_performance_kernel.cpp of a5/matmul_mxfp4_performance :297-307.)
    PTO_HD Tile &operator=(Tile &&o)
    {
        RowMaskInternal = o.RowMaskInternal;
        ColMaskInternal = o.ColMaskInternal;
        if constexpr (Loc_ == TileType::Mat && !inMemory) {
            if (o.st.bound)
                st = o.st;
        }
#if defined(PTO_VEC_TILES_IN_MEMORY)
        if (o.mem_)
            mem_ = o.mem_;
#endif
        return *this;
    }
#if defined(PTO_TILE_COPY_WRITEBACK)
    PTO_HD ~Tile()
    {
        if constexpr (!isHandle)
            if (origin_)
                origin_->st = st;
    }
#endif
    PTO_HD Storage &S() { return st; }
    PTO_HD const Storage &S() const { return st; }
    template <int RM = ValidRow, int CM = ValidCol, std::enable_if_t<RM == DYNAMIC && CM == DYNAMIC, int> = 0>
    PTO_HD Tile(size_t vr, size_t vc) : RowMaskInternal((int)vr), ColMaskInternal((int)vc)
    {}
    template <int RM = ValidRow, int CM = ValidCol, std::enable_if_t<(RM == DYNAMIC) != (CM == DYNAMIC), int> = 0>
    PTO_HD Tile(size_t v)
    {
        if constexpr (RM == DYNAMIC)
            RowMaskInternal = (int)v;
        else
            ColMaskInternal = (int)v;
    }

    PTO_HD constexpr int GetValidRow() const { return ValidRow == DYNAMIC ? RowMaskInternal : ValidRow; }
    PTO_HD constexpr int GetValidCol() const { return ValidCol == DYNAMIC ? ColMaskInternal : ValidCol; }

    // Ascend machine state that kernel sources set through a Left tile (pto_tile.hpp:1373-1401 of the reference).  TF32
    // mode makes the cube unit round fp32 operands to 11 (a2 / a3) or 10 mantissa bits before it multiplies; the fp32
    // MFMAs multiply fp32 operands exactly, which lies inside the TF32 product's own rounding error, so the mode has
    // nothing to switch.  The k-alignment flag is a layout hint of the a3 cube unit.
    PTO_HD void SetMadTF32Mode(RoundMode = RoundMode::CAST_ROUND) {}
    PTO_HD void ResetMadMode() {}
    PTO_HD bool GetKAligned() const { return true; }
    PTO_HD void SetKAligned(bool) {}

    // Mat tiles: pointer to the LDS image (swizzled, see mem_ops.hpp).  Register tiles: their fragments.
    PTO_DEV auto data()
    {
        if constexpr (Loc_ == TileType::Mat) {
            // A handle, not an address to read through (the LDS image is swizzled; TEXTRACT / TMOV / TSTORE read it): the
            // tile's byte offset in the workgroup's "L1" under a tag in the upper half, so that TASSIGN can take
            // `data() + n` apart again with integer arithmetic that the compiler folds.
            return reinterpret_cast<DType *>((uintptr_t)(detail::kMatHandleTag | (uint64_t)st.lds));
        } else {
#if defined(PTO_VEC_TILES_IN_MEMORY)
            if constexpr (inMemory)
                return mem_;
            else
#endif
                return &S();
        }
    }

    // Element `offset` of the tile's linear storage order (pto_tile.hpp:1254-1266 of the reference; Vec tiles only).
    // Every lane of the workgroup makes the call with the same arguments.  SetValue: the lane that holds the element
    // writes it.  GetValue: that lane publishes it through LDS and every lane returns it (two workgroup barriers).
    PTO_DEV void SetValue(const uint32_t offset, const DType val)
    {
        static_assert(Loc_ == TileType::Vec, "[PTO][SA] SetValue / GetValue: Vec tiles");
#if defined(PTO_VEC_TILES_IN_MEMORY)
        if (mem_ != nullptr) { // the tile is an address: one lane writes, the workgroup waits for the store
            if (hw::tid() == 0)
                mem_[offset] = val;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            return;
        }
#endif
        const uint32_t q = offset / detail::kVecChunk, e = offset % detail::kVecChunk;
        if ((uint32_t)hw::tid() == q % kBlockThreads) {
            Storage &s = S();
#pragma unroll
            for (int slot = 0; slot < Storage::Slots; ++slot)
#pragma unroll
                for (int i = 0; i < detail::kVecChunk; ++i)
                    if ((uint32_t)slot == q / kBlockThreads && (uint32_t)i == e)
                        s.v[slot][i] = val;
        }
    }
    PTO_DEV DType GetValue(const uint32_t offset)
    {
        static_assert(Loc_ == TileType::Vec, "[PTO][SA] SetValue / GetValue: Vec tiles");
#if defined(PTO_VEC_TILES_IN_MEMORY)
        if (mem_ != nullptr)
            return mem_[offset];
#endif
        __shared__ DType pto_getvalue_slot;
        const uint32_t q = offset / detail::kVecChunk, e = offset % detail::kVecChunk;
        if ((uint32_t)hw::tid() == q % kBlockThreads) {
            const Storage &s = S();
            DType v = s.v[0][0];
#pragma unroll
            for (int slot = 0; slot < Storage::Slots; ++slot)
#pragma unroll
                for (int i = 0; i < detail::kVecChunk; ++i)
                    if ((uint32_t)slot == q / kBlockThreads && (uint32_t)i == e)
                        v = s.v[slot][i];
            pto_getvalue_slot = v;
        }
        __syncthreads();
        const DType out = pto_getvalue_slot;
        __syncthreads();
        return out;
    }

private:
    PTO_HD void Bind(const Tile &o)
    {
        static_assert(isHandle || detail::kTileCopyWriteback,
                      "[PTO][SA] a register tile (Left / Right / Acc / Vec) was copied: pass it by reference, or define "
                      "PTO_TILE_COPY_WRITEBACK before including pto-inst.hpp to give copies write-back semantics");
        st = o.st;
#if defined(PTO_VEC_TILES_IN_MEMORY)
        mem_ = o.mem_;
#endif
        if constexpr (!isHandle)
            origin_ = const_cast<Tile *>(&o);
    }
};

template <typename E, int R, int C, int RV = R, int CV = C>
using TileLeft = Tile<TileType::Left, E, R, C, BLayout::ColMajor, RV, CV, SLayout::RowMajor, TileConfig::fractalABSize>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileLeftCompact = Tile<TileType::Left, E, R, C, BLayout::ColMajor, RV, CV, SLayout::RowMajor,
                             TileConfig::fractalABSize, PadValue::Null, CompactMode::Normal>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileRight = Tile<TileType::Right, E, R, C, BLayout::RowMajor, RV, CV, SLayout::ColMajor, TileConfig::fractalABSize>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileRightCompact = Tile<TileType::Right, E, R, C, BLayout::RowMajor, RV, CV, SLayout::ColMajor,
                              TileConfig::fractalABSize, PadValue::Null, CompactMode::Normal>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileAcc = Tile<TileType::Acc, E, R, C, BLayout::ColMajor, RV, CV, SLayout::RowMajor, TileConfig::fractalCSize>;
// block scales of MX operands (pto_tile.hpp:1441-1456): [rows, k / 32] for the left operand, [k / 32, cols] for the right
template <typename E, int R, int C, int RV = R, int CV = C>
using TileLeftScale = Tile<TileType::ScaleLeft, E, R, C, BLayout::RowMajor, RV, CV, SLayout::NoneBox>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileRightScale = Tile<TileType::ScaleRight, E, R, C, BLayout::ColMajor, RV, CV, SLayout::NoneBox>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileLeftScaleCompact = Tile<TileType::ScaleLeft, E, R, C, BLayout::RowMajor, RV, CV, SLayout::NoneBox, TileConfig::fractalABSize,
                                  PadValue::Null, CompactMode::Normal>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileRightScaleCompact = Tile<TileType::ScaleRight, E, R, C, BLayout::ColMajor, RV, CV, SLayout::NoneBox, TileConfig::fractalABSize,
                                   PadValue::Null, CompactMode::Normal>;
template <typename E, int R, int C, int RV = R, int CV = C>
using TileAccCompact = Tile<TileType::Acc, E, R, C, BLayout::ColMajor, RV, CV, SLayout::RowMajor,
                            TileConfig::fractalCSize, PadValue::Null, CompactMode::Normal>;

template <typename T>
struct is_tile : std::false_type {};
template <TileType L, typename E, int R, int C, BLayout B, int RV, int CV, SLayout S, int F, PadValue P, CompactMode M>
struct is_tile<Tile<L, E, R, C, B, RV, CV, S, F, P, M>> : std::true_type {};
template <typename T>
constexpr bool is_tile_data_v = is_tile<std::remove_cv_t<std::remove_reference_t<T>>>::value;

} // namespace pto
