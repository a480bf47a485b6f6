// Enumerations and scalar types of the PTO tile API, gfx950 build.
// Names and enumerator values follow the reference's public API so that kernel sources written
// against it keep compiling: include/pto/common/memory.hpp:19-43 (TileType, BLayout, SLayout) and
// include/pto/common/type.hpp:96-243 (MaskPattern ... CompactMode).
#pragma once
#include <cstddef>
#include <cstdint>
#include <type_traits>

namespace pto {

using half = _Float16;
using bfloat16_t = __bf16;
// 8-bit storage types of the MX formats (element types of `TMATMUL_MX` operands and their block scales)
struct float8_e4m3_t { uint8_t bits; };
struct float8_e5m2_t { uint8_t bits; };
struct float8_e8m0_t { uint8_t bits; }; // a power of two: 2^(bits - 127)
// two 4-bit e2m1 values (0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives): element 2i in bits 0-3, element 2i+1 in bits 4-7.
// Tile and GlobalTensor extents of this type count 4-bit elements; pointers to it advance by two elements.
struct float4_e2m1x2_t { uint8_t bits; };

constexpr int DYNAMIC = -1;

enum class TileType { Vec, Mat, Left, Right, Acc, Bias, Scaling, ScaleLeft, ScaleRight };
enum class BLayout { RowMajor = 0, ColMajor = 1 };
enum class SLayout { NoneBox = 0, RowMajor = 1, ColMajor = 2 };

// MX_A_ND / MX_B_DN: block scales of an MX matmul in memory, [rows, k / 32] row-major for the left operand and
// [k / 32, cols] column-major for the right one (type.hpp:114-119)
enum class Layout { ND, DN, NZ, MX_A_ND, MX_B_DN };

enum class MaskPattern : uint8_t { P0101 = 1, P1010 = 2, P0001 = 3, P0010 = 4, P0100 = 5, P1000 = 6, P1111 = 7 };
enum class CmpMode : uint8_t { EQ = 0, NE = 1, LT = 2, LE = 3, GT = 4, GE = 5 };
enum class STPhase : uint8_t { Unspecified = 0x0, Partial = 0x2, Final = 0x3 };
enum class AccPhase : uint8_t { Unspecified = 0x0, Unknown = Unspecified, Partial = 0x2, Final = 0x3 };
enum class RoundMode : uint8_t {
    CAST_NONE = 0,
    CAST_RINT = 1,  // nearest, ties to even
    CAST_ROUND = 2, // nearest, ties away from zero
    CAST_FLOOR = 3,
    CAST_CEIL = 4,
    CAST_TRUNC = 5,
    CAST_ODD = 6,
};
enum class AccToVecMode : uint8_t { SingleModeVec0 = 0, SingleModeVec1 = 1, DualModeSplitM = 2, DualModeSplitN = 3 };
enum class ReluPreMode : uint8_t { NoRelu = 0, NormalRelu = 1 };
enum class AtomicType : uint8_t { AtomicNone = 0, AtomicAdd = 1 };
enum class PadValue { Null, Zero, Max, Min };
enum class SaturationMode : uint8_t { ON = 0, OFF = 1 };
enum class CompactMode { Null, Normal };

namespace GlobalTensorDim {
constexpr int DIM_0 = 0, DIM_1 = 1, DIM_2 = 2, DIM_3 = 3, DIM_4 = 4, TOTAL_DIM = 5;
}

// Box ("fractal") geometry of the reference tile layouts (pto_tile.hpp:807-813).  On gfx950 the
// physical placement of a tile is free; these only feed the static shape checks and InnerRows/Cols.
struct TileConfig {
    static constexpr int alignedSize = 32;
    static constexpr int fixedRowSize = 16;
    static constexpr int fixedColSize = 16;
    static constexpr int fractalABSize = 512;
    static constexpr int fractalCSize = 1024;
};

} // namespace pto
