// Constants that kernel sources include alongside <pto/pto-inst.hpp>
// (the reference's include/pto/common/constants.hpp).  The gfx950 build needs none beyond the
// enumerations and the buffer sizes below.
#pragma once
#include "pto/common/types.hpp"

namespace pto {
// Sizes of the Ascend memory hierarchy that kernel and test sources name (the reference's constants.hpp:17-42): a
// 32-byte block, 8 blocks / 256 bytes per vector repeat, 512-byte cube fractals.  Nothing on gfx950 depends on them.
constexpr int REPEAT_BYTE = 256;
constexpr int REPEAT_MAX = 255;
constexpr int BLOCK_BYTE_SIZE = 32;
constexpr int REPEAT_STRIDE_MAX = 255;
constexpr uint64_t BLOCK_MAX_PER_REPEAT = 8;
constexpr uint64_t MASK_LEN = 64;
constexpr int BLOCK_LEN = 16;
constexpr int CUBE_BLOCK_SIZE = 512;
constexpr int C0_SIZE_BYTE = 32;
constexpr int FRACTAL_NZ_ROW = 16;
constexpr int ACC_C0_SIZE = 16;
constexpr int MX_BLOCK_SIZE = 32;

// Name of a tile type's layout pair (type.hpp:235-243, constants.hpp:248-267 of the reference)
enum class TileLayoutCustom : uint8_t { ND, DN, NZ, ZN, ZZ, NONE };
template <typename TileData>
constexpr TileLayoutCustom GetTileLayoutCustom()
{
    if constexpr (TileData::SFractal == SLayout::NoneBox)
        return TileData::isRowMajor ? TileLayoutCustom::ND : TileLayoutCustom::DN;
    else if constexpr (!TileData::isRowMajor && TileData::SFractal == SLayout::RowMajor)
        return TileLayoutCustom::NZ;
    else if constexpr (TileData::isRowMajor && TileData::SFractal == SLayout::ColMajor)
        return TileLayoutCustom::ZN;
    else if constexpr (TileData::isRowMajor && TileData::SFractal == SLayout::RowMajor)
        return TileLayoutCustom::ZZ;
    else
        return TileLayoutCustom::NONE;
}
// On-chip capacities one workgroup can address on a CU of MI355X.
constexpr int PTO_LDS_BYTES = 160 * 1024;
} // namespace pto
