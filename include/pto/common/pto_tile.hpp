// Tile, GlobalTensor and their shape types under the header name that kernel sources written for the reference include
// (include/pto/common/pto_tile.hpp of the reference: Shape / Stride / GlobalTensor :26-442, TileShape2D / BaseShape2D
// :452-616, Tile :1201-1410, the Left / Right / Acc aliases :1412-1463, GetTileOffset :1522-1552).
#pragma once
#include "pto/common/global_tensor.hpp"
#include "pto/common/tile.hpp"

namespace pto {

// Element offset of logical element (row, col) in the storage order that the reference's tile layouts define
// (plain row / column major, or 512-byte boxes in Nz / Zn / Zz order).  The LDS image of a Mat tile on gfx950 is NOT in
// this order (mem_ops.hpp): the function serves code that computes reference offsets, e.g. for SetValue / GetValue on
// unboxed Vec tiles, where the two orders coincide.
template <typename TileT>
PTO_HD constexpr size_t GetTileOffset(int row, int col)
{
    static_assert(is_tile_data_v<TileT>, "[PTO][SA] GetTileOffset: a Tile type");
    if constexpr (!TileT::isBoxedLayout) {
        return (size_t)(row * TileT::RowStride + col * TileT::ColStride);
    } else {
        const int br = row / TileT::InnerRows, bc = col / TileT::InnerCols;
        const int ir = row % TileT::InnerRows, ic = col % TileT::InnerCols;
        constexpr int nbr = TileT::Rows / TileT::InnerRows, nbc = TileT::Cols / TileT::InnerCols;
        if constexpr (!TileT::isRowMajor && TileT::isInnerRowMajor) // Nz
            return (size_t)((nbr * bc + br) * TileT::InnerNumel + ir * TileT::InnerCols + ic);
        else if constexpr (TileT::isRowMajor && TileT::isInnerColMajor) // Zn
            return (size_t)((nbc * br + bc) * TileT::InnerNumel + ic * TileT::InnerRows + ir);
        else if constexpr (TileT::isRowMajor && TileT::isInnerRowMajor) // Zz
            return (size_t)((nbc * br + bc) * TileT::InnerNumel + ir * TileT::InnerCols + ic);
        else
            static_assert(sizeof(TileT) == 0, "[PTO][SA] boxed tiles are Nz, Zn or Zz");
    }
}

} // namespace pto
