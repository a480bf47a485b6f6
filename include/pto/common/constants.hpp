// Constants that kernel sources include alongside <pto/pto-inst.hpp>
// (the reference's include/pto/common/constants.hpp).  The gfx950 build needs none beyond the
// enumerations and the buffer sizes below.
#pragma once
#include "pto/common/types.hpp"

namespace pto {
constexpr int BLOCK_BYTE_SIZE = 32;
constexpr int C0_SIZE_BYTE = 32;
constexpr int FRACTAL_NZ_ROW = 16;
// On-chip capacities one workgroup can address on a CU of MI355X.
constexpr int PTO_LDS_BYTES = 160 * 1024;
} // namespace pto
