// TileType, BLayout and SLayout under the header name of the reference (include/pto/common/memory.hpp:19-43).
#pragma once
#include "pto/common/types.hpp"
