// Integer helpers that kernel sources take from the reference's include/pto/common/utils.hpp:63-79.
#pragma once
#include "pto/gfx950/platform.hpp"

namespace pto {

PTO_HD constexpr int32_t CeilDivision(int32_t num1, int32_t num2) { return num2 == 0 ? 0 : (num1 + num2 - 1) / num2; }

template <typename T>
PTO_HD constexpr T CeilAlignment(T num1, T num2)
{
    return num2 == 0 ? 0 : (num1 + num2 - 1) / num2 * num2;
}

} // namespace pto
