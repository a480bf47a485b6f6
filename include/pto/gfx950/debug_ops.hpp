// TPRINT: a Vec tile or a GlobalTensor written to the host's standard output through the device's printf, by one lane,
// in the reference's format (npu/a2a3/TPrint.hpp:44-190: a header line, the shape, one line per row with a `|` after
// the last valid column and a line of dashes after the last valid row; floating-point values as %6.2f, integers as %6d).
// A debugging aid: every value is one call to the host.
#pragma once
#include <cstdio>

#include "pto/gfx950/vec_ops.hpp"

namespace pto {
namespace detail {

template <typename T>
PTO_DEV const char *print_type_name()
{
    if constexpr (std::is_same_v<T, float>)
        return "float32";
    else if constexpr (std::is_same_v<T, half>)
        return "float16";
    else if constexpr (std::is_same_v<T, bfloat16_t>)
        return "bfloat16";
    else if constexpr (std::is_integral_v<T>)
        return std::is_signed_v<T> ? (sizeof(T) == 4 ? "int32" : sizeof(T) == 2 ? "int16" : sizeof(T) == 1 ? "int8" : "int64") :
                                     (sizeof(T) == 4 ? "uint32" : sizeof(T) == 2 ? "uint16" : sizeof(T) == 1 ? "uint8" : "uint64");
    else
        return "unknown";
}

template <typename T>
PTO_DEV void print_value(T v, int col)
{
    if (col > 0)
        printf(" ");
    if constexpr (std::is_integral_v<T>)
        printf("%6d", (int)v);
    else
        printf("%6.2f", (double)(float)v);
}

} // namespace detail

template <typename T>
PTO_DEV void TPRINT_IMPL(T &src)
{
    if constexpr (is_global_data_v<T>) {
        using E = typename T::DType;
        if (hw::tid() == 0) {
            const int n0 = src.GetShape(0), n1 = src.GetShape(1), n2 = src.GetShape(2), n3 = src.GetShape(3), n4 = src.GetShape(4);
            const E *p = src.data();
            if constexpr (T::layout == Layout::NZ) {
                printf("=== [TPRINT GlobalTensor] Data Type: %s, Layout: %s ===\n", detail::print_type_name<E>(), "NZ");
                printf("  Logical Shape: [%d, %d]\n", n2 * n3, n0 * n1 * n4);
                for (int r = 0; r < n2 * n3; ++r) {
                    for (int c = 0; c < n0 * n1 * n4; ++c)
                        detail::print_value(p[detail::gm_elem_offset(src, r, c)], c);
                    printf("\n");
                }
            } else {
                printf("=== [TPRINT GlobalTensor] Data Type: %s, Layout: %s ===\n", detail::print_type_name<E>(), T::layout == Layout::ND ? "ND" : "DN");
                printf("  Shape: [%d, %d, %d, %d, %d]\n", n0, n1, n2, n3, n4);
                for (int i0 = 0; i0 < n0; ++i0)
                    for (int i1 = 0; i1 < n1; ++i1)
                        for (int i2 = 0; i2 < n2; ++i2) {
                            printf("  Batch [%d, %d, %d]:\n", i0, i1, i2);
                            for (int r = 0; r < n3; ++r) {
                                for (int c = 0; c < n4; ++c)
                                    detail::print_value(p[(int64_t)i0 * src.GetStride(0) + (int64_t)i1 * src.GetStride(1) + (int64_t)i2 * src.GetStride(2) +
                                                          (int64_t)r * src.GetStride(3) + (int64_t)c * src.GetStride(4)],
                                                        c);
                                printf("\n");
                            }
                        }
            }
        }
    } else {
        static_assert(T::Loc == TileType::Vec, "[PTO][SA] TPRINT: a Vec tile or a GlobalTensor");
        using E = typename T::DType;
        constexpr int kBytes = (int)sizeof(E) * T::Numel;
        E *lds = reinterpret_cast<E *>(detail::conform_buffer<(kBytes + 1023) / 1024 * 1024>());
        detail::for_each_owned<T>([&](int s, int i, int e) {
            if (e < T::Numel) {
                int r, c;
                detail::elem_rc<T>(e, r, c);
                lds[r * T::Cols + c] = src.S().v[s][i];
            }
        });
        hw::lds_barrier();
        if (hw::tid() == 0) {
            const int vr = src.GetValidRow(), vc = src.GetValidCol();
            printf("=== [TPRINT Tile] Data Type: %s, Layout: %s, TileType: %s ===\n", detail::print_type_name<E>(),
                   T::isRowMajor ? "RowMajor" : "ColMajor", "Vec");
            printf("  Shape: [%d, %d], Valid Shape: [%d, %d]\n", T::Rows, T::Cols, vr, vc);
            for (int r = 0; r < T::Rows; ++r) {
                for (int c = 0; c < T::Cols; ++c) {
                    detail::print_value(lds[r * T::Cols + c], c);
                    if (c == vc - 1 && vc > 0 && vc < T::Cols)
                        printf("|");
                }
                printf("\n");
                if (r == vr - 1 && vr > 0 && vr < T::Rows) {
                    for (int c = 0; c < T::Cols; ++c) {
                        printf(c > 0 ? " ------" : "------");
                        if (c == vc - 1 && vc > 0 && vc < T::Cols)
                            printf("|");
                    }
                    printf("\n");
                }
            }
        }
        hw::lds_barrier();
    }
}

} // namespace pto
