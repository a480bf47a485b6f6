// Shape / Stride / GlobalTensor: 5-D views of device memory with static or run-time extents.
// API surface of include/pto/common/pto_tile.hpp:26-616 in the reference (Shape, Stride,
// GlobalTensor, TileShape2D, BaseShape2D); the implementation is one generic 5-tuple.
#pragma once
#include "pto/common/types.hpp"
#include "pto/gfx950/platform.hpp"

namespace pto {

namespace detail {
// Five extents, each fixed at compile time or (DYNAMIC) taken from the constructor, in order.
template <int64_t... N>
struct Dims5 {
    static_assert(sizeof...(N) == 5, "five dimensions");
    static constexpr int64_t fixed[5] = {N...};
    static constexpr int numDynamic = ((N == DYNAMIC ? 1 : 0) + ...);
    int64_t v[5];

    PTO_HD constexpr Dims5() : v{(N == DYNAMIC ? 1 : N)...} {}
    PTO_HD constexpr Dims5(int64_t a, int64_t b, int64_t c, int64_t d, int64_t e) : v{a, b, c, d, e}
    {
        for (int i = 0; i < 5; ++i)
            if (fixed[i] != DYNAMIC)
                v[i] = fixed[i];
    }
    // Fewer arguments: they fill the DYNAMIC slots from left to right.
    template <typename... A, typename = std::enable_if_t<(sizeof...(A) >= 1 && sizeof...(A) <= 4)>>
    PTO_HD constexpr Dims5(A... args) : v{(N == DYNAMIC ? 1 : N)...}
    {
        static_assert(sizeof...(A) == numDynamic, "argument count must equal the number of DYNAMIC dimensions");
        const int64_t in[] = {static_cast<int64_t>(args)...};
        int k = 0;
        for (int i = 0; i < 5; ++i)
            if (fixed[i] == DYNAMIC)
                v[i] = in[k++];
    }
    PTO_HD constexpr int64_t get(int i) const { return fixed[i] != DYNAMIC ? fixed[i] : v[i]; }
};
} // namespace detail

template <int64_t N1 = DYNAMIC, int64_t N2 = DYNAMIC, int64_t N3 = DYNAMIC, int64_t N4 = DYNAMIC, int64_t N5 = DYNAMIC>
struct Shape : detail::Dims5<N1, N2, N3, N4, N5> {
    using Base = detail::Dims5<N1, N2, N3, N4, N5>;
    static constexpr int64_t staticShape[5] = {N1, N2, N3, N4, N5};
    PTO_HD constexpr Shape() : Base() {}
    // declared here rather than inherited: `pto::Shape(1, 1, 1, rows, cols)` without template arguments then names the
    // all-dynamic type, as with the reference's constructors (pto_tile.hpp:26-131)
    PTO_HD constexpr Shape(int64_t a, int64_t b, int64_t c, int64_t d, int64_t e) : Base(a, b, c, d, e) {}
    PTO_HD constexpr Shape(int64_t a, int64_t b, int64_t c, int64_t d) : Base(a, b, c, d) {}
    PTO_HD constexpr Shape(int64_t a, int64_t b, int64_t c) : Base(a, b, c) {}
    PTO_HD constexpr Shape(int64_t a, int64_t b) : Base(a, b) {}
    PTO_HD constexpr explicit Shape(int64_t a) : Base(a) {}
};

template <int64_t N1 = DYNAMIC, int64_t N2 = DYNAMIC, int64_t N3 = DYNAMIC, int64_t N4 = DYNAMIC, int64_t N5 = DYNAMIC>
struct Stride : detail::Dims5<N1, N2, N3, N4, N5> {
    using Base = detail::Dims5<N1, N2, N3, N4, N5>;
    static constexpr int64_t staticStride[5] = {N1, N2, N3, N4, N5};
    PTO_HD constexpr Stride() : Base() {}
    // declared here rather than inherited: `pto::Stride(1, 1, 1, rows, cols)` without template arguments then names the
    // all-dynamic type, as with the reference's constructors (pto_tile.hpp:26-131)
    PTO_HD constexpr Stride(int64_t a, int64_t b, int64_t c, int64_t d, int64_t e) : Base(a, b, c, d, e) {}
    PTO_HD constexpr Stride(int64_t a, int64_t b, int64_t c, int64_t d) : Base(a, b, c, d) {}
    PTO_HD constexpr Stride(int64_t a, int64_t b, int64_t c) : Base(a, b, c) {}
    PTO_HD constexpr Stride(int64_t a, int64_t b) : Base(a, b) {}
    PTO_HD constexpr explicit Stride(int64_t a) : Base(a) {}
};

// [1,1,1,rows,cols] extent of one 2-D tile in memory (pto_tile.hpp:452-556, ND and DN forms).
template <typename T, int64_t rows = DYNAMIC, int64_t cols = DYNAMIC, Layout L = Layout::ND>
struct TileShape2D : Shape<1, 1, 1, rows, cols> {
    using Parent = Shape<1, 1, 1, rows, cols>;
    using Parent::Parent;
    PTO_HD constexpr TileShape2D() : Parent() {}
};

// Strides of a dense [rows, cols] matrix holding such tiles: ND = row-major (.., cols, 1),
// DN = column-major (.., 1, rows)   (pto_tile.hpp:588-616).
namespace detail {
template <int64_t r, int64_t c>
constexpr int64_t mulOrDyn = (r == DYNAMIC || c == DYNAMIC) ? DYNAMIC : r * c;
}
template <typename T, int64_t rows = DYNAMIC, int64_t cols = DYNAMIC, Layout L = Layout::ND>
struct BaseShape2D;
template <typename T, int64_t rows, int64_t cols>
struct BaseShape2D<T, rows, cols, Layout::ND>
    : Stride<detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, cols, 1> {
    using Parent = Stride<detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, cols, 1>;
    PTO_HD constexpr BaseShape2D() : Parent() {}
    PTO_HD constexpr BaseShape2D(int64_t r, int64_t c) : Parent(r * c, r * c, r * c, c, 1) {}
};
template <typename T, int64_t rows, int64_t cols>
struct BaseShape2D<T, rows, cols, Layout::DN>
    : Stride<detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, 1, rows> {
    using Parent = Stride<detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, detail::mulOrDyn<rows, cols>, 1, rows>;
    PTO_HD constexpr BaseShape2D() : Parent() {}
    PTO_HD constexpr BaseShape2D(int64_t r, int64_t c) : Parent(r * c, r * c, r * c, 1, r) {}
};

// block-scale matrices of MX operands (pto_tile.hpp:651-680, 776-805): dense, the k-block index contiguous
template <typename T, int64_t rows, int64_t cols>
struct BaseShape2D<T, rows, cols, Layout::MX_A_ND> : BaseShape2D<T, rows, cols, Layout::ND> {
    using BaseShape2D<T, rows, cols, Layout::ND>::BaseShape2D;
};
template <typename T, int64_t rows, int64_t cols>
struct BaseShape2D<T, rows, cols, Layout::MX_B_DN> : BaseShape2D<T, rows, cols, Layout::DN> {
    using BaseShape2D<T, rows, cols, Layout::DN>::BaseShape2D;
};

template <typename Element_, typename Shape_, typename Stride_, Layout Layout_ = Layout::ND>
struct GlobalTensor {
    using Shape = Shape_;
    using Stride = Stride_;
    using RawDType = Element_;
    using DType = Element_;
    static constexpr Layout layout = Layout_;
    static constexpr int64_t staticShape[5] = {Shape_::fixed[0], Shape_::fixed[1], Shape_::fixed[2], Shape_::fixed[3],
                                               Shape_::fixed[4]};
    static constexpr int64_t staticStride[5] = {Stride_::fixed[0], Stride_::fixed[1], Stride_::fixed[2],
                                                Stride_::fixed[3], Stride_::fixed[4]};

    PTO_HD GlobalTensor() : data_(nullptr) {}
    PTO_HD GlobalTensor(DType *p) : data_(p) {}
    PTO_HD GlobalTensor(DType *p, const Shape_ &s) : data_(p), shape_(s) {}
    PTO_HD GlobalTensor(DType *p, const Shape_ &s, const Stride_ &st) : data_(p), shape_(s), stride_(st) {}

    PTO_HD int64_t GetShape(int dim) const { return shape_.get(dim); }
    PTO_HD int64_t GetStride(int dim) const { return stride_.get(dim); }
    template <int dim>
    PTO_HD static constexpr int64_t GetShape()
    {
        static_assert(staticShape[dim] != DYNAMIC, "dimension is dynamic: use GetShape(dim)");
        return staticShape[dim];
    }
    template <int dim>
    PTO_HD static constexpr int64_t GetStride()
    {
        static_assert(staticStride[dim] != DYNAMIC, "stride is dynamic: use GetStride(dim)");
        return staticStride[dim];
    }
    PTO_HD DType *data() const { return data_; }
    PTO_HD void SetAddr(DType *p) { data_ = p; }

private:
    DType *data_;
    Shape_ shape_{};
    Stride_ stride_{};
};

template <typename T>
struct is_global : std::false_type {};
template <typename E, typename S, typename St, Layout L>
struct is_global<GlobalTensor<E, S, St, L>> : std::true_type {};
template <typename T>
constexpr bool is_global_data_v = is_global<std::remove_cv_t<std::remove_reference_t<T>>>::value;

} // namespace pto
