// Matmul tiles of any extent: the general path of TMOV / TEXTRACT / TMATMUL* / TGEMV* / TSTORE / TLOAD for Left, Right,
// Acc and Bias tiles that are not whole MFMA blocks per wave, and for operands with a valid region inside the tile.
//
// The reference's own tests of these instructions use such tiles throughout: valid m, k, n of 40 x 50 x 60, 6 x 7 x 8,
// 127 x 128 x 63, 1 x 200 x 32 ... inside tiles rounded up to 16 rows and 32 bytes (tests/cpu/st/testcase/tmatmul/
// tmatmul_kernel.cpp:28-45, tests/npu/a2a3/src/st/testcase/tmatmul/tmatmul_kernel.cpp:27-36).  Semantics
// (include/pto/cpu/TMatmul.hpp:73-116): C[i,j] = (acc ? acc[i,j] : 0) + sum_k (CT)A[i,k] (CT)B[k,j] (+ bias[j]) over
// m, k, n = a.validRow, a.validCol, b.validCol, k ascending.
//
// A tile with plain storage (pto/common/tile.hpp: PlainStorage) is spread over the workgroup element by element like a Vec
// tile.  A matmul with any plain operand passes A and B through LDS in chunks of k ([m][kc] and [n][kc]) and every lane
// computes the elements of C it holds, whatever C's storage, with the reference's sequential k loop.  Fragment tiles take part through
// for_each_elem, which knows which (row, column) every lane's registers hold.
#pragma once
#include "pto/gfx950/matmul.hpp"
#include "pto/gfx950/mem_ops.hpp"
#include "pto/gfx950/vec_ops.hpp"

namespace pto {
namespace detail {

// Visit every element that this lane holds of a Left / Right / Acc / Bias tile: value = fn(row, col, value, owner).
// `owner` is false in the waves that hold a replica (the Left fragments of one row block are held by every wave of that
// row of the wave grid, the Right fragments by every wave of a column): exactly one lane of the workgroup sees each
// element with owner == true.
template <typename TileT, typename F>
PTO_DEV void for_each_elem(TileT &t, F &&fn)
{
    using T = typename TileT::DType;
    using S = typename TileT::Storage;
    if constexpr (is_plain_v<TileT>) {
        for_each_owned<TileT>([&](int s, int i, int e) {
            if (e < TileT::Numel) {
                int r, c;
                elem_rc<TileT>(e, r, c);
                t.S().v[s][i] = fn(r, c, t.S().v[s][i], true);
            }
        });
    } else if constexpr (TileT::Loc == TileType::Left || TileT::Loc == TileType::Right) {
        constexpr bool left = TileT::Loc == TileType::Left;
        constexpr int per = 16 / (int)sizeof(T); // elements of the lane's 16-byte chunk of a fragment
        const uint32_t lane = (uint32_t)hw::lane();
        const int l32 = (int)frag_lane_major(lane), kg = (int)frag_lane_kgroup(lane);
        const bool owner = left ? hw::wave_n() == 0 : hw::wave_m() == 0;
        constexpr int blocks = [] {
            if constexpr (left)
                return S::MB;
            else
                return S::NB;
        }();
        const int major0 = (left ? hw::wave_m() : hw::wave_n()) * (blocks * kMfmaM) + l32;
#pragma unroll
        for (int b = 0; b < blocks; ++b)
#pragma unroll
            for (int ks = 0; ks < S::KS; ++ks) {
                T tmp[per];
                __builtin_memcpy(tmp, &t.S().f[b][ks], 16);
#pragma unroll
                for (int j = 0; j < per; ++j) {
                    const int major = major0 + b * kMfmaM, k = ks * kFragK<T> + kg * per + j;
                    tmp[j] = left ? fn(major, k, tmp[j], owner) : fn(k, major, tmp[j], owner);
                }
                __builtin_memcpy(&t.S().f[b][ks], tmp, 16);
            }
    } else {
        static_assert(TileT::Loc == TileType::Acc, "[PTO][SA] for_each_elem: Left, Right, Acc or Bias tile");
        const uint32_t lane = (uint32_t)hw::lane();
        const int r0 = hw::wave_m() * (S::MB * kMfmaM) + acc_lane_row(lane), c0 = hw::wave_n() * (S::NB * kMfmaM) + acc_lane_col(lane);
#pragma unroll
        for (int mb = 0; mb < S::MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < S::NB; ++nb)
#pragma unroll
                for (int v = 0; v < kAccElems; ++v)
                    t.S().f[mb][nb][v] = fn(r0 + mb * kMfmaM + acc_elem_row(v), c0 + nb * kMfmaM, (T)t.S().f[mb][nb][v], true);
    }
}

// staging buffers of the general path; one per role, shared by every instantiation that asks for the same size
template <int Role, int Bytes>
PTO_DEV char *any_buffer()
{
    __shared__ __attribute__((aligned(16))) char buf[Bytes];
    return buf;
}
constexpr int any_round(int bytes) { return (bytes + 4095) / 4096 * 4096; }

// zero what lies outside the valid region of an operand tile (the products over the padding then add nothing)
template <typename TileT>
PTO_DEV void zero_outside_valid(TileT &t)
{
    using T = typename TileT::DType;
    const int vr = t.GetValidRow(), vc = t.GetValidCol();
    for_each_elem(t, [&](int r, int c, T v, bool) { return (r < vr && c < vc) ? v : T(0); });
}

// Mat -> plain Left / Right / Bias tile: dst[i,j] = src[idxRow + i, idxCol + j] inside dst's valid region, 0 outside
template <typename DstT, typename SrcT>
PTO_DEV void textract_any(DstT &dst, SrcT &src, uint32_t idxRow, uint32_t idxCol)
{
    static_assert(SrcT::Loc == TileType::Mat, "[PTO][SA] TEXTRACT / TMOV: source must be a Mat tile");
    static_assert(sizeof(typename DstT::DType) == sizeof(typename SrcT::DType), "[PTO][SA] TEXTRACT: dtype mismatch");
    using T = typename DstT::DType;
    using Geo = MatGeom<SrcT>;
    const char *lds = hw::lds_base() + src.st.lds;
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    for_each_elem(dst, [&](int r, int c, T, bool) {
        const uint32_t sr = idxRow + (uint32_t)r, sc = idxCol + (uint32_t)c;
        if (r < vr && c < vc && sr < (uint32_t)SrcT::Rows && sc < (uint32_t)SrcT::Cols)
            return *reinterpret_cast<const T *>(lds + Geo::elem_off(sr, sc));
        return T(0);
    });
}

// GM -> plain tile (the CPU form of a bias load: TLOAD(biasTile, global), tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:87)
template <typename TileT, typename G>
PTO_DEV void tload_any(TileT &dst, G &src)
{
    using T = typename TileT::DType;
    const T *gm = reinterpret_cast<const T *>(src.data());
    const int64_t st_r = src.GetStride(3), st_c = src.GetStride(4);
    const int vr = dst.GetValidRow(), vc = dst.GetValidCol();
    for_each_elem(dst, [&](int r, int c, T, bool) { return (r < vr && c < vc) ? gm[(int64_t)r * st_r + (int64_t)c * st_c] : T(0); });
}

// The extents of the three tiles need not agree (the GEMV forms pair a [1, k'] Left tile with a [16, n] accumulator and a
// [k, n] Right tile, k' and k rounded up differently: tmatmul_kernel.cpp:326-333 of the NPU tests): m, k, n are the valid
// extents, which must fit every tile they index.
template <bool kZeroInit, typename AccT, typename LeftT, typename RightT>
PTO_DEV void mad_any(AccT &out, AccT &in, LeftT &a, RightT &b)
{
    using A = typename LeftT::DType;
    using B = typename RightT::DType;
    using CT = typename AccT::DType;
    static_assert(sizeof(A) == sizeof(B), "[PTO][SA] TMATMUL: operands of one element size");
    constexpr int M = LeftT::Rows, KA = LeftT::Cols, KB = RightT::Rows, N = RightT::Cols;
    // k goes through LDS in chunks of KC: A as [m][KC], B as [n][KC], about 16 KiB together
    constexpr int kFit = 16 * 1024 / ((M + N) * (int)sizeof(A)) / 8 * 8;
    constexpr int KC = kFit < 8 ? 8 : (kFit > KA ? (KA + 7) / 8 * 8 : kFit);
    A *sA = reinterpret_cast<A *>(any_buffer<0, any_round((int)sizeof(A) * M * KC)>());
    B *sB = reinterpret_cast<B *>(any_buffer<1, any_round((int)sizeof(B) * N * KC)>());
    const int vm = min(a.GetValidRow(), AccT::Rows), vn = min(b.GetValidCol(), AccT::Cols);
    const int vk = min(min(a.GetValidCol(), b.GetValidRow()), min(KA, KB));
    if constexpr (kZeroInit) {
        for_each_elem(out, [&](int, int, CT, bool) { return CT(0); });
    } else {
        if (&out != &in)
            out.st = in.st;
    }
    for (int k0 = 0; k0 < vk; k0 += KC) {
        for_each_elem(a, [&](int r, int c, A v, bool owner) {
            if (owner && c >= k0 && c < k0 + KC)
                sA[r * KC + (c - k0)] = v;
            return v;
        });
        for_each_elem(b, [&](int r, int c, B v, bool owner) {
            if (owner && r >= k0 && r < k0 + KC)
                sB[c * KC + (r - k0)] = v;
            return v;
        });
        hw::lds_barrier();
        const int kn = min(KC, vk - k0);
        for_each_elem(out, [&](int r, int c, CT acc, bool) {
            if (r < vm && c < vn) {
                const A *pa = sA + r * KC;
                const B *pb = sB + c * KC;
                for (int k = 0; k < kn; ++k)
                    acc += (CT)pa[k] * (CT)pb[k];
            }
            return acc;
        });
        hw::lds_barrier();
    }
}

// C[i,j] += bias[j] (cpu/TMatmul.hpp:109-115: added after the product), for an Acc tile of either storage
template <typename AccT, typename BiasT>
PTO_DEV void add_bias_any(AccT &c, BiasT &bias)
{
    static_assert(BiasT::Loc == TileType::Bias && BiasT::Rows == 1 && BiasT::Cols == AccT::Cols, "[PTO][SA] TMATMUL_BIAS: a [1, n] Bias tile");
    using CT = typename AccT::DType;
    using BT = typename BiasT::DType;
    BT *sBias = reinterpret_cast<BT *>(any_buffer<2, any_round((int)sizeof(BT) * BiasT::Cols)>());
    for_each_elem(bias, [&](int, int col, BT v, bool) {
        sBias[col] = v;
        return v;
    });
    hw::lds_barrier();
    for_each_elem(c, [&](int, int col, CT v, bool) { return (CT)(v + (CT)sBias[col]); });
    hw::lds_barrier();
}

// plain Acc tile -> GM
template <typename TileT, typename G, AtomicType atomic, ReluPreMode relu>
PTO_DEV void tstore_any(G &dst, TileT &src)
{
    using T = typename TileT::DType;
    using GT = typename G::DType;
    GT *gm = reinterpret_cast<GT *>(dst.data());
    const int64_t st_r = dst.GetStride(3), st_c = dst.GetStride(4);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    for_each_elem(src, [&](int r, int c, T x, bool) {
        if (r < vr && c < vc) {
            T y = x;
            if constexpr (relu == ReluPreMode::NormalRelu)
                y = y < 0 ? 0 : y;
            GT *p = gm + (int64_t)r * st_r + (int64_t)c * st_c;
            if constexpr (atomic == AtomicType::AtomicAdd)
                atomic_add(p, store_cast<GT>(y));
            else
                *p = store_cast<GT>(y);
        }
        return x;
    });
}

// Mat tile: what lies outside the source's valid region becomes the destination's pad value, in LDS (the reference's
// matmul tests clear the part of an L1 tile that a ragged load left alone: tmatmul_kernel.cpp:86 of the NPU tests)
template <typename DstT, typename SrcT>
PTO_DEV void tfillpad_mat(DstT &dst, SrcT &src)
{
    static_assert(DstT::Rows == SrcT::Rows && DstT::Cols == SrcT::Cols && sizeof(typename DstT::DType) == sizeof(typename SrcT::DType),
                  "[PTO][SA] TFILLPAD on Mat tiles: one shape and element size");
    using T = typename DstT::DType;
    char *ld = hw::lds_base() + dst.st.lds;
    const char *ls = hw::lds_base() + src.st.lds;
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    const T pad = pad_value<T>(DstT::PadVal);
    hw::wait_vm0(); // asynchronous copies of a TLOAD just before
    hw::lds_barrier();
    for (int e = hw::tid(); e < DstT::Numel; e += kBlockThreads) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        T v = pad;
        if (r < vr && c < vc)
            v = *reinterpret_cast<const T *>(ls + MatGeom<SrcT>::elem_off(r, c));
        *reinterpret_cast<T *>(ld + MatGeom<DstT>::elem_off(r, c)) = v;
    }
    hw::lds_barrier();
}

} // namespace detail

// TGEMV: C[0, j] = sum_k A[0, k] B[k, j] for a Left tile of one valid row (pto_instr.hpp:529-571 of the reference).  The
// tiles' extents may differ (see mad_any); always the general path.
template <typename AccT, typename LeftT, typename RightT>
PTO_DEV void TGEMV_IMPL(AccT &c, LeftT &a, RightT &b)
{
    detail::check_mad_types<AccT, LeftT, RightT>();
    static_assert(RightT::Cols == AccT::Cols, "[PTO][SA] TGEMV: the Right and Acc tiles have one n");
    detail::mad_any<true>(c, c, a, b);
}
template <typename AccT, typename LeftT, typename RightT>
PTO_DEV void TGEMV_ACC_IMPL(AccT &cOut, AccT &cIn, LeftT &a, RightT &b)
{
    detail::check_mad_types<AccT, LeftT, RightT>();
    static_assert(RightT::Cols == AccT::Cols, "[PTO][SA] TGEMV_ACC: the Right and Acc tiles have one n");
    detail::mad_any<false>(cOut, cIn, a, b);
}
template <typename AccT, typename LeftT, typename RightT, typename BiasT>
PTO_DEV void TGEMV_BIAS_IMPL(AccT &c, LeftT &a, RightT &b, BiasT &bias)
{
    TGEMV_IMPL(c, a, b);
    detail::add_bias_any(c, bias);
}
} // namespace pto
