// TSORT32 and TMRGSORT on gfx950 Vec tiles: the sorting instructions of the reference's top-k kernel
// (kernels/manual/a2a3/topk/topk_kernel.cpp:282-331) as workgroup-wide rank computations.
//
// The reference executes them as a 32-element hardware sort and a sequential 4-way merge
// (cpu/TSort32.hpp:44-88, cpu/TMrgSort.hpp:118-178, 181-230).  Both have a closed form for where every element
// ends up: its rank = the number of elements that the comparator puts before it.  On a compute unit that is the
// natural formulation: the sources are staged in LDS, every lane computes the rank of a few elements (a scan of its
// group of 32, or a binary search in each of the other sorted lists) and scatters them into a staged image of the
// destination, which the lanes then read back into their registers.
//
// Order (cpu/TSort32.hpp:32-41, cpu/TMrgSort.hpp:106-116): score descending; TSORT32 puts equal scores in ascending
// order of index (equal pairs keep their source order); TMRGSORT compares scores only, equal scores come out in the
// order of the list number and then of the position in the list.  NaN scores have no place in that order (the
// reference's comparator is not an order for them) and are the caller's error.
// A structure is 8 bytes: (score, index) for 4-byte elements (float, int32_t), (score, 0, index & 0xffff, index >> 16)
// for 2-byte ones (half, int16_t; TMRGSORT also takes uint16_t, cpu/TMrgSort.hpp:41-46, cpu/TSort32.hpp:74-83).  The
// index is kept as its bit pattern (the form of the NPU implementation and its goldens,
// tests/npu/a2a3/src/st/testcase/tsort32/gen_data.py:20-27: struct.pack('fI') / ('e xxI'); the CPU simulation converts
// the index, or its halves, to the element type by value, which is the same thing for the integer tiles).
#pragma once
#include "pto/gfx950/vec_ops_ext.hpp"

namespace pto {

// executed structure counts of a merge (cpu/TMrgSort.hpp:22-27)
struct MrgSortExecutedNumList {
    uint16_t mrgSortList0;
    uint16_t mrgSortList1;
    uint16_t mrgSortList2;
    uint16_t mrgSortList3;
};

namespace detail {
// the unsigned integer that holds an element's bit pattern
template <typename T>
using SortBits = std::conditional_t<sizeof(T) == 4, uint32_t, uint16_t>;
template <typename T>
inline constexpr bool kSortable = std::is_same_v<T, float> || std::is_same_v<T, int32_t> || std::is_same_v<T, half> ||
                                  std::is_same_v<T, int16_t> || std::is_same_v<T, uint16_t>;
// elements of one 8-byte structure: 2 (score, index) for 4-byte elements, 4 (score, 0, index low, index high) for 2-byte ones
template <typename T>
inline constexpr int kStructElems = 8 / (int)sizeof(T);
// a structure as one 64-bit word: the score in the low bits, the index in bits 32-63
template <typename T>
PTO_DEV T score_of(uint64_t structure)
{
    return __builtin_bit_cast(T, (SortBits<T>)structure);
}
// the first ld columns of every row of a Vec tile -> LDS in (row, col) order with row stride ld (in elements)
template <typename TileT>
PTO_DEV void stage_tile_rows(TileT &t, SortBits<typename TileT::DType> *lds, int ld)
{
    using T = typename TileT::DType;
    for_each_owned<TileT>([&](int s, int i, int e) {
        if (e < TileT::Numel) {
            int r, c;
            elem_rc<TileT>(e, r, c);
            if (c < ld)
                lds[r * ld + c] = __builtin_bit_cast(SortBits<T>, t.S().v[s][i]);
        }
    });
}
// number of leading structures of a descending list whose score is > s (strict) or >= s
template <typename T, bool kStrict>
PTO_DEV int count_before(const uint64_t *list, int n, T s)
{
    int lo = 0, hi = n; // the answer lies in [lo, hi]
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const T v = score_of<T>(list[mid]);
        if (kStrict ? v > s : v >= s)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}
} // namespace detail

// The k-th pair of group g of row r goes to structure 32 g + k of row r of dst: elements (score, index) for 4-byte
// scores, (score, 0, index & 0xffff, index >> 16) for 2-byte ones
template <typename DstT, typename SrcT, typename IdxT>
PTO_DEV void TSORT32_IMPL(DstT &dst, SrcT &src, IdxT &idx)
{
    using T = typename SrcT::DType;
    using B = detail::SortBits<T>;
    constexpr int E = detail::kStructElems<T>;
    static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec && IdxT::Loc == TileType::Vec &&
                      DstT::isRowMajor && SrcT::isRowMajor && IdxT::isRowMajor,
                  "[PTO][SA] TSORT32: row-major Vec tiles");
    static_assert(std::is_same_v<typename DstT::DType, T> && detail::kSortable<T> && !std::is_same_v<T, uint16_t>,
                  "[PTO][SA] TSORT32: float, half, int32 or int16 scores, destination of the same type");
    static_assert(std::is_same_v<typename IdxT::DType, uint32_t>, "[PTO][SA] TSORT32: uint32 indices");
    static_assert(SrcT::Rows == IdxT::Rows && DstT::Rows == SrcT::Rows, "[PTO][SA] TSORT32: source, index and destination rows");
    // The valid columns decide what is sorted; the tiles' own widths may differ (the reference's top-k kernel views one
    // row buffer through a tile type twice as wide as its scores, kernels/manual/a2a3/topk/topk_kernel.cpp:132-145).
    // C: the most columns that source, index and destination (8 bytes a column) can all hold.
    constexpr int R = SrcT::Rows;
    constexpr int C0 = SrcT::Cols < IdxT::Cols ? SrcT::Cols : IdxT::Cols, C = C0 < DstT::Cols / E ? C0 : DstT::Cols / E, N = R * C;
    static_assert(C >= 1, "[PTO][SA] TSORT32: destination of 8 bytes per source element");
    uint64_t *image = reinterpret_cast<uint64_t *>(detail::stage_buffer<detail::stage_bytes(16 * N)>()); // [R][C] structures
    uint32_t *index = reinterpret_cast<uint32_t *>(image + N);
    B *score = reinterpret_cast<B *>(index + N);
    const int vr = src.GetValidRow(), vc = src.GetValidCol();
    if (vr > idx.GetValidRow() || vc > idx.GetValidCol() || vc > C)
        return; // the index tile must cover the scores (cpu/TSort32.hpp:113-115 asks for equal extents; the NPU's tests give
                // the index tile the row length rounded up to 32 bytes: tsort32_kernel.cpp:47-49); uniform over the workgroup
    detail::stage_tile_rows(src, score, C);
    detail::stage_tile_rows(idx, index, C);
    hw::lds_barrier();
    for (int e = hw::tid(); e < N; e += kBlockThreads) {
        const int r = e / C, c = e % C;
        if (r < vr && c < vc) {
            const int g0 = c & ~31, n = (vc - g0) < 32 ? (vc - g0) : 32;
            const T s = __builtin_bit_cast(T, score[e]);
            const uint32_t ix = index[e];
            int rank = 0;
            for (int k = 0; k < n; ++k) {
                const T sk = __builtin_bit_cast(T, score[r * C + g0 + k]);
                const uint32_t ik = index[r * C + g0 + k];
                const bool before = sk != s ? sk > s : (ik != ix ? ik < ix : g0 + k < c);
                rank += before ? 1 : 0;
            }
            image[r * C + g0 + rank] = (uint64_t)score[e] | ((uint64_t)ix << 32);
        }
    }
    hw::lds_barrier();
    const B *flat = reinterpret_cast<const B *>(image);
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        const int r = e / DstT::Cols, c = e % DstT::Cols;
        if (e < DstT::Numel && r < vr && c < E * vc)
            dst.S().v[s][i] = __builtin_bit_cast(T, flat[r * E * C + c]);
    });
    hw::lds_barrier();
}
// the scratch tile of the form for rows shorter than 32 is not needed
template <typename DstT, typename SrcT, typename IdxT, typename TmpT>
PTO_DEV void TSORT32_IMPL(DstT &dst, SrcT &src, IdxT &idx, TmpT &)
{
    TSORT32_IMPL(dst, src, idx);
}

// One source: every group of four consecutive blocks of blockLen elements (blockLen * sizeof(T) / 8 structures, each block
// sorted) that lies inside the destination's valid columns is merged into one sorted run (cpu/TMrgSort.hpp:181-230).
template <typename DstT, typename SrcT>
PTO_DEV void TMRGSORT_IMPL(DstT &dst, SrcT &src, uint32_t blockLen)
{
    using T = typename DstT::DType;
    using B = detail::SortBits<T>;
    constexpr int E = detail::kStructElems<T>;
    static_assert(DstT::Loc == TileType::Vec && SrcT::Loc == TileType::Vec && DstT::Rows == 1 && SrcT::Rows == 1 && DstT::isRowMajor &&
                      SrcT::isRowMajor,
                  "[PTO][SA] TMRGSORT: row-major Vec tiles of one row");
    static_assert(std::is_same_v<typename SrcT::DType, T> && detail::kSortable<T>,
                  "[PTO][SA] TMRGSORT: float, half, int32, int16 or uint16 elements");
    static_assert(DstT::Cols <= SrcT::Cols && SrcT::Cols % E == 0, "[PTO][SA] TMRGSORT: the source covers the destination");
    constexpr int N = DstT::Cols;
    uint64_t *in = reinterpret_cast<uint64_t *>(detail::stage_buffer<detail::stage_bytes((int)sizeof(T) * (SrcT::Cols + N) + 8)>());
    uint64_t *image = in + SrcT::Cols / E;
    const int maxCols = dst.GetValidCol();
    const int block = (int)blockLen, per = block / E, group = 4 * per; // per, group: in structures
    if (block == 0 || block % E != 0)
        return;
    detail::stage_tile_rows(src, reinterpret_cast<B *>(in), SrcT::Cols);
    hw::lds_barrier();
    const int merged = maxCols / (4 * block) * group; // structures that belong to complete groups
    for (int e = hw::tid(); e < merged; e += kBlockThreads) { // structure e of the source
        const int g = e / group, b = (e - g * group) / per, p = e - g * group - b * per;
        const T s = detail::score_of<T>(in[e]);
        int rank = p;
        for (int o = 0; o < 4; ++o) {
            const uint64_t *list = in + g * group + o * per;
            if (o < b)
                rank += detail::count_before<T, false>(list, per, s);
            else if (o > b)
                rank += detail::count_before<T, true>(list, per, s);
        }
        image[g * group + rank] = in[e];
    }
    hw::lds_barrier();
    const B *flat = reinterpret_cast<const B *>(image);
    detail::for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < merged * E)
            dst.S().v[s][i] = __builtin_bit_cast(T, flat[e]);
    });
    hw::lds_barrier();
}

// Two to four sorted lists (valid columns = elements, 8 bytes per structure) merged into the destination's valid columns.
// kExhausted: the merge stops right after the structure that empties one of the lists.  executed: how many
// structures of each list were taken (cpu/TMrgSort.hpp:118-178, 232-297).
namespace detail {
template <bool kExhausted, int kLists, typename DstT, typename S0, typename S1, typename S2, typename S3>
PTO_DEV void merge_lists(DstT &dst, MrgSortExecutedNumList &executed, S0 &src0, S1 &src1, S2 &src2, S3 &src3)
{
    using T = typename DstT::DType;
    using B = SortBits<T>;
    constexpr int E = kStructElems<T>;
    static_assert(DstT::Loc == TileType::Vec && DstT::Rows == 1 && DstT::isRowMajor && S0::Rows == 1 && S1::Rows == 1 && S2::Rows == 1 &&
                      S3::Rows == 1 && S0::isRowMajor && S1::isRowMajor && S2::isRowMajor && S3::isRowMajor,
                  "[PTO][SA] TMRGSORT: row-major Vec tiles of one row");
    static_assert(kSortable<T> && std::is_same_v<typename S0::DType, T> && std::is_same_v<typename S1::DType, T> &&
                      std::is_same_v<typename S2::DType, T> && std::is_same_v<typename S3::DType, T>,
                  "[PTO][SA] TMRGSORT: float, half, int32, int16 or uint16 elements, one type");
    static_assert(S0::Cols % E == 0 && S1::Cols % E == 0 && S2::Cols % E == 0 && S3::Cols % E == 0 && DstT::Cols % E == 0,
                  "[PTO][SA] TMRGSORT: whole 8-byte structures");
    // offsets and extents in structures
    constexpr int kCols[4] = {S0::Cols / E, S1::Cols / E, kLists > 2 ? S2::Cols / E : 0, kLists > 3 ? S3::Cols / E : 0};
    constexpr int kOff[4] = {0, kCols[0], kCols[0] + kCols[1], kCols[0] + kCols[1] + kCols[2]};
    constexpr int kIn = kOff[3] + kCols[3];
    uint64_t *in = reinterpret_cast<uint64_t *>(stage_buffer<stage_bytes(8 * (kIn + DstT::Cols / E) + 64)>());
    uint64_t *image = in + kIn;
    int *shared = reinterpret_cast<int *>(image + DstT::Cols / E); // [0] stop position, [1..4] executed counts
    const int n[4] = {src0.GetValidCol() / E, src1.GetValidCol() / E, kLists > 2 ? src2.GetValidCol() / E : 0,
                      kLists > 3 ? src3.GetValidCol() / E : 0};
    const int outMax = dst.GetValidCol() / E, total = n[0] + n[1] + n[2] + n[3];
    stage_tile_rows(src0, reinterpret_cast<B *>(in + kOff[0]), S0::Cols);
    stage_tile_rows(src1, reinterpret_cast<B *>(in + kOff[1]), S1::Cols);
    if constexpr (kLists > 2)
        stage_tile_rows(src2, reinterpret_cast<B *>(in + kOff[2]), S2::Cols);
    if constexpr (kLists > 3)
        stage_tile_rows(src3, reinterpret_cast<B *>(in + kOff[3]), S3::Cols);
    if (hw::tid() < 5)
        shared[hw::tid()] = hw::tid() == 0 ? (outMax < total ? outMax : total) : 0;
    hw::lds_barrier();
    auto rank_of = [&](int b, int p) {
        const T s = score_of<T>(in[kOff[b] + p]);
        int rank = p;
#pragma unroll
        for (int o = 0; o < kLists; ++o) {
            if (o < b)
                rank += count_before<T, false>(in + kOff[o], n[o], s);
            else if (o > b)
                rank += count_before<T, true>(in + kOff[o], n[o], s);
        }
        return rank;
    };
    if constexpr (kExhausted) {
        // the merge ends after the structure that empties a list: the earliest "last structure of a list"; a list that
        // is empty from the start ends it after the first structure
        if (hw::tid() < kLists) {
            const int b = hw::tid();
            const int stop = n[b] > 0 ? rank_of(b, n[b] - 1) + 1 : (total > 0 ? 1 : 0);
            atomicMin(&shared[0], stop);
        }
        hw::lds_barrier();
    }
    const int stop = shared[0];
    for (int e = hw::tid(); e < total; e += kBlockThreads) {
        int b = 0, p = e;
#pragma unroll
        for (int o = 0; o < kLists - 1; ++o)
            if (b == o && p >= n[o]) {
                p -= n[o];
                b = o + 1;
            }
        const int rank = rank_of(b, p);
        if (rank < stop) {
            image[rank] = in[kOff[b] + p];
            atomicMax(&shared[1 + b], p + 1); // ranks grow along a list: the largest taken position + 1 is the count
        }
    }
    hw::lds_barrier();
    const B *flat = reinterpret_cast<const B *>(image);
    for_each_owned<DstT>([&](int s, int i, int e) {
        if (e < E * stop)
            dst.S().v[s][i] = __builtin_bit_cast(T, flat[e]);
    });
    executed.mrgSortList0 = (uint16_t)shared[1];
    executed.mrgSortList1 = (uint16_t)shared[2];
    executed.mrgSortList2 = (uint16_t)shared[3];
    executed.mrgSortList3 = (uint16_t)shared[4];
    hw::lds_barrier();
}
} // namespace detail

template <typename DstT, typename TmpT, typename S0, typename S1, typename S2, typename S3, bool exhausted>
PTO_DEV void TMRGSORT_IMPL(DstT &dst, MrgSortExecutedNumList &executed, TmpT &, S0 &src0, S1 &src1, S2 &src2, S3 &src3)
{
    detail::merge_lists<exhausted, 4>(dst, executed, src0, src1, src2, src3);
}
template <typename DstT, typename TmpT, typename S0, typename S1, typename S2, bool exhausted>
PTO_DEV void TMRGSORT_IMPL(DstT &dst, MrgSortExecutedNumList &executed, TmpT &, S0 &src0, S1 &src1, S2 &src2)
{
    detail::merge_lists<exhausted, 3>(dst, executed, src0, src1, src2, src2);
}
template <typename DstT, typename TmpT, typename S0, typename S1, bool exhausted>
PTO_DEV void TMRGSORT_IMPL(DstT &dst, MrgSortExecutedNumList &executed, TmpT &, S0 &src0, S1 &src1)
{
    detail::merge_lists<exhausted, 2>(dst, executed, src0, src1, src1, src1);
}

} // namespace pto
