// Single-tile instruction kernels: one workgroup runs a short PTO program on one or a few tiles.
// They are the counterpart of the reference's per-instruction system tests
// (tests/cpu/st/testcase/<op>/<op>_kernel.cpp) and exist so that every instruction on the path
// can be checked against the oracle through the C ABI.
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

template <typename T, int R, int C>
using GmND = GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>>;
template <typename T, int R>
using GmCol = GlobalTensor<T, Shape<1, 1, 1, R, 1>, Stride<R, R, R, 1, R>, Layout::DN>;

// ---- streaming-softmax step on one [64, 256] fp32 score tile (stage a12 of the attention path) ----
// first != 0: M = rowmax(X), P = exp(s (X - M)), S = rowsum(P)
// else:       M' = max(M, rowmax X), alpha = exp(s (M - M')), P = exp(s (X - M')), S' = alpha S + rowsum(P)
// x_exp = half(P) with RoundMode `mode`.
constexpr int kSmRows = 64, kSmCols = 256;
__global__ __launch_bounds__(kBlockThreads) AICORE void SoftmaxStep(__gm__ half *xExpOut, __gm__ float *maxOut,
                                                                    __gm__ float *sumOut, __gm__ float *alphaOut,
                                                                    __gm__ const float *xIn, __gm__ const float *maxIn,
                                                                    __gm__ const float *sumIn, float scale, int first,
                                                                    int mode)
{
    using TileX = Tile<TileType::Vec, float, kSmRows, kSmCols, BLayout::RowMajor>;
    using TileH = Tile<TileType::Vec, half, kSmRows, kSmCols, BLayout::RowMajor>;
    using TileR = Tile<TileType::Vec, float, kSmRows, 1, BLayout::ColMajor>;
    using Tile1F = Tile<TileType::Vec, float, 1, kSmRows * kSmCols, BLayout::RowMajor>;
    using Tile1H = Tile<TileType::Vec, half, 1, kSmRows * kSmCols, BLayout::RowMajor>;
    TileX x, p;
    TileH xExp;
    TileR localMax, globalMax, expMax, localSum, globalSum;
    GmND<float, kSmRows, kSmCols> gx(const_cast<float *>(xIn));
    GmND<half, kSmRows, kSmCols> gxe(xExpOut);
    GmCol<float, kSmRows> gMaxIn(const_cast<float *>(maxIn)), gSumIn(const_cast<float *>(sumIn)), gMaxOut(maxOut),
        gSumOut(sumOut), gAlpha(alphaOut);
    TLOAD(x, gx);
    if (first) {
        TROWMAX(globalMax, x, p);
        TROWEXPANDSUB(p, x, globalMax);
        TMULS(p, p, scale);
        TEXP(p, p);
        TROWSUM(globalSum, p, x);
        TEXPANDS(expMax, 1.0f);
    } else {
        TLOAD(globalMax, gMaxIn);
        TLOAD(globalSum, gSumIn);
        TROWMAX(localMax, x, p);
        TMAX(localMax, localMax, globalMax);   // M'
        TSUB(expMax, globalMax, localMax);     // M - M'
        TMULS(globalMax, localMax, 1.0f);      // M <- M'
        TROWEXPANDSUB(p, x, localMax);
        TMULS(expMax, expMax, scale);
        TMULS(p, p, scale);
        TEXP(expMax, expMax);
        TEXP(p, p);
        TMUL(globalSum, expMax, globalSum);
        TROWSUM(localSum, p, x);
        TADD(globalSum, globalSum, localSum);
    }
    Tile1F p1;
    Tile1H xe1;
    TRESHAPE(p1, p);
    TCVT(xe1, p1, static_cast<RoundMode>(mode));
    TRESHAPE(xExp, xe1);
    TSTORE(gxe, xExp);
    TSTORE(gMaxOut, globalMax);
    TSTORE(gSumOut, globalSum);
    TSTORE(gAlpha, expMax);
}

// ---- rescale-accumulate step (stage a13): O = O alpha + PV; last: O /= S ----
constexpr int kGuRows = 64, kGuCols = 128;
__global__ __launch_bounds__(kBlockThreads) AICORE void GuStep(__gm__ float *oOut, __gm__ const float *oPrev,
                                                               __gm__ const float *pv, __gm__ const float *alpha,
                                                               __gm__ const float *sum, int last)
{
    using TileO = Tile<TileType::Vec, float, kGuRows, kGuCols, BLayout::RowMajor>;
    using TileR = Tile<TileType::Vec, float, kGuRows, 1, BLayout::ColMajor>;
    TileO o, est;
    TileR a, s;
    GmND<float, kGuRows, kGuCols> gPrev(const_cast<float *>(oPrev)), gPv(const_cast<float *>(pv)), gOut(oOut);
    GmCol<float, kGuRows> gA(const_cast<float *>(alpha)), gS(const_cast<float *>(sum));
    TLOAD(o, gPrev);
    TLOAD(est, gPv);
    TLOAD(a, gA);
    TLOAD(s, gS);
    TROWEXPANDMUL(o, o, a);
    TADD(o, o, est);
    if (last)
        TROWEXPANDDIV(o, o, s);
    TSTORE(gOut, o);
}

// ---- TTRI + TADD mask: out = x + triu(diagonal) * value ----
__global__ __launch_bounds__(kBlockThreads) AICORE void TriMask(__gm__ float *out, __gm__ const float *xIn, int diagonal,
                                                                float value, int upper)
{
    using TileX = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    TileX x, tri;
    GmND<float, 64, 128> gx(const_cast<float *>(xIn)), go(out);
    TLOAD(x, gx);
    if (upper)
        TTRI<TileX, 1>(tri, diagonal);
    else
        TTRI<TileX, 0>(tri, diagonal);
    TMULS(tri, tri, value);
    TADD(x, x, tri);
    TSTORE(go, x);
}

// ---- TQUANT<QuantType::MXFP8>: the ND-mode program of the reference's test (runTQuant<rows, cols, 0>,
// tests/npu/a5/src/st/testcase/tquant/tquant_kernel.cpp:27-80): TLOAD -> TQUANT -> TSTORE of the exponents and of the fp8 tile ----
template <int R, int C>
__global__ __launch_bounds__(kBlockThreads) AICORE void TQuantMx(__gm__ uint8_t *outE8, __gm__ uint8_t *outFp8, __gm__ float *outMax,
                                                                 __gm__ float *outScaling, __gm__ const float *in, int validRows,
                                                                 int validCols)
{
    constexpr int kGroups = R * (C / 32);
    using SrcTile = Tile<TileType::Vec, float, R, C, BLayout::RowMajor, -1, -1, SLayout::NoneBox, 512, PadValue::Zero>;
    using Fp8Tile = Tile<TileType::Vec, int8_t, R, C, BLayout::RowMajor, R, C, SLayout::NoneBox, 512, PadValue::Zero>;
    using E8Tile = Tile<TileType::Vec, uint8_t, 1, kGroups, BLayout::RowMajor, -1, -1, SLayout::NoneBox, 512, PadValue::Zero>;
    using MaxTile = Tile<TileType::Vec, float, 1, kGroups, BLayout::RowMajor, -1, -1>;
    using SrcGlobal = GlobalTensor<float, Shape<1, 1, 1, DYNAMIC, DYNAMIC>, Stride<1, 1, 1, DYNAMIC, 1>>;
    SrcTile srcTile(validRows, validCols), scalingTile(validRows, validCols);
    Fp8Tile fp8Tile;
    E8Tile e8Tile(1, kGroups);
    MaxTile maxTile(1, kGroups);
    SrcGlobal srcGlobal(const_cast<float *>(in), Shape<1, 1, 1, DYNAMIC, DYNAMIC>(validRows, validCols),
                        Stride<1, 1, 1, DYNAMIC, 1>(validCols));
    GmND<uint8_t, 1, kGroups> e8Global(outE8);
    GmND<int8_t, R, C> fp8Global(reinterpret_cast<__gm__ int8_t *>(outFp8));
    GmND<float, 1, kGroups> maxGlobal(outMax);
    GmND<float, R, C> scalingGlobal(outScaling);
    TLOAD(srcTile, srcGlobal);
    TLOAD(scalingTile, srcGlobal); // defined contents beyond the first kGroups entries
    set_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_V, EVENT_ID0);
    TQUANT<QuantType::MXFP8, Fp8Tile, SrcTile, E8Tile, MaxTile>(fp8Tile, srcTile, &e8Tile, &maxTile, &scalingTile);
    set_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    wait_flag(PIPE_V, PIPE_MTE3, EVENT_ID0);
    TSTORE(e8Global, e8Tile);
    TSTORE(fp8Global, fp8Tile);
    TSTORE(maxGlobal, maxTile);
    scalingTile = SrcTile(R, C);
    TSTORE(scalingGlobal, scalingTile);
}

// ---- mask-form TGATHER on a [16, 64] tile of 16-bit elements ----
template <MaskPattern P, int DIV>
AICORE inline void GatherMaskBody(__gm__ uint16_t *out, __gm__ const uint16_t *in)
{
    using Src = Tile<TileType::Vec, uint16_t, 16, 64, BLayout::RowMajor>;
    using Dst = Tile<TileType::Vec, uint16_t, 16, 64 / DIV, BLayout::RowMajor>;
    Src s;
    Dst d;
    GmND<uint16_t, 16, 64> gs(const_cast<uint16_t *>(in));
    GmND<uint16_t, 16, 64 / DIV> gd(out);
    TLOAD(s, gs);
    TGATHER<Dst, Src, P>(d, s);
    TSTORE(gd, d);
}
__global__ __launch_bounds__(kBlockThreads) AICORE void GatherMask(__gm__ uint16_t *out, __gm__ const uint16_t *in, int pattern)
{
    switch (pattern) {
    case 1: GatherMaskBody<MaskPattern::P0101, 2>(out, in); break;
    case 2: GatherMaskBody<MaskPattern::P1010, 2>(out, in); break;
    case 3: GatherMaskBody<MaskPattern::P0001, 4>(out, in); break;
    case 4: GatherMaskBody<MaskPattern::P0010, 4>(out, in); break;
    case 5: GatherMaskBody<MaskPattern::P0100, 4>(out, in); break;
    case 6: GatherMaskBody<MaskPattern::P1000, 4>(out, in); break;
    default: GatherMaskBody<MaskPattern::P1111, 1>(out, in); break;
    }
}

// ---- element-form MGATHER: dst[8,128] = gm[idx[8,128]] ----
__global__ __launch_bounds__(kBlockThreads) AICORE void MGatherElems(__gm__ uint16_t *out, __gm__ const uint16_t *gm,
                                                                     __gm__ const int32_t *idx, int gmElems)
{
    using Dst = Tile<TileType::Vec, uint16_t, 8, 128, BLayout::RowMajor>;
    using Idx = Tile<TileType::Vec, int32_t, 8, 128, BLayout::RowMajor>;
    Dst d;
    Idx ti;
    GmND<int32_t, 8, 128> gi(const_cast<int32_t *>(idx));
    GmND<uint16_t, 8, 128> gd(out);
    GlobalTensor<uint16_t, Shape<1, 1, 1, 1, DYNAMIC>, Stride<1, 1, 1, DYNAMIC, 1>> gsrc(
        const_cast<uint16_t *>(gm), Shape<1, 1, 1, 1, DYNAMIC>(gmElems), Stride<1, 1, 1, DYNAMIC, 1>(gmElems));
    TLOAD(ti, gi);
    MGATHER(d, gsrc, ti);
    TSTORE(gd, d);
}

// ---- TLOAD with a valid region and PadValue::Max: the whole [16, 32] tile image comes back ----
__global__ __launch_bounds__(kBlockThreads) AICORE void LoadPadImage(__gm__ float *image, __gm__ const float *gm)
{
    using Padded = Tile<TileType::Vec, float, 16, 32, BLayout::RowMajor, 10, 20, SLayout::NoneBox, 512, PadValue::Max>;
    using Full = Tile<TileType::Vec, float, 16, 32, BLayout::RowMajor>;
    Padded t;
    Full f;
    GlobalTensor<float, Shape<1, 1, 1, 10, 20>, Stride<200, 200, 200, 20, 1>> g(const_cast<float *>(gm));
    GmND<float, 16, 32> gi(image);
    TLOAD(t, g);
    TRESHAPE(f, t);
    TSTORE(gi, f);
}

// ---- 5-D GM [1,2,3,4,8] with padded strides -> [24, 8] tile -> dense [24, 8]; and back out through 5-D strides ----
__global__ __launch_bounds__(kBlockThreads) AICORE void Load5D(__gm__ float *dense, __gm__ float *strided, __gm__ const float *gm)
{
    using T = Tile<TileType::Vec, float, 24, 8, BLayout::RowMajor>;
    using G5 = GlobalTensor<float, Shape<1, 2, 3, 4, 8>, Stride<1000, 400, 100, 10, 1>>;
    T t;
    G5 g(const_cast<float *>(gm)), gOut(strided);
    GmND<float, 24, 8> gd(dense);
    TLOAD(t, g);
    TSTORE(gd, t);
    TSTORE(gOut, t);
}

// ---- TEXTRACT windows: C = A[:, col0 : col0+64] (through Left) x I, and C = I x B[row0 : row0+64, :] (through Right) ----
__global__ __launch_bounds__(kBlockThreads) AICORE void ExtractWindows(__gm__ float *outLeft, __gm__ float *outRight,
                                                                       __gm__ const half *a, __gm__ const half *bT,
                                                                       __gm__ const half *eyeB, __gm__ const half *eyeA,
                                                                       int col0, int row0)
{
    // a [128, 256] row-major; bT [256 cols][256 rows] (column-major 256 x 256); eyeB: [256][64] column-major 64 x 256
    // identity-like (eyeB(k, n) = k == n); eyeA [128, 64] with eyeA(r, k) = r == k
    using MatA = Tile<TileType::Mat, half, 128, 256, BLayout::ColMajor, 128, 256, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, half, 256, 256, BLayout::RowMajor, 256, 256, SLayout::ColMajor>;
    using MatEyeB = Tile<TileType::Mat, half, 64, 256, BLayout::RowMajor, 64, 256, SLayout::ColMajor>;
    using MatEyeA = Tile<TileType::Mat, half, 128, 64, BLayout::ColMajor, 128, 64, SLayout::RowMajor>;
    MatA am;
    MatB bm;
    MatEyeB eb;
    MatEyeA ea;
    TASSIGN(am, 0u);
    TASSIGN(eb, 64u * 1024);
    TASSIGN(ea, 96u * 1024);
    TileLeft<half, 128, 64> l;
    TileRight<half, 64, 256> r;
    TileAcc<float, 128, 256> c;
    GmND<half, 128, 256> ga(const_cast<half *>(a));
    GlobalTensor<half, Shape<1, 1, 1, 64, 256>, Stride<1, 1, 1, 1, 64>, Layout::DN> geb(const_cast<half *>(eyeB));
    GmND<half, 128, 64> gea(const_cast<half *>(eyeA));
    GmND<float, 128, 256> gl(outLeft), gr(outRight);
    TLOAD(am, ga);
    TLOAD(eb, geb);
    TLOAD(ea, gea);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TEXTRACT(l, am, 0, (uint16_t)col0);
    TMOV(r, eb);
    TMATMUL(c, l, r);
    TSTORE(gl, c);
    // reuse the A region for B once everyone has read it
    set_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID0);
    wait_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID0);
    TASSIGN(bm, 0u);
    GlobalTensor<half, Shape<1, 1, 1, 256, 256>, Stride<1, 1, 1, 1, 256>, Layout::DN> gb(const_cast<half *>(bT));
    // the B image spans 128 KiB: it would overwrite the identity tiles, so fetch them again afterwards
    TLOAD(bm, gb);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID1);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID1);
    TEXTRACT(r, bm, (uint16_t)row0, 0);
    set_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1);
    wait_flag(PIPE_MTE1, PIPE_MTE2, EVENT_ID1);
    TASSIGN(ea, 0u);
    TLOAD(ea, gea);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID2);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID2);
    TMOV(l, ea);
    TMATMUL(c, l, r);
    TSTORE(gr, c);
}

// ---- one-block matmul [128, K] x [K, 256] with bias, fp16 or bf16, ordered by Event objects ----
template <typename T, int K>
__global__ __launch_bounds__(kBlockThreads) AICORE void MatmulBias(__gm__ float *out, __gm__ const T *a, __gm__ const T *bT,
                                                                   __gm__ const float *bias)
{
    using MatA = Tile<TileType::Mat, T, 128, K, BLayout::ColMajor, 128, K, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, T, K, 256, BLayout::RowMajor, K, 256, SLayout::ColMajor>;
    MatA am;
    MatB bm;
    TASSIGN(am, 0u);
    TASSIGN(bm, 128u * K * sizeof(T));
    TileLeft<T, 128, K> l;
    TileRight<T, K, 256> r;
    TileAcc<float, 128, 256> c;
    GmND<T, 128, K> ga(const_cast<T *>(a));
    GlobalTensor<T, Shape<1, 1, 1, K, 256>, Stride<1, 1, 1, 1, K>, Layout::DN> gb(const_cast<T *>(bT));
    GmND<float, 128, 256> gc(out);
    Event<Op::TLOAD, Op::TEXTRACT> loaded;
    Event<Op::TEXTRACT, Op::TMATMUL> extracted;
    Event<Op::TMATMUL, Op::TSTORE_ACC> computed;
    TLOAD(am, ga);
    loaded = TLOAD(bm, gb);
    TEXTRACT(l, am, 0, 0, loaded);
    extracted = TEXTRACT(r, bm, 0, 0);
    if (bias != nullptr)
        computed = TMATMUL_BIAS(c, l, r, BiasRow{bias}, extracted);
    else
        computed = TMATMUL(c, l, r, extracted);
    TSTORE(gc, c, computed);
}

// ---- one-block matmul [128, K] x [K, 256] for the other operand types of TMATMUL: int8 -> int32, fp32 -> fp32 ----
// (tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp with the int8 and float cases of its gen_data.py:92-99).  K is taken
// in two halves: TMATMUL on the first, TMATMUL_ACC on the second.  relu: the store clamps negative results to zero
// (TSTORE<..., AtomicType::AtomicNone, ReluPreMode::NormalRelu, STPhase::Final>).
template <typename T, typename CT, int K>
__global__ __launch_bounds__(kBlockThreads) AICORE void MatmulTyped(__gm__ CT *out, __gm__ const T *a, __gm__ const T *bT, int relu)
{
    constexpr int KH = K / 2;
    using MatA = Tile<TileType::Mat, T, 128, K, BLayout::ColMajor, 128, K, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, T, K, 256, BLayout::RowMajor, K, 256, SLayout::ColMajor>;
    MatA am;
    MatB bm;
    TASSIGN(am, 0u);
    TASSIGN(bm, 128u * K * sizeof(T));
    TileLeft<T, 128, KH> l;
    TileRight<T, KH, 256> r;
    TileAcc<CT, 128, 256> c;
    GmND<T, 128, K> ga(const_cast<T *>(a));
    GlobalTensor<T, Shape<1, 1, 1, K, 256>, Stride<1, 1, 1, 1, K>, Layout::DN> gb(const_cast<T *>(bT));
    GmND<CT, 128, 256> gc(out);
    TLOAD(am, ga);
    TLOAD(bm, gb);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TEXTRACT(l, am, 0, 0);
    TEXTRACT(r, bm, 0, 0);
    TMATMUL(c, l, r);
    TEXTRACT(l, am, 0, KH);
    TEXTRACT(r, bm, KH, 0);
    TMATMUL_ACC(c, c, l, r);
    using AccT = TileAcc<CT, 128, 256>;
    using GmC = GmND<CT, 128, 256>;
    if (relu)
        TSTORE<AccT, GmC, AtomicType::AtomicNone, ReluPreMode::NormalRelu, STPhase::Final>(gc, c);
    else
        TSTORE<AccT, GmC, AtomicType::AtomicNone, STPhase::Final>(gc, c);
}

// ---- one-block MX matmul [128, 256] x [256, 128], fp8 operands (formats may differ) with e8m0 block scales ----
// (tests/npu/a5/src/st/testcase/tmatmul_mx/tmatmul_mx_kernel.cpp: TLOAD -> TEXTRACT -> TMATMUL_MX -> TSTORE).  K is taken
// in two halves of 128: TMATMUL_MX on the first, the accumulating form on the second.  VIA_MAT == false: the scale tiles
// are loaded whole from memory (MX_A_ND / MX_B_DN) into registers and windowed per half; true: the scales are TLOADed
// into Mat tiles (as the reference kernels stage them in L1) and each half's scale tiles TEXTRACTed from there.
// bias != nullptr: the first half is the bias form of TMATMUL_MX with the row bias[0 .. 127] in a Bias tile.
template <typename FA, typename FB, bool VIA_MAT>
__global__ __launch_bounds__(kBlockThreads) AICORE void MatmulMx(__gm__ float *out, __gm__ const FA *a, __gm__ const FB *bT,
                                                                 __gm__ const float8_e8m0_t *sa, __gm__ const float8_e8m0_t *sbT,
                                                                 __gm__ const float *bias)
{
    constexpr int M = 128, N = 128, K = 256, KH = 128, KB = K / 32;
    using X = float8_e8m0_t;
    using MatA = Tile<TileType::Mat, FA, M, K, BLayout::ColMajor, M, K, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, FB, K, N, BLayout::RowMajor, K, N, SLayout::ColMajor>;
    MatA am;
    MatB bm;
    TASSIGN(am, 0u);
    TASSIGN(bm, (uint32_t)(M * K));
    TileLeft<FA, M, KH> l;
    TileRight<FB, KH, N> r;
    TileLeftScale<X, M, KB> lsAll;
    TileRightScale<X, KB, N> rsAll;
    TileLeftScale<X, M, KH / 32> ls;
    TileRightScale<X, KH / 32, N> rs;
    TileAcc<float, M, N> c;
    GmND<FA, M, K> ga(const_cast<FA *>(a));
    GlobalTensor<FB, Shape<1, 1, 1, K, N>, Stride<1, 1, 1, 1, K>, Layout::DN> gb(const_cast<FB *>(bT));
    GlobalTensor<X, TileShape2D<X, M, KB, Layout::MX_A_ND>, BaseShape2D<X, M, KB, Layout::MX_A_ND>, Layout::MX_A_ND> gsa(const_cast<X *>(sa));
    GlobalTensor<X, TileShape2D<X, KB, N, Layout::MX_B_DN>, BaseShape2D<X, KB, N, Layout::MX_B_DN>, Layout::MX_B_DN> gsb(const_cast<X *>(sbT));
    GmND<float, M, N> gc(out);
    Tile<TileType::Mat, X, M, KB, BLayout::RowMajor, M, KB, SLayout::NoneBox> lsMat;
    Tile<TileType::Mat, X, KB, N, BLayout::ColMajor, KB, N, SLayout::NoneBox> rsMat;
    TASSIGN(lsMat, (uint32_t)(M * K + K * N));
    TASSIGN(rsMat, (uint32_t)(M * K + K * N + M * KB));
    TLOAD(am, ga);
    TLOAD(bm, gb);
    if constexpr (VIA_MAT) {
        TLOAD(lsMat, gsa);
        TLOAD(rsMat, gsb);
    } else {
        TLOAD(lsAll, gsa);
        TLOAD(rsAll, gsb);
    }
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TEXTRACT(l, am, 0, 0);
    TEXTRACT(r, bm, 0, 0);
    if constexpr (VIA_MAT) {
        TEXTRACT(ls, lsMat, 0, 0);
        TEXTRACT(rs, rsMat, 0, 0);
    } else {
        TEXTRACT(ls, lsAll, 0, 0);
        TEXTRACT(rs, rsAll, 0, 0);
    }
    if (bias != nullptr) {
        Tile<TileType::Bias, float, 1, N, BLayout::RowMajor, 1, N> biasTile;
        GlobalTensor<float, Shape<1, 1, 1, 1, N>, Stride<N, N, N, N, 1>> gBias(const_cast<float *>(bias));
        TLOAD(biasTile, gBias);
        TMATMUL_MX(c, l, ls, r, rs, biasTile);
    } else {
        TMATMUL_MX(c, l, ls, r, rs);
    }
    TEXTRACT(l, am, 0, KH);
    TEXTRACT(r, bm, KH, 0);
    if constexpr (VIA_MAT) {
        TEXTRACT(ls, lsMat, 0, KH / 32);
        TEXTRACT(rs, rsMat, KH / 32, 0);
    } else {
        TEXTRACT(ls, lsAll, 0, KH / 32);
        TEXTRACT(rs, rsAll, KH / 32, 0);
    }
    TMATMUL_MX(c, c, l, ls, r, rs);
    TSTORE(gc, c);
}

// ---- one Vec instruction on [64, 128] fp32 tiles; `vec` is a per-row ([64]) or per-column ([128]) operand ----
enum VecOp : int {
    kAbs = 0, kNeg, kRelu, kSqrt, kRsqrt, kLog, kRecip, kExp,
    kAdd = 20, kSub, kMul, kDiv, kMax, kMin, kPrelu, kCmpEq, kCmpNe, kCmpLt, kCmpLe, kCmpGt, kCmpGe, kSels,
    kAdds = 40, kSubs, kMuls, kDivs, kMaxs, kMins, kLrelu,
    kRowExpand = 60, kRowSub, kRowMul, kRowDiv, kRowAdd, kRowMax, kRowMin, kRowExpDif,
    kColExpand = 80, kColSub, kColMul, kColDiv, kColAdd, kColMax, kColMin, kColExpDif,
};
__global__ __launch_bounds__(kBlockThreads) AICORE void VecOpKernel(__gm__ float *out, __gm__ const float *aIn, __gm__ const float *bIn,
                                                                    __gm__ const float *vecIn, float k, int op)
{
    using TileX = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    using TileR = Tile<TileType::Vec, float, 64, 1, BLayout::ColMajor>;
    using TileC = Tile<TileType::Vec, float, 1, 128, BLayout::RowMajor>;
    TileX a, b, o;
    TileR rv;
    TileC cv;
    GmND<float, 64, 128> ga(const_cast<float *>(aIn)), gb(const_cast<float *>(bIn)), go(out);
    TLOAD(a, ga);
    if (op >= kAdd && op < kAdds)
        TLOAD(b, gb);
    if (op >= kRowExpand && op < kColExpand) {
        GmCol<float, 64> gr(const_cast<float *>(vecIn));
        TLOAD(rv, gr);
    }
    if (op >= kColExpand) {
        GmND<float, 1, 128> gc(const_cast<float *>(vecIn));
        TLOAD(cv, gc);
    }
    switch (op) {
    case kAbs: TABS(o, a); break;
    case kNeg: TNEG(o, a); break;
    case kRelu: TRELU(o, a); break;
    case kSqrt: TSQRT(o, a); break;
    case kRsqrt: TRSQRT(o, a); break;
    case kLog: TLOG(o, a); break;
    case kRecip: TRECIP(o, a); break;
    case kExp: TEXP(o, a); break;
    case kAdd: TADD(o, a, b); break;
    case kSub: TSUB(o, a, b); break;
    case kMul: TMUL(o, a, b); break;
    case kDiv: TDIV(o, a, b); break;
    case kMax: TMAX(o, a, b); break;
    case kMin: TMIN(o, a, b); break;
    case kPrelu: TPRELU(o, a, b); break;
    case kCmpEq: TCMP(o, a, b, CmpMode::EQ); break;
    case kCmpNe: TCMP(o, a, b, CmpMode::NE); break;
    case kCmpLt: TCMP(o, a, b, CmpMode::LT); break;
    case kCmpLe: TCMP(o, a, b, CmpMode::LE); break;
    case kCmpGt: TCMP(o, a, b, CmpMode::GT); break;
    case kCmpGe: TCMP(o, a, b, CmpMode::GE); break;
    case kSels: TSELS(o, a, b, (uint8_t)k); break;
    case kAdds: TADDS(o, a, k); break;
    case kSubs: TSUBS(o, a, k); break;
    case kMuls: TMULS(o, a, k); break;
    case kDivs: TDIVS(o, a, k); break;
    case kMaxs: TMAXS(o, a, k); break;
    case kMins: TMINS(o, a, k); break;
    case kLrelu: TLRELU(o, a, k); break;
    case kRowExpand: TROWEXPAND(o, rv); break;
    case kRowSub: TROWEXPANDSUB(o, a, rv); break;
    case kRowMul: TROWEXPANDMUL(o, a, rv); break;
    case kRowDiv: TROWEXPANDDIV(o, a, rv); break;
    case kRowAdd: TROWEXPANDADD(o, a, rv); break;
    case kRowMax: TROWEXPANDMAX(o, a, rv); break;
    case kRowMin: TROWEXPANDMIN(o, a, rv); break;
    case kRowExpDif: TROWEXPANDEXPDIF(o, a, rv); break;
    case kColExpand: TCOLEXPAND(o, cv); break;
    case kColSub: TCOLEXPANDSUB(o, a, cv); break;
    case kColMul: TCOLEXPANDMUL(o, a, cv); break;
    case kColDiv: TCOLEXPANDDIV(o, a, cv); break;
    case kColAdd: TCOLEXPANDADD(o, a, cv); break;
    case kColMax: TCOLEXPANDMAX(o, a, cv); break;
    case kColMin: TCOLEXPANDMIN(o, a, cv); break;
    case kColExpDif: TCOLEXPANDEXPDIF(o, a, cv); break;
    default: TMULS(o, a, 0.0f); break;
    }
    TSTORE(go, o);
}

// ---- row / column reductions of the valid region [vr, vc] of a [64, 128] fp32 tile ----
// op 0..2: TROWMAX / TROWMIN / TROWSUM -> out[64]; 3..5: TCOLMAX / TCOLMIN / TCOLSUM -> out[128].
// Entries outside the valid region are left as the caller set them.
__global__ __launch_bounds__(kBlockThreads) AICORE void ReduceKernel(__gm__ float *out, __gm__ const float *aIn, int vr, int vc, int op)
{
    using TileX = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    using TileR = Tile<TileType::Vec, float, 64, 1, BLayout::ColMajor, DYNAMIC, 1>;
    using TileC = Tile<TileType::Vec, float, 1, 128, BLayout::RowMajor, 1, DYNAMIC>;
    TileX a(vr, vc), tmp(vr, vc);
    GlobalTensor<float, Shape<1, 1, 1, DYNAMIC, DYNAMIC>, Stride<1, 1, 1, 128, 1>> ga(const_cast<float *>(aIn), Shape<1, 1, 1, DYNAMIC, DYNAMIC>(vr, vc));
    TLOAD(a, ga);
    if (op < 3) {
        TileR r(vr);
        if (op == 0)
            TROWMAX(r, a, tmp);
        else if (op == 1)
            TROWMIN(r, a, tmp);
        else
            TROWSUM(r, a, tmp);
        GlobalTensor<float, Shape<1, 1, 1, DYNAMIC, 1>, Stride<1, 1, 1, 1, 64>, Layout::DN> gr(out, Shape<1, 1, 1, DYNAMIC, 1>(vr));
        TSTORE(gr, r);
    } else {
        TileC c(vc);
        if (op == 3)
            TCOLMAX(c, a);
        else if (op == 4)
            TCOLMIN(c, a);
        else
            TCOLSUM(c, a);
        GlobalTensor<float, Shape<1, 1, 1, 1, DYNAMIC>, Stride<1, 1, 1, 128, 1>> gc(out, Shape<1, 1, 1, 1, DYNAMIC>(vc));
        TSTORE(gc, c);
    }
}

// ---- TCMPS into a packed bit mask, then TSEL with that mask: bits[64][16] and sel = bit ? a : b ----
__global__ __launch_bounds__(kBlockThreads) AICORE void CmpsSelKernel(__gm__ float *sel, __gm__ uint8_t *bits, __gm__ const float *aIn,
                                                                      __gm__ const float *bIn, float scalar, int mode)
{
    using TileX = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    using TileM = Tile<TileType::Vec, uint8_t, 64, 32, BLayout::RowMajor, 64, 16>;
    TileX a, b, o;
    TileM m;
    GmND<float, 64, 128> ga(const_cast<float *>(aIn)), gb(const_cast<float *>(bIn)), go(sel);
    GlobalTensor<uint8_t, Shape<1, 1, 1, 64, 16>, Stride<1024, 1024, 1024, 16, 1>> gm(bits);
    TLOAD(a, ga);
    TLOAD(b, gb);
    TCMPS(m, a, scalar, static_cast<CmpMode>(mode));
    TSEL(o, m, a, b);
    TSTORE(gm, m);
    TSTORE(go, o);
}

// ---- TFILLPAD: [64, 128] tile whose valid region [vr, vc] comes from GM, the rest is the pad value ----
template <PadValue PAD>
__global__ __launch_bounds__(kBlockThreads) AICORE void FillPadKernel(__gm__ float *out, __gm__ const float *aIn, int vr, int vc)
{
    using TileS = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    using TileD = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, 64, 128, SLayout::NoneBox, 512, PAD>;
    TileS a(vr, vc);
    TileD d;
    GlobalTensor<float, Shape<1, 1, 1, DYNAMIC, DYNAMIC>, Stride<1, 1, 1, 128, 1>> ga(const_cast<float *>(aIn), Shape<1, 1, 1, DYNAMIC, DYNAMIC>(vr, vc));
    GmND<float, 64, 128> go(out);
    TLOAD(a, ga);
    TFILLPAD(d, a);
    TSTORE(go, d);
}

// ---- [64, 64] x [64, 128] fp16 matmul, accumulator moved to a Vec tile (optionally clamped at zero), scaled, stored ----
__global__ __launch_bounds__(kBlockThreads) AICORE void MatmulMovKernel(__gm__ float *out, __gm__ const half *a, __gm__ const half *bT,
                                                                        int relu, float scale)
{
    using MatA = Tile<TileType::Mat, half, 64, 64, BLayout::ColMajor, 64, 64, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, half, 64, 128, BLayout::RowMajor, 64, 128, SLayout::ColMajor>;
    using TileV = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    MatA am;
    MatB bm;
    TASSIGN(am, 0u);
    TASSIGN(bm, 64u * 64u * sizeof(half));
    TileLeft<half, 64, 64> l;
    TileRight<half, 64, 128> r;
    TileAcc<float, 64, 128> c;
    TileV v;
    GmND<half, 64, 64> ga(const_cast<half *>(a));
    GlobalTensor<half, Shape<1, 1, 1, 64, 128>, Stride<1, 1, 1, 1, 64>, Layout::DN> gb(const_cast<half *>(bT));
    GmND<float, 64, 128> go(out);
    TLOAD(am, ga);
    TLOAD(bm, gb);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TMOV(l, am);
    TMOV(r, bm);
    TMATMUL(c, l, r);
    if (relu)
        TMOV<TileV, TileAcc<float, 64, 128>, ReluPreMode::NormalRelu>(v, c);
    else
        TMOV(v, c);
    TMULS(v, v, scale);
    TSTORE(go, v);
}


// ---- two-stage pipeline through FIFOs, the shape of the attention kernel's Cube -> Vec -> Cube hand-offs
// (fa_performance_kernel.cpp:346-583): for t in {0, 1}
//   S = a x b[t]                       [64,64] x [64,128] fp16 -> fp32 accumulator
//   TPUSH(S)  ->  TPOP as a Vec tile   (global-memory FIFO, or an LDS FIFO when LDS_FIFO)
//   P = fp16(0.25 S)                   TMULS, TCVT
//   TPUSH(P)  ->  TPOP as a Mat tile   (global-memory FIFO)
//   O (+)= P x v[t]                    [64,128] x [128,64]
template <bool LDS_FIFO>
__global__ __launch_bounds__(kBlockThreads) AICORE void PushPopKernel(__gm__ float *out, __gm__ const half *a, __gm__ const half *bT,
                                                                      __gm__ const half *vT, __gm__ float *qkFifoMem, __gm__ half *pFifoMem)
{
    using MatA = Tile<TileType::Mat, half, 64, 64, BLayout::ColMajor, 64, 64, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, half, 64, 128, BLayout::RowMajor, 64, 128, SLayout::ColMajor>;
    using MatP = Tile<TileType::Mat, half, 64, 128, BLayout::ColMajor, 64, 128, SLayout::RowMajor>;
    using MatV = Tile<TileType::Mat, half, 128, 64, BLayout::RowMajor, 128, 64, SLayout::ColMajor>;
    using VecS = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    using VecP = Tile<TileType::Vec, half, 64, 128, BLayout::RowMajor>;
    using AccS = TileAcc<float, 64, 128>;
    using AccO = TileAcc<float, 64, 64>;
    constexpr uint32_t kA = 0, kB = 8192, kP = kB + 16384, kV = kP + 16384, kFifo = kV + 16384;
    MatA am;
    MatB bm;
    MatP pm;
    MatV vm;
    TASSIGN(am, kA);
    TASSIGN(bm, kB);
    TASSIGN(pm, kP);
    TASSIGN(vm, kV);
    using QkFifo = DataFIFO<float, LDS_FIFO ? FIFOType::VEC_FIFO : FIFOType::GM_FIFO, 2, 1>;
    using PFifo = DataFIFO<half, FIFOType::GM_FIFO, 2, 1>;
    using QkSync = TFIFOSync<0, QkFifo, TSyncOpType::TSTORE_C2GM, TSyncOpType::TLOAD>;
    using PSync = TFIFOSync<2, PFifo, TSyncOpType::TSTORE_V2GM, TSyncOpType::TLOAD>;
    QkFifo qkFifo = LDS_FIFO ? QkFifo(kFifo, 0) : QkFifo(qkFifoMem);
    PFifo pFifo(pFifoMem);
    typename QkSync::Producer qkProd;
    typename QkSync::Consumer qkCons;
    typename PSync::Producer pProd;
    typename PSync::Consumer pCons;

    TileLeft<half, 64, 64> aLeft;
    TileRight<half, 64, 128> bRight;
    TileLeft<half, 64, 128> pLeft;
    TileRight<half, 128, 64> vRight;
    AccS sAcc;
    AccO oAcc;
    VecS sVec;
    VecP pVec;
    GmND<half, 64, 64> ga(const_cast<half *>(a));
    TLOAD(am, ga);
    for (int t = 0; t < 2; ++t) {
        GlobalTensor<half, Shape<1, 1, 1, 64, 128>, Stride<1, 1, 1, 1, 64>, Layout::DN> gb(const_cast<half *>(bT) + t * 128 * 64);
        GlobalTensor<half, Shape<1, 1, 1, 128, 64>, Stride<1, 1, 1, 1, 128>, Layout::DN> gv(const_cast<half *>(vT) + t * 64 * 128);
        pipe_barrier(PIPE_ALL); // everyone has left the Mat tiles of the previous step
        TLOAD(bm, gb);
        TLOAD(vm, gv);
        set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
        TMOV(aLeft, am);
        TMOV(bRight, bm);
        TMATMUL(sAcc, aLeft, bRight);
        TPUSH(qkProd, sAcc, qkFifo);
        TPOP(qkCons, sVec, qkFifo);
        TMULS(sVec, sVec, 0.25f);
        TCVT(pVec, sVec, RoundMode::CAST_RINT);
        TPUSH(pProd, pVec, pFifo);
        TPOP(pCons, pm, pFifo);
        TMOV(pLeft, pm);
        TMOV(vRight, vm);
        if (t == 0)
            TMATMUL(oAcc, pLeft, vRight);
        else
            TMATMUL_ACC(oAcc, oAcc, pLeft, vRight);
    }
    GmND<float, 64, 64> go(out);
    TSTORE(go, oAcc);
}

} // namespace

PTO_DEVICE_CODE_END

#define PTO_ST_NONNULL(...)                          \
    do {                                             \
        const void *ptrs[] = {__VA_ARGS__};          \
        for (const void *p : ptrs)                   \
            if (p == nullptr)                        \
                return PTO_ERR_BAD_ARG;              \
    } while (0)

extern "C" int pto_st_softmax_step_f32_64x256(void *stream, uint16_t *x_exp, float *max_out, float *sum_out, float *alpha_out,
                                              const float *x, const float *max_in, const float *sum_in, float scale,
                                              int first, int round_mode)
{
    PTO_ST_NONNULL(x_exp, max_out, sum_out, alpha_out, x);
    if (!first)
        PTO_ST_NONNULL(max_in, sum_in);
    if (round_mode < PTO_CAST_RINT || round_mode > PTO_CAST_ODD)
        return PTO_ERR_BAD_ARG;
    SoftmaxStep<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<half *>(x_exp), max_out, sum_out, alpha_out, x, max_in, sum_in, scale, first, round_mode);
    return pto_amd::check_launch();
}

extern "C" int pto_st_gu_step_f32_64x128(void *stream, float *o_out, const float *o_prev, const float *pv,
                                         const float *alpha, const float *sum, int last)
{
    PTO_ST_NONNULL(o_out, o_prev, pv, alpha, sum);
    GuStep<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(o_out, o_prev, pv, alpha, sum, last);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tri_mask_f32_64x128(void *stream, float *out, const float *x, int diagonal, float value, int upper)
{
    PTO_ST_NONNULL(out, x);
    TriMask<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, x, diagonal, value, upper);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tgather_mask_b16_16x64(void *stream, uint16_t *out, const uint16_t *src, int pattern)
{
    PTO_ST_NONNULL(out, src);
    if (pattern < 1 || pattern > 7)
        return PTO_ERR_BAD_ARG;
    GatherMask<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, src, pattern);
    return pto_amd::check_launch();
}

// shape: 0 = 32 x 32, 1 = 32 x 64, 2 = 64 x 128, 3 = 128 x 128 (the ND cases of the reference's test, tquant/main.cpp:236-251)
extern "C" int pto_st_tquant_mxfp8(void *stream, uint8_t *out_e8m0, uint8_t *out_fp8, float *out_max, float *out_scaling, const float *src,
                                   int shape, int valid_rows, int valid_cols)
{
    PTO_ST_NONNULL(out_e8m0, out_fp8, out_max, out_scaling, src);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PTO_ST_TQUANT_CASE(ID, R, C)                                                                                          \
    if (shape == ID) {                                                                                                        \
        if (valid_rows < 1 || valid_rows > R || valid_cols < 1 || valid_cols > C)                                             \
            return PTO_ERR_BAD_ARG;                                                                                           \
        TQuantMx<R, C><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out_e8m0, out_fp8, out_max, out_scaling, src, valid_rows, valid_cols); \
        return pto_amd::check_launch();                                                                                       \
    }
    PTO_ST_TQUANT_CASE(0, 32, 32)
    PTO_ST_TQUANT_CASE(1, 32, 64)
    PTO_ST_TQUANT_CASE(2, 64, 128)
    PTO_ST_TQUANT_CASE(3, 128, 128)
#undef PTO_ST_TQUANT_CASE
    return PTO_ERR_BAD_ARG;
}

extern "C" int pto_st_mgather_b16_8x128(void *stream, uint16_t *out, const uint16_t *gm, const int32_t *idx, int gm_elems)
{
    PTO_ST_NONNULL(out, gm, idx);
    MGatherElems<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, gm, idx, gm_elems);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tload_pad_f32_16x32(void *stream, float *image, const float *gm)
{
    PTO_ST_NONNULL(image, gm);
    LoadPadImage<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(image, gm);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tload_5d_f32(void *stream, float *dense, float *strided, const float *gm)
{
    PTO_ST_NONNULL(dense, strided, gm);
    Load5D<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(dense, strided, gm);
    return pto_amd::check_launch();
}

extern "C" int pto_st_textract_windows_f16(void *stream, float *out_left, float *out_right, const uint16_t *a,
                                           const uint16_t *b_t, const uint16_t *eye_b, const uint16_t *eye_a, int col0, int row0)
{
    PTO_ST_NONNULL(out_left, out_right, a, b_t, eye_b, eye_a);
    if (col0 < 0 || col0 % 8 || col0 + 64 > 256 || row0 < 0 || row0 % 8 || row0 + 64 > 256)
        return PTO_ERR_UNSUPPORTED;
    constexpr int lds = 128 * 1024;
    static const int attr = pto_amd::allow_lds(ExtractWindows, lds);
    if (attr != PTO_OK)
        return attr;
    ExtractWindows<<<dim3(1), dim3(kBlockThreads), lds, static_cast<hipStream_t>(stream)>>>(
        out_left, out_right, reinterpret_cast<const half *>(a), reinterpret_cast<const half *>(b_t),
        reinterpret_cast<const half *>(eye_b), reinterpret_cast<const half *>(eye_a), col0, row0);
    return pto_amd::check_launch();
}

extern "C" int pto_st_matmul_s8_128x128x256(void *stream, int32_t *out, const int8_t *a, const int8_t *b_t, int relu)
{
    PTO_ST_NONNULL(out, a, b_t);
    constexpr int lds = 128 * 128 + 128 * 256;
    MatmulTyped<int8_t, int32_t, 128><<<dim3(1), dim3(kBlockThreads), lds, static_cast<hipStream_t>(stream)>>>(out, a, b_t, relu);
    return pto_amd::check_launch();
}

extern "C" int pto_st_matmul_f32_128x32x256(void *stream, float *out, const float *a, const float *b_t, int relu)
{
    PTO_ST_NONNULL(out, a, b_t);
    constexpr int lds = (128 * 32 + 32 * 256) * 4;
    MatmulTyped<float, float, 32><<<dim3(1), dim3(kBlockThreads), lds, static_cast<hipStream_t>(stream)>>>(out, a, b_t, relu);
    return pto_amd::check_launch();
}

static int matmul_mx_128x256x128(void *stream, float *out, const uint8_t *a, const uint8_t *b_t, const uint8_t *scale_a,
                                 const uint8_t *scale_b_t, const float *bias, int format_a, int format_b, int scales_via_lds)
{
    PTO_ST_NONNULL(out, a, b_t, scale_a, scale_b_t);
    if (format_a < 0 || format_a > 1 || format_b < 0 || format_b > 1)
        return PTO_ERR_BAD_ARG;
    constexpr int lds = 128 * 256 + 256 * 128 + 2 * 128 * 8;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const float8_e8m0_t *sa = reinterpret_cast<const float8_e8m0_t *>(scale_a), *sb = reinterpret_cast<const float8_e8m0_t *>(scale_b_t);
#define PTO_ST_MX(FA, FB)                                                                                                     \
    do {                                                                                                                      \
        static const int attr0 = pto_amd::allow_lds(MatmulMx<FA, FB, false>, lds);                                            \
        static const int attr1 = pto_amd::allow_lds(MatmulMx<FA, FB, true>, lds);                                             \
        if (attr0 != PTO_OK || attr1 != PTO_OK)                                                                               \
            return attr0 != PTO_OK ? attr0 : attr1;                                                                           \
        if (scales_via_lds)                                                                                                   \
            MatmulMx<FA, FB, true><<<dim3(1), dim3(kBlockThreads), lds, st>>>(out, reinterpret_cast<const FA *>(a),           \
                                                                              reinterpret_cast<const FB *>(b_t), sa, sb, bias); \
        else                                                                                                                  \
            MatmulMx<FA, FB, false><<<dim3(1), dim3(kBlockThreads), lds, st>>>(out, reinterpret_cast<const FA *>(a),          \
                                                                               reinterpret_cast<const FB *>(b_t), sa, sb, bias); \
    } while (0)
    if (format_a == 0 && format_b == 0)
        PTO_ST_MX(float8_e4m3_t, float8_e4m3_t);
    else if (format_a == 0)
        PTO_ST_MX(float8_e4m3_t, float8_e5m2_t);
    else if (format_b == 0)
        PTO_ST_MX(float8_e5m2_t, float8_e4m3_t);
    else
        PTO_ST_MX(float8_e5m2_t, float8_e5m2_t);
#undef PTO_ST_MX
    return pto_amd::check_launch();
}

extern "C" int pto_st_matmul_mx_128x256x128(void *stream, float *out, const uint8_t *a, const uint8_t *b_t, const uint8_t *scale_a,
                                            const uint8_t *scale_b_t, int format_a, int format_b, int scales_via_lds)
{
    return matmul_mx_128x256x128(stream, out, a, b_t, scale_a, scale_b_t, nullptr, format_a, format_b, scales_via_lds);
}

extern "C" int pto_st_matmul_mx_bias_128x256x128(void *stream, float *out, const uint8_t *a, const uint8_t *b_t, const uint8_t *scale_a,
                                                 const uint8_t *scale_b_t, const float *bias, int format_a, int format_b)
{
    PTO_ST_NONNULL(bias);
    return matmul_mx_128x256x128(stream, out, a, b_t, scale_a, scale_b_t, bias, format_a, format_b, 0);
}

extern "C" int pto_st_matmul_bias_128x64x256(void *stream, float *out, const uint16_t *a, const uint16_t *b_t,
                                             const float *bias, int bf16)
{
    PTO_ST_NONNULL(out, a, b_t);
    constexpr int lds = (128 * 64 + 64 * 256) * 2;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (bf16)
        MatmulBias<bfloat16_t, 64><<<dim3(1), dim3(kBlockThreads), lds, st>>>(
            out, reinterpret_cast<const bfloat16_t *>(a), reinterpret_cast<const bfloat16_t *>(b_t), bias);
    else
        MatmulBias<half, 64><<<dim3(1), dim3(kBlockThreads), lds, st>>>(out, reinterpret_cast<const half *>(a),
                                                                         reinterpret_cast<const half *>(b_t), bias);
    return pto_amd::check_launch();
}

// The arithmetic subset of the Vec instructions on fp16 and int32 tiles (the reference's per-instruction tests run
// them on half, float, int32 and int16: e.g. tests/cpu/st/testcase/tadd/main.cpp).
template <typename T>
__global__ __launch_bounds__(kBlockThreads) AICORE void VecOpTyped(__gm__ T *out, __gm__ const T *aIn, __gm__ const T *bIn,
                                                                   __gm__ const T *vecIn, T k, int op)
{
    using TileX = Tile<TileType::Vec, T, 64, 128, BLayout::RowMajor>;
    using TileR = Tile<TileType::Vec, T, 64, 1, BLayout::ColMajor>;
    using TileC = Tile<TileType::Vec, T, 1, 128, BLayout::RowMajor>;
    TileX a, b, o;
    TileR rv;
    TileC cv;
    GmND<T, 64, 128> ga(const_cast<T *>(aIn)), gb(const_cast<T *>(bIn)), go(out);
    TLOAD(a, ga);
    if (op >= kAdd && op < kAdds)
        TLOAD(b, gb);
    if (op >= kRowExpand && op < kColExpand) {
        GmCol<T, 64> gr(const_cast<T *>(vecIn));
        TLOAD(rv, gr);
    }
    if (op >= kColExpand) {
        GmND<T, 1, 128> gc(const_cast<T *>(vecIn));
        TLOAD(cv, gc);
    }
    bool floatOp = false;
    if constexpr (!std::is_integral_v<T>) { // the transcendental and division instructions: floating-point tiles
        floatOp = true;
        switch (op) {
        case kSqrt: TSQRT(o, a); break;
        case kRsqrt: TRSQRT(o, a); break;
        case kLog: TLOG(o, a); break;
        case kRecip: TRECIP(o, a); break;
        case kExp: TEXP(o, a); break;
        case kDiv: TDIV(o, a, b); break;
        case kDivs: TDIVS(o, a, k); break;
        default: floatOp = false; break;
        }
    }
    if (!floatOp)
    switch (op) {
    case kAbs: TABS(o, a); break;
    case kNeg: TNEG(o, a); break;
    case kRelu: TRELU(o, a); break;
    case kAdd: TADD(o, a, b); break;
    case kSub: TSUB(o, a, b); break;
    case kMul: TMUL(o, a, b); break;
    case kMax: TMAX(o, a, b); break;
    case kMin: TMIN(o, a, b); break;
    case kAdds: TADDS(o, a, k); break;
    case kSubs: TSUBS(o, a, k); break;
    case kMuls: TMULS(o, a, k); break;
    case kMaxs: TMAXS(o, a, k); break;
    case kMins: TMINS(o, a, k); break;
    case kRowExpand: TROWEXPAND(o, rv); break;
    case kRowSub: TROWEXPANDSUB(o, a, rv); break;
    case kRowMul: TROWEXPANDMUL(o, a, rv); break;
    case kRowAdd: TROWEXPANDADD(o, a, rv); break;
    case kRowMax: TROWEXPANDMAX(o, a, rv); break;
    case kRowMin: TROWEXPANDMIN(o, a, rv); break;
    case kColExpand: TCOLEXPAND(o, cv); break;
    case kColSub: TCOLEXPANDSUB(o, a, cv); break;
    case kColMul: TCOLEXPANDMUL(o, a, cv); break;
    case kColAdd: TCOLEXPANDADD(o, a, cv); break;
    case kColMax: TCOLEXPANDMAX(o, a, cv); break;
    case kColMin: TCOLEXPANDMIN(o, a, cv); break;
    default: TSUB(o, a, a); break;
    }
    TSTORE(go, o);
}

extern "C" int pto_st_vec_op_typed_64x128(void *stream, void *out, const void *a, const void *b, const void *vec, float scalar, int op,
                                          int dtype)
{
    PTO_ST_NONNULL(out, a);
    const bool known = (op >= kAbs && op <= kRelu) || (op >= kAdd && op <= kMin && op != kDiv) ||
                       (op >= kAdds && op <= kMins && op != kDivs) || (op >= kRowExpand && op <= kRowMin && op != kRowDiv) ||
                       (op >= kColExpand && op <= kColMin && op != kColDiv);
    const bool floatOnly = (op >= kSqrt && op <= kExp) || op == kDiv || op == kDivs;
    if (!(known || (floatOnly && dtype == 0)) || dtype < 0 || dtype > 1)
        return PTO_ERR_BAD_ARG;
    if (op >= kAdd && op <= kMin)
        PTO_ST_NONNULL(b);
    if (op >= kRowExpand)
        PTO_ST_NONNULL(vec);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        VecOpTyped<half><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<half *>(out), static_cast<const half *>(a),
                                                                  static_cast<const half *>(b), static_cast<const half *>(vec),
                                                                  (half)scalar, op);
    else
        VecOpTyped<int32_t><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<int32_t *>(out), static_cast<const int32_t *>(a),
                                                                     static_cast<const int32_t *>(b), static_cast<const int32_t *>(vec),
                                                                     (int32_t)scalar, op);
    return pto_amd::check_launch();
}

// Bitwise, shift, remainder and three-operand Vec instructions (the reference tests them per instruction:
// tests/cpu/st/testcase/{tand,tor,txor,tnot,tshl,tshr,trem,taddc,tsubc,tands,...}/): int32 tiles run every op, fp32 tiles
// the remainder and three-operand ones.
enum BitOp : int {
    kBitAnd = 0, kBitOr, kBitXor, kBitShl, kBitShr, kBitRem, kBitNot, kBitAnds, kBitOrs, kBitXors, kBitShls, kBitShrs, kBitRems,
    kBitAddc, kBitSubc, kBitAddsc, kBitSubsc, kBitOpCount
};
template <typename T>
__global__ __launch_bounds__(kBlockThreads) AICORE void VecBitOp(__gm__ T *out, __gm__ const T *aIn, __gm__ const T *bIn,
                                                                 __gm__ const T *cIn, T k, int op)
{
    using TileX = Tile<TileType::Vec, T, 64, 128, BLayout::RowMajor>;
    TileX a, b, c, o, tmp;
    GmND<T, 64, 128> ga(const_cast<T *>(aIn)), gb(const_cast<T *>(bIn)), gc(const_cast<T *>(cIn)), go(out);
    TLOAD(a, ga);
    TLOAD(b, gb);
    TLOAD(c, gc);
    if constexpr (std::is_integral_v<T>) {
        switch (op) {
        case kBitAnd: TAND(o, a, b); break;
        case kBitOr: TOR(o, a, b); break;
        case kBitXor: TXOR(o, a, b, tmp); break;
        case kBitShl: TSHL(o, a, b); break;
        case kBitShr: TSHR(o, a, b); break;
        case kBitNot: TNOT(o, a); break;
        case kBitAnds: TANDS(o, a, k); break;
        case kBitOrs: TORS(o, a, k); break;
        case kBitXors: TXORS(o, a, k, tmp); break;
        case kBitShls: TSHLS(o, a, k); break;
        case kBitShrs: TSHRS(o, a, k); break;
        default: break;
        }
    }
    switch (op) {
    case kBitRem: TREM(o, a, b); break;
    case kBitRems: TREMS(o, a, k); break;
    case kBitAddc: TADDC(o, a, b, c); break;
    case kBitSubc: TSUBC(o, a, b, c); break;
    case kBitAddsc: TADDSC(o, a, k, c); break;
    case kBitSubsc: TSUBSC(o, a, k, c); break;
    default: break;
    }
    TSTORE(go, o);
}

// dtype 0: fp32 (scalar_f), 1: int32 (scalar_i); a, b and c are all read
extern "C" int pto_st_vec_bitop_64x128(void *stream, void *out, const void *a, const void *b, const void *c, float scalar_f,
                                       int scalar_i, int op, int dtype)
{
    PTO_ST_NONNULL(out, a, b, c);
    if (op < 0 || op >= kBitOpCount || dtype < 0 || dtype > 1)
        return PTO_ERR_BAD_ARG;
    const bool forFloat = op == kBitRem || op == kBitRems || op >= kBitAddc;
    if (dtype == 0 && !forFloat)
        return PTO_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == 0)
        VecBitOp<float><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<float *>(out), static_cast<const float *>(a),
                                                                 static_cast<const float *>(b), static_cast<const float *>(c), scalar_f, op);
    else
        VecBitOp<int32_t><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<int32_t *>(out), static_cast<const int32_t *>(a),
                                                                   static_cast<const int32_t *>(b), static_cast<const int32_t *>(c),
                                                                   scalar_i, op);
    return pto_amd::check_launch();
}

extern "C" int pto_st_vec_op_f32_64x128(void *stream, float *out, const float *a, const float *b, const float *vec, float scalar, int op)
{
    PTO_ST_NONNULL(out, a);
    const bool known = (op >= kAbs && op <= kExp) || (op >= kAdd && op <= kSels) || (op >= kAdds && op <= kLrelu) ||
                       (op >= kRowExpand && op <= kRowExpDif) || (op >= kColExpand && op <= kColExpDif);
    if (!known)
        return PTO_ERR_BAD_ARG;
    if (op >= kAdd && op <= kSels)
        PTO_ST_NONNULL(b);
    if (op >= kRowExpand)
        PTO_ST_NONNULL(vec);
    VecOpKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, a, b, vec, scalar, op);
    return pto_amd::check_launch();
}

extern "C" int pto_st_reduce_f32_64x128(void *stream, float *out, const float *a, int valid_rows, int valid_cols, int op)
{
    PTO_ST_NONNULL(out, a);
    if (valid_rows < 1 || valid_rows > 64 || valid_cols < 1 || valid_cols > 128 || op < 0 || op > 5)
        return PTO_ERR_BAD_ARG;
    ReduceKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, a, valid_rows, valid_cols, op);
    return pto_amd::check_launch();
}

extern "C" int pto_st_cmps_sel_f32_64x128(void *stream, float *sel, uint8_t *bits, const float *a, const float *b, float scalar, int cmp_mode)
{
    PTO_ST_NONNULL(sel, bits, a, b);
    if (cmp_mode < 0 || cmp_mode > 5)
        return PTO_ERR_BAD_ARG;
    CmpsSelKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(sel, bits, a, b, scalar, cmp_mode);
    return pto_amd::check_launch();
}

extern "C" int pto_st_fillpad_f32_64x128(void *stream, float *out, const float *a, int valid_rows, int valid_cols, int pad_kind)
{
    PTO_ST_NONNULL(out, a);
    if (valid_rows < 1 || valid_rows > 64 || valid_cols < 1 || valid_cols > 128 || pad_kind < 1 || pad_kind > 3)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (pad_kind == 1)
        FillPadKernel<PadValue::Zero><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, a, valid_rows, valid_cols);
    else if (pad_kind == 2)
        FillPadKernel<PadValue::Max><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, a, valid_rows, valid_cols);
    else
        FillPadKernel<PadValue::Min><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, a, valid_rows, valid_cols);
    return pto_amd::check_launch();
}

// Matmul whose operands arrive as Vec tiles and are moved into Left / Right with TMOV (the operand path of the Auto-mode
// programs: cpu/TMov.hpp Vec -> Left / Right), the result moved Acc -> Left and multiplied once more, and TTRANS:
//   out = (A B) B2 with A [64,64], B [64,128], B2 = B^T [128,64] made by TTRANS; fp16 operands, fp32 accumulators;
//   the intermediate A B is cast to fp16 by the Acc -> Left move.
__global__ __launch_bounds__(kBlockThreads) AICORE void MatmulVecOperands(__gm__ float *out, __gm__ float *mid, __gm__ const half *a,
                                                                          __gm__ const half *b)
{
    using VA = Tile<TileType::Vec, half, 64, 64, BLayout::RowMajor>;
    using VB = Tile<TileType::Vec, half, 64, 128, BLayout::RowMajor>;
    using VBT = Tile<TileType::Vec, half, 128, 64, BLayout::RowMajor>;
    VA va;
    VB vb;
    VBT vbt;
    GmND<half, 64, 64> ga(const_cast<half *>(a));
    GmND<half, 64, 128> gb(const_cast<half *>(b));
    TLOAD(va, ga);
    TLOAD(vb, gb);
    TileLeft<half, 64, 64> l;
    TileRight<half, 64, 128> r;
    TMOV(l, va);
    TMOV(r, vb);
    TileAcc<float, 64, 128> c;
    TMATMUL(c, l, r);
    GmND<float, 64, 128> gmid(mid);
    TSTORE(gmid, c);
    TTRANS(vbt, vb, vb);
    TileLeft<half, 64, 128> l2;
    TileRight<half, 128, 64> r2;
    TMOV(l2, c);
    TMOV(r2, vbt);
    TileAcc<float, 64, 64> c2;
    TMATMUL(c2, l2, r2);
    GmND<float, 64, 64> go(out);
    TSTORE(go, c2);
}

// TTRANS alone on fp32: out [128,64] = in [64,128] transposed
__global__ __launch_bounds__(kBlockThreads) AICORE void TransKernel(__gm__ float *out, __gm__ const float *in)
{
    Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor> x;
    Tile<TileType::Vec, float, 128, 64, BLayout::RowMajor> y;
    GmND<float, 64, 128> gi(const_cast<float *>(in));
    GmND<float, 128, 64> go(out);
    TLOAD(x, gi);
    TTRANS(y, x, x);
    TSTORE(go, y);
}

// TPREFETCH (the tile then holds the region, as after a TLOAD), TPACK to 16 and to 8 bits, and, when asked, TPRINT of
// the [4, 16] corner tile and of the matching corner of the input in memory
__global__ __launch_bounds__(kBlockThreads) AICORE void PackKernel(__gm__ int16_t *out16, __gm__ int8_t *out8, __gm__ const int32_t *in, int print)
{
    Tile<TileType::Vec, int32_t, 16, 64, BLayout::RowMajor> x;
    Tile<TileType::Vec, int16_t, 16, 64, BLayout::RowMajor> y16;
    Tile<TileType::Vec, int8_t, 16, 64, BLayout::RowMajor> y8;
    GmND<int32_t, 16, 64> gi(const_cast<int32_t *>(in));
    GmND<int16_t, 16, 64> go16(out16);
    GmND<int8_t, 16, 64> go8(out8);
    TPREFETCH(x, gi);
    TPACK(y16, x);
    TPACK(y8, y16);
    TSTORE(go16, y16);
    TSTORE(go8, y8);
    if (print) {
        Tile<TileType::Vec, int32_t, 4, 16, BLayout::RowMajor, -1, -1> corner(3, 10);
        GlobalTensor<int32_t, Shape<1, 1, 1, 4, 16>, Stride<64 * 16, 64 * 16, 64 * 16, 64, 1>> gc(const_cast<int32_t *>(in));
        TLOAD(corner, gc);
        TPRINT(corner);
        GlobalTensor<int32_t, Shape<1, 1, 1, 2, 4>, Stride<64 * 16, 64 * 16, 64 * 16, 64, 1>> gs(const_cast<int32_t *>(in));
        TPRINT(gs);
    }
}

// ---- TSORT32 on an [8, 128] tile with valid region [vr, vc]; out [8, 256] (4-byte scores) or [8, 512] (2-byte) is loaded first so that the elements the
// instruction leaves alone keep what the caller put there ----
template <typename T>
__global__ __launch_bounds__(kBlockThreads) AICORE void Sort32Kernel(__gm__ T *out, __gm__ const T *srcIn, __gm__ const uint32_t *idxIn,
                                                                    int vr, int vc)
{
    using Full = Tile<TileType::Vec, T, 8, 128, BLayout::RowMajor>;
    using FullI = Tile<TileType::Vec, uint32_t, 8, 128, BLayout::RowMajor>;
    using Src = Tile<TileType::Vec, T, 8, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    using Idx = Tile<TileType::Vec, uint32_t, 8, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    constexpr int kDstCols = 128 * 8 / (int)sizeof(T);
    using Dst = Tile<TileType::Vec, T, 8, kDstCols, BLayout::RowMajor>;
    Full sf;
    FullI xf;
    Dst d;
    GmND<T, 8, 128> gs(const_cast<T *>(srcIn));
    GmND<uint32_t, 8, 128> gi(const_cast<uint32_t *>(idxIn));
    GmND<T, 8, kDstCols> go(out);
    TLOAD(sf, gs);
    TLOAD(xf, gi);
    TLOAD(d, go);
    Src s(vr, vc);
    Idx x(vr, vc);
    s.st = sf.st;
    x.st = xf.st;
    TSORT32(d, s, x);
    TSTORE(go, d);
}

// ---- TMRGSORT, one source: [1, COLS] tile (8 KiB), the destination's valid columns and the block length at run time ----
template <typename T>
__global__ __launch_bounds__(kBlockThreads) AICORE void MergeBlocksKernel(__gm__ T *out, __gm__ const T *srcIn, int validCols, int blockLen)
{
    constexpr int COLS = 4096 / (int)sizeof(T);
    using Full = Tile<TileType::Vec, T, 1, COLS, BLayout::RowMajor>;
    using Dst = Tile<TileType::Vec, T, 1, COLS, BLayout::RowMajor, 1, DYNAMIC>;
    Full s, d0;
    GmND<T, 1, COLS> gs(const_cast<T *>(srcIn)), go(out);
    TLOAD(s, gs);
    TLOAD(d0, go);
    Dst d(validCols);
    d.st = d0.st;
    TMRGSORT(d, s, (uint32_t)blockLen);
    d0.st = d.st;
    TSTORE(go, d0);
}

// ---- TMRGSORT, two to four lists of up to 128 structures each into a destination of up to 512 ----
template <typename T, int LISTS, bool EXHAUSTED>
__global__ __launch_bounds__(kBlockThreads) AICORE void MergeListsKernel(__gm__ T *out, __gm__ uint32_t *executedOut, __gm__ const T *in0,
                                                                         __gm__ const T *in1, __gm__ const T *in2, __gm__ const T *in3, int c0,
                                                                         int c1, int c2, int c3, int outCols)
{
    constexpr int LC = 1024 / (int)sizeof(T), DC = 4 * LC;
    using Full = Tile<TileType::Vec, T, 1, LC, BLayout::RowMajor>;
    using List = Tile<TileType::Vec, T, 1, LC, BLayout::RowMajor, 1, DYNAMIC>;
    using FullD = Tile<TileType::Vec, T, 1, DC, BLayout::RowMajor>;
    using Dst = Tile<TileType::Vec, T, 1, DC, BLayout::RowMajor, 1, DYNAMIC>;
    Full f;
    FullD d0, tmp;
    List l0(c0), l1(c1), l2(c2), l3(c3);
    GmND<T, 1, DC> go(out);
    const T *ins[4] = {in0, in1, in2, in3};
    List *lists[4] = {&l0, &l1, &l2, &l3};
#pragma unroll
    for (int i = 0; i < LISTS; ++i) {
        GmND<T, 1, LC> g(const_cast<T *>(ins[i]));
        TLOAD(f, g);
        lists[i]->st = f.st;
    }
    TLOAD(d0, go);
    Dst d(outCols);
    d.st = d0.st;
    MrgSortExecutedNumList executed = {};
    if constexpr (LISTS == 4)
        TMRGSORT<Dst, FullD, List, List, List, List, EXHAUSTED>(d, executed, tmp, l0, l1, l2, l3);
    else if constexpr (LISTS == 3)
        TMRGSORT<Dst, FullD, List, List, List, EXHAUSTED>(d, executed, tmp, l0, l1, l2);
    else
        TMRGSORT<Dst, FullD, List, List, EXHAUSTED>(d, executed, tmp, l0, l1);
    d0.st = d.st;
    TSTORE(go, d0);
    if (hw::tid() == 0) {
        executedOut[0] = executed.mrgSortList0;
        executedOut[1] = executed.mrgSortList1;
        executedOut[2] = executed.mrgSortList2;
        executedOut[3] = executed.mrgSortList3;
    }
}

// ---- TPARTADD / TPARTMAX / TPARTMIN on [64, 128] fp32 tiles whose three valid regions come at run time; out is loaded
// first so that the elements outside the destination's valid region keep what the caller put there ----
__global__ __launch_bounds__(kBlockThreads) AICORE void PartOpKernel(__gm__ float *out, __gm__ const float *aIn, __gm__ const float *bIn,
                                                                     int op, int dvr, int dvc, int avr, int avc, int bvr, int bvc)
{
    using Full = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    using Dyn = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    Full fa, fb, fo;
    GmND<float, 64, 128> ga(const_cast<float *>(aIn)), gb(const_cast<float *>(bIn)), go(out);
    TLOAD(fa, ga);
    TLOAD(fb, gb);
    TLOAD(fo, go);
    Dyn a(avr, avc), b(bvr, bvc), d(dvr, dvc);
    a.st = fa.st;
    b.st = fb.st;
    d.st = fo.st;
    if (op == 0)
        TPARTADD(d, a, b);
    else if (op == 1)
        TPARTMAX(d, a, b);
    else
        TPARTMIN(d, a, b);
    fo.st = d.st;
    TSTORE(go, fo);
}

extern "C" int pto_st_tpart_f32_64x128(void *stream, float *out, const float *a, const float *b, int op, int dst_valid_rows,
                                       int dst_valid_cols, int a_valid_rows, int a_valid_cols, int b_valid_rows, int b_valid_cols)
{
    PTO_ST_NONNULL(out, a, b);
    const int v[6] = {dst_valid_rows, dst_valid_cols, a_valid_rows, a_valid_cols, b_valid_rows, b_valid_cols};
    for (int i = 0; i < 6; ++i)
        if (v[i] < 0 || v[i] > (i % 2 ? 128 : 64))
            return PTO_ERR_BAD_ARG;
    if (op < 0 || op > 2)
        return PTO_ERR_BAD_ARG;
    PartOpKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, a, b, op, v[0], v[1], v[2], v[3], v[4], v[5]);
    return pto_amd::check_launch();
}

// ---- TSCATTER on [64, 128] fp32 tiles (valid region of the source at run time), MSCATTER of the same tile into memory,
// TCI on a [1, 1024] int32 tile ----
__global__ __launch_bounds__(kBlockThreads) AICORE void ScatterKernel(__gm__ float *out, __gm__ const float *srcIn, __gm__ const int32_t *idxIn,
                                                                      int vr, int vc, int toMemory)
{
    using Full = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
    using FullI = Tile<TileType::Vec, int32_t, 64, 128, BLayout::RowMajor>;
    using Dyn = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    using DynI = Tile<TileType::Vec, int32_t, 64, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    Full fs, fo;
    FullI fi;
    GmND<float, 64, 128> gs(const_cast<float *>(srcIn)), go(out);
    GmND<int32_t, 64, 128> gi(const_cast<int32_t *>(idxIn));
    TLOAD(fs, gs);
    TLOAD(fi, gi);
    Dyn s(vr, vc), d(vr, vc);
    DynI x(vr, vc);
    s.st = fs.st;
    x.st = fi.st;
    if (toMemory) {
        MSCATTER(go, s, x);
        return;
    }
    TLOAD(fo, go);
    d.st = fo.st;
    TSCATTER(d, s, x);
    fo.st = d.st;
    TSTORE(go, fo);
}

// ---- TGATHERB: dst [16, 128] fp32 (run-time valid region) from a [32, 64] source tile with [16, 16] byte offsets ----
__global__ __launch_bounds__(kBlockThreads) AICORE void GatherBKernel(__gm__ float *out, __gm__ const float *srcIn, __gm__ const uint32_t *offIn,
                                                                      int vr, int vc)
{
    using Full = Tile<TileType::Vec, float, 16, 128, BLayout::RowMajor>;
    using Dyn = Tile<TileType::Vec, float, 16, 128, BLayout::RowMajor, DYNAMIC, DYNAMIC>;
    Full f;
    Tile<TileType::Vec, float, 32, 64, BLayout::RowMajor> s;
    Tile<TileType::Vec, uint32_t, 16, 16, BLayout::RowMajor> o;
    GmND<float, 16, 128> go(out);
    GmND<float, 32, 64> gs(const_cast<float *>(srcIn));
    GmND<uint32_t, 16, 16> gof(const_cast<uint32_t *>(offIn));
    TLOAD(f, go);
    TLOAD(s, gs);
    TLOAD(o, gof);
    Dyn d(vr, vc);
    d.st = f.st;
    TGATHERB(d, s, o);
    f.st = d.st;
    TSTORE(go, f);
}

template <int DESC>
__global__ __launch_bounds__(kBlockThreads) AICORE void CiKernel(__gm__ int32_t *out, int32_t start, int vc)
{
    using Full = Tile<TileType::Vec, int32_t, 1, 1024, BLayout::RowMajor>;
    using Dyn = Tile<TileType::Vec, int32_t, 1, 1024, BLayout::RowMajor, 1, DYNAMIC>;
    Full f;
    GmND<int32_t, 1, 1024> go(out);
    TLOAD(f, go);
    Dyn d(vc);
    d.st = f.st;
    TCI<Dyn, int32_t, DESC>(d, start);
    f.st = d.st;
    TSTORE(go, f);
}

extern "C" int pto_st_scatter_f32_64x128(void *stream, float *out, const float *src, const int32_t *idx, int valid_rows, int valid_cols,
                                         int to_memory)
{
    PTO_ST_NONNULL(out, src, idx);
    if (valid_rows < 0 || valid_rows > 64 || valid_cols < 0 || valid_cols > 128)
        return PTO_ERR_BAD_ARG;
    ScatterKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, src, idx, valid_rows, valid_cols, to_memory != 0);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tgatherb_f32_16x128(void *stream, float *out, const float *src, const uint32_t *offsets, int valid_rows, int valid_cols)
{
    PTO_ST_NONNULL(out, src, offsets);
    if (valid_rows < 0 || valid_rows > 16 || valid_cols < 0 || valid_cols > 128 || valid_cols % 8)
        return PTO_ERR_BAD_ARG;
    GatherBKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, src, offsets, valid_rows, valid_cols);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tci_s32_1x1024(void *stream, int32_t *out, int32_t start, int descending, int valid_cols)
{
    PTO_ST_NONNULL(out);
    if (valid_cols < 0 || valid_cols > 1024)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (descending)
        CiKernel<1><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, start, valid_cols);
    else
        CiKernel<0><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, start, valid_cols);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tsort32_8x128(void *stream, void *out, const void *src, const uint32_t *idx, int valid_rows, int valid_cols, int dtype)
{
    PTO_ST_NONNULL(out, src, idx);
    if (valid_rows < 0 || valid_rows > 8 || valid_cols < 0 || valid_cols > 128 || dtype < 0 || dtype > 3)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PTO_ST_SORT32(T) \
    Sort32Kernel<T><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<T *>(out), static_cast<const T *>(src), idx, valid_rows, valid_cols)
    if (dtype == 0)
        PTO_ST_SORT32(float);
    else if (dtype == 1)
        PTO_ST_SORT32(int32_t);
    else if (dtype == 2)
        PTO_ST_SORT32(half);
    else
        PTO_ST_SORT32(int16_t);
#undef PTO_ST_SORT32
    return pto_amd::check_launch();
}

extern "C" int pto_st_tmrgsort_blocks_f32_1x1024(void *stream, float *out, const float *src, int valid_cols, int block_len)
{
    PTO_ST_NONNULL(out, src);
    if (valid_cols < 0 || valid_cols > 1024 || block_len < 0 || block_len > 256)
        return PTO_ERR_BAD_ARG;
    MergeBlocksKernel<float><<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, src, valid_cols, block_len);
    return pto_amd::check_launch();
}

extern "C" int pto_st_tmrgsort_blocks_16_1x2048(void *stream, void *out, const void *src, int valid_cols, int block_len, int dtype)
{
    PTO_ST_NONNULL(out, src);
    if (valid_cols < 0 || valid_cols > 2048 || block_len < 0 || block_len > 512 || dtype < 0 || dtype > 2)
        return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PTO_ST_BLOCKS(T) \
    MergeBlocksKernel<T><<<dim3(1), dim3(kBlockThreads), 0, st>>>(static_cast<T *>(out), static_cast<const T *>(src), valid_cols, block_len)
    if (dtype == 0)
        PTO_ST_BLOCKS(half);
    else if (dtype == 1)
        PTO_ST_BLOCKS(uint16_t);
    else
        PTO_ST_BLOCKS(int16_t);
#undef PTO_ST_BLOCKS
    return pto_amd::check_launch();
}

namespace {
template <typename T>
int merge_lists_launch(void *stream, T *out, uint32_t *executed, const T *src0, const T *src1, const T *src2, const T *src3, int cols0,
                       int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted)
{
    constexpr int E = 8 / (int)sizeof(T), LC = 1024 / (int)sizeof(T);
    PTO_ST_NONNULL(out, executed, src0, src1);
    if (lists < 2 || lists > 4 || (lists > 2 && !src2) || (lists > 3 && !src3) || out_cols < 0 || out_cols > 4 * LC)
        return PTO_ERR_BAD_ARG;
    const int cols[4] = {cols0, cols1, cols2, cols3};
    for (int i = 0; i < lists; ++i)
        if (cols[i] < 0 || cols[i] > LC || cols[i] % E)
            return PTO_ERR_BAD_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PTO_ST_MERGE(L, X) \
    MergeListsKernel<T, L, X><<<dim3(1), dim3(kBlockThreads), 0, st>>>(out, executed, src0, src1, src2, src3, cols0, cols1, cols2, cols3, out_cols)
    if (lists == 4 && exhausted)
        PTO_ST_MERGE(4, true);
    else if (lists == 4)
        PTO_ST_MERGE(4, false);
    else if (lists == 3 && exhausted)
        PTO_ST_MERGE(3, true);
    else if (lists == 3)
        PTO_ST_MERGE(3, false);
    else if (exhausted)
        PTO_ST_MERGE(2, true);
    else
        PTO_ST_MERGE(2, false);
#undef PTO_ST_MERGE
    return pto_amd::check_launch();
}
} // namespace

extern "C" int pto_st_tmrgsort_lists_f32(void *stream, float *out, uint32_t *executed, const float *src0, const float *src1, const float *src2,
                                         const float *src3, int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted)
{
    return merge_lists_launch<float>(stream, out, executed, src0, src1, src2, src3, cols0, cols1, cols2, cols3, out_cols, lists, exhausted);
}

extern "C" int pto_st_tmrgsort_lists_16(void *stream, void *out, uint32_t *executed, const void *src0, const void *src1, const void *src2,
                                        const void *src3, int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted,
                                        int dtype)
{
    if (dtype < 0 || dtype > 1)
        return PTO_ERR_BAD_ARG;
    if (dtype == 0)
        return merge_lists_launch<half>(stream, static_cast<half *>(out), executed, static_cast<const half *>(src0),
                                        static_cast<const half *>(src1), static_cast<const half *>(src2), static_cast<const half *>(src3), cols0,
                                        cols1, cols2, cols3, out_cols, lists, exhausted);
    return merge_lists_launch<uint16_t>(stream, static_cast<uint16_t *>(out), executed, static_cast<const uint16_t *>(src0),
                                        static_cast<const uint16_t *>(src1), static_cast<const uint16_t *>(src2),
                                        static_cast<const uint16_t *>(src3), cols0, cols1, cols2, cols3, out_cols, lists, exhausted);
}

extern "C" int pto_st_matmul_vec_operands_f16_64x64x128(void *stream, float *out, float *mid, const uint16_t *a, const uint16_t *b)
{
    PTO_ST_NONNULL(out, mid, a, b);
    MatmulVecOperands<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, mid, reinterpret_cast<const half *>(a),
                                                                                            reinterpret_cast<const half *>(b));
    return pto_amd::check_launch();
}

extern "C" int pto_st_ttrans_f32_64x128(void *stream, float *out, const float *in)
{
    PTO_ST_NONNULL(out, in);
    TransKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, in);
    return pto_amd::check_launch();
}

extern "C" int pto_st_prefetch_pack_print_s32_16x64(void *stream, int16_t *out16, int8_t *out8, const int32_t *in, int print)
{
    PTO_ST_NONNULL(out16, out8, in);
    PackKernel<<<dim3(1), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out16, out8, in, print);
    return pto_amd::check_launch();
}

extern "C" int pto_st_matmul_tmov_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, int relu, float scale)
{
    PTO_ST_NONNULL(out, a, b_t);
    MatmulMovKernel<<<dim3(1), dim3(kBlockThreads), (64 * 64 + 64 * 128) * sizeof(half), static_cast<hipStream_t>(stream)>>>(
        out, reinterpret_cast<const half *>(a), reinterpret_cast<const half *>(b_t), relu, scale);
    return pto_amd::check_launch();
}

extern "C" int pto_st_pushpop_f16_64x64x128(void *stream, float *out, const uint16_t *a, const uint16_t *b_t, const uint16_t *v_t,
                                            float *qk_fifo, uint16_t *p_fifo, int lds_fifo)
{
    PTO_ST_NONNULL(out, a, b_t, v_t, p_fifo);
    if (!lds_fifo)
        PTO_ST_NONNULL(qk_fifo);
    hipStream_t st = static_cast<hipStream_t>(stream);
    constexpr int ldsPlain = 8192 + 3 * 16384, ldsFifo = ldsPlain + 2 * 64 * 128 * 4;
    const half *ha = reinterpret_cast<const half *>(a), *hb = reinterpret_cast<const half *>(b_t), *hv = reinterpret_cast<const half *>(v_t);
    half *hp = reinterpret_cast<half *>(p_fifo);
    if (lds_fifo) {
        static const int attr = pto_amd::allow_lds(PushPopKernel<true>, ldsFifo);
        if (attr != PTO_OK)
            return attr;
        PushPopKernel<true><<<dim3(1), dim3(kBlockThreads), ldsFifo, st>>>(out, ha, hb, hv, qk_fifo, hp);
    } else {
        PushPopKernel<false><<<dim3(1), dim3(kBlockThreads), ldsPlain, st>>>(out, ha, hb, hv, qk_fifo, hp);
    }
    return pto_amd::check_launch();
}

// A Mat tile walked over a larger one by `data() + k * bytes`, the way pto_macro_matmul.hpp:176-177 of the reference walks an
// L1 panel: chunk 0 is accepted (the start of an image is an image), a later chunk ends the kernel with a message.
// flags[0] = 1 when the kernel has started, flags[1] = 1 when it has reached its end.
PTO_DEVICE_CODE_BEGIN
__global__ __launch_bounds__(kBlockThreads) AICORE void MatViewWalk(__gm__ uint32_t *flags, int chunks, uint32_t step)
{
    using Whole = Tile<TileType::Mat, half, 128, 128, BLayout::ColMajor, 128, 128, SLayout::RowMajor>;
    using Chunk = Tile<TileType::Mat, half, 128, 64, BLayout::ColMajor, 128, 64, SLayout::RowMajor>;
    Whole whole;
    Chunk chunk;
    TASSIGN(whole, 0x0);
    if (hw::tid() == 0)
        flags[0] = 1;
    for (int k = 0; k < chunks; ++k)
        TASSIGN(chunk, (uint64_t)whole.data() + (uint64_t)k * step); // (a step the compiler does not know: the run-time form)
    if (hw::tid() == 0)
        flags[1] = 1 + (uint32_t)(chunk.data() - whole.data());
}
PTO_DEVICE_CODE_END

extern "C" int pto_st_mat_view_walk(void *stream, uint32_t *flags, int chunks)
{
    PTO_ST_NONNULL(flags);
    if (chunks < 1 || chunks > 2)
        return PTO_ERR_UNSUPPORTED;
    MatViewWalk<<<dim3(1), dim3(kBlockThreads), 128 * 128 * sizeof(half), static_cast<hipStream_t>(stream)>>>(flags, chunks, 128 * 64 * (uint32_t)sizeof(half));
    return pto_amd::check_launch();
}
