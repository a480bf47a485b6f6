// C-ABI harness around the REFERENCE's own CPU-simulation headers.
// TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile (target `ref`) with
//   clang++ -std=c++20 -D__CPU_SIM -I<reference>/include
// from the reference sources where they lie; the output (oracle/_ref/libpto_ref.so)
// is used to validate the plain-C restatement in pto_oracle.c and as the CPU
// baseline of the benchmark.  Nothing from the reference is copied here: this file
// only instantiates its public templates (pto::Tile, pto::GlobalTensor, TLOAD, ...)
// at the shapes the tests use.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <memory>
#include <pto/pto-inst.hpp>

using namespace pto;

namespace {

template <typename T, int R, int C>
using GmND = GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>, Layout::ND>;
// column-major view of a buffer stored [C][R]
template <typename T, int R, int C>
using GmDN = GlobalTensor<T, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, 1, R>, Layout::DN>;

// ---- GEMM tile path: TLOAD(ND->Nz A, DN->Zn B) -> TEXTRACT -> TMATMUL[_ACC] per K-step -> TSTORE ----
// A [M,K] row-major fp16, B stored [N,K] (column-major K x N), C [M,N] fp32.  KS = K-step
// (one TMATMUL for the first step, TMATMUL_ACC after), as the manual GEMM kernel does.
template <int M, int K, int N, int KS>
void gemm_tile(float *c, const uint16_t *a, const uint16_t *b)
{
    using MatA = Tile<TileType::Mat, half, M, KS, BLayout::ColMajor, M, KS, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, half, KS, N, BLayout::RowMajor, KS, N, SLayout::ColMajor>;
    using L = TileLeft<half, M, KS, M, KS>;
    using R = TileRight<half, KS, N, KS, N>;
    using Acc = TileAcc<float, M, N, M, N>;
    using GA = GlobalTensor<half, Shape<1, 1, 1, M, KS>, Stride<M * K, M * K, M * K, K, 1>, Layout::ND>;
    using GB = GlobalTensor<half, Shape<1, 1, 1, KS, N>, Stride<N * K, N * K, N * K, 1, K>, Layout::DN>;
    auto am = std::make_unique<MatA>();
    auto bm = std::make_unique<MatB>();
    auto al = std::make_unique<L>();
    auto br = std::make_unique<R>();
    auto acc = std::make_unique<Acc>();
    for (int k0 = 0; k0 < K; k0 += KS) {
        GA ga(reinterpret_cast<half *>(const_cast<uint16_t *>(a)) + k0);
        GB gb(reinterpret_cast<half *>(const_cast<uint16_t *>(b)) + k0);
        TLOAD(*am, ga);
        TLOAD(*bm, gb);
        TEXTRACT(*al, *am, 0, 0);
        TEXTRACT(*br, *bm, 0, 0);
        if (k0 == 0)
            TMATMUL(*acc, *al, *br);
        else
            TMATMUL_ACC(*acc, *acc, *al, *br);
    }
    GmND<float, M, N> gc(c);
    TSTORE(gc, *acc);
}

// ---- valid-region matmul as in the tmatmul ST: plain [vM,vK] x [vK,vN], both row-major ----
template <typename TO, typename TI, int vM, int vK, int vN, bool kBias>
void matmul_valid(TO *out, const TI *a, const TI *b, const TO *bias)
{
    constexpr int al = sizeof(TI) == 1 ? 32 : 16;
    constexpr int M = (vM + al - 1) / al * al, K = (vK + al - 1) / al * al, N = (vN + al - 1) / al * al;
    using MatA = Tile<TileType::Mat, TI, M, K, BLayout::ColMajor, vM, vK, SLayout::RowMajor, 512>;
    using MatB = Tile<TileType::Mat, TI, K, N, BLayout::ColMajor, vK, vN, SLayout::RowMajor, 512>;
    using L = TileLeft<TI, M, K, vM, vK>;
    using R = TileRight<TI, K, N, vK, vN>;
    using Acc = TileAcc<TO, M, N, vM, vN>;
    using Bias = Tile<TileType::Bias, TO, 1, N, BLayout::RowMajor, 1, vN>;
    auto am = std::make_unique<MatA>();
    auto bm = std::make_unique<MatB>();
    auto lt = std::make_unique<L>();
    auto rt = std::make_unique<R>();
    auto acc = std::make_unique<Acc>();
    GmND<TI, vM, vK> ga(const_cast<TI *>(a));
    GmND<TI, vK, vN> gb(const_cast<TI *>(b));
    TLOAD(*am, ga);
    TLOAD(*bm, gb);
    TMOV(*lt, *am);
    TMOV(*rt, *bm);
    if constexpr (kBias) {
        auto bt = std::make_unique<Bias>();
        GlobalTensor<TO, Shape<1, 1, 1, 1, vN>, Stride<vN, vN, vN, vN, 1>> gbias(const_cast<TO *>(bias));
        TLOAD(*bt, gbias);
        TMATMUL_BIAS(*acc, *lt, *rt, *bt);
    } else {
        TMATMUL(*acc, *lt, *rt);
    }
    GmND<TO, vM, vN> gc(out);
    TSTORE(gc, *acc);
}

// ---- elementwise conversion over an [R,C] row-major tensor, one Vec tile ----
template <typename D, typename S, int R, int C>
void cvt_tile(D *dst, const S *src)
{
    using TS = Tile<TileType::Vec, S, R, C, BLayout::RowMajor>;
    using TD = Tile<TileType::Vec, D, R, C, BLayout::RowMajor>;
    auto s = std::make_unique<TS>();
    auto d = std::make_unique<TD>();
    GmND<S, R, C> gs(const_cast<S *>(src));
    GmND<D, R, C> gd(dst);
    TLOAD(*s, gs);
    TCVT(*d, *s, RoundMode::CAST_RINT);
    TSTORE(gd, *d);
}

// ---- index gather: dst[R,C] = src0[R0,C0].flat[idx[R,C]] ----
template <typename T, int R0, int C0, int R, int C>
void gather_index(T *dst, const T *src0, const int32_t *idx)
{
    using T0 = Tile<TileType::Vec, T, R0, C0, BLayout::RowMajor>;
    using TI = Tile<TileType::Vec, int32_t, R, C, BLayout::RowMajor>;
    using TD = Tile<TileType::Vec, T, R, C, BLayout::RowMajor>;
    auto s0 = std::make_unique<T0>();
    auto ti = std::make_unique<TI>();
    auto td = std::make_unique<TD>();
    GmND<T, R0, C0> g0(const_cast<T *>(src0));
    GmND<int32_t, R, C> gi(const_cast<int32_t *>(idx));
    GmND<T, R, C> gd(dst);
    TLOAD(*s0, g0);
    TLOAD(*ti, gi);
    TGATHER(*td, *s0, *ti);
    TSTORE(gd, *td);
}

// ---- mask gather over [R,C] -> [R, C/div] ----
template <typename T, int R, int C, MaskPattern P, int Div>
void gather_mask(T *dst, const T *src)
{
    using TS = Tile<TileType::Vec, T, R, C, BLayout::RowMajor>;
    using TD = Tile<TileType::Vec, T, R, C / Div, BLayout::RowMajor>;
    auto s = std::make_unique<TS>();
    auto d = std::make_unique<TD>();
    GmND<T, R, C> gs(const_cast<T *>(src));
    GmND<T, R, C / Div> gd(dst);
    TLOAD(*s, gs);
    TGATHER<TD, TS, P>(*d, *s);
    TSTORE(gd, *d);
}

// ---- MGATHER: dst[R,C] = gm[idx[R,C]] ----
template <typename T, int R, int C, int GN>
void mgather(T *dst, const T *gm, const int32_t *idx)
{
    using TI = Tile<TileType::Vec, int32_t, R, C, BLayout::RowMajor>;
    using TD = Tile<TileType::Vec, T, R, C, BLayout::RowMajor>;
    auto ti = std::make_unique<TI>();
    auto td = std::make_unique<TD>();
    GmND<int32_t, R, C> gi(const_cast<int32_t *>(idx));
    GmND<T, 1, GN> gsrc(const_cast<T *>(gm));
    GmND<T, R, C> gd(dst);
    TLOAD(*ti, gi);
    MGATHER(*td, gsrc, *ti);
    TSTORE(gd, *td);
}

// ---- suffix-window TEXTRACT Mat(Nz) [R,C] -> Left [R-r0, C-c0] -> plain out ----
template <int R, int C, int R0, int C0>
void extract_suffix(uint16_t *out, const uint16_t *in)
{
    using Src = Tile<TileType::Mat, half, R, C, BLayout::ColMajor, R, C, SLayout::RowMajor>;
    using Dst = TileLeft<half, R, C, R - R0, C - C0>;
    using Pl = Tile<TileType::Vec, half, R, C, BLayout::RowMajor, R - R0, C - C0>;
    auto s = std::make_unique<Src>();
    auto d = std::make_unique<Dst>();
    auto p = std::make_unique<Pl>();
    GmND<half, R, C> gs(reinterpret_cast<half *>(const_cast<uint16_t *>(in)));
    TLOAD(*s, gs);
    TEXTRACT(*d, *s, R0, C0);
    TMOV(*p, *d);
    GlobalTensor<half, Shape<1, 1, 1, R - R0, C - C0>,
                 Stride<(R - R0) * (C - C0), (R - R0) * (C - C0), (R - R0) * (C - C0), C - C0, 1>>
        go(reinterpret_cast<half *>(out));
    TSTORE(go, *p);
}

// ---- raw tile images: what TLOAD leaves in tile storage (layout + pad) ----
template <typename TileT, typename GmT>
void load_image(typename TileT::DType *image, typename TileT::DType *gm)
{
    auto t = std::make_unique<TileT>();
    GmT g(gm);
    TLOAD(*t, g);
    std::memcpy(image, t->data(), sizeof(typename TileT::DType) * TileT::Numel);
}

// ---- Auto-Mode attention on one [S,D] fp32 head (the op sequence of the tflashattn ST) ----
template <int S, int D>
void fa_auto(float *out, const float *q, const float *k, const float *v)
{
    using QP = Tile<TileType::Vec, float, S, D, BLayout::RowMajor, S, D, SLayout::NoneBox>;
    using KT = Tile<TileType::Vec, float, D, S, BLayout::RowMajor, D, S, SLayout::NoneBox>;
    using SP = Tile<TileType::Vec, float, S, S, BLayout::RowMajor, S, S, SLayout::NoneBox>;
    using RR = Tile<TileType::Vec, float, S, S, BLayout::ColMajor, S, S, SLayout::NoneBox>;
    auto qt = std::make_unique<QP>();
    auto kt = std::make_unique<QP>();
    auto vt = std::make_unique<QP>();
    auto ktt = std::make_unique<KT>();
    auto ql = std::make_unique<TileLeft<float, S, D, S, D>>();
    auto kr = std::make_unique<TileRight<float, D, S, D, S>>();
    auto sa = std::make_unique<TileAcc<float, S, S, S, S>>();
    auto sc = std::make_unique<SP>();
    auto cen = std::make_unique<SP>();
    auto ex = std::make_unique<SP>();
    auto pr = std::make_unique<SP>();
    auto rmax = std::make_unique<RR>();
    auto rsum = std::make_unique<RR>();
    auto pl = std::make_unique<TileLeft<float, S, S, S, S>>();
    auto vr = std::make_unique<TileRight<float, S, D, S, D>>();
    auto oa = std::make_unique<TileAcc<float, S, D, S, D>>();
    GmND<float, S, D> gq(const_cast<float *>(q)), gk(const_cast<float *>(k)), gv(const_cast<float *>(v)), go(out);
    const float scale = 1.0f / std::sqrt(static_cast<float>(D));
    TLOAD(*qt, gq);
    TLOAD(*kt, gk);
    TLOAD(*vt, gv);
    TMOV(*ql, *qt);
    TTRANS(*ktt, *kt, *kt);
    TMOV(*kr, *ktt);
    TMATMUL(*sa, *ql, *kr);
    TMOV(*sc, *sa);
    TMULS(*sc, *sc, scale);
    TROWMAX(*rmax, *sc, *sc);
    TROWEXPANDSUB(*cen, *sc, *rmax);
    TEXP(*ex, *cen);
    TROWSUM(*rsum, *ex, *ex);
    TROWEXPANDDIV(*pr, *ex, *rsum);
    TMOV(*pl, *pr);
    TMOV(*vr, *vt);
    TMATMUL(*oa, *pl, *vr);
    TSTORE(go, *oa);
}


// ---- multi-latent attention on one head, the instruction sequence of the reference's Auto-mode demo
// (demos/cpu/mla_attention_demo), at its sizes S = 64, D = 32, R = 16 ----
template <int S, int D, int R>
void mla_auto(float *out, const float *q, const float *k, const float *v, const float *wq, const float *wk, const float *wv,
              const float *wo)
{
    using XP = Tile<TileType::Vec, float, S, D, BLayout::RowMajor, S, D, SLayout::NoneBox>;
    using WP = Tile<TileType::Vec, float, D, R, BLayout::RowMajor, D, R, SLayout::NoneBox>;
    using WOP = Tile<TileType::Vec, float, R, D, BLayout::RowMajor, R, D, SLayout::NoneBox>;
    using LP = Tile<TileType::Vec, float, S, R, BLayout::RowMajor, S, R, SLayout::NoneBox>;
    using LTP = Tile<TileType::Vec, float, R, S, BLayout::RowMajor, R, S, SLayout::NoneBox>;
    using SP = Tile<TileType::Vec, float, S, S, BLayout::RowMajor, S, S, SLayout::NoneBox>;
    using RR = Tile<TileType::Vec, float, S, S, BLayout::ColMajor, S, S, SLayout::NoneBox>;
    using AccL = TileAcc<float, S, R, S, R>;
    auto x = std::make_unique<XP>();
    auto w = std::make_unique<WP>();
    auto w2 = std::make_unique<WOP>();
    auto xl = std::make_unique<TileLeft<float, S, D, S, D>>();
    auto wr = std::make_unique<TileRight<float, D, R, D, R>>();
    auto wor = std::make_unique<TileRight<float, R, D, R, D>>();
    std::unique_ptr<AccL> lat[3] = {std::make_unique<AccL>(), std::make_unique<AccL>(), std::make_unique<AccL>()};
    const float *xs[3] = {q, k, v}, *ws[3] = {wq, wk, wv};
    for (int i = 0; i < 3; ++i) {
        GmND<float, S, D> gx(const_cast<float *>(xs[i]));
        GmND<float, D, R> gw(const_cast<float *>(ws[i]));
        TLOAD(*x, gx);
        TLOAD(*w, gw);
        TMOV(*xl, *x);
        TMOV(*wr, *w);
        TMATMUL(*lat[i], *xl, *wr);
    }
    auto ql = std::make_unique<TileLeft<float, S, R, S, R>>();
    auto kp = std::make_unique<LP>();
    auto kt = std::make_unique<LTP>();
    auto ktr = std::make_unique<TileRight<float, R, S, R, S>>();
    auto sa = std::make_unique<TileAcc<float, S, S, S, S>>();
    auto sc = std::make_unique<SP>();
    auto pr = std::make_unique<SP>();
    auto rmax = std::make_unique<RR>();
    auto rsum = std::make_unique<RR>();
    TMOV(*ql, *lat[0]);
    TMOV(*kp, *lat[1]);
    TTRANS(*kt, *kp, *kp);
    TMOV(*ktr, *kt);
    TMATMUL(*sa, *ql, *ktr);
    TMOV(*sc, *sa);
    TMULS(*sc, *sc, 1.0f / std::sqrt(static_cast<float>(R)));
    TROWMAX(*rmax, *sc, *sc);
    TROWEXPANDSUB(*pr, *sc, *rmax);
    TEXP(*pr, *pr);
    TROWSUM(*rsum, *pr, *pr);
    TROWEXPANDDIV(*pr, *pr, *rsum);
    auto pl = std::make_unique<TileLeft<float, S, S, S, S>>();
    auto vr = std::make_unique<TileRight<float, S, R, S, R>>();
    auto ctx = std::make_unique<AccL>();
    auto cl = std::make_unique<TileLeft<float, S, R, S, R>>();
    auto oa = std::make_unique<TileAcc<float, S, D, S, D>>();
    TMOV(*pl, *pr);
    TMOV(*vr, *lat[2]);
    TMATMUL(*ctx, *pl, *vr);
    TMOV(*cl, *ctx);
    GmND<float, R, D> gwo(const_cast<float *>(wo));
    TLOAD(*w2, gwo);
    TMOV(*wor, *w2);
    TMATMUL(*oa, *cl, *wor);
    GmND<float, S, D> go(out);
    TSTORE(go, *oa);
}

// ---- further Vec instructions on [64,128] fp32 tiles (op codes: PTO_VOP_* of include/pto_amd.h) ----
using VX = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor>;
using VRow = Tile<TileType::Vec, float, 64, 1, BLayout::ColMajor>;   // one value per row
using VCol = Tile<TileType::Vec, float, 1, 128, BLayout::RowMajor>;  // one value per column

void vec_op_64x128(float *out, const float *a, const float *b, const float *vec, float k, int op)
{
    auto ta = std::make_unique<VX>(), tb = std::make_unique<VX>(), to = std::make_unique<VX>();
    auto rv = std::make_unique<VRow>();
    auto cv = std::make_unique<VCol>();
    GmND<float, 64, 128> ga(const_cast<float *>(a)), go(out);
    TLOAD(*ta, ga);
    if (b) {
        GmND<float, 64, 128> gb(const_cast<float *>(b));
        TLOAD(*tb, gb);
    }
    if (op >= 60 && op < 80) {
        GmDN<float, 64, 1> gr(const_cast<float *>(vec));
        TLOAD(*rv, gr);
    }
    if (op >= 80) {
        GmND<float, 1, 128> gc(const_cast<float *>(vec));
        TLOAD(*cv, gc);
    }
    switch (op) {
    case 0: TABS(*to, *ta); break;
    case 1: TNEG(*to, *ta); break;
    case 2: TRELU(*to, *ta); break;
    case 3: TSQRT(*to, *ta); break;
    case 4: TRSQRT(*to, *ta); break;
    case 5: TLOG(*to, *ta); break;
    case 6: TRECIP(*to, *ta); break;
    case 7: TEXP(*to, *ta); break;
    case 20: TADD(*to, *ta, *tb); break;
    case 21: TSUB(*to, *ta, *tb); break;
    case 22: TMUL(*to, *ta, *tb); break;
    case 23: TDIV(*to, *ta, *tb); break;
    case 24: TMAX(*to, *ta, *tb); break;
    case 25: TMIN(*to, *ta, *tb); break;
    case 26: TPRELU_IMPL(*to, *ta, *tb); break; // the front end of TPRELU takes a scratch tile and returns nothing
    case 27: TCMP(*to, *ta, *tb, CmpMode::EQ); break;
    case 28: TCMP(*to, *ta, *tb, CmpMode::NE); break;
    case 29: TCMP(*to, *ta, *tb, CmpMode::LT); break;
    case 30: TCMP(*to, *ta, *tb, CmpMode::LE); break;
    case 31: TCMP(*to, *ta, *tb, CmpMode::GT); break;
    case 32: TCMP(*to, *ta, *tb, CmpMode::GE); break;
    case 33: TSELS(*to, *ta, *tb, k); break;
    case 40: TADDS(*to, *ta, k); break;
    case 41: TSUBS(*to, *ta, k); break;
    case 42: TMULS(*to, *ta, k); break;
    case 43: TDIVS(*to, *ta, k); break;
    case 44: TMAXS(*to, *ta, k); break;
    case 45: TMINS(*to, *ta, k); break;
    case 46: TLRELU(*to, *ta, k); break;
    case 60: TROWEXPAND(*to, *rv); break;
    case 61: TROWEXPANDSUB(*to, *ta, *rv); break;
    case 62: TROWEXPANDMUL(*to, *ta, *rv); break;
    case 63: TROWEXPANDDIV(*to, *ta, *rv); break;
    case 64: TROWEXPANDADD(*to, *ta, *rv); break;
    case 65: TROWEXPANDMAX(*to, *ta, *rv); break;
    case 66: TROWEXPANDMIN(*to, *ta, *rv); break;
    case 67: TROWEXPANDEXPDIF(*to, *ta, *rv); break;
    case 80: TCOLEXPAND(*to, *cv); break;
    case 81: TCOLEXPANDSUB(*to, *ta, *cv); break;
    case 82: TCOLEXPANDMUL(*to, *ta, *cv); break;
    case 83: TCOLEXPANDDIV(*to, *ta, *cv); break;
    case 84: TCOLEXPANDADD(*to, *ta, *cv); break;
    case 85: TCOLEXPANDMAX(*to, *ta, *cv); break;
    case 86: TCOLEXPANDMIN(*to, *ta, *cv); break;
    case 87: TCOLEXPANDEXPDIF(*to, *ta, *cv); break;
    default: return;
    }
    TSTORE(go, *to);
}

// reductions of the valid region [vr, vc]; out holds vr (row ops) or vc (column ops) values
void reduce_64x128(float *out, const float *a, int vr, int vc, int op)
{
    using VD = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, -1, -1>;
    using RD = Tile<TileType::Vec, float, 64, 1, BLayout::ColMajor, -1, 1>;
    using CD = Tile<TileType::Vec, float, 1, 128, BLayout::RowMajor, 1, -1>;
    auto ta = std::make_unique<VD>(vr, vc), tmp = std::make_unique<VD>(vr, vc);
    for (int r = 0; r < vr; ++r)
        for (int c = 0; c < vc; ++c)
            ta->data()[r * 128 + c] = a[r * 128 + c];
    if (op < 3) {
        auto r = std::make_unique<RD>(vr);
        if (op == 0)
            TROWMAX(*r, *ta, *tmp);
        else if (op == 1)
            TROWMIN(*r, *ta, *tmp);
        else
            TROWSUM(*r, *ta, *tmp);
        for (int i = 0; i < vr; ++i)
            out[i] = r->data()[i];
    } else {
        auto c = std::make_unique<CD>(vc);
        if (op == 3)
            TCOLMAX(*c, *ta);
        else if (op == 4)
            TCOLMIN(*c, *ta);
        else
            TCOLSUM(*c, *ta);
        for (int j = 0; j < vc; ++j)
            out[j] = c->data()[j];
    }
}

} // namespace

extern "C" {

#define REF_GEMM(M, K, N, KS)                                                          \
    void ref_gemm_##M##x##K##x##N##_ks##KS(float *c, const uint16_t *a, const uint16_t *b) \
    {                                                                                  \
        gemm_tile<M, K, N, KS>(c, a, b);                                               \
    }
REF_GEMM(128, 64, 256, 64)
REF_GEMM(128, 256, 256, 64)
REF_GEMM(128, 512, 128, 64)
REF_GEMM(256, 256, 256, 256)
REF_GEMM(1536, 1536, 1536, 1536)
REF_GEMM(1536, 1536, 1536, 64)

void ref_matmul_f16_40x50x60(float *o, const uint16_t *a, const uint16_t *b)
{
    matmul_valid<float, half, 40, 50, 60, false>(o, reinterpret_cast<const half *>(a),
                                                 reinterpret_cast<const half *>(b), nullptr);
}
void ref_matmul_s8_6x7x8(int32_t *o, const int8_t *a, const int8_t *b)
{
    matmul_valid<int32_t, int8_t, 6, 7, 8, false>(o, a, b, nullptr);
}
void ref_matmul_f32_120x110x50(float *o, const float *a, const float *b)
{
    matmul_valid<float, float, 120, 110, 50, false>(o, a, b, nullptr);
}
void ref_matmul_bias_f16_26x100x94(float *o, const uint16_t *a, const uint16_t *b, const float *bias)
{
    matmul_valid<float, half, 26, 100, 94, true>(o, reinterpret_cast<const half *>(a),
                                                 reinterpret_cast<const half *>(b), bias);
}

// fp32 -> fp16 over n elements, n a multiple of 4096 (64 x 64 tiles)
void ref_tcvt_f32_f16(uint16_t *dst, const float *src, size_t n)
{
    for (size_t i = 0; i + 4096 <= n; i += 4096)
        cvt_tile<half, float, 64, 64>(reinterpret_cast<half *>(dst) + i, src + i);
}
void ref_tcvt_f16_f32(float *dst, const uint16_t *src, size_t n)
{
    for (size_t i = 0; i + 4096 <= n; i += 4096)
        cvt_tile<float, half, 64, 64>(dst + i, reinterpret_cast<const half *>(src) + i);
}

void ref_tgather_index_f16_16x1024_16x128(uint16_t *dst, const uint16_t *src0, const int32_t *idx)
{
    gather_index<half, 16, 1024, 16, 128>(reinterpret_cast<half *>(dst), reinterpret_cast<const half *>(src0), idx);
}
void ref_tgather_index_f32_32x64_32x64(float *dst, const float *src0, const int32_t *idx)
{
    gather_index<float, 32, 64, 32, 64>(dst, src0, idx);
}
void ref_tgather_mask_f16_16x64_p0101(uint16_t *dst, const uint16_t *src)
{
    gather_mask<half, 16, 64, MaskPattern::P0101, 2>(reinterpret_cast<half *>(dst),
                                                     reinterpret_cast<const half *>(src));
}
void ref_tgather_mask_f32_8x64_p1000(float *dst, const float *src)
{
    gather_mask<float, 8, 64, MaskPattern::P1000, 4>(dst, src);
}
void ref_tgather_mask_f32_8x64_p1111(float *dst, const float *src)
{
    gather_mask<float, 8, 64, MaskPattern::P1111, 1>(dst, src);
}
void ref_mgather_f16_8x128(uint16_t *dst, const uint16_t *gm, const int32_t *idx)
{
    mgather<half, 8, 128, 65536>(reinterpret_cast<half *>(dst), reinterpret_cast<const half *>(gm), idx);
}

void ref_textract_suffix_64x64_16_32(uint16_t *out, const uint16_t *in) { extract_suffix<64, 64, 16, 32>(out, in); }
void ref_textract_suffix_128x256_0_192(uint16_t *out, const uint16_t *in) { extract_suffix<128, 256, 0, 192>(out, in); }

// raw tile images (element order in tile storage)
void ref_image_nz_f16_32x48(uint16_t *image, const uint16_t *gm)
{
    using T = Tile<TileType::Mat, half, 32, 48, BLayout::ColMajor, 32, 48, SLayout::RowMajor>;
    load_image<T, GmND<half, 32, 48>>(reinterpret_cast<half *>(image), reinterpret_cast<half *>(const_cast<uint16_t *>(gm)));
}
void ref_image_zn_f16_48x32(uint16_t *image, const uint16_t *gm)
{ // gm stored [32][48] (column-major 48 x 32)
    using T = Tile<TileType::Mat, half, 48, 32, BLayout::RowMajor, 48, 32, SLayout::ColMajor>;
    load_image<T, GmDN<half, 48, 32>>(reinterpret_cast<half *>(image), reinterpret_cast<half *>(const_cast<uint16_t *>(gm)));
}
void ref_image_nz_f32_32x16(float *image, const float *gm)
{
    using T = Tile<TileType::Mat, float, 32, 16, BLayout::ColMajor, 32, 16, SLayout::RowMajor>;
    load_image<T, GmND<float, 32, 16>>(image, const_cast<float *>(gm));
}
void ref_image_pad_f32_16x32_valid_10x20(float *image, const float *gm)
{ // PadValue::Max fills everything outside the 10 x 20 valid region with +inf
    using T = Tile<TileType::Vec, float, 16, 32, BLayout::RowMajor, 10, 20, SLayout::NoneBox, 512, PadValue::Max>;
    using G = GlobalTensor<float, Shape<1, 1, 1, 10, 20>, Stride<200, 200, 200, 20, 1>>;
    load_image<T, G>(image, const_cast<float *>(gm));
}
void ref_image_5d_f32_2x3x4x8(float *image, const float *gm)
{ // 5-D GM [1,2,3,4,8] with padded strides -> plain [24, 8] tile
    using T = Tile<TileType::Vec, float, 24, 8, BLayout::RowMajor>;
    using G = GlobalTensor<float, Shape<1, 2, 3, 4, 8>, Stride<1000, 400, 100, 10, 1>>;
    load_image<T, G>(image, const_cast<float *>(gm));
}

void ref_fa_auto_64x32(float *out, const float *q, const float *k, const float *v) { fa_auto<64, 32>(out, q, k, v); }
void ref_mla_auto_64x32x16(float *out, const float *q, const float *k, const float *v, const float *wq, const float *wk,
                           const float *wv, const float *wo)
{
    mla_auto<64, 32, 16>(out, q, k, v, wq, wk, wv, wo);
}
// ---- TSORT32 / TMRGSORT on the tiles of the single-tile programs: [8,128] sources with a run-time valid region,
// [1,1024] one-source merges, two to four [1,256] lists into [1,1024] ----
extern "C++" {
template <typename T>
void sort32_8x128(T *out, const T *src, const uint32_t *idx, int vr, int vc)
{
    using S = Tile<TileType::Vec, T, 8, 128, BLayout::RowMajor, -1, -1>;
    using I = Tile<TileType::Vec, uint32_t, 8, 128, BLayout::RowMajor, -1, -1>;
    constexpr int DC = 128 * 8 / (int)sizeof(T); // 8 bytes of destination per source element
    using D = Tile<TileType::Vec, T, 8, DC, BLayout::RowMajor>;
    auto s = std::make_unique<S>(vr, vc);
    auto x = std::make_unique<I>(vr, vc);
    auto d = std::make_unique<D>();
    std::memcpy(s->data(), src, sizeof(T) * 8 * 128);
    std::memcpy(x->data(), idx, sizeof(uint32_t) * 8 * 128);
    std::memcpy(d->data(), out, sizeof(T) * 8 * DC);
    TSORT32(*d, *s, *x);
    std::memcpy(out, d->data(), sizeof(T) * 8 * DC);
}
} // extern "C++"
void ref_tsort32_f32_8x128(float *out, const float *src, const uint32_t *idx, int vr, int vc) { sort32_8x128<float>(out, src, idx, vr, vc); }
void ref_tsort32_s32_8x128(int32_t *out, const int32_t *src, const uint32_t *idx, int vr, int vc)
{
    sort32_8x128<int32_t>(out, src, idx, vr, vc);
}
// 2-byte scores: out [8,512]
void ref_tsort32_f16_8x128(uint16_t *out, const uint16_t *src, const uint32_t *idx, int vr, int vc)
{
    sort32_8x128<half>(reinterpret_cast<half *>(out), reinterpret_cast<const half *>(src), idx, vr, vc);
}
void ref_tsort32_s16_8x128(int16_t *out, const int16_t *src, const uint32_t *idx, int vr, int vc)
{
    sort32_8x128<int16_t>(out, src, idx, vr, vc);
}
void ref_tpart_f32_64x128(float *out, const float *a, const float *b, int op, int dvr, int dvc, int avr, int avc, int bvr, int bvc)
{
    using Dyn = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, -1, -1>;
    auto ta = std::make_unique<Dyn>(avr, avc), tb = std::make_unique<Dyn>(bvr, bvc), td = std::make_unique<Dyn>(dvr, dvc);
    std::memcpy(ta->data(), a, sizeof(float) * 64 * 128);
    std::memcpy(tb->data(), b, sizeof(float) * 64 * 128);
    std::memcpy(td->data(), out, sizeof(float) * 64 * 128);
    if (op == 0)
        TPARTADD(*td, *ta, *tb);
    else if (op == 1)
        TPARTMAX(*td, *ta, *tb);
    else
        TPARTMIN(*td, *ta, *tb);
    std::memcpy(out, td->data(), sizeof(float) * 64 * 128);
}
void ref_tscatter_f32_64x128(float *out, const float *src, const int32_t *idx, int vr, int vc)
{
    using Dyn = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, -1, -1>;
    using DynI = Tile<TileType::Vec, int32_t, 64, 128, BLayout::RowMajor, -1, -1>;
    auto ts = std::make_unique<Dyn>(vr, vc), td = std::make_unique<Dyn>(vr, vc);
    auto ti = std::make_unique<DynI>(vr, vc);
    std::memcpy(ts->data(), src, sizeof(float) * 64 * 128);
    std::memcpy(ti->data(), idx, sizeof(int32_t) * 64 * 128);
    std::memcpy(td->data(), out, sizeof(float) * 64 * 128);
    TSCATTER(*td, *ts, *ti);
    std::memcpy(out, td->data(), sizeof(float) * 64 * 128);
}
void ref_mscatter_f32_64x128(float *out, const float *src, const int32_t *idx, int vr, int vc)
{
    using Dyn = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, -1, -1>;
    using DynI = Tile<TileType::Vec, int32_t, 64, 128, BLayout::RowMajor, -1, -1>;
    auto ts = std::make_unique<Dyn>(vr, vc);
    auto ti = std::make_unique<DynI>(vr, vc);
    std::memcpy(ts->data(), src, sizeof(float) * 64 * 128);
    std::memcpy(ti->data(), idx, sizeof(int32_t) * 64 * 128);
    GmND<float, 64, 128> go(out);
    MSCATTER(go, *ts, *ti);
}
void ref_tgatherb_f32_16x128(float *out, const float *src, const uint32_t *offsets, int vr, int vc)
{
    using D = Tile<TileType::Vec, float, 16, 128, BLayout::RowMajor, -1, -1>;
    auto td = std::make_unique<D>(vr, vc);
    auto ts = std::make_unique<Tile<TileType::Vec, float, 32, 64, BLayout::RowMajor>>();
    auto to = std::make_unique<Tile<TileType::Vec, uint32_t, 16, 16, BLayout::RowMajor>>();
    std::memcpy(td->data(), out, sizeof(float) * 16 * 128);
    std::memcpy(ts->data(), src, sizeof(float) * 32 * 64);
    std::memcpy(to->data(), offsets, sizeof(uint32_t) * 16 * 16);
    TGATHERB(*td, *ts, *to);
    std::memcpy(out, td->data(), sizeof(float) * 16 * 128);
}
void ref_tci_s32_1x1024(int32_t *out, int32_t start, int descending, int vc)
{
    using Dyn = Tile<TileType::Vec, int32_t, 1, 1024, BLayout::RowMajor, 1, -1>;
    auto td = std::make_unique<Dyn>(vc);
    std::memcpy(td->data(), out, sizeof(int32_t) * 1024);
    if (descending)
        TCI<Dyn, int32_t, 1>(*td, start);
    else
        TCI<Dyn, int32_t, 0>(*td, start);
    std::memcpy(out, td->data(), sizeof(int32_t) * 1024);
}
extern "C++" {
// one source of 4 KiB: [1,1024] 4-byte or [1,2048] 2-byte elements
template <typename T>
void mrgsort_blocks(T *out, const T *src, int valid_cols, int block_len)
{
    constexpr int N = 4096 / (int)sizeof(T);
    using S = Tile<TileType::Vec, T, 1, N, BLayout::RowMajor>;
    using D = Tile<TileType::Vec, T, 1, N, BLayout::RowMajor, 1, -1>;
    auto s = std::make_unique<S>();
    auto d = std::make_unique<D>(valid_cols);
    std::memcpy(s->data(), src, sizeof(T) * N);
    std::memcpy(d->data(), out, sizeof(T) * N);
    TMRGSORT(*d, *s, static_cast<uint32_t>(block_len));
    std::memcpy(out, d->data(), sizeof(T) * N);
}
// lists of 1 KiB (up to 128 structures) into a destination of 4 KiB
template <typename T, bool EXH>
void mrgsort_lists(T *out, uint32_t *executed, const T *const *src, const int *cols, int out_cols, int lists)
{
    constexpr int LC = 1024 / (int)sizeof(T), DC = 4 * LC;
    using L = Tile<TileType::Vec, T, 1, LC, BLayout::RowMajor, 1, -1>;
    using D = Tile<TileType::Vec, T, 1, DC, BLayout::RowMajor, 1, -1>;
    using Tmp = Tile<TileType::Vec, T, 1, DC, BLayout::RowMajor>;
    std::unique_ptr<L> l[4];
    for (int i = 0; i < 4; ++i) {
        l[i] = std::make_unique<L>(i < lists ? cols[i] : 0);
        if (i < lists)
            std::memcpy(l[i]->data(), src[i], sizeof(T) * LC);
    }
    auto d = std::make_unique<D>(out_cols);
    auto tmp = std::make_unique<Tmp>();
    std::memcpy(d->data(), out, sizeof(T) * DC);
    MrgSortExecutedNumList ex = {};
    if (lists == 4)
        TMRGSORT<D, Tmp, L, L, L, L, EXH>(*d, ex, *tmp, *l[0], *l[1], *l[2], *l[3]);
    else if (lists == 3)
        TMRGSORT<D, Tmp, L, L, L, EXH>(*d, ex, *tmp, *l[0], *l[1], *l[2]);
    else
        TMRGSORT<D, Tmp, L, L, EXH>(*d, ex, *tmp, *l[0], *l[1]);
    std::memcpy(out, d->data(), sizeof(T) * DC);
    executed[0] = ex.mrgSortList0;
    executed[1] = ex.mrgSortList1;
    executed[2] = ex.mrgSortList2;
    executed[3] = ex.mrgSortList3;
}
template <typename T>
void mrgsort_lists_any(void *out, uint32_t *executed, const void *src0, const void *src1, const void *src2, const void *src3, int cols0,
                       int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted)
{
    const T *src[4] = {static_cast<const T *>(src0), static_cast<const T *>(src1), static_cast<const T *>(src2), static_cast<const T *>(src3)};
    const int cols[4] = {cols0, cols1, cols2, cols3};
    if (exhausted)
        mrgsort_lists<T, true>(static_cast<T *>(out), executed, src, cols, out_cols, lists);
    else
        mrgsort_lists<T, false>(static_cast<T *>(out), executed, src, cols, out_cols, lists);
}
} // extern "C++"
void ref_tmrgsort_blocks_f32_1x1024(float *out, const float *src, int valid_cols, int block_len)
{
    mrgsort_blocks<float>(out, src, valid_cols, block_len);
}
// dtype 0 = half, 1 = uint16_t, 2 = int16_t
void ref_tmrgsort_blocks_16_1x2048(void *out, const void *src, int valid_cols, int block_len, int dtype)
{
    if (dtype == 0)
        mrgsort_blocks<half>(static_cast<half *>(out), static_cast<const half *>(src), valid_cols, block_len);
    else if (dtype == 1)
        mrgsort_blocks<uint16_t>(static_cast<uint16_t *>(out), static_cast<const uint16_t *>(src), valid_cols, block_len);
    else
        mrgsort_blocks<int16_t>(static_cast<int16_t *>(out), static_cast<const int16_t *>(src), valid_cols, block_len);
}
void ref_tmrgsort_lists_f32(float *out, uint32_t *executed, const float *src0, const float *src1, const float *src2, const float *src3,
                            int cols0, int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted)
{
    mrgsort_lists_any<float>(out, executed, src0, src1, src2, src3, cols0, cols1, cols2, cols3, out_cols, lists, exhausted);
}
// dtype 0 = half, 1 = uint16_t
void ref_tmrgsort_lists_16(void *out, uint32_t *executed, const void *src0, const void *src1, const void *src2, const void *src3, int cols0,
                           int cols1, int cols2, int cols3, int out_cols, int lists, int exhausted, int dtype)
{
    if (dtype == 0)
        mrgsort_lists_any<half>(out, executed, src0, src1, src2, src3, cols0, cols1, cols2, cols3, out_cols, lists, exhausted);
    else
        mrgsort_lists_any<uint16_t>(out, executed, src0, src1, src2, src3, cols0, cols1, cols2, cols3, out_cols, lists, exhausted);
}
void ref_fa_auto_128x64(float *out, const float *q, const float *k, const float *v) { fa_auto<128, 64>(out, q, k, v); }


void ref_vec_op_f32_64x128(float *out, const float *a, const float *b, const float *vec, float k, int op)
{
    vec_op_64x128(out, a, b, vec, k, op);
}
void ref_reduce_f32_64x128(float *out, const float *a, int vr, int vc, int op) { reduce_64x128(out, a, vr, vc, op); }
// TCMPS into a [64,128] uint8 tile whose first 16 valid columns take the packed bits, then TSEL with that mask
void ref_cmps_sel_f32_64x128(float *sel, uint8_t *bits, const float *a, const float *b, float scalar, int mode)
{
    using MB = Tile<TileType::Vec, uint8_t, 64, 128, BLayout::RowMajor, 64, 16>;
    using MS = Tile<TileType::Vec, uint8_t, 64, 32, BLayout::RowMajor, 64, 16>;
    auto ta = std::make_unique<VX>(), tb = std::make_unique<VX>(), to = std::make_unique<VX>();
    auto m = std::make_unique<MB>();
    auto ms = std::make_unique<MS>();
    GmND<float, 64, 128> ga(const_cast<float *>(a)), gb(const_cast<float *>(b)), go(sel);
    TLOAD(*ta, ga);
    TLOAD(*tb, gb);
    TCMPS(*m, *ta, scalar, static_cast<CmpMode>(mode));
    for (int r = 0; r < 64; ++r)
        for (int c = 0; c < 16; ++c) {
            bits[r * 16 + c] = m->data()[r * 128 + c];
            ms->data()[r * 32 + c] = m->data()[r * 128 + c];
        }
    TSEL(*to, *ms, *ta, *tb);
    TSTORE(go, *to);
}
void ref_fillpad_f32_64x128(float *out, const float *a, int vr, int vc, int pad_kind)
{
    using VS = Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, -1, -1>;
    auto ts = std::make_unique<VS>(vr, vc);
    for (int r = 0; r < vr; ++r)
        for (int c = 0; c < vc; ++c)
            ts->data()[r * 128 + c] = a[r * 128 + c];
    GmND<float, 64, 128> go(out);
    if (pad_kind == 1) {
        auto td = std::make_unique<Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, 64, 128, SLayout::NoneBox, 512, PadValue::Zero>>();
        TFILLPAD(*td, *ts);
        TSTORE(go, *td);
    } else if (pad_kind == 2) {
        auto td = std::make_unique<Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, 64, 128, SLayout::NoneBox, 512, PadValue::Max>>();
        TFILLPAD(*td, *ts);
        TSTORE(go, *td);
    } else {
        auto td = std::make_unique<Tile<TileType::Vec, float, 64, 128, BLayout::RowMajor, 64, 128, SLayout::NoneBox, 512, PadValue::Min>>();
        TFILLPAD(*td, *ts);
        TSTORE(go, *td);
    }
}
// accumulator tile -> Vec tile with ReluPreMode
void ref_tmov_acc_vec_f32_64x128(float *out, const float *acc_rowmajor, int relu)
{
    using Acc = TileAcc<float, 64, 128, 64, 128>;
    auto c = std::make_unique<Acc>();
    auto v = std::make_unique<VX>();
    for (int r = 0; r < 64; ++r)
        for (int col = 0; col < 128; ++col)
            c->data()[GetTileElementOffset<Acc>(r, col)] = acc_rowmajor[r * 128 + col];
    if (relu)
        TMOV<VX, Acc, ReluPreMode::NormalRelu>(*v, *c);
    else
        TMOV(*v, *c);
    GmND<float, 64, 128> go(out);
    TSTORE(go, *v);
}

} // extern "C"
