// Multi-latent attention on one workgroup per (batch, head), written as an Auto-mode PTO program: every intermediate is
// a tile, matmuls are chained with TMOV (Vec / Acc -> Left / Right), the softmax runs on Vec tiles.
//
// Counterpart of the reference's CPU demo demos/cpu/mla_attention_demo/mla_attention_demo.cpp:227-397 (mla_pto), same
// sizes (S = 64 positions, D = 32 head dim, R = 16 latent dim, fp32) and the same instruction sequence:
//   Q_lat = Q Wq, K_lat = K Wk, V_lat = V Wv   [S,D] x [D,R]
//   P = softmax(Q_lat K_lat^T / sqrt(R))       [S,S]
//   O = (P V_lat) Wo                           [S,R] x [R,D]
// Four wavefronts stacked along the rows (16 rows of every result per wave) on v_mfma_f32_16x16x4_f32.
#define PTO_WAVES_M 4
#define PTO_WAVES_N 1
#define PTO_MFMA_M 16
#include <pto/pto-inst.hpp>

#include "common.hpp"

using namespace pto;

PTO_DEVICE_CODE_BEGIN

namespace {

constexpr int kS = 64, kD = 32, kR = 16;

template <int R, int C>
using Gm = GlobalTensor<float, Shape<1, 1, 1, R, C>, Stride<R * C, R * C, R * C, C, 1>>;
template <int R, int C>
using Plain = Tile<TileType::Vec, float, R, C, BLayout::RowMajor, R, C, SLayout::NoneBox>;

__global__ __launch_bounds__(kBlockThreads) AICORE void MlaAttention(__gm__ float *out, __gm__ const float *q, __gm__ const float *k,
                                                                     __gm__ const float *v, __gm__ const float *wq,
                                                                     __gm__ const float *wk, __gm__ const float *wv,
                                                                     __gm__ const float *wo)
{
    const size_t head = (size_t)get_block_idx() * kS * kD;
    // the column-major [S,S] tile of the reference program: a reduction leaves one value per row in its first column
    using RowStat = Tile<TileType::Vec, float, kS, kS, BLayout::ColMajor, kS, kS, SLayout::NoneBox>;

    // ---- projection weights as right-hand operands ----
    TileRight<float, kD, kR> wqR, wkR, wvR;
    TileRight<float, kR, kD> woR;
    {
        Plain<kD, kR> w;
        Gm<kD, kR> gq(const_cast<float *>(wq)), gk(const_cast<float *>(wk)), gv(const_cast<float *>(wv));
        TLOAD(w, gq);
        TMOV(wqR, w);
        TLOAD(w, gk);
        TMOV(wkR, w);
        TLOAD(w, gv);
        TMOV(wvR, w);
        Plain<kR, kD> w2;
        Gm<kR, kD> go(const_cast<float *>(wo));
        TLOAD(w2, go);
        TMOV(woR, w2);
    }

    // ---- latent projections [S,D] x [D,R] ----
    TileAcc<float, kS, kR> qLat, kLat, vLat;
    {
        Plain<kS, kD> x;
        TileLeft<float, kS, kD> xL;
        Gm<kS, kD> gq(const_cast<float *>(q) + head), gk(const_cast<float *>(k) + head), gv(const_cast<float *>(v) + head);
        TLOAD(x, gq);
        TMOV(xL, x);
        TMATMUL(qLat, xL, wqR);
        TLOAD(x, gk);
        TMOV(xL, x);
        TMATMUL(kLat, xL, wkR);
        TLOAD(x, gv);
        TMOV(xL, x);
        TMATMUL(vLat, xL, wvR);
    }

    // ---- scores = Q_lat K_lat^T / sqrt(R) ----
    Plain<kS, kS> scores;
    {
        TileLeft<float, kS, kR> qL;
        TMOV(qL, qLat);
        Plain<kS, kR> kPlain;
        Plain<kR, kS> kT;
        TileRight<float, kR, kS> kTR;
        TMOV(kPlain, kLat);
        TTRANS(kT, kPlain, kPlain);
        TMOV(kTR, kT);
        TileAcc<float, kS, kS> sAcc;
        TMATMUL(sAcc, qL, kTR);
        TMOV(scores, sAcc);
        TMULS(scores, scores, 0.25f); // 1 / sqrt(16)
    }

    // ---- softmax over every row ----
    Plain<kS, kS> probs;
    {
        RowStat rowMax, rowSum;
        TROWMAX(rowMax, scores, scores);
        TROWEXPANDSUB(probs, scores, rowMax);
        TEXP(probs, probs);
        TROWSUM(rowSum, probs, probs);
        TROWEXPANDDIV(probs, probs, rowSum);
    }

    // ---- context in the latent space, then the output projection ----
    TileLeft<float, kS, kS> pL;
    TileRight<float, kS, kR> vR;
    TMOV(pL, probs);
    TMOV(vR, vLat);
    TileAcc<float, kS, kR> ctx;
    TMATMUL(ctx, pL, vR);
    TileLeft<float, kS, kR> ctxL;
    TMOV(ctxL, ctx);
    TileAcc<float, kS, kD> oAcc;
    TMATMUL(oAcc, ctxL, woR);
    Gm<kS, kD> gOut(out + head);
    TSTORE(gOut, oAcc);
}

// The reference's other Auto-mode attention program (demos/cpu/flash_attention_demo/flash_attention_demo.cpp:169-258,
// flash_attention_pto; the same sequence is its tflashattn system test): O = softmax(Q K^T / sqrt(D)) V on one
// [S, D] fp32 head per workgroup, scores and probabilities as whole [S, S] tiles.
template <int S, int D>
__global__ __launch_bounds__(kBlockThreads) AICORE void AttentionAuto(__gm__ float *out, __gm__ const float *q, __gm__ const float *k,
                                                                      __gm__ const float *v)
{
    const size_t head = (size_t)get_block_idx() * S * D;
    using RowStat = Tile<TileType::Vec, float, S, S, BLayout::ColMajor, S, S, SLayout::NoneBox>;
    Gm<S, D> gq(const_cast<float *>(q) + head), gk(const_cast<float *>(k) + head), gv(const_cast<float *>(v) + head), go(out + head);
    TileAcc<float, S, S> sAcc;
    {
        Plain<S, D> x;
        Plain<D, S> kT;
        TileLeft<float, S, D> qL;
        TileRight<float, D, S> kR;
        TLOAD(x, gq);
        TMOV(qL, x);
        TLOAD(x, gk);
        TTRANS(kT, x, x);
        TMOV(kR, kT);
        TMATMUL(sAcc, qL, kR);
    }
    Plain<S, S> p;
    TMOV(p, sAcc);
    TMULS(p, p, 1.0f / __builtin_sqrtf((float)D));
    {
        RowStat rowMax, rowSum;
        TROWMAX(rowMax, p, p);
        TROWEXPANDSUB(p, p, rowMax);
        TEXP(p, p);
        TROWSUM(rowSum, p, p);
        TROWEXPANDDIV(p, p, rowSum);
    }
    TileLeft<float, S, S> pL;
    TMOV(pL, p);
    TileRight<float, S, D> vR;
    {
        Plain<S, D> x;
        TLOAD(x, gv);
        TMOV(vR, x);
    }
    TileAcc<float, S, D> oAcc;
    TMATMUL(oAcc, pL, vR);
    TSTORE(go, oAcc);
}

} // namespace

PTO_DEVICE_CODE_END

extern "C" int pto_mla_attention_f32_s64_d32_r16(void *stream, float *out, const float *q, const float *k, const float *v, const float *wq,
                                                 const float *wk, const float *wv, const float *wo, int batch, int heads)
{
    if (!out || !q || !k || !v || !wq || !wk || !wv || !wo || batch <= 0 || heads <= 0)
        return PTO_ERR_BAD_ARG;
    const long long blocks = (long long)batch * heads;
    if (blocks > 0x7fffffffLL)
        return PTO_ERR_UNSUPPORTED;
    MlaAttention<<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream)>>>(out, q, k, v, wq, wk, wv, wo);
    return pto_amd::check_launch();
}

extern "C" int pto_attention_auto_f32(void *stream, float *out, const float *q, const float *k, const float *v, int batch, int heads,
                                      int seq, int head_dim)
{
    if (!out || !q || !k || !v || batch <= 0 || heads <= 0)
        return PTO_ERR_BAD_ARG;
    const long long blocks = (long long)batch * heads;
    if (blocks > 0x7fffffffLL)
        return PTO_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (seq == 64 && head_dim == 32)
        AttentionAuto<64, 32><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, st>>>(out, q, k, v);
    else if (seq == 128 && head_dim == 64)
        AttentionAuto<128, 64><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, st>>>(out, q, k, v);
    else
        return PTO_ERR_UNSUPPORTED;
    return pto_amd::check_launch();
}
