// Flash-attention forward for MI355X: one fused kernel built from PTO tile instructions.
//
// Arithmetic follows the reference's streaming softmax and rescale stages
// (kernels/manual/common/flash_atten/pto_macro_fa_softmax.hpp:47-215, pto_macro_fa_gu.hpp:33-56):
//   per key tile X = q k^T (fp32);  M' = max(M, rowmax X);  alpha = exp(s (M - M'));
//   P = exp(s (X - M'));  S = alpha S + rowsum P;  O = alpha O + half(P) v;  at the end O /= S,
// s = 1/sqrt(head_dim), causal mask = -3.40282e38 added to the hidden scores.
//
// Structure.  The reference runs the four stages on two kinds of cores that hand tiles over
// through global-memory FIFOs (fa_performance_kernel.cpp:607-963).  A CDNA4 compute unit does
// matrix and vector work itself, so here a workgroup owns 128 query rows of one head and keeps
// scores, probabilities and the output accumulator in registers for the whole sweep over the keys:
//   * wave grid 1 x 4: every wave owns 32 queries and sees every key of the tile,
//   * the score tile is computed transposed, X^T = K Q^T (TMATMUL with K as the Left operand and
//     Q^T as the Right operand), so that in the MFMA accumulator layout one lane holds one query
//     and the per-query quantities (max, sum, alpha) are per-lane scalars: the row reductions of
//     the softmax are in-register, plus one exchange between the two half-waves for the max,
//   * P^T in accumulator layout already is a Right (B) operand for O^T = V^T P^T up to a
//     permutation of the keys inside a 16-key step; V^T is read from the row-major V tile in LDS
//     with the transposing ds_read_b64_tr_b16 using the same permutation, so P never moves,
//   * K and V tiles are double-buffered in LDS by asynchronous TLOADs.
#define PTO_WAVES_M 1
#define PTO_WAVES_N 4
#include <pto/pto-inst.hpp>

#include "fa_kernels.hpp"

#if defined(PTO_ST_HOOKS)
// Tuning hook (not part of the public header).
extern "C" int pto_fa_fwd_f16_variant(void *stream, void *o, float *lse, const uint16_t *q, const uint16_t *k,
                                      const uint16_t *v, int batch, int heads, int seq_q, int seq_kv, int head_dim,
                                      int causal, int variant)
{
    if (!o || !q || !k || !v || batch <= 0 || heads <= 0 || seq_q <= 0 || seq_kv <= 0)
        return PTO_ERR_BAD_ARG;
    if (causal && seq_kv < seq_q)
        return PTO_ERR_UNSUPPORTED;
    const int causalOff = seq_kv - seq_q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *hq = reinterpret_cast<const half *>(q), *hk = reinterpret_cast<const half *>(k),
               *hv = reinterpret_cast<const half *>(v);
#define PTO_FA_VARIANT(VV, DD, CC, MB)                           \
    if (variant == VV && head_dim == DD && (causal != 0) == CC) \
        return launch_fa<DD, CC, false, MB>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    PTO_FA_VARIANT(1, 128, false, 1)
    PTO_FA_VARIANT(2, 128, false, 2)
    PTO_FA_VARIANT(2, 128, true, 2)
    PTO_FA_VARIANT(1, 64, true, 1)
    PTO_FA_VARIANT(2, 64, true, 2)
    PTO_FA_VARIANT(5, 64, true, 3)
#undef PTO_FA_VARIANT
    if (variant == 10 && head_dim == 128)
        return pto_amd::fa_fwd_d128_w8(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causal != 0, false, causalOff);
    if (variant == 20 && head_dim == 128)
        return pto_amd::fa_fwd_d128_w8m16(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causal != 0, false, causalOff);
    if (variant == 21 && head_dim == 128) // fp32 output and LSE
        return pto_amd::fa_fwd_d128_w8m16(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causal != 0, true, causalOff);
    if (variant == 6 && head_dim == 128 && !causal)
        return launch_fa<128, false, false, 2, 32>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    if (variant == 6 && head_dim == 64 && causal)
        return launch_fa<64, true, false, 3, 32>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    if (variant == 8 && head_dim == 64 && causal) // 64 queries per wave
        return launch_fa<64, true, false, 2, 64, false, 2>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    if (variant == 8 && head_dim == 64 && !causal)
        return launch_fa<64, false, false, 2, 64, false, 2>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    return PTO_ERR_BAD_ARG;
}
#endif // PTO_ST_HOOKS

extern "C" int pto_fa_fwd_f16(void *stream, void *o, float *lse, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                              int batch, int heads, int seq_q, int seq_kv, int head_dim, int causal, int o_fp32)
{
    if (!o || !q || !k || !v || batch <= 0 || heads <= 0 || seq_q <= 0 || seq_kv <= 0)
        return PTO_ERR_BAD_ARG;
    if ((head_dim != 64 && head_dim != 128) || seq_q % kBQ1 || seq_kv % kBKVDefault)
        return PTO_ERR_UNSUPPORTED;
    // causal == 1: the diagonal ends in the last key (query i sees keys j <= i + seq_kv - seq_q; needs seq_kv >= seq_q);
    // causal == 2: the diagonal starts in the first key (j <= i, the rule of the reference's kernel and generator:
    // fa_performance_kernel.cpp:298-299 and :757, scripts/gen_data.py:53), any seq_kv.  The same when seq_kv == seq_q.
    if (causal != 0 && causal != 1 && causal != 2)
        return PTO_ERR_BAD_ARG;
    if (causal == 1 && seq_kv < seq_q)
        return PTO_ERR_UNSUPPORTED;
    const int causalOff = causal == 2 ? 0 : seq_kv - seq_q;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half *hq = reinterpret_cast<const half *>(q), *hk = reinterpret_cast<const half *>(k),
               *hv = reinterpret_cast<const half *>(v);
    // head_dim 128 with enough work to give every compute unit a workgroup of eight wavefronts (256 queries): the
    // K / V tiles are shared by twice the queries and the two waves of a SIMD alternate between MFMA and softmax
    // phases (measured +10-15 % at B1 H16 S4096 over workgroups of four waves)
    if (head_dim == 128 && seq_q % 256 == 0) {
        static const int cus = [] {
            int dev = 0, n = 0;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
                n = 256;
            return n;
        }();
        if ((long long)batch * heads * (seq_q / 256) >= cus) {
            // the same schedule on 16 x 16 x 32 MFMAs: +1.5 .. 3.6 % without a mask and for long causal sequences
            // (interleaved runs; B2 H16 S2048 causal is 6 % slower on it and stays on the 32 x 32 x 16 kernel)
            if (!causal || seq_kv >= 4096)
                return pto_amd::fa_fwd_d128_w8m16(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causal != 0, o_fp32 != 0, causalOff);
            return pto_amd::fa_fwd_d128_w8(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causal != 0, o_fp32 != 0, causalOff);
        }
    }
    // otherwise workgroups of four wavefronts (128 queries): two per compute unit at head_dim 128, three at 64
#define PTO_FA_CASE(DD, CC, FF)                                                                      \
    if (head_dim == DD && (causal != 0) == CC && (o_fp32 != 0) == FF)                                \
        return launch_fa<DD, CC, FF, (DD == 128 ? 2 : 3)>(st, o, lse, hq, hk, hv, batch, heads, seq_q, seq_kv, causalOff);
    PTO_FA_CASE(128, false, false)
    PTO_FA_CASE(128, false, true)
    PTO_FA_CASE(128, true, false)
    PTO_FA_CASE(128, true, true)
    PTO_FA_CASE(64, false, false)
    PTO_FA_CASE(64, false, true)
    PTO_FA_CASE(64, true, false)
    PTO_FA_CASE(64, true, true)
#undef PTO_FA_CASE
    return PTO_ERR_UNSUPPORTED;
}
