// Flash-attention forward with eight wavefronts per workgroup (wave grid 1 x 8): 256 queries of one head per
// workgroup share every K / V tile, so each wave issues half the asynchronous copies per key tile and the
// L2 -> LDS traffic per flop halves.  Waves w and w+4 share a SIMD and run in opposite phases: one issues
// MFMAs while the other runs its softmax.  Same kernel template as pto_fa.hip.
#define PTO_WAVES_M 1
#define PTO_WAVES_N 8
#include <pto/pto-inst.hpp>

#include "fa_kernels.hpp"

namespace pto_amd {
int fa_fwd_d128_w8(hipStream_t st, void *o, float *lse, const half *q, const half *k, const half *v, int batch, int heads, int seqQ,
                   int seqKv, bool causal, bool oFp32, int causalOff)
{
    if (causal)
        return oFp32 ? launch_fa<128, true, true, 1, kBKVDefault, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff)
                     : launch_fa<128, true, false, 1, kBKVDefault, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff);
    return oFp32 ? launch_fa<128, false, true, 1, kBKVDefault, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff)
                 : launch_fa<128, false, false, 1, kBKVDefault, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff);
}
} // namespace pto_amd
