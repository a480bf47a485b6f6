// Flash-attention forward, head dimension 128, eight wavefronts per workgroup on v_mfma_f32_16x16x32_f16
// (fa_kernels_m16.hpp): the kernel of pto_fa_w8.hip re-tiled for the MFMA shape that sustains the higher clock.
#define PTO_WAVES_M 1
#define PTO_WAVES_N 8
#define PTO_MFMA_M 16
#include <pto/pto-inst.hpp>

#include "fa_kernels_m16.hpp"

namespace pto_amd {
int fa_fwd_d128_w8m16(hipStream_t st, void *o, float *lse, const half *q, const half *k, const half *v, int batch, int heads, int seqQ,
                      int seqKv, bool causal, bool oFp32, int causalOff)
{
    if (causal)
        return oFp32 ? launch_fa_m16<128, true, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff)
                     : launch_fa_m16<128, true, false>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff);
    return oFp32 ? launch_fa_m16<128, false, true>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff)
                 : launch_fa_m16<128, false, false>(st, o, lse, q, k, v, batch, heads, seqQ, seqKv, causalOff);
}
} // namespace pto_amd
