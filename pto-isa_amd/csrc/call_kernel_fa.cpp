// `call_kernel` of the flash-attention demo (demos/torch_jit/flash_atten/fa_kernel.cpp:1017-1092): one head,
// q [s0, 128], k and v [s1, 128] fp16, o_out [s0, 128] fp32.  Same signature.  The workspace arguments are the
// reference's global-memory FIFOs and intermediates; this back end keeps scores and probabilities on chip and
// does not touch them.  The causal mask follows the reference's rule (key j is visible to query i iff j <= i, whatever
// s1 is: fa_kernel.cpp's runTFA skips tiles with s1_index > s0_index).  Unsupported parameters return without launching, as the reference does
// (fa_kernel.cpp:1050-1058); pto_last_status_fa() tells why.
#include <cstdint>

#include "pto_amd.h"

static int g_last = PTO_OK;

extern "C" int pto_last_status_fa(void) { return g_last; }

extern "C" void call_kernel(void *stream, int headSize, int s0, int s1, bool is_causal, uint8_t *q, uint8_t *k, uint8_t *v,
                            uint8_t *o_out, float *outDevice, uint16_t *xexpDevice, float *pOutFp32Device, float *out2Device,
                            float *gSumDevice, float *expMaxDevice, float *oPartsDevice)
{
    (void)outDevice;
    (void)xexpDevice;
    (void)pOutFp32Device;
    (void)out2Device;
    (void)gSumDevice;
    (void)expMaxDevice;
    (void)oPartsDevice;
    if (headSize != 128 || (s0 % 128) != 0) { // the reference's own checks
        g_last = PTO_ERR_UNSUPPORTED;
        return;
    }
    g_last = pto_fa_fwd_f16(stream, o_out, nullptr, reinterpret_cast<const uint16_t *>(q), reinterpret_cast<const uint16_t *>(k),
                            reinterpret_cast<const uint16_t *>(v), 1, 1, s0, s1, headSize, is_causal ? 2 : 0, 1);
}
