// `call_kernel` of the GEMM demo (demos/torch_jit/gemm/gemm_kernel.cpp:236-262): the entry point that the reference's
// JIT demo loads with ctypes.  Same signature; the problem size is the demo's fixed m = n = k = 6144.  blockDim is the
// Ascend core count and has no meaning here (the launch geometry is chosen by the library).
#include <cstdint>

#include "pto_amd.h"

extern "C" void call_kernel(uint32_t blockDim, void *stream, uint8_t *out, uint8_t *src0, uint8_t *src1)
{
    (void)blockDim;
    (void)pto_gemm_f16f32(stream, reinterpret_cast<float *>(out), reinterpret_cast<const uint16_t *>(src0),
                          reinterpret_cast<const uint16_t *>(src1), 6144, 6144, 6144);
}
