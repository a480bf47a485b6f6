// The one call of Ascend's runtime header that the reference's flash-attention host program makes
// (kernels/manual/common/flash_atten/main.cpp:244-246): the address of the cross-core synchronisation registers, which its
// launcher hands to the kernel.  Cube and Vec roles share a workgroup here, so there is no such block: address 0, length 0.
#ifndef PTO_HOST_RUNTIME_RT_H
#define PTO_HOST_RUNTIME_RT_H
#include <cstdint>

static inline int rtGetC2cCtrlAddr(uint64_t *addr, uint32_t *len)
{
    if (addr)
        *addr = 0;
    if (len)
        *len = 0;
    return 0;
}
#endif // PTO_HOST_RUNTIME_RT_H
