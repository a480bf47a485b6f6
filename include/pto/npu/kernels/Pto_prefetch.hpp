// PTO_PREFETCH of the reference (include/pto/npu/kernels/Pto_prefetch.hpp:78-95): a host call that warms the L2 with a
// tensor before the kernel that reads it.  On gfx950 the first workgroups to touch a line bring it into the L2 of their
// XCD; there is nothing to do ahead of time.
#pragma once
#include <cstdint>

#include "pto/host/acl_hip.h"

template <bool UseSdma = true, int AivCores = 40>
inline void PTO_PREFETCH(void *tensor, uint64_t tensor_bytes, aclrtStream stream)
{
    (void)tensor;
    (void)tensor_bytes;
    (void)stream;
}
