/* Host-side shim: the Ascend runtime calls that the reference's host programs make
 * (kernels/manual/a2a3/gemm_performance/main.cpp:26-72, kernels/manual/common/flash_atten/main.cpp:120-260,
 * tests/cpu/st/testcase/.../main.cpp) expressed on the HIP runtime, so that those programs build against this back end
 * with `#include <pto/host/acl_hip.h>` in place of <acl/acl.h>.  Error codes: 0 on success, the HIP error otherwise. */
#ifndef PTO_HOST_ACL_HIP_H
#define PTO_HOST_ACL_HIP_H
#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

typedef hipStream_t aclrtStream;
typedef int aclError;
typedef uint16_t aclFloat16; /* fp16 bit pattern on the host, as in the reference's host code */
enum { ACL_SUCCESS = 0 };
typedef enum aclrtMemMallocPolicy {
    ACL_MEM_MALLOC_HUGE_FIRST = 0,
    ACL_MEM_MALLOC_HUGE_ONLY = 1,
    ACL_MEM_MALLOC_NORMAL_ONLY = 2
} aclrtMemMallocPolicy;
typedef enum aclrtMemcpyKind {
    ACL_MEMCPY_HOST_TO_HOST = 0,
    ACL_MEMCPY_HOST_TO_DEVICE = 1,
    ACL_MEMCPY_DEVICE_TO_HOST = 2,
    ACL_MEMCPY_DEVICE_TO_DEVICE = 3
} aclrtMemcpyKind;

static inline aclError aclInit(const char *config) { (void)config; return (aclError)hipInit(0); }
static inline aclError aclFinalize(void) { return ACL_SUCCESS; }
static inline aclError aclrtSetDevice(int32_t device) { return (aclError)hipSetDevice(device); }
static inline aclError aclrtResetDevice(int32_t device) { (void)device; return (aclError)hipDeviceSynchronize(); }
/* default priority only: streams of other priorities are not used by this back end */
static inline aclError aclrtCreateStream(aclrtStream *stream) { return (aclError)hipStreamCreate(stream); }
static inline aclError aclrtDestroyStream(aclrtStream stream) { return (aclError)hipStreamDestroy(stream); }
static inline aclError aclrtSynchronizeStream(aclrtStream stream) { return (aclError)hipStreamSynchronize(stream); }
static inline aclError aclrtSynchronizeDevice(void) { return (aclError)hipDeviceSynchronize(); }
static inline aclError aclrtMalloc(void **ptr, size_t size, aclrtMemMallocPolicy policy)
{
    (void)policy;
    return (aclError)hipMalloc(ptr, size);
}
static inline aclError aclrtFree(void *ptr) { return (aclError)hipFree(ptr); }
/* pinned host memory is allocated, never registered after the fact */
static inline aclError aclrtMallocHost(void **ptr, size_t size) { return (aclError)hipHostMalloc(ptr, size, hipHostMallocDefault); }
static inline aclError aclrtFreeHost(void *ptr) { return (aclError)hipHostFree(ptr); }
static inline hipMemcpyKind pto_acl_kind(aclrtMemcpyKind kind)
{
    switch (kind) {
    case ACL_MEMCPY_HOST_TO_HOST: return hipMemcpyHostToHost;
    case ACL_MEMCPY_HOST_TO_DEVICE: return hipMemcpyHostToDevice;
    case ACL_MEMCPY_DEVICE_TO_HOST: return hipMemcpyDeviceToHost;
    default: return hipMemcpyDeviceToDevice;
    }
}
static inline aclError aclrtMemcpy(void *dst, size_t destMax, const void *src, size_t count, aclrtMemcpyKind kind)
{
    if (count > destMax)
        return (aclError)hipErrorInvalidValue;
    return (aclError)hipMemcpy(dst, src, count, pto_acl_kind(kind));
}
static inline aclError aclrtMemcpyAsync(void *dst, size_t destMax, const void *src, size_t count, aclrtMemcpyKind kind,
                                        aclrtStream stream)
{
    if (count > destMax)
        return (aclError)hipErrorInvalidValue;
    return (aclError)hipMemcpyAsync(dst, src, count, pto_acl_kind(kind), stream);
}
static inline aclError aclrtMemset(void *ptr, size_t maxCount, int32_t value, size_t count)
{
    if (count > maxCount)
        return (aclError)hipErrorInvalidValue;
    return (aclError)hipMemset(ptr, value, count);
}
#endif /* PTO_HOST_ACL_HIP_H */
