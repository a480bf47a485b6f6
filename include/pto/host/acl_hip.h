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
/* conversions of the Ascend runtime between that pattern and float (every value of fp16 is a float; to fp16 rounds to nearest even) */
static inline float aclFloat16ToFloat(aclFloat16 value)
{
    const uint32_t sign = (uint32_t)(value & 0x8000u) << 16, exp = (value >> 10) & 0x1Fu, man = value & 0x3FFu;
    uint32_t bits;
    if (exp == 0x1Fu) {
        bits = sign | 0x7F800000u | (man << 13); /* infinity, NaN */
    } else if (exp != 0) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else { /* subnormal: man x 2^-24 */
        uint32_t m = man, e = 113u;
        while ((m & 0x400u) == 0) {
            m <<= 1;
            --e;
        }
        bits = sign | (e << 23) | ((m & 0x3FFu) << 13);
    }
    float f;
    __builtin_memcpy(&f, &bits, sizeof f);
    return f;
}
static inline aclFloat16 aclFloatToFloat16(float value)
{
    uint32_t x;
    __builtin_memcpy(&x, &value, sizeof x);
    const uint32_t sign = (x >> 16) & 0x8000u, mag = x & 0x7FFFFFFFu;
    if (mag >= 0x7F800000u) /* infinity, NaN */
        return (aclFloat16)(sign | 0x7C00u | (mag > 0x7F800000u ? 0x200u : 0u));
    if (mag >= 0x477FF000u) /* rounds to 65520 or more: infinity */
        return (aclFloat16)(sign | 0x7C00u);
    if (mag < 0x33000001u) /* at most 2^-25: zero */
        return (aclFloat16)sign;
    const int e = (int)(mag >> 23) - 127;
    const uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;
    const int shift = e >= -14 ? 13 : 13 + (-14 - e); /* bits dropped below the fp16 mantissa */
    const uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t r = kept + ((rest > half || (rest == half && (kept & 1u))) ? 1u : 0u);
    /* normal: implicit bit of `kept` adds one to the exponent field; subnormal: the field starts at 0 and a carry makes it 1 */
    const uint32_t bits = e >= -14 ? (((uint32_t)(e + 14) << 10) + r) : r;
    return (aclFloat16)(sign | bits);
}
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
