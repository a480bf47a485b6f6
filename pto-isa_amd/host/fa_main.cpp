// Host program of the flash-attention kernel with the reference's file protocol
// (kernels/manual/common/flash_atten/main.cpp:229-233, 340, 610-614): reads <dir>/q.bin (Q [s0, head] fp16),
// <dir>/kt.bin (K stored [s1, head] fp16) and <dir>/v.bin (V [s1, head] fp16), runs the kernel on one head, writes
// <dir>/o_out.bin (O [s0, head] fp32) and compares it with <dir>/o.bin (ResultCmp, eps 1e-3).  The reference's
// intermediate dumps (QK, P, per-tile sums) have no counterpart: scores and probabilities never leave the chip here.
// Prints "test success" or "test failed".
//
//   fa_main [dir [head s0 s1 [causal]]]        defaults: dir = ".", head = 128, s0 = 128, s1 = 1024, causal = 0
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include <pto/host/acl_hip.h>
#include <pto/host/test_common.h>

#include "pto_amd.h"

using namespace PtoTestCommon;

int main(int argc, char **argv)
{
    const std::string dir = argc > 1 ? argv[1] : ".";
    int head = 128, s0 = 128, s1 = 1024, causal = 0;
    if (argc > 4) {
        head = std::atoi(argv[2]);
        s0 = std::atoi(argv[3]);
        s1 = std::atoi(argv[4]);
    }
    if (argc > 5)
        causal = std::atoi(argv[5]);
    size_t qSize = (size_t)s0 * head * sizeof(uint16_t), kSize = (size_t)s1 * head * sizeof(uint16_t), vSize = kSize;
    size_t oSize = (size_t)s0 * head * sizeof(float);

    aclInit(nullptr);
    aclrtSetDevice(0);
    if (pto_init() != PTO_OK) {
        std::printf("test failed (pto_init: not a gfx950 device)\n");
        return 2;
    }
    aclrtStream stream;
    aclrtCreateStream(&stream);

    uint8_t *qHost, *kHost, *vHost, *oHost, *qDevice, *kDevice, *vDevice, *oDevice;
    aclrtMallocHost((void **)(&qHost), qSize);
    aclrtMallocHost((void **)(&kHost), kSize);
    aclrtMallocHost((void **)(&vHost), vSize);
    aclrtMallocHost((void **)(&oHost), oSize);
    aclrtMalloc((void **)&qDevice, qSize, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void **)&kDevice, kSize, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void **)&vDevice, vSize, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void **)&oDevice, oSize, ACL_MEM_MALLOC_HUGE_FIRST);

    bool ok = ReadFile(dir + "/q.bin", qSize, qHost, qSize);
    ok = ReadFile(dir + "/kt.bin", kSize, kHost, kSize) && ok;
    ok = ReadFile(dir + "/v.bin", vSize, vHost, vSize) && ok;
    if (!ok) {
        std::printf("test failed (inputs)\n");
        return 2;
    }
    aclrtMemcpy(qDevice, qSize, qHost, qSize, ACL_MEMCPY_HOST_TO_DEVICE);
    aclrtMemcpy(kDevice, kSize, kHost, kSize, ACL_MEMCPY_HOST_TO_DEVICE);
    aclrtMemcpy(vDevice, vSize, vHost, vSize, ACL_MEMCPY_HOST_TO_DEVICE);
    const int status = pto_fa_fwd_f16(stream, oDevice, nullptr, reinterpret_cast<const uint16_t *>(qDevice),
                                      reinterpret_cast<const uint16_t *>(kDevice), reinterpret_cast<const uint16_t *>(vDevice), 1, 1, s0,
                                      s1, head, causal, 1);
    aclrtSynchronizeStream(stream);
    aclrtMemcpy(oHost, oSize, oDevice, oSize, ACL_MEMCPY_DEVICE_TO_HOST);
    WriteFile(dir + "/o_out.bin", oHost, oSize);

    aclrtFree(qDevice);
    aclrtFree(kDevice);
    aclrtFree(vDevice);
    aclrtFree(oDevice);
    aclrtFreeHost(qHost);
    aclrtFreeHost(kHost);
    aclrtFreeHost(vHost);
    aclrtFreeHost(oHost);
    aclrtDestroyStream(stream);
    aclrtResetDevice(0);
    aclFinalize();
    if (status != PTO_OK) {
        std::printf("test failed (kernel status %d)\n", status);
        return 2;
    }

    const size_t count = (size_t)s0 * head;
    std::vector<float> golden(count), devFinal(count);
    size_t goldenFileSize = oSize, devFileSize = oSize;
    ok = ReadFile(dir + "/o.bin", goldenFileSize, golden.data(), oSize);
    ok = ReadFile(dir + "/o_out.bin", devFileSize, devFinal.data(), oSize) && ok;
    if (ok && ResultCmp<float>(golden, devFinal, 0.001f)) {
        std::printf("test success\n");
        return 0;
    }
    std::printf("test failed\n");
    return 1;
}
