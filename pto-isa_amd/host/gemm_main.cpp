// Host program of the GEMM kernel with the reference's file protocol
// (kernels/manual/a2a3/gemm_performance/main.cpp:17-105): reads <dir>/input/x1_gm.bin (A [m,k] fp16) and
// <dir>/input/x2_gm.bin (B stored [n,k] fp16), runs the kernel, writes <dir>/output/output_z.bin (C [m,n] fp32) and
// compares it with <dir>/output/golden.bin (ResultCmp, eps 1e-3).  Prints "test success" or "test failed".
//
//   gemm_main [dir [m k n]]        defaults: dir = "..", m = k = n = 6144 (the reference's build)
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include <pto/host/acl_hip.h>
#include <pto/host/test_common.h>

#include "pto_amd.h"

using namespace PtoTestCommon;

namespace {
uint32_t gM = 6144, gK = 6144, gN = 6144;
int gStatus = PTO_OK;
}

// same name and argument meaning as the reference's launcher (gemm_performance_kernel.cpp:243-264)
template <typename T>
void LaunchGEMME2E(uint8_t *out, uint8_t *src0, uint8_t *src1, void *stream)
{
    gStatus = pto_gemm_f16f32(stream, reinterpret_cast<float *>(out), reinterpret_cast<const uint16_t *>(src0),
                              reinterpret_cast<const uint16_t *>(src1), (int)gM, (int)gN, (int)gK);
}

int main(int argc, char **argv)
{
    const std::string dir = argc > 1 ? argv[1] : "..";
    if (argc > 4) {
        gM = (uint32_t)std::atoi(argv[2]);
        gK = (uint32_t)std::atoi(argv[3]);
        gN = (uint32_t)std::atoi(argv[4]);
    }
    size_t aFileSize = (size_t)gM * gK * sizeof(uint16_t), bFileSize = (size_t)gK * gN * sizeof(uint16_t);
    size_t cFileSize = (size_t)gM * gN * sizeof(float);

    aclInit(nullptr);
    aclrtSetDevice(0);
    if (pto_init() != PTO_OK) {
        std::printf("test failed (pto_init: not a gfx950 device)\n");
        return 2;
    }
    aclrtStream stream;
    aclrtCreateStream(&stream);

    uint8_t *dstHost, *src0Host, *src1Host, *dstDevice, *src0Device, *src1Device;
    aclrtMallocHost((void **)(&dstHost), cFileSize);
    aclrtMallocHost((void **)(&src0Host), aFileSize);
    aclrtMallocHost((void **)(&src1Host), bFileSize);
    aclrtMalloc((void **)&dstDevice, cFileSize, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void **)&src0Device, aFileSize, ACL_MEM_MALLOC_HUGE_FIRST);
    aclrtMalloc((void **)&src1Device, bFileSize, ACL_MEM_MALLOC_HUGE_FIRST);

    bool ok = ReadFile(dir + "/input/x1_gm.bin", aFileSize, src0Host, aFileSize);
    ok = ReadFile(dir + "/input/x2_gm.bin", bFileSize, src1Host, bFileSize) && ok;
    if (!ok) {
        std::printf("test failed (inputs)\n");
        return 2;
    }
    aclrtMemcpy(src0Device, aFileSize, src0Host, aFileSize, ACL_MEMCPY_HOST_TO_DEVICE);
    aclrtMemcpy(src1Device, bFileSize, src1Host, bFileSize, ACL_MEMCPY_HOST_TO_DEVICE);
    LaunchGEMME2E<uint16_t>(dstDevice, src0Device, src1Device, stream);
    aclrtSynchronizeStream(stream);
    aclrtMemcpy(dstHost, cFileSize, dstDevice, cFileSize, ACL_MEMCPY_DEVICE_TO_HOST);
    WriteFile(dir + "/output/output_z.bin", dstHost, cFileSize);

    aclrtFree(dstDevice);
    aclrtFree(src0Device);
    aclrtFree(src1Device);
    aclrtFreeHost(dstHost);
    aclrtFreeHost(src0Host);
    aclrtFreeHost(src1Host);
    aclrtDestroyStream(stream);
    aclrtResetDevice(0);
    aclFinalize();
    if (gStatus != PTO_OK) {
        std::printf("test failed (pto_gemm_f16f32 returned %d)\n", gStatus);
        return 1;
    }

    const size_t count = (size_t)gM * gN;
    std::vector<float> golden(count), devFinal(count);
    ok = ReadFile(dir + "/output/golden.bin", cFileSize, golden.data(), cFileSize);
    ok = ReadFile(dir + "/output/output_z.bin", cFileSize, devFinal.data(), cFileSize) && ok;
    const bool ret = ok && ResultCmp(golden, devFinal, 0.001f);
    std::printf(ret ? "test success\n" : "test failed\n");
    return ret ? 0 : 1;
}
