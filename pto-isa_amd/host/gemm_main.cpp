// GEMM through the C ABI on files in the layout of the reference's gemm_performance example
// (kernels/manual/a2a3/gemm_performance/main.cpp:42-78; scripts/gen_data.py): <dir>/input/x1_gm.bin = A [m,k] fp16,
// <dir>/input/x2_gm.bin = B stored [n,k] fp16 -> <dir>/output/output_z.bin = C [m,n] fp32, compared with
// <dir>/output/golden.bin by the reference's rule (ResultCmp, eps 1e-3).  Prints "test success" or "test failed".
// (The reference's own main.cpp, compiled where it lies against include/acl/acl.h, is build/ported/host/gemm_performance_main.)
//
//   gemm_main [dir [m k n]]        defaults: dir = "..", m = k = n = 6144
#include <cstdlib>

#include <pto/host/test_common.h>

#include "host_util.hpp"
#include "pto_amd.h"

namespace {
struct Problem {
    std::string dir = "..";
    int m = 6144, k = 6144, n = 6144;
};

Problem ParseArgs(int argc, char **argv)
{
    Problem p;
    if (argc > 1)
        p.dir = argv[1];
    if (argc > 4) {
        p.m = std::atoi(argv[2]);
        p.k = std::atoi(argv[3]);
        p.n = std::atoi(argv[4]);
    }
    return p;
}

// 0: matches the golden file, 1: does not; exceptions: the set-up failed or the kernel refused the shape
int Run(const Problem &p)
{
    using namespace host_util;
    const size_t elemsC = (size_t)p.m * p.n;
    DeviceBuffer a(ReadExactly(p.dir + "/input/x1_gm.bin", (size_t)p.m * p.k * sizeof(uint16_t)));
    DeviceBuffer b(ReadExactly(p.dir + "/input/x2_gm.bin", (size_t)p.n * p.k * sizeof(uint16_t)));
    DeviceBuffer c(elemsC * sizeof(float));
    hipStream_t stream;
    Check(hipStreamCreate(&stream), "hipStreamCreate");
    const int status = pto_gemm_f16f32(stream, c.as<float>(), a.as<uint16_t>(), b.as<uint16_t>(), p.m, p.n, p.k);
    Check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    Check(hipStreamDestroy(stream), "hipStreamDestroy");
    if (status != PTO_OK)
        throw std::runtime_error("pto_gemm_f16f32 returned " + std::to_string(status));
    const std::vector<float> result = c.ToHost<float>();
    WriteAll(p.dir + "/output/output_z.bin", result.data(), result.size() * sizeof(float));
    const std::vector<uint8_t> goldenBytes = ReadExactly(p.dir + "/output/golden.bin", elemsC * sizeof(float));
    const float *golden = reinterpret_cast<const float *>(goldenBytes.data());
    return PtoTestCommon::ResultCmp(std::vector<float>(golden, golden + elemsC), result, 0.001f) ? 0 : 1;
}
} // namespace

int main(int argc, char **argv)
{
    if (pto_init() != PTO_OK) {
        std::printf("test failed (pto_init: not a gfx950 device)\n");
        return 2;
    }
    try {
        const int rc = Run(ParseArgs(argc, argv));
        std::printf(rc == 0 ? "test success\n" : "test failed\n");
        return rc;
    } catch (const std::exception &e) {
        std::printf("test failed (%s)\n", e.what());
        return 2;
    }
}
