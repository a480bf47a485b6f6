// Flash-attention forward of one head through the C ABI on files in the layout of the reference's flash_atten example
// (kernels/manual/common/flash_atten/main.cpp:229-233, 340, 610-614; scripts/gen_data.py): <dir>/q.bin = Q [s0, head] fp16,
// <dir>/kt.bin = K stored [s1, head] fp16, <dir>/v.bin = V [s1, head] fp16 -> <dir>/o_out.bin = O [s0, head] fp32, compared
// with <dir>/o.bin by the reference's rule (ResultCmp, eps 1e-3).  The reference's intermediate dumps (QK, P, per-tile
// sums) have no counterpart: scores and probabilities never leave the chip here.  Prints "test success" or "test failed".
// (The reference's own main.cpp, compiled where it lies against include/acl/acl.h, is build/ported/host/flash_atten_main.)
//
//   fa_main [dir [head s0 s1 [causal]]]        defaults: dir = ".", head = 128, s0 = 128, s1 = 1024, causal = 0
#include <cstdlib>

#include <pto/host/test_common.h>

#include "host_util.hpp"
#include "pto_amd.h"

namespace {
struct Problem {
    std::string dir = ".";
    int head = 128, s0 = 128, s1 = 1024, causal = 0;
};

Problem ParseArgs(int argc, char **argv)
{
    Problem p;
    if (argc > 1)
        p.dir = argv[1];
    if (argc > 4) {
        p.head = std::atoi(argv[2]);
        p.s0 = std::atoi(argv[3]);
        p.s1 = std::atoi(argv[4]);
    }
    if (argc > 5)
        p.causal = std::atoi(argv[5]);
    return p;
}

// 0: matches the golden file, 1: does not; exceptions: the set-up failed or the kernel refused the shape
int Run(const Problem &p)
{
    using namespace host_util;
    const size_t elemsO = (size_t)p.s0 * p.head;
    DeviceBuffer q(ReadExactly(p.dir + "/q.bin", (size_t)p.s0 * p.head * sizeof(uint16_t)));
    DeviceBuffer k(ReadExactly(p.dir + "/kt.bin", (size_t)p.s1 * p.head * sizeof(uint16_t)));
    DeviceBuffer v(ReadExactly(p.dir + "/v.bin", (size_t)p.s1 * p.head * sizeof(uint16_t)));
    DeviceBuffer o(elemsO * sizeof(float));
    hipStream_t stream;
    Check(hipStreamCreate(&stream), "hipStreamCreate");
    const int status = pto_fa_fwd_f16(stream, o.as<void>(), nullptr, q.as<uint16_t>(), k.as<uint16_t>(), v.as<uint16_t>(), 1, 1, p.s0,
                                      p.s1, p.head, p.causal, 1);
    Check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    Check(hipStreamDestroy(stream), "hipStreamDestroy");
    if (status != PTO_OK)
        throw std::runtime_error("pto_fa_fwd_f16 returned " + std::to_string(status));
    const std::vector<float> result = o.ToHost<float>();
    WriteAll(p.dir + "/o_out.bin", result.data(), result.size() * sizeof(float));
    const std::vector<uint8_t> goldenBytes = ReadExactly(p.dir + "/o.bin", elemsO * sizeof(float));
    const float *golden = reinterpret_cast<const float *>(goldenBytes.data());
    return PtoTestCommon::ResultCmp<float>(std::vector<float>(golden, golden + elemsO), result, 0.001f) ? 0 : 1;
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
