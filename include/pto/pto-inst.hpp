// PTO tile instructions, MI355X (gfx950) back end.  Compile with hipcc --offload-arch=gfx950.
//
//   #include <pto/pto-inst.hpp>
//   using namespace pto;
//
// Define PTO_WAVES_M / PTO_WAVES_N before the include to choose the wave grid of a workgroup
// (default 2 x 2 = 256 threads); launch kernels with pto::kBlockThreads threads per block and the
// bytes of LDS that the TASSIGN'ed Mat tiles span as dynamic shared memory.
#pragma once
#include "pto/common/constants.hpp"
#include "pto/common/pto_instr.hpp"

// Kernel sources written for the Ascend toolchain mark device functions with AICORE only, which is
// empty here.  Bracket the device part of a translation unit (kernels and their helpers, not the
// host launch code) with these two macros: every function in between is compiled for the device.
#define PTO_DEVICE_CODE_BEGIN _Pragma("clang force_cuda_host_device begin")
#define PTO_DEVICE_CODE_END _Pragma("clang force_cuda_host_device end")
