// Library bookkeeping of the C ABI: device check, version, last HIP error.
#include "common.hpp"

#include <cstring>

namespace pto_amd {
thread_local int g_last_hip_error = 0;
}

extern "C" int pto_init(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        pto_amd::g_last_hip_error = static_cast<int>(e);
        return PTO_ERR_HIP;
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) {
        pto_amd::g_last_hip_error = static_cast<int>(e);
        return PTO_ERR_HIP;
    }
    // the kernels are built for gfx950 only
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return PTO_ERR_UNSUPPORTED;
    return PTO_OK;
}

extern "C" const char *pto_version(void) { return "pto-amd 0.1 (gfx950)"; }

extern "C" int pto_last_hip_error(void) { return pto_amd::g_last_hip_error; }
