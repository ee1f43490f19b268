// Entry points of the C ABI that launch no kernel: error names and device facts.
#include "common.hpp"
#include <string.h>

extern "C" const char *mi355_error_string(int code) {
    switch (code) {
        case MI355_OK: return "ok";
        case MI355_EINVAL: return "invalid argument (null pointer, negative size or unknown enum)";
        case MI355_ESHAPE: return "shape or stride breaks a precondition of the operator";
        case MI355_EALIGN: return "pointer or leading dimension not aligned for the requested kernel";
        case MI355_EWORKSPACE: return "workspace missing, misaligned or too small";
        case MI355_ELAUNCH: return "HIP runtime refused the launch";
        case MI355_EUNSUPPORTED: return "no kernel variant covers this request";
        case MI355_ESCRATCH: return "the launch needs more scratch than the no-allocation entry point holds";
        default: return "unknown error code";
    }
}

extern "C" int mi355_device_info(int device, int64_t out[8]) {
    if (!out) return MI355_EINVAL;
    if (device < 0 && hipGetDevice(&device) != hipSuccess) return MI355_ELAUNCH;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return MI355_ELAUNCH;
    out[0] = prop.multiProcessorCount;
    out[1] = prop.clockRate;
    out[2] = (int64_t)prop.sharedMemPerBlockOptin > 0 ? (int64_t)prop.sharedMemPerBlockOptin : (int64_t)prop.maxSharedMemoryPerMultiProcessor;
    out[3] = prop.l2CacheSize;
    out[4] = prop.memoryClockRate;
    out[5] = prop.memoryBusWidth;
    out[6] = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
    out[7] = (int64_t)prop.totalGlobalMem;
    return MI355_OK;
}
