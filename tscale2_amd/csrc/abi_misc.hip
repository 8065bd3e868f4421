// Library-level queries of the C ABI.
#include "common.h"
#include "internal.h"

extern "C" int ts2_device_info(int *cuCount, int *clockMHz)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        return TS2_ERR_LAUNCH;
    }
    if (cuCount) {
        *cuCount = prop.multiProcessorCount;
    }
    if (clockMHz) {
        *clockMHz = prop.clockRate / 1000;
    }
    // the library's per-device set-up that is not stream work, so that no later entry point has to do it under a caller's capture
    return Ts2MoeRouteSetup();
}

extern "C" const char *ts2_version(void)
{
    return "ts2amd 0.1 (gfx950)";
}
