// The error channel and device check of the library.
#include "common.h"
#include "api.h"
#include <stdarg.h>
#include <string.h>

static thread_local char g_error[512] = "";

void picolm_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* picolm_last_error(void) { return g_error; }

extern "C" int picolm_abi_version(void) { return 1; }

extern "C" int picolm_device_check(void) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    PICOLM_REQUIRE(e == hipSuccess, "no HIP device: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    PICOLM_REQUIRE(e == hipSuccess, "cannot query device %d: %s", dev, hipGetErrorString(e));
    PICOLM_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
                   "device %d is %s; these kernels are built for gfx950 only", dev, prop.gcnArchName);
    return 0;
}
