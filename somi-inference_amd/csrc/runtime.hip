// Error text and device queries of the kernel library.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[1024] = "";

extern "C" const char* somi_last_error() { return g_error; }

int somi_fail(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
    return 1;
}

// Name of the architecture the current device reports ("gfx950:sramecc+:xnack-").
extern "C" int somi_device_arch(char* out, int capacity) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return somi_fail("hipGetDevice: %s", hipGetErrorString(err));
    hipDeviceProp_t prop;
    err = hipGetDeviceProperties(&prop, device);
    if (err != hipSuccess) return somi_fail("hipGetDeviceProperties: %s", hipGetErrorString(err));
    snprintf(out, capacity, "%s", prop.gcnArchName);
    return 0;
}

// Compute units of the current device (256 on an MI355X); what launch shapes aim their workgroup counts at.
extern "C" int somi_compute_units() {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return -1;
    return prop.multiProcessorCount;
}

int somi_units() {
    static int cached[64];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    if (cached[device] == 0) {
        hipDeviceProp_t prop;
        cached[device] = hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0
                             ? prop.multiProcessorCount : 256;
    }
    return cached[device];
}

extern "C" int somi_abi_version() { return 1; }
