// Error text, version and device facts of the kernel library.
#include "common.h"
#include "api.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace {
thread_local char g_error[512] = "";
}

void fsie_set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
}

extern "C" const char* fsie_last_error(void) { return g_error; }

extern "C" int fsie_version(void) { return 1; }

int fsie_compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        cached[dev] = n;
    }
    return cached[dev];
}

extern "C" int fsie_device_compute_units(void) { return fsie_compute_units(); }

extern "C" int fsie_device_info(char* arch_out, int arch_len, int* n_compute_units) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        fsie_set_error("device_info: %s", hipGetErrorString(e));
        return 2;
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) {
        fsie_set_error("device_info: %s", hipGetErrorString(e));
        return 2;
    }
    if (arch_out && arch_len > 0) {
        strncpy(arch_out, prop.gcnArchName, static_cast<size_t>(arch_len) - 1);
        arch_out[arch_len - 1] = '\0';
    }
    if (n_compute_units) *n_compute_units = prop.multiProcessorCount;
    return 0;
}
