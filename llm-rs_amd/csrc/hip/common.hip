#include "common.h"

static thread_local char g_error[512];

char* llmrs_error_buffer() { return g_error; }

int llmrs_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return -1;
}

extern "C" const char* llmrs_hip_error() { return g_error; }

int llmrs_compute_units() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) ? prop.multiProcessorCount : 256;
    }
    return n;
}

// Name of the architecture the current device reports, for the loader's check
// that this library and the device fit each other.
extern "C" int llmrs_device_arch(char* out, int cap) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return llmrs_fail("no HIP device");
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return llmrs_fail("cannot read device properties");
    snprintf(out, cap, "%s", prop.gcnArchName);
    return prop.multiProcessorCount;
}
