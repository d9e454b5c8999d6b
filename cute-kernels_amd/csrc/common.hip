// Error slot, version and device-property queries of libfma_hip.so.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace fmahip {

static thread_local char g_error[512] = {0};

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int launch_status(const char* what) {
    hipError_t err = hipGetLastError();
    if (err == hipSuccess) return FMA_OK;
    fail((int)err, "%s: launch failed: %s", what, hipGetErrorString(err));
    return (int)err;
}

int num_compute_units() {
    // one cached value per device; a benign race only ever stores the same number twice
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (dev < 0 || dev >= 64) dev = 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace fmahip

extern "C" {

const char* fma_last_error_string(void) { return fmahip::g_error; }

int fma_abi_version(void) { return 2; }

int fma_num_compute_units(void) { return fmahip::num_compute_units(); }

}  // extern "C"
