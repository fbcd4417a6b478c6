// The error channel of the kernel library.
#include "zi_common.h"
#include <stdarg.h>

static thread_local char zi_error_buf[1024] = "";

extern "C" const char* zi_last_error() { return zi_error_buf; }

int zi_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(zi_error_buf, sizeof(zi_error_buf), fmt, ap);
    va_end(ap);
    return 1;
}

int zi_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return zi_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

extern "C" int zi_abi_version() { return 1; }

// Compute units of the current device (what launch cuts and tile choices are balanced over), read once per
// device; ZI_DEFAULT_COMPUTE_UNITS when there is no device to ask (a host-only process that plans launches).
#include <atomic>
extern "C" int zi_compute_units() {
    static std::atomic<int> known[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return ZI_DEFAULT_COMPUTE_UNITS;
    }
    int cus = known[dev].load(std::memory_order_relaxed);
    if (cus <= 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            return ZI_DEFAULT_COMPUTE_UNITS;
        }
        known[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}
