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
