// Error channel and identity of the kernel library.
#include "common.h"
#include "pta_kernels.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[1024] = "";

int pta_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return 1;
}

int pta_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return pta_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// compute units of the current device (asked once per device; 256 if the runtime will not say)
int pta_compute_units() {
    static int units[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (units[dev] == 0) {
        int n = 0;
        units[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
    }
    return units[dev];
}

extern "C" const char* pta_last_error(void) { return g_error; }

extern "C" int pta_abi_version(void) { return PTA_ABI_VERSION; }

extern "C" int pta_page_size(void) { return PTA_PAGE; }
