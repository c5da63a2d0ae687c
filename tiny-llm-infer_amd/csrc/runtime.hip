// Error channel and small queries of the C ABI.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

extern "C" const char* tli_last_error() { return g_error; }

int tli_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return 1;
}

int tli_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return tli_fail("%s: %s", what, hipGetErrorString(e));
    return 0;
}

extern "C" int tli_abi_version() { return 1; }

int tli_compute_units() {
    static int units = 0;
    if (units == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n >= TLI_DIES)
            units = n;
        else
            units = 256;                     // (no device to ask: the chip this library is written for)
        (void)hipGetLastError();
    }
    return units;
}

extern "C" int tli_device_compute_units() { return tli_compute_units(); }
