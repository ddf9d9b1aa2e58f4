// The error channel and the identification of the library.
#include "common.hpp"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void pl_set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
}

extern "C" const char* pl_last_error() { return g_error; }

// The compute units of the current device, asked once a device.  (Where no device answers, the count of
// the chip this library is built for, so that the host-side choices that use it stay defined.)
int pl_compute_units() {
    constexpr int kDevices = 64, kFallback = 256;
    static int known[kDevices] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kDevices) return kFallback;
    if (known[device] == 0) {
        int units = 0;
        if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
            return kFallback;
        known[device] = units;
    }
    return known[device];
}

// Bumped when an entry point changes its arguments, so that a stale build is rebuilt.
extern "C" int pl_abi_version() { return 1; }
