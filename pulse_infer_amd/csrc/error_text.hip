// The error channel of the C entry points: a message per thread, read with pulse_last_error().
#include "common.h"

#include <cstdarg>
#include <cstdio>

static thread_local char g_error[512] = "";

extern "C" const char* pulse_last_error() { return g_error; }

void pulse_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// Compute units of the current device, asked once per device (the dispatch rules count workgroups against them).
int pulse_compute_units() {
    constexpr int MAX_DEVICES = 64;
    static int cached[MAX_DEVICES] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= MAX_DEVICES) return 256;
    if (cached[device] == 0) {
        int units = 0;
        if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
            units = 256;
        cached[device] = units;
    }
    return cached[device];
}
