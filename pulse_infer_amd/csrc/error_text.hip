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
