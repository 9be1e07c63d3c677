// Host-side odds and ends of the kernel library: the error text and the interface version.
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

static thread_local char g_error[512] = "";

void ri_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* ri_last_error(void) { return g_error; }
extern "C" int ri_abi_version(void) { return 1; }
