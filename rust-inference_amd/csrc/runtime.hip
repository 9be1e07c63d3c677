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

// Compute units of the device that is current on the calling thread, asked once per device.  The rules that
// size launches (how many row tiles a workgroup takes, into how many stretches K is cut, when attention tiles
// are halved) count workgroups against this number.  Where there is no device (a build machine), the MI355X's 256.
extern "C" int ri_compute_units(void) {
    static int known[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();                 // the failed query must not be reported by the next launch check
        return 256;
    }
    if (known[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        known[dev] = n;
    }
    return known[dev];
}
