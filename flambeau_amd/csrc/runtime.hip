// Host-side pieces of the kernel library: error text and version.
#include "common.h"
#include "api.h"
#include <stdarg.h>

static thread_local char g_error[512] = "";

void fl_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* fl_last_error(void) { return g_error; }

extern "C" int fl_abi_version(void) { return 1; }

// Compute units of the current device, asked once (256 where no device answers, as on an MI355X).
// Block shapes, K-splits and the splits of the attention kernels are planned against this number.
int fl_units(void) {
    static int units = 0;
    if (!units) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        units = n;
    }
    return units;
}

extern "C" int fl_compute_units(void) { return fl_units(); }
