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
