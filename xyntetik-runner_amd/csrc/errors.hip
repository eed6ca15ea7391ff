// The error text of the calling thread, and the library's version.
// Every shared object of the kernel library links this file once.
#include "common.h"

static thread_local char g_err[512] = "";

extern "C" const char* xr_last_error() { return g_err; }

void xr_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" int xr_abi_version() { return 1; }
