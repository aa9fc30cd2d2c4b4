// Error text of the last rejected call (per host thread) and the library version string.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/mf_decode.h"

static thread_local char g_err[512] = "";

void mf_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char* mf_last_error(void) { return g_err; }
extern "C" const char* mf_version(void) { return "mf_decode 0.1 (gfx950)"; }
