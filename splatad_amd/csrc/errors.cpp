// Thread-local error message and ABI version of libsplatad_hip.so.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/splatad_hip.h"

static thread_local char g_last_error[512] = "";

void splatad_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

extern "C" const char *splatad_last_error(void) { return g_last_error; }

extern "C" int splatad_abi_version(void) { return 11; }
