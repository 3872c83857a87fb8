// The error channel of the C entry points: a message per thread, and the ABI version.
#include "common.h"
#include "api.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void ia_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* ia_last_error(void) { return g_error; }

extern "C" int ia_abi_version(void) { return IA_ABI_VERSION; }
