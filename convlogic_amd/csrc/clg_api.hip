// Error reporting and version of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "clg_common.h"

namespace {
thread_local char g_error[512] = "";
}

void clg_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char *clg_last_error(void) { return g_error; }
extern "C" int clg_abi_version(void) { return 1; }
