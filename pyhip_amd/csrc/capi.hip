// Library-wide pieces of the C ABI: version, last-error string.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_last_error[512] = "";

extern "C" void pyhip_set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* pyhip_moe_last_error(void) { return g_last_error; }

extern "C" int pyhip_moe_abi_version(void) { return 9; }
