// Error reporting and version of the C ABI (host only).
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_last_error[512] = "";

void ezl_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* ezl_last_error(void) { return g_last_error; }

extern "C" int ezl_version(void) { return 100; }
