// Error message of the last failed entry point on this thread.
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_msg[1024] = "";

extern "C" const char* ri_last_error() { return g_msg; }

int ri_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_msg, sizeof(g_msg), fmt, ap);
    va_end(ap);
    return 1;
}

extern "C" int ri_abi_version() { return 1; }
