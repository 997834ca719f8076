#include "common.h"

static thread_local char g_error[512] = "";

extern "C" const char* spy_last_error() { return g_error; }

int spy_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return 1;
}

extern "C" int spy_abi_version() { return 1; }
