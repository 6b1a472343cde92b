#include "t12_host.h"
#include <cstring>

static thread_local char g_err[512] = "";

void t12_set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}

extern "C" const char* t12_last_error(void) { return g_err; }
extern "C" const char* t12_version(void) { return "turbo12-gfx950 0.1"; }
