// Error reporting and version of libmoe_mi355.so.
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace {
thread_local char g_err[512] = "";
}

namespace moe {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}
}  // namespace moe

extern "C" const char* moe_last_error(void) { return g_err; }
extern "C" const char* moe_version(void) { return "moe_mi355 0.1 (gfx950)"; }
