// Error text and version for libats_gfx950.
#include <stdarg.h>
#include <stdio.h>

#include "ats_common.hpp"

namespace ats {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
}  // namespace ats

extern "C" int ats_version(void) { return 100; }
extern "C" const char* ats_last_error_string(void) { return ats::g_err; }
