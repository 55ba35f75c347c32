// Version and error reporting of the C ABI (include/smh.h).
#include <stdarg.h>
#include <stdio.h>

#include "smh_common.hpp"

namespace smh {
static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
}  // namespace smh

extern "C" int smh_version(void) { return SMH_VERSION; }
extern "C" const char *smh_last_error_string(void) { return smh::g_error; }
