// Library-level entry points: version and the thread-local error string.
#include "bsrl_common.h"
#include <string.h>

namespace { thread_local char g_err[512] = ""; }

void bsrl_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" int bsrl_version(void) { return 17; }
extern "C" const char* bsrl_last_error(void) { return g_err; }
