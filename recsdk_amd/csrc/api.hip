// Library-level entry points: version and per-thread error text.
#include <stdarg.h>

#include "common.h"

namespace recsdk {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

}  // namespace recsdk

extern "C" int recsdk_version(void) { return 1; }

extern "C" const char* recsdk_last_error(void) { return recsdk::g_err; }
