// Thread-local error message and version query of libdnatok_hip.
#include "common.hpp"

#include <stdarg.h>

namespace dnatok {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

}  // namespace dnatok

extern "C" int dnatok_version(void) { return DNATOK_VERSION; }

extern "C" const char *dnatok_last_error(void) { return dnatok::g_error; }
