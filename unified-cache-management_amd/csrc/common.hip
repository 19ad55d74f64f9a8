// Error text storage and version of the HIP library.
#include "common.h"

#include <cstring>

namespace ucm {

namespace {
thread_local char g_err[512] = {0};
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_err[0] = 0; }

}  // namespace ucm

extern "C" int ucm_version(void) { return 100; }

extern "C" const char* ucm_last_error(void) { return ucm::g_err; }
