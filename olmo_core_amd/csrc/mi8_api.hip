// Library-wide pieces of the C ABI: version, per-thread error text, launch status.
#include <stdarg.h>
#include <stdio.h>

#include "mi8_common.h"

namespace mi8 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int launch_status(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return MI8_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return MI8_ERR_LAUNCH;
}

}  // namespace mi8

extern "C" int mi8_version(void) { return MI8_VERSION; }

extern "C" const char* mi8_last_error(void) { return mi8::g_error; }
