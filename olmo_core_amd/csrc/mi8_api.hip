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

int reserve_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* what)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return MI8_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
        set_error("%s: cannot reserve %d bytes of LDS: %s", what, bytes, hipGetErrorString(e));
        return MI8_ERR_LAUNCH;
    }
    done.fetch_or(bit, std::memory_order_release);
    return MI8_OK;
}

int num_compute_units()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    std::atomic<int>& slot = cached[dev & 63];
    int n = slot.load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        slot.store(n, std::memory_order_relaxed);
    }
    return n;
}

}  // namespace mi8

extern "C" int mi8_version(void) { return MI8_VERSION; }

extern "C" const char* mi8_last_error(void) { return mi8::g_error; }
