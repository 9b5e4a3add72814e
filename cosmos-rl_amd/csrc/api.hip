// Version, error reporting and device check of libcosmosfp8.
#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "cfp8_common.h"

namespace cfp8 {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(CFP8_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return CFP8_OK;
}

int check_device() {
    // one flag per device ordinal: 0 unknown, 1 good, 2 bad.  Relaxed atomics: two threads that race on
    // the first call both query the device and store the same answer.
    static std::atomic<int8_t> cache[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return set_error(CFP8_EARCH, "no HIP device is current");
    }
    const bool cached = dev >= 0 && dev < 64;
    if (cached && cache[dev].load(std::memory_order_relaxed) == 1) return CFP8_OK;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return set_error(CFP8_EARCH, "cannot query device %d", dev);
    }
    const bool ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    if (cached) cache[dev].store(ok ? 1 : 2, std::memory_order_relaxed);
    if (!ok) return set_error(CFP8_EARCH, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
    return CFP8_OK;
}

}  // namespace cfp8

extern "C" int cfp8_version(void) { return 101; }

extern "C" const char* cfp8_last_error(void) { return cfp8::g_err; }
