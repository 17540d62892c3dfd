// Library-level entry points: version and thread-local error string.
#include "common.h"

#include <atomic>

static thread_local char g_err[512] = "";

int ptj_set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Compute units of the current device, asked once per device and kept.  Grid sizes of persistent
// and grid-stride kernels are multiples of it.  Without a device (planning calls on a machine that
// has none) the MI355X's 256.
int ptj_num_cus() {
    constexpr int DEFAULT_CUS = 256, MAX_DEVICES = 64;
    static std::atomic<int> cached[MAX_DEVICES] = {};   // 0 = not asked yet; every thread that asks stores the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        (void)hipGetLastError();
        return DEFAULT_CUS;
    }
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = DEFAULT_CUS;
        }
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

extern "C" {
int ptj_version(void) { return 1; }
const char* ptj_last_error(void) { return g_err; }
}
