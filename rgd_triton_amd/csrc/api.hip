// Library-wide pieces of the C ABI: version, thread-local error text, device properties.
#include "common.h"

#include <atomic>

namespace {
thread_local char g_error[512] = "";
std::atomic<int> g_num_cus{0};
}  // namespace

void rgd_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// compute units of the current device; 256 (MI355X) when no device can be queried
int rgd_num_cus() {
    int n = g_num_cus.load(std::memory_order_relaxed);
    if (n > 0) return n;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) {
        g_num_cus.store(cus, std::memory_order_relaxed);
        return cus;
    }
    (void)hipGetLastError();
    return 256;
}

extern "C" {
int rgd_version(void) { return 1000; }
const char* rgd_last_error(void) { return g_error; }
}
