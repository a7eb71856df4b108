// Library-wide pieces of the C ABI: version, thread-local error text, one-time set-up.
#include "common.h"

#include <atomic>
#include <mutex>

// attn_f16.hip / attn_bf16.hip: LDS size attribute of every attention kernel instantiation of one element type
template <typename T> int attn_configure_all();
template <typename T> int attn_configure_cls();  // attn_cls_f16.hip / attn_cls_bf16.hip
// rows_wide.hip: address of the library-owned scratch array on the current device
int wide_noalloc_setup(void** out);

namespace {
thread_local char g_error[512] = "";
std::once_flag g_once;
std::atomic<int> g_init_rc{1};  // 1 = set-up has not run
int g_num_cus = 256;

void init_once() {
    int rc = RGD_OK;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) {
        g_num_cus = cus;
        // kernels with more than 48 KB of dynamic LDS need the attribute before their first launch
        rc = attn_configure_all<f16_t>();
        if (rc == RGD_OK) rc = attn_configure_all<bf16_t>();
        if (rc == RGD_OK) rc = attn_configure_cls<f16_t>();
        if (rc == RGD_OK) rc = attn_configure_cls<bf16_t>();
        if (rc == RGD_OK) rc = wide_noalloc_setup(nullptr);
    } else {
        // no usable device (a CPU-only process that checks arguments): launches will fail with their own error
        (void)hipGetLastError();
    }
    g_init_rc.store(rc, std::memory_order_release);
}
}  // namespace

void rgd_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int rgd_ensure_init() {
    int rc = g_init_rc.load(std::memory_order_acquire);
    if (rc <= 0) return rc;
    std::call_once(g_once, init_once);
    return g_init_rc.load(std::memory_order_acquire);
}

int rgd_num_cus() {
    (void)rgd_ensure_init();
    return g_num_cus;
}

int rgd_launch_status(const char* what, hipError_t e) {
    if (e == hipSuccess) return RGD_OK;
    rgd_set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return RGD_ERR_LAUNCH;
}

extern "C" {
int rgd_version(void) { return 3000; }
const char* rgd_last_error(void) { return g_error; }
int rgd_init(void) {
    const int rc = rgd_ensure_init();
    if (rc != RGD_OK && g_error[0] == 0) rgd_set_error("rgd_init: set-up failed earlier on another thread (%d)", rc);
    return rc;
}
}
