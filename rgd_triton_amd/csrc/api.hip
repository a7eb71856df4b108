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
std::mutex g_init_mutex;
std::atomic<int> g_init_done{0};  // 1 once a device has been seen and the set-up below has run
int g_num_cus = 256;
// what the attention kernels' set-up returned, kept apart from the rest: the row kernels need none of it
int g_attn_rc = RGD_OK;
char g_attn_error[256] = "";

void init_locked() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        // no usable device yet (a CPU-only process that checks arguments or asks for a workspace size): nothing is
        // latched, so that the first call with a device still sets the kernels up
        (void)hipGetLastError();
        return;
    }
    g_num_cus = cus;
    // kernels with more than 48 KB of dynamic LDS need the attribute before their first launch
    int rc = attn_configure_all<f16_t>();
    if (rc == RGD_OK) rc = attn_configure_all<bf16_t>();
    if (rc == RGD_OK) rc = attn_configure_cls<f16_t>();
    if (rc == RGD_OK) rc = attn_configure_cls<bf16_t>();
    if (rc != RGD_OK) {
        g_attn_rc = rc;
        snprintf(g_attn_error, sizeof(g_attn_error), "%s", g_error);
    }
    // the scratch array of rgd_rms_bwd_noalloc on this device; a failure is reported by that entry point, which
    // resolves the address again
    (void)wide_noalloc_setup(nullptr);
    g_error[0] = 0;
    g_init_done.store(1, std::memory_order_release);
}
}  // namespace

void rgd_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

void rgd_ensure_init() {
    if (g_init_done.load(std::memory_order_acquire)) return;
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (!g_init_done.load(std::memory_order_relaxed)) init_locked();
}

int rgd_attn_ready() {
    rgd_ensure_init();
    if (g_attn_rc != RGD_OK) rgd_set_error("attention kernels: set-up failed when the library was initialised: %s", g_attn_error);
    return g_attn_rc;
}

int rgd_num_cus() {
    rgd_ensure_init();
    return g_num_cus;
}

int rgd_launch_status(const char* what, hipError_t e) {
    if (e == hipSuccess) return RGD_OK;
    rgd_set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    // the runtime keeps a failed launch as the thread's last error: taken back here, so that the caller's next
    // check of its own work does not report this one (a launch that succeeded makes no such call)
    (void)hipGetLastError();
    return RGD_ERR_LAUNCH;
}

extern "C" {
int rgd_version(void) { return 3000; }
const char* rgd_last_error(void) { return g_error; }
int rgd_init(void) {
    rgd_ensure_init();
    if (!g_init_done.load(std::memory_order_acquire)) {
        rgd_set_error("rgd_init: no usable device (hipGetDevice or its compute-unit count failed)");
        return RGD_ERR_LAUNCH;
    }
    return rgd_attn_ready();
}
}
