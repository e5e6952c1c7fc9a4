// Error channel, stopwatch and the host-side table initialisers of libint64gemm.so.
#include "gemm.h"
#include "../../include/int64gemm.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <mutex>

namespace zk {

static std::mutex g_err_mutex;
static int g_err_code = kOk;
static char g_err_text[512] = "";

void set_error(int code, const char *fmt, ...)
{
    std::lock_guard<std::mutex> lock(g_err_mutex);
    if (g_err_code != kOk) return;
    g_err_code = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err_text, sizeof(g_err_text), fmt, ap);
    va_end(ap);
    if (getenv("ZK_VERBOSE")) fprintf(stderr, "libint64gemm: %s\n", g_err_text);
}

// Errors that only a kernel can detect travel through pinned host memory: the kernel stores 1 into its flag, and the
// next look at the error channel after that store has landed records the error.
static int *g_deferred = nullptr;
static bool g_deferred_tried = false;
static const char *const kDeferredText[kDeferredCount] = {
    "moe_dispatch: an expert index lies outside [0, E); its entries were left out (they read row 0 in moe_combine)",
};

int *deferred_error_flag(int which)
{
    std::lock_guard<std::mutex> lock(g_err_mutex);
    if (!g_deferred_tried) {
        g_deferred_tried = true;
        if (hipHostMalloc(&g_deferred, kDeferredCount * sizeof(int), hipHostMallocDefault) == hipSuccess) {
            for (int i = 0; i < kDeferredCount; i++) g_deferred[i] = 0;
        } else {
            (void)hipGetLastError();
            g_deferred = nullptr;
        }
    }
    return g_deferred ? g_deferred + which : nullptr;
}

static void take_deferred_errors()
{
    if (!g_deferred) return;
    for (int i = 0; i < kDeferredCount; i++) {
        volatile int *f = g_deferred + i;
        if (*f) { *f = 0; set_error(kBadArgument, "%s", kDeferredText[i]); }
    }
}

bool check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return true;
    set_error(kLaunchFailure, "%s: %s", what, hipGetErrorString(e));
    return false;
}

static hipEvent_t g_t0 = nullptr, g_t1 = nullptr;

}  // namespace zk

extern "C" {

int zk_last_error(void)
{
    zk::take_deferred_errors();
    std::lock_guard<std::mutex> lock(zk::g_err_mutex);
    return zk::g_err_code;
}

const char *zk_last_error_string(void) { return zk::g_err_text; }

void zk_clear_error(void)
{
    std::lock_guard<std::mutex> lock(zk::g_err_mutex);
    zk::g_err_code = zk::kOk;
    zk::g_err_text[0] = 0;
}

size_t zk_workspace_bytes(void)
{
    return zk::gemm_mfma_workspace_bytes(nullptr) + zk::gemm_rows16_workspace_bytes() + zk::act_workspace_bytes();
}

size_t zk_prepared_weights_bytes(void)
{
    size_t prepared = 0;
    (void)zk::gemm_mfma_workspace_bytes(&prepared);
    return prepared;
}

void zk_release_workspace(void)
{
    zk::gemm_mfma_release_workspace();       // waits for the device first
    zk::gemm_rows16_release_workspace();
    zk::act_release_workspace();
}

void zk_reload_env(void)
{
    zk::gemm_mfma_reload_switches();
    zk::gemm_rows16_reload_switches();
}

void zk_timer_start(void)
{
    if (!zk::g_t0) {
        if (hipEventCreate(&zk::g_t0) != hipSuccess || hipEventCreate(&zk::g_t1) != hipSuccess) {
            zk::set_error(zk::kLaunchFailure, "zk_timer_start: hipEventCreate failed");
            return;
        }
    }
    if (hipEventRecord(zk::g_t0, 0) != hipSuccess) zk::set_error(zk::kLaunchFailure, "zk_timer_start: hipEventRecord failed");
}

float zk_timer_stop_ms(void)
{
    if (!zk::g_t0) return -1.0f;
    float ms = -1.0f;
    if (hipEventRecord(zk::g_t1, 0) != hipSuccess || hipEventSynchronize(zk::g_t1) != hipSuccess ||
        hipEventElapsedTime(&ms, zk::g_t0, zk::g_t1) != hipSuccess) {
        zk::set_error(zk::kLaunchFailure, "zk_timer_stop_ms: event timing failed");
        return -1.0f;
    }
    return ms;
}

// The four tables are filled on the host, like the reference's (it passes a CPU tensor's pointer and
// uploads afterwards).  pow() is evaluated in double: the exponent is a float expression promoted to
// double, exactly representable for every i.
void softmax_init_q21(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(std::pow(2.0, (double)(-i) / 256.0) * 2097152.0);
}

void softmax_init_q19(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(std::pow(2.0, (double)(-i) / 256.0) * 524288.0);
}

void silu_init_q25(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(std::pow(2.0, (double)i / 256.0) * 33554432.0);
}

void silu_init_q23(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(std::pow(2.0, (double)i / 256.0) * 8388608.0);
}

}  // extern "C"
