// Host-side plumbing of the C ABI: version, per-thread error text, launch checks.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "dagx_common.h"

namespace dagx {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return DAGX_ERR_LAUNCH;
    }
    return DAGX_OK;
}

static std::atomic<int> g_log_domain{-1};   // -1: not decided yet (environment), 0: tile kernels, 1: log-domain kernels only

bool force_log_domain() {
    int v = g_log_domain.load(std::memory_order_relaxed);
    if (v < 0) {
        const char *e = getenv("DAGX_EXACT_SWEEP");
        const int from_env = (e && e[0] == '1') ? 1 : 0;
        int expected = -1;
        g_log_domain.compare_exchange_strong(expected, from_env);   // a concurrent dagx_force_log_domain() wins
        v = g_log_domain.load(std::memory_order_relaxed);
    }
    return v == 1;
}

}  // namespace dagx

extern "C" int dagx_force_log_domain(int on) {
    const int before = dagx::force_log_domain() ? 1 : 0;
    dagx::g_log_domain.store(on ? 1 : 0);
    return before;
}

extern "C" const char *dagx_version(void) { return "dagx 0.1 (gfx950)"; }
extern "C" const char *dagx_last_error(void) { return dagx::g_error; }
