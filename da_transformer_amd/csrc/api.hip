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

// -1: not decided yet (environment), 0: tile kernels, 1: log-domain kernels only, 2: as 0, but dagx_best_alignment treats every
// sample as one the tile pipeline gave up on (so that the route of such samples can be tested without making a pipeline fail)
static std::atomic<int> g_log_domain{-1};

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

bool redo_every_sample() { return g_log_domain.load(std::memory_order_relaxed) == 2; }

// -1: not decided yet (environment), 0: dagx_loss_fwd starts with the float32 tile sweeps, 1: with the float64 ones
static std::atomic<int> g_float64_first{-1};

bool float64_first() {
    int v = g_float64_first.load(std::memory_order_relaxed);
    if (v < 0) {
        const char *e = getenv("DAGX_FLOAT64_FIRST");
        int expected = -1;
        g_float64_first.compare_exchange_strong(expected, (e && e[0] == '1') ? 1 : 0);   // a concurrent setter wins
        v = g_float64_first.load(std::memory_order_relaxed);
    }
    return v == 1;
}

}  // namespace dagx

extern "C" int dagx_force_log_domain(int on) {
    dagx::force_log_domain();   // (settles the environment's say first)
    const int before = dagx::g_log_domain.load();
    dagx::g_log_domain.store(on == 2 ? 2 : on ? 1 : 0);
    return before;
}

extern "C" int dagx_loss_float64_first(int on) {
    const int before = dagx::float64_first() ? 1 : 0;   // (settles the environment's say first)
    dagx::g_float64_first.store(on ? 1 : 0);
    return before;
}

extern "C" const char *dagx_version(void) { return "dagx 0.3 (gfx950)"; }
extern "C" const char *dagx_last_error(void) { return dagx::g_error; }
