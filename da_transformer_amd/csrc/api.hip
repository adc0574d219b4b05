// Host-side plumbing of the C ABI: version, per-thread error text, launch checks.
#include <stdarg.h>
#include <stdio.h>

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

}  // namespace dagx

extern "C" const char *dagx_version(void) { return "dagx 0.1 (gfx950)"; }
extern "C" const char *dagx_last_error(void) { return dagx::g_error; }
