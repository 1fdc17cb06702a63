// Host-side plumbing shared by the entry points: version, thread-local error text, launch check.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace kernl {

static thread_local char g_error[512] = {0};

int set_error(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(KERNL_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return KERNL_OK;
}

}  // namespace kernl

extern "C" int kernl_version(void) { return 0 * 10000 + 1 * 100 + 0; }

extern "C" const char *kernl_last_error_string(void) { return kernl::g_error; }
