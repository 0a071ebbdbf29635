// Version and error-string entry points of the C ABI.
#include "common.h"

static thread_local char g_err[512] = "";

int hyena_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hyena_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        hyena_fail((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

extern "C" const char* hyena_version(void) { return "hyena-mi355x 0.1 (gfx950)"; }
extern "C" const char* hyena_last_error_string(void) { return g_err; }
