// Version and error-string entry points of the C ABI.
#include <atomic>
#include <string.h>

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

// Launch-shape overrides: process-wide, set explicitly through the C ABI (nothing is read from the environment).
namespace {
const char* const kOverrideNames[HYENA_OV_COUNT] = {"mr_nseg", "cl_nseg", "se_nt", "mr_nt", "li_nt", "cl_nt",
                                                    "li_cpw", "li_coop", "li_xcd", "cl_ns", "cl_f32_mfma"};
std::atomic<int64_t> g_override[HYENA_OV_COUNT] = {{-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}};
}  // namespace

int64_t hyena_override(int id) { return g_override[id].load(std::memory_order_relaxed); }

extern "C" int hyena_set_launch_override(const char* name, int64_t value) {
    if (!name) return hyena_fail(HYENA_EINVAL, "hyena_set_launch_override: null name");
    for (int i = 0; i < HYENA_OV_COUNT; ++i)
        if (strcmp(name, kOverrideNames[i]) == 0) {
            g_override[i].store(value < 0 ? -1 : value, std::memory_order_relaxed);
            return 0;
        }
    return hyena_fail(HYENA_EINVAL, "hyena_set_launch_override: unknown name '%s'", name);
}
