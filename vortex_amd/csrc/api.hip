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

// Plain device copy with the same access shape as the Hyena kernels (16 bytes per lane,
// 1 KiB per wavefront instruction).  Used to calibrate hardware traffic counters and as the
// achievable-bandwidth yardstick next to the kernels' own figures.
namespace {
__global__ __launch_bounds__(256) void copy_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}
}  // namespace

extern "C" int hyena_copy_probe(const void* src, void* dst, int64_t nbytes, void* stream) {
    if (!src || !dst || nbytes < 0 || nbytes % 16 != 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
        return hyena_fail(HYENA_EINVAL, "hyena_copy_probe: need 16-byte aligned pointers and a multiple of 16 bytes");
    const int64_t n16 = nbytes / 16;
    if (n16 == 0) return 0;
    const int64_t nblk = (n16 + 255) / 256;
    if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "hyena_copy_probe: too large");
    hipLaunchKernelGGL(copy_probe_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4*)src, (u32x4*)dst, n16);
    return hyena_check_launch("hyena_copy_probe");
}
