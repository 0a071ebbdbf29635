// Plain device copy with the same access shape as the Hyena kernels (16 bytes per lane, 1 KiB per wavefront
// instruction).  Built into its own small library, libhyena_probe.so: it is the calibration launch for hardware
// traffic counters and the achievable-bandwidth yardstick of the benchmark, not part of the operator ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;

namespace {
__global__ __launch_bounds__(256) void copy_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}
}  // namespace

// 0 on success, -1 for a rejected argument, a positive hipError_t if the launch failed.
extern "C" int hyena_copy_probe(const void* src, void* dst, int64_t nbytes, void* stream) {
    if (!src || !dst || nbytes < 0 || nbytes % 16 != 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return -1;
    const int64_t n16 = nbytes / 16;
    if (n16 == 0) return 0;
    const int64_t nblk = (n16 + 255) / 256;
    if (nblk > 0x7fffffffLL) return -1;
    hipLaunchKernelGGL(copy_probe_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4*)src, (u32x4*)dst, n16);
    return (int)hipGetLastError();
}
