// Access-pattern probes: kernels that move the bytes of a gated long convolution (3 reads + 1 write of 2 bytes per
// element over D rows of L samples, 16 bytes per lane, non-temporal) with no arithmetic, in the access orders a
// scan along L can or cannot take.  They measure what the memory system delivers for each order, which is the
// ceiling a kernel with that order can reach.  Part of libhyena_probe.so (measurement aid, not the operator ABI).
//
//   pattern 0  whole rows:  one block (4 wavefronts) per set of R rows walks them from start to end, 2048 samples per
//              block step, two steps prefetched -- the order a one-pass scan with a carried state imposes
//   pattern 1  segments:    one block per (row set, segment of `seg` samples), segments of a row set on consecutive
//              blocks -- the order of a kernel whose blocks are independent (Hyena-MR); a carried state would have
//              to be handed from block to block
//   pattern 2  one row per block:  the four wavefronts of a block walk ONE row together, 4 KiB each per step
//              (16 KiB of the row per block step, two steps prefetched); `seg` = blocks resident per CU (1, 2, 4
//              or 8, enforced with an LDS request), i.e. 256 .. 2048 rows in flight on the chip -- the order of a
//              scan whose block shares one row and passes the state between its wavefronts
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef unsigned short bf16_t;

namespace {
constexpr int R = 4, PF = 2;

__device__ __forceinline__ u32x4 ldnt(const bf16_t* p) { return __builtin_nontemporal_load((const u32x4*)p); }
__device__ __forceinline__ void stnt(bf16_t* p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4*)p); }

// unit u of this block -> element offset of row r (or -1 when the unit does not exist)
struct Walk {
    int64_t L, nsets, seg; int nseg; int64_t nunits;
    int xcd;       // != 0: XCD x (block id mod 8) takes the x-th eighth of the block order instead of every eighth block
    __device__ __forceinline__ uint32_t block() const {
        const uint32_t bid = blockIdx.x;
        return (xcd && (gridDim.x & 7u) == 0) ? (bid & 7u) * (gridDim.x >> 3) + (bid >> 3) : bid;
    }
    template <int PATTERN>
    __device__ __forceinline__ int64_t at(int64_t u, int w, int lane) const {     // row 0 of the unit; row r is r*L further
        int64_t set, t;                                            // 32-bit index arithmetic (64-bit division is emulated)
        const uint32_t bid = block(), uu = (uint32_t)u;
        if (PATTERN == 0) { set = bid; t = (int64_t)uu * 2048; }
        else { set = bid / (uint32_t)nseg; t = (int64_t)(bid % (uint32_t)nseg) * seg + (int64_t)uu * 2048; }
        return set * R * L + t + 512 * w + lane * 8;
    }
};

template <int PATTERN>
__global__ __launch_bounds__(256) void stream_probe_kernel(const bf16_t* a, const bf16_t* b, const bf16_t* c, bf16_t* o,
                                                           Walk wk) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    u32x4 x[PF][R], y[PF][R], z[PF][R];
    int64_t cur[PF];                                               // offset of the unit held in each register stage
#pragma unroll
    for (int p = 0; p < PF; ++p) {
        cur[p] = p < wk.nunits ? wk.at<PATTERN>(p, w, lane) : -1;
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (cur[p] >= 0) { const int64_t t = cur[p] + r * wk.L; x[p][r] = ldnt(a + t); y[p][r] = ldnt(b + t); z[p][r] = ldnt(c + t); }
    }
    // Rotations in which every unit and every refill exists run without a branch around any memory instruction: only
    // then can the compiler count the younger requests that may still be in flight when a stage is consumed; with the
    // tests of the loop below around them it waits for all outstanding requests at every step, which makes the
    // prefetch depth meaningless.  (One wait for everything first: the prologue's requests were conditional.)
    int64_t u0 = 0;
    __builtin_amdgcn_s_waitcnt(0x0F70);                            // vmcnt(0)
    for (; u0 + 2 * PF <= wk.nunits; u0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
            const int64_t t0 = cur[p], tn0 = wk.at<PATTERN>(u0 + p + PF, w, lane);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                stnt(o + t0 + r * wk.L, x[p][r] ^ y[p][r] ^ z[p][r]);
                const int64_t tn = tn0 + r * wk.L;
                x[p][r] = ldnt(a + tn); y[p][r] = ldnt(b + tn); z[p][r] = ldnt(c + tn);
            }
            cur[p] = tn0;
            __syncthreads();
        }
    }
    for (; u0 < wk.nunits; u0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
            const int64_t u = u0 + p;
            if (u >= wk.nunits) break;
            const int64_t t0 = cur[p], tn0 = u + PF < wk.nunits ? wk.at<PATTERN>(u + PF, w, lane) : -1;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (t0 >= 0) stnt(o + t0 + r * wk.L, x[p][r] ^ y[p][r] ^ z[p][r]);
                if (tn0 >= 0) { const int64_t tn = tn0 + r * wk.L; x[p][r] = ldnt(a + tn); y[p][r] = ldnt(b + tn); z[p][r] = ldnt(c + tn); }
            }
            cur[p] = tn0;
            __syncthreads();      // the wavefronts of a block stay together, as a carried state would force
        }
    }
}
// pattern 2: block = one row, wavefront w takes samples [2048 w, 2048 w + 2048) of each 8192-sample block step
__global__ __launch_bounds__(256) void row_probe_kernel(const bf16_t* a, const bf16_t* b, const bf16_t* c, bf16_t* o, int64_t L,
                                                        int xcd) {
    extern __shared__ char occupancy_limit[];
    constexpr int K = 4;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t step = 4 * K * 512, nsteps = L / step;
    const uint32_t bid = (xcd && (gridDim.x & 7u) == 0) ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const int64_t base = (int64_t)bid * L + (int64_t)w * K * 512 + lane * 8;
    u32x4 x[PF][K], y[PF][K], z[PF][K];
#pragma unroll
    for (int p = 0; p < PF; ++p)
#pragma unroll
        for (int j = 0; j < K; ++j)
            if (p < nsteps) { const int64_t t = base + p * step + j * 512; x[p][j] = ldnt(a + t); y[p][j] = ldnt(b + t); z[p][j] = ldnt(c + t); }
    int64_t u0 = 0;
    __builtin_amdgcn_s_waitcnt(0x0F70);                            // vmcnt(0); whole rotations as in stream_probe_kernel
    for (; u0 + 2 * PF <= nsteps; u0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int64_t t = base + (u0 + p) * step + j * 512, tn = t + PF * step;
                stnt(o + t, x[p][j] ^ y[p][j] ^ z[p][j]);
                x[p][j] = ldnt(a + tn); y[p][j] = ldnt(b + tn); z[p][j] = ldnt(c + tn);
            }
            __syncthreads();
        }
    }
    for (; u0 < nsteps; u0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
            const int64_t u = u0 + p;
            if (u >= nsteps) break;
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int64_t t = base + u * step + j * 512;
                stnt(o + t, x[p][j] ^ y[p][j] ^ z[p][j]);
                if (u + PF < nsteps) { const int64_t tn = t + PF * step; x[p][j] = ldnt(a + tn); y[p][j] = ldnt(b + tn); z[p][j] = ldnt(c + tn); }
            }
            __syncthreads();      // the wavefronts of a block stay together, as a state passed between them would force
        }
    }
}
}  // namespace

// a, b, c, o: D rows of L bf16 samples each (contiguous); D % 4 == 0, L % 2048 == 0.
// pattern + 8: the same order with XCD x (block id mod 8) taking the x-th eighth of the blocks.
// pattern 0: seg ignored.  pattern 1: seg a multiple of 2048 dividing L.  pattern 2: seg = blocks per CU (1, 2, 4, 8), L % 8192 == 0.
// 0 on success, -1 for a rejected argument, a positive hipError_t if the launch failed.
extern "C" int hyena_stream_probe(const void* a, const void* b, const void* c, void* o, int64_t D, int64_t L, int pattern,
                                  int64_t seg, void* stream) {
    const int xcd = pattern >= 0 ? (pattern >> 3) & 1 : 0;         // pattern + 8: the XCD-contiguous block order
    if (pattern >= 0) pattern &= ~8;
    if (!a || !b || !c || !o || D <= 0 || D % R || L <= 0 || L % 2048 || pattern < 0 || pattern > 2) return -1;
    Walk wk = {};
    wk.xcd = xcd;
    wk.L = L; wk.nsets = D / R;
    int64_t grid;
    if (pattern == 0) { wk.nunits = L / 2048; grid = wk.nsets; }
    else if (pattern == 1) {
        if (seg <= 0 || seg % 2048 || L % seg) return -1;
        wk.seg = seg; wk.nseg = (int)(L / seg); wk.nunits = seg / 2048; grid = wk.nsets * wk.nseg;
    }
    else {
        if (L % 8192 || (seg != 1 && seg != 2 && seg != 4 && seg != 8) || D > 0x7fffffffLL) return -1;
        const size_t lds = seg == 1 ? 100000 : seg == 2 ? 70000 : seg == 4 ? 36000 : 0;      // of 160 KiB per CU
        hipLaunchKernelGGL(row_probe_kernel, dim3((unsigned)D), dim3(256), lds, (hipStream_t)stream, (const bf16_t*)a,
                           (const bf16_t*)b, (const bf16_t*)c, (bf16_t*)o, L, xcd);
        return (int)hipGetLastError();
    }
    if (grid > 0x7fffffffLL) return -1;
#define GO(P) hipLaunchKernelGGL(stream_probe_kernel<P>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)a, \
                              (const bf16_t*)b, (const bf16_t*)c, (bf16_t*)o, wk)
    if (pattern == 0) GO(0); else GO(1);
#undef GO
    return (int)hipGetLastError();
}
