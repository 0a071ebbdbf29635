// Channel-last gated FIR in direct form for float32 and float16 tensors: the (batch, seqlen, groups, group_dim)
// operator of vortex/ops/hyena_se/fwd.py:17-43 for the element types its reference grid runs in
// (vortex/ops/hyena_se/tests/test_fwd.py:25-54: float16 and float32, filters of 4, 32 and 128 taps drawn from N(0, 1)).
//
// float32 inputs cannot go through one bf16 or fp16 MFMA term at that grid's tolerance (1e-2 absolute on outputs whose
// accumulation runs over magnitudes of sqrt(K) ~ 11).  Two float32 forms: the float32 matrix-core kernel at the end of
// this file (16-channel filter groups, K <= 128, no inner bias), and this direct-form kernel for everything else, which
// accumulates in float32 on the vector ALUs with float32 operands: out = x2 * (sum_k h[g][k] * (x1*v)[t-k]), nothing rounded below float32.  float16 tensors take
// the same kernel for shapes the MFMA form does not cover (filter groups that are not multiples of 16 channels,
// unaligned strides), with the roundings of float16 tensor arithmetic: bx = f16(x1*v), z = f16(conv), out = f16(x2*z).
//
// Block = 64 channels x 128 output samples.  bx of the tile and up to 127 samples of history sit in LDS as float32
// [row][channel] (a lane reads its own channel: consecutive banks), the taps as [lag][channel], or as one row where
// the block's channels share a filter; the LDS is sized by the filter length, so short filters fit several blocks per CU.
// Global requests go out in batches with clamped addresses and no branch around them (rows of bx sixteen per thread at
// a time, the output gate's thirty-two at the start), so that a batch costs one memory round trip, not one per row.  A thread owns one
// channel and 32 consecutive outputs; it walks the lags 32 at a time with a 63-sample window of bx in registers, so
// every product has compile-time register operands: 63 + 32 LDS reads per 1024 FMAs.  Filters longer than 128 taps
// run as blocks of 128 lags: the same LDS tile is refilled with the rows 128 samples further back and the next 128
// taps, and the sums carry on in the same registers.  That covers the filter lengths no MFMA kernel is built for
// (vortex/model/engine.py:174-187 takes any length through its FFT, :339-349 any long_fir_threshold), in bfloat16 too.
#include <type_traits>

#include "common.h"

namespace {

constexpr int DT = 128;        // output samples per block
constexpr int DC = 64;         // channels per block
constexpr int DK = 128;        // lags the tap table is padded to

template <typename T> struct ElT;
template <> struct ElT<float> {
    static __device__ __forceinline__ float rnd(float f) { return f; }
};
template <> struct ElT<_Float16> {
    static __device__ __forceinline__ float rnd(float f) { return (float)(_Float16)f; }     // round to nearest even
};
template <> struct ElT<__bf16> {
    static __device__ __forceinline__ float rnd(float f) { return round_bf(f); }
};

template <typename T>
struct ClMapT {                // channel-last operand: (b, t, d) at ptr + b*bs + t*ts + d
    const T* ptr;
    int64_t bs, ts;
};

// NGB = filter groups a block of 64 channels can touch: its tap table is [lag][NGB], read as a broadcast by the lanes
// of one group (one column when groups are multiples of 64 channels, 64 columns with one filter per channel).
template <typename T>
__global__ __launch_bounds__(256) void fir_cl_direct_kernel(ClMapT<T> x1, ClMapT<T> x2, ClMapT<T> v,
                                                            const float* __restrict__ h, int K, int reversed,
                                                            const float* __restrict__ bias, int bias_mode,
                                                            T* __restrict__ out, T* __restrict__ y2_out,
                                                            T* __restrict__ bx_out, int64_t bx_from, int64_t L,
                                                            int64_t D, int dg, int ndb, int ntt, int KP, int NGB,
                                                            int G) {
    // KP = lags per lag block held in LDS: min(K, 128) rounded up to 32.  bx rows: DT + KP - 1; tap rows: KP.
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const bx_lds = smem;
    float* const h_lds = smem + (DT + KP - 1) * DC;
    const int tid = threadIdx.x, c = tid & (DC - 1), tq = tid >> 6;
    const uint32_t bid = blockIdx.x;
    const uint32_t db = bid % (uint32_t)ndb;
    const uint32_t tt = (bid / (uint32_t)ndb) % (uint32_t)ntt;
    const int64_t b = bid / ((uint32_t)ndb * (uint32_t)ntt);
    const int64_t d = (int64_t)db * DC + c;
    const bool ch_ok = d < D;
    const int64_t dcl = ch_ok ? d : D - 1;             // a channel that exists, for requests whose result is dropped
    const int64_t t0 = (int64_t)tt * DT;
    const bool pre = v.ptr != nullptr, post = x2.ptr != nullptr;
    const int nrows = DT + KP - 1;

    const int g0 = (int)(((uint32_t)db * DC) / (uint32_t)dg);              // first filter group of the block
    const int gl = (int)((uint32_t)dcl / (uint32_t)dg) - g0;             // this thread's column of the tap table
    // outputs j = 0..31 at t0 + 32*tq + j; LDS row of output j at lag k of the current lag block: base + j - k
    const int base = (KP - 1) + 32 * tq;
    float acc[32], ucur[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) { acc[j] = 0.f; ucur[j] = 0.f; }
    // the output gate of this thread's 32 samples: requested now, used at the end (clamped addresses, no branch around
    // a request: the thirty-two travel together instead of one round trip each)
    T gate[32];
    if (post) {
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            int64_t t = t0 + 32 * tq + j;
            t = t < L ? t : L - 1;
            gate[j] = x2.ptr[b * x2.bs + t * x2.ts + dcl];
        }
    }
    // lag blocks of KP <= 128: block lb holds lags KP*lb .. KP*lb + KP - 1.  LDS row r holds sample
    // t0 - KP*lb - (KP-1) + r, so that row base + j - k is sample (t0 + 32*tq + j) - (KP*lb + k).
    for (int lb = 0; lb * KP < K; ++lb) {
        if (lb) __syncthreads();                       // the tile of the block before has been consumed
        const int kofs = lb * KP;
        // taps by lag (0 = the current sample), zero from K on
        for (int e = tid; e < KP * NGB; e += 256) {
            const int kk = e / NGB, gc = e - kk * NGB;
            const int k = kofs + kk, gg = g0 + gc;
            const int kc = k < K ? k : K - 1, gcl = gg < G ? gg : G - 1;
            const float val = h[(int64_t)gcl * K + (reversed ? K - 1 - kc : kc)];
            h_lds[e] = (k < K && gg < G) ? val : 0.f;
        }
        // rows of bx, sixteen per thread at a time: every request of a pass goes out before the first is used
        const int64_t tfirst = t0 - kofs - (KP - 1);
        for (int r0 = 0; r0 < nrows; r0 += 64) {
            T xa[16], va[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                int64_t t = tfirst + r0 + tq + 4 * i;
                t = t < 0 ? 0 : (t < L ? t : L - 1);
                xa[i] = x1.ptr[b * x1.bs + t * x1.ts + dcl];
                if (pre) va[i] = v.ptr[b * v.bs + t * v.ts + dcl];
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int r = r0 + tq + 4 * i;
                const int64_t t = tfirst + r;
                float val = (float)xa[i];
                if (pre) val = ElT<T>::rnd(val * (float)va[i]);
                if (!(ch_ok && t >= 0 && t < L)) val = 0.f;
                if (r < nrows) {
                    bx_lds[r * DC + c] = val;
                    if (lb == 0 && bx_out && ch_ok && r >= KP - 1 && t < L && t >= bx_from)
                        bx_out[(b * (L - bx_from) + (t - bx_from)) * D + d] = (T)val;
                }
            }
        }
        __syncthreads();
        if (lb == 0) {
#pragma unroll
            for (int j = 0; j < 32; ++j) ucur[j] = bx_lds[(base + j) * DC + c];      // u at the outputs (gated bias)
        }
        const int kend = (K - kofs < KP) ? K - kofs : KP;
        for (int kb = 0; kb < kend; kb += 32) {
            float win[63];
#pragma unroll
            for (int i = 0; i < 63; ++i) win[i] = bx_lds[(base - kb - 31 + i) * DC + c];      // row >= (KP-1) - (KP-32) - 31 = 0
#pragma unroll
            for (int kk = 0; kk < 32; ++kk) {
                const float hk = h_lds[(kb + kk) * NGB + gl];
#pragma unroll
                for (int j = 0; j < 32; ++j) acc[j] = fmaf(hk, win[j - kk + 31], acc[j]);
            }
        }
    }

    const float bz = bias_mode != HYENA_BIAS_NONE ? bias[dcl] : 0.f;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        const int64_t t = t0 + 32 * tq + j;
        const float u = ucur[j];
        float z;
        switch (bias_mode) {
            case HYENA_BIAS_ADD:        z = ElT<T>::rnd(ElT<T>::rnd(acc[j]) + bz); break;
            case HYENA_BIAS_ADD_FP32:   z = ElT<T>::rnd(acc[j] + bz); break;
            case HYENA_BIAS_GATED_FP32: z = ElT<T>::rnd(fmaf(bz, u, acc[j])); break;
            case HYENA_BIAS_GATED_BF16: z = ElT<T>::rnd(ElT<T>::rnd(acc[j]) + ElT<T>::rnd(bz * u)); break;   // element-type tensor arithmetic
            default:                    z = ElT<T>::rnd(acc[j]);
        }
        if (ch_ok && t < L) {
            const int64_t o = (b * L + t) * D + d;
            if (y2_out) y2_out[o] = (T)z;
            if (post) z = ElT<T>::rnd(z * (float)gate[j]);
            out[o] = (T)z;
        }
    }
}

template <typename T>
int direct_launch(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h, int taps_reversed,
                  const float* bias, int bias_mode, void* out, void* y2_out, void* bx_out, int64_t bx_from, int64_t B,
                  int64_t L, int64_t D, int64_t G, int K, void* stream, const char* who) {
    const int64_t ndb = (D + DC - 1) / DC, ntt = (L + DT - 1) / DT;
    if (B * ndb * ntt > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);
    ClMapT<T> m1 = {(const T*)x1->ptr, x1->batch_stride, x1->time_stride};
    ClMapT<T> m2 = {nullptr, 0, 0}, mv = {nullptr, 0, 0};
    if (x2 && x2->ptr) m2 = {(const T*)x2->ptr, x2->batch_stride, x2->time_stride};
    if (v && v->ptr) mv = {(const T*)v->ptr, v->batch_stride, v->time_stride};
    const int KP = ((K < DK ? K : DK) + 31) / 32 * 32;
    const int64_t dg = D / G;
    // filter groups a block of 64 consecutive channels (starting at a multiple of 64) can touch
    const int NGB = dg % DC == 0 ? 1 : (DC % dg == 0 ? (int)(DC / dg) : (int)((DC - 1) / dg + 2));
    const size_t lds = ((size_t)(DT + KP - 1) * DC + (size_t)KP * NGB) * sizeof(float);
    const dim3 grid((unsigned)(B * ndb * ntt));
    // more than the default dynamic LDS: asked for once per device and instantiation (the attribute belongs to the
    // function as loaded on one device)
    static bool big[64] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev < 0 || !big[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)fir_cl_direct_kernel<T>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024);
        if (e != hipSuccess) return hyena_fail((int)e, "%s: hipFuncSetAttribute: %s", who, hipGetErrorString(e));
        if (dev >= 0) big[dev] = true;
    }
    hipLaunchKernelGGL((fir_cl_direct_kernel<T>), grid, dim3(256), lds, (hipStream_t)stream, m1, m2, mv, h, K,
                       taps_reversed, bias, bias_mode, (T*)out, (T*)y2_out, (T*)bx_out, bx_from, L, D, (int)dg, (int)ndb,
                       (int)ntt, KP, NGB, (int)G);
    return hyena_check_launch(who);
}


// ------------------------------------------------------------------ float32 on the matrix cores
// The same operator for float32 tensors whose filter groups are multiples of 16 channels (the reference grid's are
// 1024 .. 4096 wide), K <= 128, no inner bias: v_mfma_f32_16x16x4_f32 with full float32 operands.  A block takes 64
// channels x 128 outputs; bx = x1*v of the tile and its 128 samples of history sits in LDS as [channel][256 rows]
// (row r = sample t0 - 128 + r; row stride 260 floats, so the sixteen channels x four row quads of a B operand fall
// into 64 different banks).  Wavefront w owns channels 16w .. 16w+15 and all eight 16-sample output blocks.  Output
// block b at lags 0 .. 127 reads rows 16b .. 16b+143, nine groups of 16 rows; group G meets the 16 x 16 Toeplitz
// block A_G[i][j] = h[128 + i - 16G - j], which does not depend on b, so the 36 A operands (nine groups x four
// slices of four rows) stay in registers and every 16-row group of the tile is read from LDS once (one 16-byte read
// per lane: the K index of slice q is rows 4k + q, k = lane / 16) and used by up to eight output blocks: 288 MFMAs
// and 16 LDS reads per wavefront and tile.  Results leave through LDS again (the wavefront's own history rows, dead
// by then) so that the gate and the stores run channel-last with 16 bytes per lane.
constexpr int MRS = 260;       // LDS row stride of one channel (floats)
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float ff4;

// GMIN: row groups below it only meet lags >= K (short filters) and are neither staged nor multiplied
template <int GMIN>
__global__ __launch_bounds__(256, 2) void fir_cl_f32_mfma_kernel(ClMapT<float> x1, ClMapT<float> x2, ClMapT<float> v,
                                                                 const float* __restrict__ h, int K, int reversed,
                                                                 float* __restrict__ out, float* __restrict__ y2_out,
                                                                 float* __restrict__ bx_out, int64_t bx_from, int64_t L,
                                                                 int64_t D, int dg, int ndb, int ntt) {
    extern __shared__ __attribute__((aligned(16))) float smem[];       // [64][MRS]
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bid = blockIdx.x;
    const uint32_t db = bid % (uint32_t)ndb;
    const uint32_t tt = (bid / (uint32_t)ndb) % (uint32_t)ntt;
    const int64_t b = bid / ((uint32_t)ndb * (uint32_t)ntt);
    const int64_t d0 = (int64_t)db * DC, t0 = (int64_t)tt * DT;
    const bool pre = v.ptr != nullptr, post = x2.ptr != nullptr;

    // ---- staging: thread = 4 channels x one row of each pass of 16 rows; four passes of requests in flight
    const int c4 = tid & 15, rr = tid >> 4;
    const int64_t dq = d0 + 4 * c4;
    const bool q_ok = dq < D;                                  // D is a multiple of 4: a quad exists whole or not at all
    const int64_t dql = q_ok ? dq : 0;
    const ff4 zero = {0.f, 0.f, 0.f, 0.f};
    constexpr int NB = 16;                                     // passes of 16 rows requested together: the whole tile in one round trip
#pragma unroll
    for (int p0 = GMIN; p0 < 16; p0 += NB) {
        ff4 xa[NB], va[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (p0 + i >= 16) continue;
            int64_t t = t0 - 128 + 16 * (p0 + i) + rr;
            t = t < 0 ? 0 : (t < L ? t : L - 1);
            xa[i] = *(const ff4*)(x1.ptr + b * x1.bs + t * x1.ts + dql);
            if (pre) va[i] = *(const ff4*)(v.ptr + b * v.bs + t * v.ts + dql);
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (p0 + i >= 16) continue;
            const int r = 16 * (p0 + i) + rr;
            const int64_t t = t0 - 128 + r;
            ff4 val = xa[i];
            if (pre) val = val * va[i];
            if (!(q_ok && t >= 0 && t < L)) val = zero;
#pragma unroll
            for (int e = 0; e < 4; ++e) smem[(4 * c4 + e) * MRS + r] = val[e];
            if (bx_out && q_ok && r >= 128 && t < L && t >= bx_from)
                *(ff4*)(bx_out + (b * (L - bx_from) + (t - bx_from)) * D + dq) = val;
        }
    }
    // the output gate of this thread's eight (row, quad) pieces: requested now, used at the end
    ff4 gate[8];
    if (post) {
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            int64_t t = t0 + 16 * p + rr;
            t = t < L ? t : L - 1;
            gate[p] = *(const ff4*)(x2.ptr + b * x2.bs + t * x2.ts + dql);
        }
    }

    // ---- Toeplitz operands of this wavefront's filter group
    const int n = lane & 15, k = lane >> 4;
    const int64_t dw = d0 + 16 * w;
    const bool w_ok = dw < D;                                  // wave-uniform
    const int g = (int)((uint32_t)(w_ok ? dw : 0) / (uint32_t)dg);
    float A[9][4];
#pragma unroll
    for (int G = 0; G < 9; ++G)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int lag = 128 + n - 16 * G - 4 * k - q;       // output row i = n of the block, input row 16G + 4k + q
            const int lc = lag < 0 ? 0 : (lag < K ? lag : K - 1);
            const float hv = h[(int64_t)g * K + (reversed ? K - 1 - lc : lc)];
            A[G][q] = (lag >= 0 && lag < K) ? hv : 0.f;
        }
    __syncthreads();

    ff4 acc[8];
#pragma unroll
    for (int bb = 0; bb < 8; ++bb) acc[bb] = zero;
    float* const mine = smem + (16 * w + n) * MRS;
    if (w_ok) {
#pragma unroll
        for (int J = GMIN; J < 16; ++J) {
            const ff4 Bq = *(const ff4*)(mine + 16 * J + 4 * k);
#pragma unroll
            for (int bb = 0; bb < 8; ++bb) {
                const int G = J - bb;
                if (G < GMIN || G > 8) continue;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[bb] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[G][q], Bq[q], acc[bb], 0, 0, 0);
            }
        }
        // lane (n, k) holds outputs 16bb + 4k .. + 3 of channel 16w + n: into this channel's history rows, which no
        // other wavefront reads (an LDS read and write of one wavefront complete in order)
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) *(ff4*)(mine + 16 * bb + 4 * k) = acc[bb];
    }
    __syncthreads();

    // ---- channel-last output: the staging layout again (4 channels x one row of each pass)
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const int tl = 16 * p + rr;
        const int64_t t = t0 + tl;
        ff4 z;
#pragma unroll
        for (int e = 0; e < 4; ++e) z[e] = smem[(4 * c4 + e) * MRS + tl];
        if (q_ok && t < L) {
            const int64_t o = (b * L + t) * D + dq;
            if (y2_out) *(ff4*)(y2_out + o) = z;
            if (post) z = z * gate[p];
            *(ff4*)(out + o) = z;
        }
    }
}


// The same arithmetic as fir_cl_f32_mfma_kernel for launches with many tiles along L: a block walks `seg_tiles`
// consecutive 128-output tiles of its 64 channels.  The two 128-row halves of the LDS tile form a ring -- the half
// staged for one tile is the next tile's history, and the half that held the history takes the results on their way
// out and then the next tile's rows -- so every sample is staged once (plus 128 samples at the start of a segment),
// and the next tile's rows are requested ahead of the MFMAs of this one and travel during them.
template <int GMIN>
__global__ __launch_bounds__(256, 2) void fir_cl_f32_ring_kernel(ClMapT<float> x1, ClMapT<float> x2, ClMapT<float> v,
                                                                 const float* __restrict__ h, int K, int reversed,
                                                                 float* __restrict__ out, float* __restrict__ y2_out,
                                                                 float* __restrict__ bx_out, int64_t bx_from, int64_t L,
                                                                 int64_t D, int dg, int ndb, int ntt, int nseg,
                                                                 int seg_tiles) {
    extern __shared__ __attribute__((aligned(16))) float smem[];       // [64][MRS]: rows 0..127 and 128..255 are the ring's halves
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bid = blockIdx.x;
    const uint32_t db = bid % (uint32_t)ndb;
    const uint32_t seg = (bid / (uint32_t)ndb) % (uint32_t)nseg;
    const int64_t b = bid / ((uint32_t)ndb * (uint32_t)nseg);
    const int i0 = (int)seg * seg_tiles;
    const int i1 = i0 + seg_tiles < ntt ? i0 + seg_tiles : ntt;
    if (i0 >= i1) return;                                      // the whole block leaves: no barrier is skipped
    const int64_t d0 = (int64_t)db * DC;
    const bool pre = v.ptr != nullptr, post = x2.ptr != nullptr;
    const int c4 = tid & 15, rr = tid >> 4;
    const int64_t dq = d0 + 4 * c4;
    const bool q_ok = dq < D;
    const int64_t dql = q_ok ? dq : 0;
    const ff4 zero = {0.f, 0.f, 0.f, 0.f};
    const float* const px1 = x1.ptr + b * x1.bs + dql;
    const float* const pxv = pre ? v.ptr + b * v.bs + dql : nullptr;
    const float* const px2 = post ? x2.ptr + b * x2.bs + dql : nullptr;

    const int n = lane & 15, k = lane >> 4;
    const int64_t dw = d0 + 16 * w;
    const bool w_ok = dw < D;
    const int g = (int)((uint32_t)(w_ok ? dw : 0) / (uint32_t)dg);
    float A[9][4];
#pragma unroll
    for (int G = 0; G < 9; ++G)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int lag = 128 + n - 16 * G - 4 * k - q;
            const int lc = lag < 0 ? 0 : (lag < K ? lag : K - 1);
            const float hv = h[(int64_t)g * K + (reversed ? K - 1 - lc : lc)];
            A[G][q] = (lag >= 0 && lag < K) ? hv : 0.f;
        }

    // eight passes of 16 rows: the 128 samples that start at ts
    ff4 xa[8], va[8];
    auto request = [&](const int64_t ts) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            int64_t t = ts + 16 * p + rr;
            t = t < 0 ? 0 : (t < L ? t : L - 1);
            xa[p] = *(const ff4*)(px1 + t * x1.ts);
            if (pre) va[p] = *(const ff4*)(pxv + t * v.ts);
        }
    };
    auto stage = [&](const int64_t ts, const int half, const bool store_bx, const int p_first) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            if (p < p_first) continue;
            const int r = 128 * half + 16 * p + rr;
            const int64_t t = ts + 16 * p + rr;
            ff4 val = xa[p];
            if (pre) val = val * va[p];
            if (!(q_ok && t >= 0 && t < L)) val = zero;
#pragma unroll
            for (int e = 0; e < 4; ++e) smem[(4 * c4 + e) * MRS + r] = val[e];
            if (store_bx && bx_out && q_ok && t < L && t >= bx_from)
                *(ff4*)(bx_out + (b * (L - bx_from) + (t - bx_from)) * D + dq) = val;
        }
    };
    // history of the segment's first tile -> the half that tile does not stage (row groups below GMIN meet no tap)
    request((int64_t)i0 * DT - 128);
    stage((int64_t)i0 * DT - 128, 1, false, GMIN);
    request((int64_t)i0 * DT);

    float* const mine = smem + (16 * w + n) * MRS;
    for (int i = i0; i < i1; ++i) {
        const int64_t t0 = (int64_t)i * DT;
        const int c = (i - i0) & 1;                            // the half this tile's rows go to; its history is in the other
        stage(t0, c, true, 0);
        __syncthreads();
        ff4 gate[8];
        if (post) {
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                int64_t t = t0 + 16 * p + rr;
                t = t < L ? t : L - 1;
                gate[p] = *(const ff4*)(px2 + t * x2.ts);
            }
        }
        if (i + 1 < i1) request(t0 + DT);                      // travels during the MFMAs below

        ff4 acc[8];
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) acc[bb] = zero;
        float* const hist = mine + 128 * (c ^ 1);
        float* const cur = mine + 128 * c;
        if (w_ok) {
#pragma unroll
            for (int J = GMIN; J < 16; ++J) {
                const ff4 Bq = *(const ff4*)((J < 8 ? hist : cur) + 16 * (J & 7) + 4 * k);
#pragma unroll
                for (int bb = 0; bb < 8; ++bb) {
                    const int G = J - bb;
                    if (G < GMIN || G > 8) continue;
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        acc[bb] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[G][q], Bq[q], acc[bb], 0, 0, 0);
                }
            }
            // results into the history half, which is dead now (only this wavefront reads its channels' rows)
#pragma unroll
            for (int bb = 0; bb < 8; ++bb) *(ff4*)(hist + 16 * bb + 4 * k) = acc[bb];
        }
        __syncthreads();
        const int zb = 128 * (c ^ 1);
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int tl = 16 * p + rr;
            const int64_t t = t0 + tl;
            ff4 z;
#pragma unroll
            for (int e = 0; e < 4; ++e) z[e] = smem[(4 * c4 + e) * MRS + zb + tl];
            if (q_ok && t < L) {
                const int64_t o = (b * L + t) * D + dq;
                if (y2_out) *(ff4*)(y2_out + o) = z;
                if (post) z = z * gate[p];
                *(ff4*)(out + o) = z;
            }
        }
        __syncthreads();                                       // the next tile stages its rows over these results
    }
}

// dynamic LDS beyond the default for the ring kernels, once per device
int big_ring_ready(const char* who) {
    static bool big[64] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev >= 0 && big[dev]) return 0;
    const void* fns[4] = {(const void*)fir_cl_f32_ring_kernel<0>, (const void*)fir_cl_f32_ring_kernel<3>,
                          (const void*)fir_cl_f32_ring_kernel<5>, (const void*)fir_cl_f32_ring_kernel<6>};
    for (const void* f : fns) {
        const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(DC * MRS * sizeof(float)));
        if (e != hipSuccess) return hyena_fail((int)e, "%s: hipFuncSetAttribute: %s", who, hipGetErrorString(e));
    }
    if (dev >= 0) big[dev] = true;
    return 0;
}

int f32_mfma_launch(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h, int taps_reversed,
                    void* out, void* y2_out, void* bx_out, int64_t bx_from, int64_t B, int64_t L, int64_t D, int64_t G,
                    int K, void* stream, const char* who) {
    const int64_t ndb = (D + DC - 1) / DC, ntt = (L + DT - 1) / DT;
    if (B * ndb * ntt > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);
    ClMapT<float> m1 = {(const float*)x1->ptr, x1->batch_stride, x1->time_stride};
    ClMapT<float> m2 = {nullptr, 0, 0}, mv = {nullptr, 0, 0};
    if (x2 && x2->ptr) m2 = {(const float*)x2->ptr, x2->batch_stride, x2->time_stride};
    if (v && v->ptr) mv = {(const float*)v->ptr, v->batch_stride, v->time_stride};
    const size_t lds = (size_t)DC * MRS * sizeof(float);
    static bool big[64] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev < 0 || !big[dev]) {
        const void* fns[4] = {(const void*)fir_cl_f32_mfma_kernel<0>, (const void*)fir_cl_f32_mfma_kernel<3>,
                              (const void*)fir_cl_f32_mfma_kernel<5>, (const void*)fir_cl_f32_mfma_kernel<6>};
        for (const void* f : fns) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return hyena_fail((int)e, "%s: hipFuncSetAttribute: %s", who, hipGetErrorString(e));
        }
        if (dev >= 0) big[dev] = true;
    }
    // row group G meets lags 113 - 16G .. 143 - 16G: groups with 113 - 16G >= K hold no tap
    const int gz = K <= 113 ? (113 - K) / 16 + 1 : 0;           // all-zero groups ahead of the first live one
    // many tiles along L: blocks that walk a segment of them (about two blocks per CU, at least four tiles each)
    {
        const int64_t rows = B * ndb;
        int64_t nseg = (512 + rows - 1) / rows;
        nseg = nseg < 1 ? 1 : (nseg > ntt ? ntt : nseg);
        int64_t seg_tiles = (ntt + nseg - 1) / nseg;
        if (seg_tiles < 4) seg_tiles = ntt < 4 ? ntt : 4;
        nseg = (ntt + seg_tiles - 1) / seg_tiles;
        const int64_t x = hyena_override(HYENA_OV_CL_F32_MFMA);
        // (short filters skip most of the history in the one-tile form, which then measured 5 % faster: 219 against 231 us
        // at B = 2, L = 8192, D = 4096, K = 4; at K = 128 the ring takes 267 against 315 us)
        if ((x == 2 || (x < 0 && seg_tiles >= 4 && gz < 5)) && x != 1) {
            if (int rc = big_ring_ready(who)) return rc;
            const dim3 rgrid((unsigned)(rows * nseg));
#define F32_RING(GM)                                                                                                \
    hipLaunchKernelGGL(fir_cl_f32_ring_kernel<GM>, rgrid, dim3(256), lds, (hipStream_t)stream, m1, m2, mv, h, K,     \
                       taps_reversed, (float*)out, (float*)y2_out, (float*)bx_out, bx_from, L, D, (int)(D / G), (int)ndb, \
                       (int)ntt, (int)nseg, (int)seg_tiles)
            if (gz >= 6) F32_RING(6); else if (gz >= 5) F32_RING(5); else if (gz >= 3) F32_RING(3); else F32_RING(0);
#undef F32_RING
            return hyena_check_launch(who);
        }
    }
    const dim3 grid((unsigned)(B * ndb * ntt));
#define F32_GO(GM)                                                                                                  \
    hipLaunchKernelGGL(fir_cl_f32_mfma_kernel<GM>, grid, dim3(256), lds, (hipStream_t)stream, m1, m2, mv, h, K,       \
                       taps_reversed, (float*)out, (float*)y2_out, (float*)bx_out, bx_from, L, D, (int)(D / G), (int)ndb, \
                       (int)ntt)
    if (gz >= 6) F32_GO(6); else if (gz >= 5) F32_GO(5); else if (gz >= 3) F32_GO(3); else F32_GO(0);
#undef F32_GO
    return hyena_check_launch(who);
}

// whether the matrix-core form takes a float32 launch: 16-channel filter groups, at most 128 taps, no inner bias, and
// 16-byte pieces of four channels everywhere
bool f32_mfma_ok(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, int bias_mode, const void* out,
                 const void* y2_out, const void* bx_out, int64_t D, int64_t G, int K) {
    auto cl4 = [](const hyena_cl* c) {
        return !c || !c->ptr || ((((uintptr_t)c->ptr) & 15) == 0 && c->batch_stride % 4 == 0 && c->time_stride % 4 == 0);
    };
    return K >= 1 && K <= 128 && (D / G) % 16 == 0 && bias_mode == HYENA_BIAS_NONE && cl4(x1) && cl4(x2) && cl4(v) &&
           !((((uintptr_t)out) | ((uintptr_t)y2_out) | ((uintptr_t)bx_out)) & 15);
}

}  // namespace

// Direct-form launch for channel-last tensors of any of the three element types, any K >= 1; arguments as
// hyena_fir_cl_fwd_dtype, already validated by the caller.
int hyena_fir_cl_direct(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h, int taps_reversed,
                        const float* bias, int bias_mode, void* out, void* y2_out, void* bx_out, int64_t bx_from,
                        int64_t B, int64_t L, int64_t D, int64_t G, int K, int dtype, void* stream, const char* who) {
    if (dtype == HYENA_DTYPE_F32 && hyena_override(HYENA_OV_CL_F32_MFMA) != 0 &&
        f32_mfma_ok(x1, x2, v, bias_mode, out, y2_out, bx_out, D, G, K))
        return f32_mfma_launch(x1, x2, v, h, taps_reversed, out, y2_out, bx_out, bx_from, B, L, D, G, K, stream, who);
    if (dtype == HYENA_DTYPE_F32)
        return direct_launch<float>(x1, x2, v, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D,
                                    G, K, stream, who);
    if (dtype == HYENA_DTYPE_BF16)
        return direct_launch<__bf16>(x1, x2, v, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D,
                                     G, K, stream, who);
    return direct_launch<_Float16>(x1, x2, v, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D, G,
                                   K, stream, who);
}
