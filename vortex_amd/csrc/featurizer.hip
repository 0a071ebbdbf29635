// Featurizer short FIR: depthwise causal FIR (K <= 8) over the 3D channels of the
// input projection, fused with the layout change the caller needs.  Input is
// channel-last [B][L][C] (what the dense projection writes), output is
// sequence-last [B][C][L] (what the Hyena operators read), so the transpose that
// vortex/model/engine.py:189-190 does as a separate permute never touches HBM.
// Reads are coalesced along C, writes along L; the transpose happens in LDS.
#include "common.h"

namespace {

constexpr int TT = 128;      // samples per tile
constexpr int TC = 128;      // channels per tile
constexpr int TBP = 136;     // row stride (elements) of the transposed LDS tile: 272 B

template <int K, bool BIAS>
__global__ __launch_bounds__(256) void featurizer_kernel(const bf16_t* __restrict__ u, int64_t u_bs, int64_t u_ts,
                                                         const float* __restrict__ taps, int dg,
                                                         const float* __restrict__ bias, bf16_t* __restrict__ z,
                                                         int64_t C, int64_t L, int interleave3, int pad) {
    // L counts output columns; column t holds input sample t - pad, the first `pad` columns are zeros
    constexpr int ROWS = TT + K - 1;
    constexpr int A_ELEMS = ROWS * TC, B_ELEMS = TC * TBP;
    __shared__ __attribute__((aligned(16))) bf16_t lds[A_ELEMS > B_ELEMS ? A_ELEMS : B_ELEMS];
    const int tid = threadIdx.x;
    const int64_t c0 = (int64_t)blockIdx.x * TC, t0 = (int64_t)blockIdx.y * TT, b = blockIdx.z;
    const bf16_t* ub = u + b * u_bs;

    // phase 1: [time][channel] tile, rows t0-(K-1) .. t0+TT-1
    for (int e = tid; e < ROWS * (TC / 8); e += 256) {
        const int row = e / (TC / 8), lc = e - row * (TC / 8);
        const int64_t t = t0 - (K - 1) + row - pad, c = c0 + 8 * lc;
        u32x4 q = {0, 0, 0, 0};
        if (t >= 0 && t < L - pad && c < C) q = *(const u32x4*)(ub + t * u_ts + c);
        *(u32x4*)(lds + row * TC + 8 * lc) = q;
    }
    __syncthreads();

    // phase 2: this thread filters channels 2*cp, 2*cp+1 over 32 samples
    const int cp = tid & 63, tg = tid >> 6;
    const int64_t ch = c0 + 2 * cp;
    float w0[K], w1[K];
    const bool chan_ok = ch < C;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        w0[k] = chan_ok ? taps[(ch / dg) * K + k] : 0.f;
        w1[k] = chan_ok ? taps[((ch + 1) / dg) * K + k] : 0.f;
    }
    float b0 = 0.f, b1 = 0.f;
    if (BIAS && chan_ok) { b0 = bias[ch]; b1 = bias[ch + 1]; }
    float win0[K], win1[K];
    const uint32_t* col = (const uint32_t*)(lds) + cp;          // dword = channel pair, row stride TC/2 dwords
#pragma unroll
    for (int k = 0; k < K - 1; ++k) {
        const uint32_t p = col[(tg * 32 + k) * (TC / 2)];
        win0[k] = bf_lo(p);
        win1[k] = bf_hi(p);
    }
    uint32_t o0[16], o1[16];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const uint32_t p = col[(tg * 32 + i + K - 1) * (TC / 2)];
        win0[K - 1] = bf_lo(p);
        win1[K - 1] = bf_hi(p);
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            a0 = fmaf(w0[k], win0[k], a0);
            a1 = fmaf(w1[k], win1[k], a1);
        }
#pragma unroll
        for (int k = 0; k < K - 1; ++k) {
            win0[k] = win0[k + 1];
            win1[k] = win1[k + 1];
        }
        a0 = round_bf(a0);
        a1 = round_bf(a1);
        if (BIAS) {
            const bool live = t0 + tg * 32 + i >= pad;       // padding columns stay zero, bias or not
            a0 = live ? a0 + b0 : 0.f;
            a1 = live ? a1 + b1 : 0.f;
        }
        if (i & 1) {
            o0[i >> 1] = pack_bf2(__uint_as_float(o0[i >> 1]), a0);
            o1[i >> 1] = pack_bf2(__uint_as_float(o1[i >> 1]), a1);
        } else {
            o0[i >> 1] = __float_as_uint(a0);
            o1[i >> 1] = __float_as_uint(a1);
        }
    }
    __syncthreads();                     // every read of the [time][channel] tile is done

    // transposed tile [channel][time]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const u32x4 v0 = {o0[4 * q], o0[4 * q + 1], o0[4 * q + 2], o0[4 * q + 3]};
        const u32x4 v1 = {o1[4 * q], o1[4 * q + 1], o1[4 * q + 2], o1[4 * q + 3]};
        *(u32x4*)(lds + (2 * cp) * TBP + tg * 32 + 8 * q) = v0;
        *(u32x4*)(lds + (2 * cp + 1) * TBP + tg * 32 + 8 * q) = v1;
    }
    __syncthreads();

    // phase 3: coalesced stores along L
    const int oc = tid & 15, r0 = tid >> 4;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int r = r0 + 16 * k;
        const int64_t c = c0 + r, t = t0 + 8 * oc;
        // interleave3: channel 3j+i of the projection lands in row i*C/3 + j (vortex/model/utils.py:26-38)
        const int64_t row = interleave3 ? (c % 3) * (C / 3) + c / 3 : c;
        if (c < C && t < L) *(u32x4*)(z + (b * C + row) * L + t) = *(const u32x4*)(lds + r * TBP + 8 * oc);
    }
}

}  // namespace

extern "C" int hyena_featurizer_fwd(const void* u, int64_t u_batch_stride, int64_t u_time_stride, const float* taps,
                                    const float* bias, int interleave3, void* out, int64_t B, int64_t L, int64_t C,
                                    int64_t G, int K, int front_pad, void* stream) {
    if (!u || !taps || !out) return hyena_fail(HYENA_EINVAL, "hyena_featurizer_fwd: u, taps and out are required");
    if (B < 0 || L < 0 || C <= 0 || G <= 0 || C % G != 0)
        return hyena_fail(HYENA_EINVAL, "hyena_featurizer_fwd: bad sizes B=%lld L=%lld C=%lld G=%lld", (long long)B,
                          (long long)L, (long long)C, (long long)G);
    if (K < 2 || K > 8) return hyena_fail(HYENA_ENOSUP, "hyena_featurizer_fwd: K=%d outside 2..8", K);
    if (front_pad < 0 || front_pad > 7) return hyena_fail(HYENA_EINVAL, "hyena_featurizer_fwd: front_pad %d outside 0..7", front_pad);
    if (L > 0) L += front_pad;            // from here on L counts output columns
    if (C % 8 != 0 || L % 8 != 0 || u_batch_stride % 8 != 0 || u_time_stride % 8 != 0 || ((uintptr_t)u & 15) ||
        ((uintptr_t)out & 15))
        return hyena_fail(HYENA_EALIGN, "hyena_featurizer_fwd: C, L + front_pad, strides must be multiples of 8, pointers 16-byte aligned");
    if (interleave3 && C % 3 != 0) return hyena_fail(HYENA_EINVAL, "hyena_featurizer_fwd: interleave needs C %% 3 == 0");
    if (B > 65535 || (L + TT - 1) / TT > 65535) return hyena_fail(HYENA_EINVAL, "hyena_featurizer_fwd: grid too large");
    if (B == 0 || L == 0) return 0;
    dim3 grid((unsigned)((C + TC - 1) / TC), (unsigned)((L + TT - 1) / TT), (unsigned)B);
    hipStream_t s = (hipStream_t)stream;
    const int dg = (int)(C / G);
#define FZ_CASE(KK)                                                                                                \
    case KK:                                                                                                        \
        if (bias)                                                                                                   \
            hipLaunchKernelGGL((featurizer_kernel<KK, true>), grid, dim3(256), 0, s, (const bf16_t*)u,              \
                               u_batch_stride, u_time_stride, taps, dg, bias, (bf16_t*)out, C, L, interleave3, front_pad);                  \
        else                                                                                                        \
            hipLaunchKernelGGL((featurizer_kernel<KK, false>), grid, dim3(256), 0, s, (const bf16_t*)u,             \
                               u_batch_stride, u_time_stride, taps, dg, bias, (bf16_t*)out, C, L, interleave3, front_pad);                  \
        break;
    switch (K) { FZ_CASE(2) FZ_CASE(3) FZ_CASE(4) FZ_CASE(5) FZ_CASE(6) FZ_CASE(7) FZ_CASE(8) }
#undef FZ_CASE
    return hyena_check_launch("hyena_featurizer_fwd");
}
