// Cached decode step: FIR over a ring-buffer cache and the modal IIR state
// update, each fused with the gating multiplies.  Both are HBM-bound: the FIR
// step has to read its whole cache once per token, but it writes back one slot
// instead of shifting the cache as vortex/model/engine.py:443-447 does.
#include "common.h"

namespace {

// ---------------------------------------------------------------- FIR step
// Block = NSG wavefronts over the same 512 channels; wavefront sg handles cache
// slots sg, sg+NSG, ... so every load instruction reads 1 KiB of one slot row.
// NSG = 8 for deep caches (enough loads in flight to cover HBM latency), 2 for shallow ones.
// Ring layout [B][R][D]: channels contiguous, so the slot written back is one
// coalesced row per batch element.
template <bool PRE, bool POST, int BIAS, bool GROUPED, int NSG>
__global__ __launch_bounds__(64 * NSG) void fir_step_kernel(const bf16_t* __restrict__ x1, const bf16_t* __restrict__ x2,
                                                       const bf16_t* __restrict__ v, int64_t in_bs,
                                                       bf16_t* __restrict__ ring, int R, int pos,
                                                       const float* __restrict__ w, const float* __restrict__ bias,
                                                       bf16_t* __restrict__ out, int64_t out_bs, int64_t D, int dg) {
    extern __shared__ float smem[];
    const int tid = threadIdx.x, oc = tid & 63, sg = tid >> 6;
    const int64_t dblk = (int64_t)blockIdx.x * 512;
    const int64_t d0 = dblk + oc * 8;
    const int64_t b = blockIdx.y;
    const bool live = d0 < D;
    const int W = R + 1;

    const int ng = GROUPED ? (512 / dg) : 0;
    float* wl = smem;                       // [W][ng]  taps of the block's groups, transposed
    float* red = smem + (GROUPED ? W * ng : 0);   // [NSG-1][64][8]
    const int gl = GROUPED ? (oc * 8) / dg : 0;
    constexpr int UF = 8;                   // cache slots in flight per lane
    const bf16_t* rb = ring + (b * R) * D + d0;
    const u32x4 zero4 = {0, 0, 0, 0};

    auto load_batch = [&](int i, u32x4* q) {
#pragma unroll
        for (int k = 0; k < UF; ++k) {
            const int ii = i + NSG * k;
            int s = pos + ii;
            if (s >= R) s -= R;
            q[k] = (live && ii < R) ? *(const u32x4*)(rb + (int64_t)s * D) : zero4;
        }
    };
    float acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = 0.f;
    auto fma_batch = [&](int i, const u32x4* q) {
#pragma unroll
        for (int k = 0; k < UF; ++k) {
            int ii = i + NSG * k;
            if (ii >= R) ii = R - 1;        // the slot was loaded as zeros; any finite tap will do
            if (GROUPED) {
                const float t = wl[ii * ng + gl];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[2 * j] = fmaf(t, bf_lo(q[k][j]), acc[2 * j]);
                    acc[2 * j + 1] = fmaf(t, bf_hi(q[k][j]), acc[2 * j + 1]);
                }
            } else if (live) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[2 * j] = fmaf(w[(d0 + 2 * j) * W + ii], bf_lo(q[k][j]), acc[2 * j]);
                    acc[2 * j + 1] = fmaf(w[(d0 + 2 * j + 1) * W + ii], bf_hi(q[k][j]), acc[2 * j + 1]);
                }
            }
        }
    };

    // the first batch of cache reads goes out before the tap table is staged, so HBM is busy from the start
    u32x4 q0[UF];
    load_batch(sg, q0);
    if (GROUPED) {
        const int64_t g0 = dblk / dg;
        const int64_t gmax = (D + dg - 1) / dg;
        if ((W & 3) == 0) {
            for (int e = tid; e < (W / 4) * ng; e += 64 * NSG) {
                const int gl2 = e / (W / 4), i4 = (e - gl2 * (W / 4)) * 4;
                f32x4 t = {0.f, 0.f, 0.f, 0.f};
                if (g0 + gl2 < gmax) t = *(const f32x4*)(w + (g0 + gl2) * W + i4);
#pragma unroll
                for (int k = 0; k < 4; ++k) wl[(i4 + k) * ng + gl2] = t[k];
            }
        } else {
            for (int e = tid; e < W * ng; e += 64 * NSG) {
                const int gl2 = e / W, i = e - gl2 * W;
                wl[i * ng + gl2] = (g0 + gl2 < gmax) ? w[(g0 + gl2) * W + i] : 0.f;
            }
        }
        __syncthreads();
    }
    fma_batch(sg, q0);
    for (int i = sg + UF * NSG; i < R; i += UF * NSG) {
        u32x4 q[UF];
        load_batch(i, q);
        fma_batch(i, q);
    }
    if (sg > 0) {
#pragma unroll
        for (int c = 0; c < 8; ++c) red[((sg - 1) * 64 + oc) * 8 + c] = acc[c];
    }
    __syncthreads();          // also orders every read of slot `pos` before its overwrite below
    if (sg != 0 || !live) return;
#pragma unroll
    for (int k = 0; k < NSG - 1; ++k)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] += red[(k * 64 + oc) * 8 + c];

    const u32x4 a1 = *(const u32x4*)(x1 + b * in_bs + d0);
    u32x4 av = {0, 0, 0, 0}, a2 = {0, 0, 0, 0};
    if (PRE) av = *(const u32x4*)(v + b * in_bs + d0);
    if (POST) a2 = *(const u32x4*)(x2 + b * in_bs + d0);
    uint32_t up[4], o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float uu[2], y[2];
        uu[0] = PRE ? round_bf(bf_lo(a1[j]) * bf_lo(av[j])) : bf_lo(a1[j]);
        uu[1] = PRE ? round_bf(bf_hi(a1[j]) * bf_hi(av[j])) : bf_hi(a1[j]);
        up[j] = PRE ? pack_bf2(uu[0], uu[1]) : a1[j];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int c = 2 * j + e;
            const float h0 = GROUPED ? wl[R * ng + gl] : w[(d0 + c) * W + R];
            float yy = fmaf(h0, uu[e], acc[c]);
            if (BIAS == HYENA_BIAS_GATED_FP32) yy = fmaf(bias[d0 + c], uu[e], yy);
            if (BIAS == HYENA_BIAS_ADD) yy += bias[d0 + c];
            yy = round_bf(yy);
            if (POST) yy *= (e ? bf_hi(a2[j]) : bf_lo(a2[j]));
            y[e] = yy;
        }
        o[j] = pack_bf2(y[0], y[1]);
    }
    const u32x4 ov = {o[0], o[1], o[2], o[3]};
    *(u32x4*)(out + b * out_bs + d0) = ov;
    const u32x4 uv = {up[0], up[1], up[2], up[3]};
    *(u32x4*)(ring + (b * R + pos) * D + d0) = uv;
}

// ---------------------------------------------------------------- IIR step
// LPB lanes share one (batch, channel): each holds 16 bytes of its modal state
// (4 real or 2 complex states), so state traffic is fully coalesced.  The
// residue-weighted sum is reduced with xor shuffles inside the lane group.
template <int S, bool CPLX>
__global__ __launch_bounds__(256) void iir_step_kernel(const bf16_t* __restrict__ x1, const bf16_t* __restrict__ x2,
                                                       const bf16_t* __restrict__ v, int64_t in_bs,
                                                       float* __restrict__ state, const float* __restrict__ poles,
                                                       const float* __restrict__ residues,
                                                       const float* __restrict__ Dcoef, int d_is_bf16,
                                                       void* __restrict__ out, int out_is_fp32, int64_t out_bs,
                                                       int64_t B, int64_t D, int dg) {
    constexpr int LPB = CPLX ? S / 2 : S / 4;      // lanes per (b, d)
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int q = (int)(idx % LPB);
    int64_t bd = idx / LPB;
    const bool live = bd < B * D;
    if (!live) bd = 0;
    const int64_t b = bd / D, d = bd - b * D;
    const int64_t g = d / dg;
    constexpr int FPS = CPLX ? 2 : 1;              // floats per state
    float* sp = state + (bd * S) * FPS + q * 4;
    const f32x4 st = *(const f32x4*)sp;
    const f32x4 pp = *(const f32x4*)(poles + (g * S) * FPS + q * 4);
    const f32x4 rr = *(const f32x4*)(residues + (g * S) * FPS + q * 4);
    const float a = bf_to_f(x1[b * in_bs + d]), c = bf_to_f(v[b * in_bs + d]);
    const float x1v = round_bf(a * c);
    f32x4 ns;
    float part;
    if (CPLX) {
        // (pr + i pi)(sr + i si) + x1v
        ns[0] = fmaf(pp[0], st[0], -pp[1] * st[1]) + x1v;
        ns[1] = fmaf(pp[0], st[1], pp[1] * st[0]);
        ns[2] = fmaf(pp[2], st[2], -pp[3] * st[3]) + x1v;
        ns[3] = fmaf(pp[2], st[3], pp[3] * st[2]);
        part = (rr[0] * ns[0] - rr[1] * ns[1]) + (rr[2] * ns[2] - rr[3] * ns[3]);   // Re(r*s)
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) ns[k] = fmaf(pp[k], st[k], x1v);
        part = (rr[0] * ns[0] + rr[1] * ns[1]) + (rr[2] * ns[2] + rr[3] * ns[3]);
    }
    if (live) *(f32x4*)sp = ns;
#pragma unroll
    for (int m = 1; m < LPB; m <<= 1) part += __shfl_xor(part, m, 64);
    if (live && q == 0) {
        float dx = Dcoef[d] * x1v;
        if (d_is_bf16) dx = round_bf(dx);
        const float y = bf_to_f(x2[b * in_bs + d]) * (part + dx);
        if (out_is_fp32) ((float*)out)[b * out_bs + d] = y;
        else ((bf16_t*)out)[b * out_bs + d] = (bf16_t)f_to_bf_bits(y);
    }
}

}  // namespace

extern "C" int hyena_fir_step(const void* x1, const void* x2, const void* v, int64_t in_bs, void* ring, int64_t R,
                              int64_t pos, const float* w, const float* bias, int bias_mode, void* out,
                              int64_t out_bs, int64_t B, int64_t D, int64_t G, void* stream) {
    if (!x1 || !ring || !w || !out) return hyena_fail(HYENA_EINVAL, "hyena_fir_step: x1, ring, w, out are required");
    if (B < 0 || D <= 0 || G <= 0 || D % G != 0 || R < 1 || R > 4096 || pos < 0 || pos >= R)
        return hyena_fail(HYENA_EINVAL, "hyena_fir_step: bad sizes B=%lld D=%lld G=%lld R=%lld pos=%lld", (long long)B,
                          (long long)D, (long long)G, (long long)R, (long long)pos);
    if (bias_mode < 0 || bias_mode > 2 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "hyena_fir_step: bias_mode %d needs a bias pointer", bias_mode);
    if (D % 8 != 0 || in_bs % 8 != 0 || out_bs % 8 != 0 || ((uintptr_t)x1 & 15) || ((uintptr_t)ring & 15) ||
        ((uintptr_t)out & 15) || (x2 && ((uintptr_t)x2 & 15)) || (v && ((uintptr_t)v & 15)))
        return hyena_fail(HYENA_EALIGN, "hyena_fir_step: D and strides must be multiples of 8, pointers 16-byte aligned");
    if (B > 65535) return hyena_fail(HYENA_EINVAL, "hyena_fir_step: B > 65535");
    if (B == 0) return 0;
    const int dg = (int)(D / G);
    const bool grouped = (dg % 8 == 0) && (512 % dg == 0);
    if (!grouped && G != D)
        return hyena_fail(HYENA_ENOSUP, "hyena_fir_step: D/G=%d needs per-channel taps (pass G=D)", dg);
    const bool pre = v != nullptr, post = x2 != nullptr;
    dim3 grid((unsigned)((D + 511) / 512), (unsigned)B);
    const int nsg = R >= 32 ? 8 : 2;
    size_t sh = (size_t)(nsg - 1) * 64 * 8 * sizeof(float) + (grouped ? (size_t)(R + 1) * (512 / dg) * sizeof(float) : 0);
    if (sh > 160 * 1024) return hyena_fail(HYENA_ENOSUP, "hyena_fir_step: R too large for the LDS tap table");
    hipStream_t s = (hipStream_t)stream;
    const bf16_t *p1 = (const bf16_t*)x1, *p2 = (const bf16_t*)x2, *pv = (const bf16_t*)v;
    bool ok = false;
#define FS_GO(P, Q, M, GR, N)                                                                                 \
    hipLaunchKernelGGL((fir_step_kernel<P, Q, M, GR, N>), grid, dim3(64 * N), sh, s, p1, p2, pv, in_bs,       \
                       (bf16_t*)ring, (int)R, (int)pos, w, bias, (bf16_t*)out, out_bs, D, dg)
#define FS_CASE(P, Q, M)                                                                                      \
    if (pre == P && post == Q && bias_mode == M) {                                                            \
        if (grouped && nsg == 8) FS_GO(P, Q, M, true, 8);                                                     \
        else if (grouped) FS_GO(P, Q, M, true, 2);                                                            \
        else if (nsg == 8) FS_GO(P, Q, M, false, 8);                                                          \
        else FS_GO(P, Q, M, false, 2);                                                                        \
        ok = true;                                                                                            \
    }
    FS_CASE(true, true, HYENA_BIAS_NONE)
    FS_CASE(true, true, HYENA_BIAS_GATED_FP32)
    FS_CASE(false, false, HYENA_BIAS_NONE)
    FS_CASE(false, false, HYENA_BIAS_ADD)
    FS_CASE(false, false, HYENA_BIAS_GATED_FP32)
    FS_CASE(true, true, HYENA_BIAS_ADD)
#undef FS_CASE
#undef FS_GO
    if (!ok) return hyena_fail(HYENA_ENOSUP, "hyena_fir_step: this gate/bias combination has no kernel");
    return hyena_check_launch("hyena_fir_step");
}

extern "C" int hyena_iir_step(const void* x1, const void* x2, const void* v, int64_t in_bs, float* state,
                              const float* poles, const float* residues, int is_complex, const float* Dcoef,
                              int d_is_bf16, void* out, int out_is_fp32, int64_t out_bs, int64_t B, int64_t D,
                              int64_t G, int64_t S, void* stream) {
    if (!x1 || !x2 || !v || !state || !poles || !residues || !Dcoef || !out)
        return hyena_fail(HYENA_EINVAL, "hyena_iir_step: all pointers are required");
    if (B < 0 || D <= 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "hyena_iir_step: bad sizes B=%lld D=%lld G=%lld", (long long)B, (long long)D,
                          (long long)G);
    if (S != 16 && S != 8 && S != 32)
        return hyena_fail(HYENA_ENOSUP, "hyena_iir_step: state size %lld (8, 16 or 32 supported)", (long long)S);
    if (((uintptr_t)state & 15) || ((uintptr_t)poles & 15) || ((uintptr_t)residues & 15))
        return hyena_fail(HYENA_EALIGN, "hyena_iir_step: state, poles, residues must be 16-byte aligned");
    if (B == 0) return 0;
    const int dg = (int)(D / G);
    const int lpb = is_complex ? (int)S / 2 : (int)S / 4;
    const int64_t nthr = B * D * lpb;
    dim3 grid((unsigned)((nthr + 255) / 256));
    hipStream_t s = (hipStream_t)stream;
    const bf16_t *p1 = (const bf16_t*)x1, *p2 = (const bf16_t*)x2, *pv = (const bf16_t*)v;
#define IIR_CASE(SS, C)                                                                                        \
    if (S == SS && (is_complex != 0) == C)                                                                      \
        hipLaunchKernelGGL((iir_step_kernel<SS, C>), grid, dim3(256), 0, s, p1, p2, pv, in_bs, state, poles,    \
                           residues, Dcoef, d_is_bf16, out, out_is_fp32, out_bs, B, D, dg);
    IIR_CASE(8, false) IIR_CASE(16, false) IIR_CASE(32, false)
    IIR_CASE(8, true) IIR_CASE(16, true) IIR_CASE(32, true)
#undef IIR_CASE
    return hyena_check_launch("hyena_iir_step");
}
