// Hyena-LI prefill: long gated convolution with an implicit modal filter
// h[t] = Re sum_s r_s p_s^t, computed in one pass over L as a chunked modal scan:
//
//   chunk c (128 samples):  y_c = T * u_c  +  Pout * X_c ,   X_{c+1} = p^128 (.) X_c + Pin * u_c
//
//   T    [128 x 128]  lower-triangular Toeplitz of the filter head h[0..127]
//   Pin  [2S  x 128]  rows (Re, Im) of p_s^(127-j): the chunk's contribution to the state
//   Pout [128 x 2S ]  (Re, -Im) of r_s p_s^(i+1):  what the incoming state adds to sample i
//   X_c  [2S]         complex modal state after the samples before chunk c
//
// All three contractions run on bf16 MFMA with fp32 accumulation.  To keep the
// fp32 long-convolution output within 1e-4 of an fp32 evaluation, every fp32
// coefficient is split into two bf16 terms (hi + lo) and the state, which is not
// bf16-exact, is split as well (hi*hi + hi*lo + lo*hi); the inputs u = bf16(x1*v)
// are exact.  The state recurrence itself is carried in fp32 registers.  The final
// X is the decode state of vortex/model/engine.py:525-559 for free.
//
// One block (4 wavefronts) owns 16 channels of one filter group and walks the
// whole sequence in 512-sample steps (4 chunks); global traffic is the same
// coalesced 16 B/lane pattern as the Hyena-MR kernel: x1, v, x2 read once, out
// written once.
#include "common.h"

namespace {

constexpr int TL = 512;
constexpr int C = 128;         // chunk
constexpr int URS = 520;       // u_lds / z_lds row stride (elements): 1040 B = 16 * 65
constexpr int S = 16;          // modal state size (poles per group)
constexpr int R2 = 2 * S;      // real rows of the state

// workspace layout per group (floats)
constexpr int WS_HEAD = 0;                 // [128]
constexpr int WS_PIN = WS_HEAD + C;        // [32][128]
constexpr int WS_POUT = WS_PIN + R2 * C;   // [128][32]
constexpr int WS_PC = WS_POUT + C * R2;    // [16][2]
constexpr int WS_PINV = WS_PC + 2 * S;     // [16][2]  1/p
constexpr int WS_GROUP = WS_PINV + 2 * S;  // 8384 floats

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) {
    union { u32x4 u; bf16x8 b; } c;
    c.u = x;
    return c.b;
}

template <bool PRE>
__device__ __forceinline__ u32x4 gate_mul(u32x4 a, u32x4 b) {
    if (!PRE) return a;
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = pack_bf2(bf_lo(a[j]) * bf_lo(b[j]), bf_hi(a[j]) * bf_hi(b[j]));
    return r;
}

// hi/lo bf16 split of eight fp32 values produced by f(e), e = 0..7
template <typename F>
__device__ __forceinline__ void split8(F f, bf16x8& hi, bf16x8& lo) {
    u32x4 ph, pl;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = f(2 * j), b = f(2 * j + 1);
        const float ah = round_bf(a), bh = round_bf(b);
        ph[j] = (__float_as_uint(ah) >> 16) | (__float_as_uint(bh) & 0xffff0000u);
        pl[j] = pack_bf2(a - ah, b - bh);
    }
    hi = as_bf16x8(ph);
    lo = as_bf16x8(pl);
}

// ------------------------------------------------------------------ plan kernel
// One block per group; coefficients evaluated in double from the fp32 parameters.
__global__ __launch_bounds__(256) void li_plan_kernel(const float* __restrict__ log_poles,   // [G][S][2]
                                                      const float* __restrict__ residues,    // [G][S][2]
                                                      float* __restrict__ ws) {
    const int g = blockIdx.x, tid = threadIdx.x;
    float* w = ws + (size_t)g * WS_GROUP;
    const float* lp = log_poles + (size_t)g * S * 2;
    const float* rs = residues + (size_t)g * S * 2;
    // p^k = exp(k*lr) * (cos(k*th), sin(k*th))
    auto ppow = [&](int s, int k, double& re, double& im) {
        const double m = exp((double)k * (double)lp[2 * s]);
        const double a = (double)k * (double)lp[2 * s + 1];
        re = m * cos(a);
        im = m * sin(a);
    };
    if (tid < C) {                                  // filter head
        double acc = 0.0;
        for (int s = 0; s < S; ++s) {
            double re, im;
            ppow(s, tid, re, im);
            acc += (double)rs[2 * s] * re - (double)rs[2 * s + 1] * im;
        }
        w[WS_HEAD + tid] = (float)acc;
    }
    for (int e = tid; e < S * C; e += 256) {        // Pin and Pout
        const int s = e / C, j = e - s * C;
        double re, im;
        ppow(s, C - 1 - j, re, im);
        w[WS_PIN + s * C + j] = (float)re;
        w[WS_PIN + (S + s) * C + j] = (float)im;
        ppow(s, j + 1, re, im);                     // here j plays the role of the output sample i
        const double rr = rs[2 * s], ri = rs[2 * s + 1];
        w[WS_POUT + j * R2 + s] = (float)(rr * re - ri * im);          //  Re(r p^(i+1))
        w[WS_POUT + j * R2 + S + s] = (float)(-(rr * im + ri * re));   // -Im(r p^(i+1))
    }
    if (tid < S) {
        double re, im;
        ppow(tid, C, re, im);
        w[WS_PC + 2 * tid] = (float)re;
        w[WS_PC + 2 * tid + 1] = (float)im;
        ppow(tid, -1, re, im);
        w[WS_PINV + 2 * tid] = (float)re;
        w[WS_PINV + 2 * tid + 1] = (float)im;
    }
}

// ------------------------------------------------------------------ main kernel
struct LiArgs {
    RowMap x1, x2, v;
    const float* ws;          // plan workspace
    const float* Dcoef;       // [D] or null
    bf16_t* out;              // [B][D][L]
    float* y32;               // optional [B][D][L] fp32 convolution output (before any rounding)
    float* state_out;         // optional [B][D][S][2]
    int64_t D, L;
    int dg;
    int d_is_bf16;
};

template <int W, bool PRE, bool POST>
__device__ __forceinline__ void li_body(const LiArgs& a, bf16_t* u_lds, bf16_t* z_lds, float* l_lds, bf16_t* xh_lds,
                                        bf16_t* xl_lds) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int64_t nslab = a.D / 16;
    const int64_t slab = blockIdx.x % nslab, b = blockIdx.x / nslab;
    const int64_t d0 = slab * 16;
    const int g = (int)(d0 / a.dg);
    const float* ws = a.ws + (size_t)g * WS_GROUP;
    const int64_t L = a.L;

    // ---- A fragments -----------------------------------------------------------------
    const int n = lane & 31, hh = lane >> 5;
    const int i_time = 16 * ((n >> 2) & 1) + 4 * (n >> 3) + (n & 3);   // sample owned through MFMA row n
    bf16x8 Th[8], Tl[8];                 // Toeplitz blocks, delta = -1..6 at index delta+1
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        split8([&](int e) {
            const int lag = 16 * (q - 1) + i_time - (8 * hh + e);
            return (lag >= 0 && lag < C) ? ws[WS_HEAD + lag] : 0.f;
        }, Th[q], Tl[q]);
    }
    constexpr int I0 = W, I1 = 3 - W;    // 32-row output blocks of this wavefront (column group 0 / 1)
    bf16x8 Poh[2][2], Pol[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int k = 0; k < 2; ++k)
            split8([&](int e) { return ws[WS_POUT + (32 * (t ? I1 : I0) + i_time) * R2 + 16 * k + 8 * hh + e]; },
                   Poh[t][k], Pol[t][k]);
    const int m16 = lane & 15, q4 = lane >> 4;
    bf16x8 Pih[2][4], Pil[2][4];
#pragma unroll
    for (int mu = 0; mu < 2; ++mu)
#pragma unroll
        for (int k = 0; k < 4; ++k)
            split8([&](int e) { return ws[WS_PIN + (16 * mu + m16) * C + 32 * k + 8 * q4 + e]; }, Pih[mu][k],
                   Pil[mu][k]);

    // ---- state owned by this thread: channel sc, pole ss
    const int sc = tid >> 4, ss = tid & 15;
    float Xr = 0.f, Xi = 0.f;
    const float pcr = ws[WS_PC + 2 * ss], pci = ws[WS_PC + 2 * ss + 1];

    // ---- coalesced layout: 16 B of rows 4*r4 + W
    const bf16_t *p1[4], *pv[4], *p2[4];
    bf16_t* po[4];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        const int64_t d = d0 + 4 * r4 + W;
        p1[r4] = a.x1.row(b, d) + lane * 8;
        pv[r4] = PRE ? a.v.row(b, d) + lane * 8 : nullptr;
        p2[r4] = POST ? a.x2.row(b, d) + lane * 8 : nullptr;
        po[r4] = a.out + (b * a.D + d) * L + lane * 8;
    }
    const u32x4 zero4 = {0, 0, 0, 0};
    u32x4 c1[4], cv[4];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        const bool ok = lane * 8 < L;
        c1[r4] = ok ? *(const u32x4*)(p1[r4]) : zero4;
        cv[r4] = (PRE && ok) ? *(const u32x4*)(pv[r4]) : zero4;
    }
    const int c = n & 15, s = n >> 4;
    float dco = 0.f;
    if (a.Dcoef) dco = a.Dcoef[d0 + c];

    for (int64_t ts = 0; ts < L; ts += TL) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
            *(u32x4*)(u_lds + (4 * r4 + W) * URS + lane * 8) = gate_mul<PRE>(c1[r4], cv[r4]);
        __syncthreads();                                                      // (1) u ready

        u32x4 c2[4];
        {
            const int64_t tn = ts + TL;
            const bool okn = tn + lane * 8 < L, okc = ts + lane * 8 < L;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                c1[r4] = okn ? *(const u32x4*)(p1[r4] + tn) : zero4;
                cv[r4] = (PRE && okn) ? *(const u32x4*)(pv[r4] + tn) : zero4;
                c2[r4] = (POST && okc) ? *(const u32x4*)(p2[r4] + ts) : zero4;
            }
        }

        // ---- state-in of chunk W: Pin[32 x 128] * u_chunk[128 x 16], 16x16x32 MFMA
        {
            f32x4 l0 = {0, 0, 0, 0}, l1 = {0, 0, 0, 0};
            const bf16_t* ub = u_lds + m16 * URS + C * W + 8 * q4;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const bf16x8 bf = *(const bf16x8*)(ub + 32 * k);
                l0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pih[0][k], bf, l0, 0, 0, 0);
                l0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pil[0][k], bf, l0, 0, 0, 0);
                l1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pih[1][k], bf, l1, 0, 0, 0);
                l1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pil[1][k], bf, l1, 0, 0, 0);
            }
            // lane (column m16, quad q4) holds state rows 4*q4..+3 of each half
            float* lp = l_lds + (W * 16 + m16) * R2 + 4 * q4;
            *(f32x4*)lp = l0;
            *(f32x4*)(lp + 16) = l1;
        }

        // ---- Toeplitz: tile 0 = (column group 0, rows I0), tile 1 = (column group 1, rows I1)
        f32x16 acc0, acc1;
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
        {
            const bf16_t* ub0 = u_lds + c * URS + C * s + 8 * hh;            // chunks 0,1
            const bf16_t* ub1 = ub0 + 2 * C;                                  // chunks 2,3
#pragma unroll
            for (int J = 0; J <= 2 * I0 + 1; ++J) {
                const bf16x8 bf = *(const bf16x8*)(ub0 + 16 * J);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Th[2 * I0 - J + 1], bf, acc0, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Tl[2 * I0 - J + 1], bf, acc0, 0, 0, 0);
            }
#pragma unroll
            for (int J = 0; J <= 2 * I1 + 1; ++J) {
                const bf16x8 bf = *(const bf16x8*)(ub1 + 16 * J);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Th[2 * I1 - J + 1], bf, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Tl[2 * I1 - J + 1], bf, acc1, 0, 0, 0);
            }
        }
        __syncthreads();                                                      // (2) chunk contributions ready

        // ---- state scan over the 4 chunks of this step (thread = one channel x one pole)
        {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float xrh = round_bf(Xr), xih = round_bf(Xi);
                const int o = (k * 16 + sc) * R2;
                xh_lds[o + ss] = (bf16_t)(__float_as_uint(xrh) >> 16);
                xh_lds[o + S + ss] = (bf16_t)(__float_as_uint(xih) >> 16);
                xl_lds[o + ss] = (bf16_t)f_to_bf_bits(Xr - xrh);
                xl_lds[o + S + ss] = (bf16_t)f_to_bf_bits(Xi - xih);
                const float lr = l_lds[o + ss], li = l_lds[o + S + ss];
                const float nr = fmaf(pcr, Xr, fmaf(-pci, Xi, lr));
                const float ni = fmaf(pcr, Xi, fmaf(pci, Xr, li));
                Xr = nr;
                Xi = ni;
            }
        }
        __syncthreads();                                                      // (3) chunk states ready

        // ---- state-out: Pout[rows x 32] * X[32 x columns], three bf16 products
        {
            const bf16_t* xb0h = xh_lds + ((0 + s) * 16 + c) * R2 + 8 * hh;
            const bf16_t* xb0l = xl_lds + ((0 + s) * 16 + c) * R2 + 8 * hh;
            const bf16_t* xb1h = xh_lds + ((2 + s) * 16 + c) * R2 + 8 * hh;
            const bf16_t* xb1l = xl_lds + ((2 + s) * 16 + c) * R2 + 8 * hh;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const bf16x8 h0 = *(const bf16x8*)(xb0h + 16 * k), l0 = *(const bf16x8*)(xb0l + 16 * k);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Poh[0][k], h0, acc0, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Poh[0][k], l0, acc0, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Pol[0][k], h0, acc0, 0, 0, 0);
                const bf16x8 h1 = *(const bf16x8*)(xb1h + 16 * k), l1 = *(const bf16x8*)(xb1l + 16 * k);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Poh[1][k], h1, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Poh[1][k], l1, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Pol[1][k], h1, acc1, 0, 0, 0);
            }
        }

        // ---- epilogue: y = bf16(conv); z = bf16(y + bf16(D*u)) -> LDS (engine.py:352-353)
#pragma unroll
        for (int tau = 0; tau < 2; ++tau) {
            const int tcol = C * (2 * tau + s) + 32 * (tau ? I1 : I0) + 16 * hh;
            const f32x16 acc = tau ? acc1 : acc0;
            if (a.y32) {
                const int64_t t0 = ts + tcol;
                float* yp = a.y32 + (b * a.D + d0 + c) * L + t0;
#pragma unroll
                for (int r = 0; r < 16; r += 4)
                    if (t0 + r < L) {
                        const f32x4 q = {acc[r], acc[r + 1], acc[r + 2], acc[r + 3]};
                        *(f32x4*)(yp + r) = q;
                    }
            }
            const u32x4 ua = *(const u32x4*)(u_lds + c * URS + tcol);
            const u32x4 ub2 = *(const u32x4*)(u_lds + c * URS + tcol + 8);
            u32x4 z0, z1;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t uw = j < 4 ? ua[j] : ub2[j - 4];
                float y0 = round_bf(acc[2 * j]), y1 = round_bf(acc[2 * j + 1]);
                float t0 = dco * bf_lo(uw), t1 = dco * bf_hi(uw);
                if (a.d_is_bf16) { t0 = round_bf(t0); t1 = round_bf(t1); }
                const uint32_t p = pack_bf2(y0 + t0, y1 + t1);
                if (j < 4) z0[j] = p; else z1[j - 4] = p;
            }
            *(u32x4*)(z_lds + c * URS + tcol) = z0;
            *(u32x4*)(z_lds + c * URS + tcol + 8) = z1;
        }
        __syncthreads();                                                      // (4) z ready, u and X consumed

        if (ts + lane * 8 < L) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const u32x4 zz = *(const u32x4*)(z_lds + (4 * r4 + W) * URS + lane * 8);
                u32x4 o = zz;
                if (POST) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[j] = pack_bf2(bf_lo(zz[j]) * bf_lo(c2[r4][j]), bf_hi(zz[j]) * bf_hi(c2[r4][j]));
                }
                *(u32x4*)(po[r4] + ts) = o;
            }
        }
    }

    if (a.state_out) {
        // the scan ran over ceil(L/512)*512 samples with zero inputs past L: undo the padding, X *= p^-pad
        int pad = (int)(((L + TL - 1) / TL) * TL - L);
        float qr = ws[WS_PINV + 2 * ss], qi = ws[WS_PINV + 2 * ss + 1];
        float fr = 1.f, fi = 0.f;
        while (pad) {
            if (pad & 1) { const float t = fr * qr - fi * qi; fi = fr * qi + fi * qr; fr = t; }
            const float t = qr * qr - qi * qi; qi = 2.f * qr * qi; qr = t;
            pad >>= 1;
        }
        float* sp = a.state_out + ((b * a.D + d0 + sc) * S + ss) * 2;
        sp[0] = Xr * fr - Xi * fi;
        sp[1] = Xr * fi + Xi * fr;
    }
}

template <bool PRE, bool POST>
__global__ __launch_bounds__(256, 1) void li_kernel(LiArgs a) {
    __shared__ __attribute__((aligned(16))) bf16_t u_lds[16 * URS];
    __shared__ __attribute__((aligned(16))) bf16_t z_lds[16 * URS];
    __shared__ __attribute__((aligned(16))) float l_lds[4 * 16 * R2];
    __shared__ __attribute__((aligned(16))) bf16_t xh_lds[4 * 16 * R2];
    __shared__ __attribute__((aligned(16))) bf16_t xl_lds[4 * 16 * R2];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    switch (w) {
        case 0: li_body<0, PRE, POST>(a, u_lds, z_lds, l_lds, xh_lds, xl_lds); break;
        case 1: li_body<1, PRE, POST>(a, u_lds, z_lds, l_lds, xh_lds, xl_lds); break;
        case 2: li_body<2, PRE, POST>(a, u_lds, z_lds, l_lds, xh_lds, xl_lds); break;
        default: li_body<3, PRE, POST>(a, u_lds, z_lds, l_lds, xh_lds, xl_lds); break;
    }
}

}  // namespace

extern "C" int64_t hyena_li_plan_bytes(int64_t G, int64_t S_) {
    if (G <= 0 || S_ != S) return 0;
    return (int64_t)G * WS_GROUP * (int64_t)sizeof(float);
}

extern "C" int hyena_li_plan(const float* log_poles, const float* residues, int64_t G, int64_t S_, void* workspace,
                             void* stream) {
    if (!log_poles || !residues || !workspace) return hyena_fail(HYENA_EINVAL, "hyena_li_plan: null pointer");
    if (G <= 0 || G > 0x7fffffff) return hyena_fail(HYENA_EINVAL, "hyena_li_plan: bad G=%lld", (long long)G);
    if (S_ != S) return hyena_fail(HYENA_ENOSUP, "hyena_li_plan: state size %lld (only 16)", (long long)S_);
    hipLaunchKernelGGL(li_plan_kernel, dim3((unsigned)G), dim3(256), 0, (hipStream_t)stream, log_poles, residues,
                       (float*)workspace);
    return hyena_check_launch("hyena_li_plan");
}

extern "C" int hyena_li_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const void* workspace,
                            const float* Dcoef, int d_is_bf16, void* out, float* y_conv_fp32, float* state_out,
                            int64_t B, int64_t D, int64_t L, int64_t G, int64_t S_, void* stream) {
    if (!x1 || !x1->ptr || !workspace || !out)
        return hyena_fail(HYENA_EINVAL, "hyena_li_fwd: x1, workspace and out are required");
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "hyena_li_fwd: bad sizes B=%lld D=%lld L=%lld G=%lld", (long long)B,
                          (long long)D, (long long)L, (long long)G);
    if (S_ != S) return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd: state size %lld (only 16)", (long long)S_);
    if ((D / G) % 16 != 0)
        return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd: D/G=%lld must be a multiple of 16", (long long)(D / G));
    if (L % 8 != 0 || !rows_aligned8(x1) || !rows_aligned8(x2) || !rows_aligned8(v) || (((uintptr_t)out) & 15) ||
        (((uintptr_t)y_conv_fp32) & 15))
        return hyena_fail(HYENA_EALIGN, "hyena_li_fwd: L and strides must be multiples of 8, pointers 16-byte aligned");
    if (B == 0 || L == 0) return 0;
    const bool pre = v && v->ptr, post = x2 && x2->ptr;
    const int64_t nblk = B * (D / 16);
    if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "hyena_li_fwd: problem too large for one launch");
    LiArgs a;
    a.x1 = make_rowmap(x1);
    a.x2 = make_rowmap(post ? x2 : nullptr);
    a.v = make_rowmap(pre ? v : nullptr);
    a.ws = (const float*)workspace;
    a.Dcoef = Dcoef;
    a.out = (bf16_t*)out;
    a.y32 = y_conv_fp32;
    a.state_out = state_out;
    a.D = D;
    a.L = L;
    a.dg = (int)(D / G);
    a.d_is_bf16 = d_is_bf16;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)nblk);
    if (pre && post) hipLaunchKernelGGL((li_kernel<true, true>), grid, dim3(256), 0, s, a);
    else if (!pre && !post) hipLaunchKernelGGL((li_kernel<false, false>), grid, dim3(256), 0, s, a);
    else return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd: pass both v and x2 or neither");
    return hyena_check_launch("hyena_li_fwd");
}
