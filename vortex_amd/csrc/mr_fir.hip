// Hyena-MR: gated causal depthwise FIR, K <= 128, as a block-Toeplitz
// contraction on bf16 MFMA (v_mfma_f32_32x32x16_bf16) with fp32 accumulation.
//
// For 32 output samples starting at T and filter lags 0..127 the inputs are the
// ten 16-sample blocks that start at T-128+16m, m = 0..9, and the 32x16
// Toeplitz block that weights block m, A_m[i][j] = h[i - j + 128 - 16m], does
// not depend on T.  A wavefront therefore keeps all ten A_m of its filter group
// in registers for the whole kernel and streams u = bf16(x1*v) through the B
// operand.  The MFMA N dimension (32 columns) is 16 channels of the group x 2
// time offsets.  This is the two-pass chunked Toeplitz form of
// vortex/ops/hyena_se/ref_fwd.py:216-266 with the all-zero blocks of T and T^
// dropped and the two passes merged into one accumulator.
//
// Data path per 512-sample step of a block (4 wavefronts, 16 channels):
//   global (coalesced 16 B/lane) -> u = bf16(x1*v) -> LDS row-major [16][128+512]
//   -> B fragments (ds_read_b128) -> MFMA -> z = bf16(acc + D*u) -> LDS
//   -> coalesced read, * x2, 16 B/lane store.
// The 128-sample tail of a step stays in LDS as the next step's halo, so each
// input is read from HBM once per segment.
#include <type_traits>

#include "common.h"

namespace {

constexpr int TL = 512;        // samples per step
constexpr int HALO = 128;      // samples kept from the previous step
constexpr int URS = 648;       // u_lds row stride (elements): 1296 B = 16 * 81
constexpr int ZRS = 520;       // z_lds row stride (elements): 1040 B = 16 * 65

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) {
    union { u32x4 u; bf16x8 b; } c;
    c.u = x;
    return c.b;
}

// streaming accesses: every activation is touched once, so keep it out of the caches' way
template <bool NT>
__device__ __forceinline__ u32x4 ld16(const bf16_t* p) {
    return NT ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
}
template <bool NT>
__device__ __forceinline__ void st16(bf16_t* p, u32x4 v) {
    if (NT) __builtin_nontemporal_store(v, (u32x4*)p); else *(u32x4*)p = v;
}

template <bool PRE>
__device__ __forceinline__ u32x4 gate_mul(u32x4 a, u32x4 b) {
    if (!PRE) return a;
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = pack_bf2(bf_lo(a[j]) * bf_lo(b[j]), bf_hi(a[j]) * bf_hi(b[j]));
    return r;
}

// Three-tap featurizer FIR on one 16-byte piece (8 samples of a raw projection row): hw holds the two samples ahead
// of it.  fp32 FMAs, oldest sample first, one rounding to bf16: the arithmetic of the other featurizer kernels.
__device__ __forceinline__ u32x4 feat3(const u32x4 cc, const uint32_t hw, const float w0, const float w1, const float w2) {
    float rr[10];
    rr[0] = bf_lo(hw);
    rr[1] = bf_hi(hw);
#pragma unroll
    for (int j = 0; j < 4; ++j) { rr[2 + 2 * j] = bf_lo(cc[j]); rr[3 + 2 * j] = bf_hi(cc[j]); }
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float f0 = fmaf(w2, rr[2 * j + 2], fmaf(w1, rr[2 * j + 1], fmaf(w0, rr[2 * j], 0.f)));
        const float f1 = fmaf(w2, rr[2 * j + 3], fmaf(w1, rr[2 * j + 2], fmaf(w0, rr[2 * j + 1], 0.f)));
        o[j] = pack_bf2(f0, f1);
    }
    return o;
}

// FEAT = 3: the rows are the raw projection of the layer, stored sequence-major, and the three-tap featurizer FIR of
// vortex/model/model.py:233-246 (vortex/model/engine.py:188-223 with gate = False) runs on every 16-byte piece as the
// step consumes it.  A wavefront instruction covers 512 consecutive samples of one row, so a lane's two samples of
// history are the last dword of the lane to its left (a wavefront shift); lane 0 takes them from the piece the
// wavefront consumed one step earlier, carried in a scalar register, and at the start of a segment from memory.
template <bool PRE, bool POST, int BIAS, bool NT, bool FULL, int FEAT = 0>
__global__ __launch_bounds__(256, 3) void mr_fir_kernel(RowMap x1, RowMap x2, RowMap v, const float* __restrict__ h,
                                                        int K, int reversed, const float* __restrict__ bias,
                                                        bf16_t* __restrict__ out, int64_t D, int64_t L, int dg,
                                                        int64_t seg_len, int nseg, const float* __restrict__ ftaps) {
    static_assert(FEAT == 0 || (FEAT == 3 && PRE && POST), "featurizer: three taps, all three gates");
    __shared__ __attribute__((aligned(16))) bf16_t u_lds[16 * URS];
    __shared__ __attribute__((aligned(16))) bf16_t z_lds[16 * ZRS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // A slab is 16 channels of one filter group.  Groups whose size is not a multiple of 16 get a last slab
    // with fewer live channels (their rows are read as zeros and never stored).
    const uint32_t spg = ((uint32_t)dg + 15) / 16;              // slabs per group
    const uint32_t nslab = (uint32_t)(D / dg) * spg;
    // Workgroups are dealt to the 8 XCDs in turn (id mod 8).  For tensors that stream through the caches XCD x takes
    // the x-th eighth of the (batch, slab, segment) order, so that each XCD (and its L2) walks one contiguous part of
    // the tensors instead of every eighth piece of all of them: 340 -> 334 us at the config-2 shape.  Cache-resident
    // shapes measured 4-5 % slower that way and keep the plain order.
    uint32_t bid = blockIdx.x;
    if (NT && (gridDim.x & 7u) == 0) bid = (bid & 7u) * (gridDim.x >> 3) + (bid >> 3);
    const int seg = (int)(bid % (uint32_t)nseg);
    const uint32_t slab = (bid / (uint32_t)nseg) % nslab;
    const int64_t b = bid / ((uint32_t)nseg * nslab);
    const int g = (int)(slab / spg);
    const int c_base = 16 * (int)(slab % spg);                 // first channel of the slab inside its group
    const int64_t d0 = (int64_t)g * dg + c_base;
    const int c_live = dg - c_base < 16 ? dg - c_base : 16;    // live channels of this slab

    // ---- Toeplitz fragments of this group's filter (A operand, 32 x 16 each)
    const int n = lane & 31, hh = lane >> 5;
    // accumulator register r of lane (n, hh) is MFMA row 8*(r/4) + 4*hh + r%4; feeding the
    // A rows in the order below makes that lane own the 16 consecutive samples 16*hh + r.
    const int i_time = 16 * ((n >> 2) & 1) + 4 * (n >> 3) + (n & 3);
    bf16x8 A[10];
    // blocks below m_min are all zero; FULL (K > 98) means every block is live and the MFMA chain is branch-free
    const int m_min = FULL ? 0 : ((114 - K) > 0 ? (114 - K + 15) / 16 : 0);
#pragma unroll
    for (int m = 0; m < 10; ++m) {
        u32x4 pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int lag = i_time - (8 * hh + 2 * j + e) + 128 - 16 * m;
                float val = 0.f;
                if (lag >= 0 && lag < K) val = h[g * K + (reversed ? K - 1 - lag : lag)];
                t[e] = val;
            }
            pk[j] = pack_bf2(t[0], t[1]);
        }
        A[m] = as_bf16x8(pk);
    }

    // ---- coalesced layout: this thread moves 16 B of rows 4*r4 + w, r4 = 0..3
    const bf16_t *p1[4], *pv[4], *p2[4];
    bf16_t* po[4];
    bool rlive[4];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        rlive[r4] = 4 * r4 + w < c_live;
        const int64_t d = rlive[r4] ? d0 + 4 * r4 + w : d0;
        p1[r4] = x1.row(b, d);
        pv[r4] = PRE ? v.row(b, d) : nullptr;
        p2[r4] = POST ? x2.row(b, d) : nullptr;
        po[r4] = out + (b * D + d) * L;
    }
    // The row bases above are the same for every lane of the wavefront; a lane adds its 32-bit byte offset at each
    // access (scalar base + vector offset addressing), so no 64-bit address per lane and row is held across the loop.
    const uint32_t lane_b = (uint32_t)lane * 16u;
    auto at = [](const bf16_t* base, int64_t t, uint32_t off) __attribute__((always_inline)) {
        return (const bf16_t*)((const char*)(base + t) + off);
    };
    const int64_t t_begin = (int64_t)seg * seg_len;
    const int64_t t_end = (t_begin + seg_len < L) ? t_begin + seg_len : L;
    if (t_begin >= t_end) return;

    // ---- FEAT: taps of this wavefront's four rows (wave-uniform) and the dwords carried from piece to piece
    float fw[FEAT ? 3 : 1][4][3];
    uint32_t car1[4], carv[4], car2[4];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        car1[r4] = carv[r4] = car2[r4] = 0u;
        if constexpr (FEAT != 0) {
            const int64_t d = rlive[r4] ? d0 + 4 * r4 + w : d0;
#pragma unroll
            for (int i = 0; i < 3; ++i)
#pragma unroll
                for (int k = 0; k < 3; ++k)
                    fw[i][r4][k] = __uint_as_float((uint32_t)__builtin_amdgcn_readfirstlane(
                        (int)__float_as_uint(ftaps[((int64_t)i * D + d) * 3 + k])));
            if (t_begin > 0) {          // the two samples ahead of the segment (t_begin is a multiple of 8: aligned dwords)
                car1[r4] = (uint32_t)__builtin_amdgcn_readfirstlane((int)*(const uint32_t*)(p1[r4] + t_begin - 2));
                carv[r4] = (uint32_t)__builtin_amdgcn_readfirstlane((int)*(const uint32_t*)(pv[r4] + t_begin - 2));
                car2[r4] = (uint32_t)__builtin_amdgcn_readfirstlane((int)*(const uint32_t*)(p2[r4] + t_begin - 2));
            }
        }
    }
    auto feat = [&](const u32x4 cc, uint32_t& carry, const float (&wt)[3]) __attribute__((always_inline)) -> u32x4 {
        const uint32_t hw = (uint32_t)__builtin_amdgcn_update_dpp((int)carry, (int)cc[3], 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
        carry = (uint32_t)__builtin_amdgcn_readlane((int)cc[3], 63);
        return feat3(cc, hw, wt[0], wt[1], wt[2]);
    };

    // ---- halo of the segment: the 128 samples before t_begin (zeros at the sequence start)
    {
        const int ch = tid >> 4, tt = (tid & 15) * 8;
        u32x4 hu = {0, 0, 0, 0};
        if (t_begin > 0 && ch < c_live) {
            const bf16_t* r1 = x1.row(b, d0 + ch) + t_begin - HALO + tt;
            u32x4 a = *(const u32x4*)r1;
            u32x4 c = {0, 0, 0, 0};
            if (PRE) c = *(const u32x4*)(v.row(b, d0 + ch) + t_begin - HALO + tt);
            if constexpr (FEAT != 0) {
                // every thread fetches its own two samples of history here (once per segment)
                const bf16_t* rv = v.row(b, d0 + ch) + t_begin - HALO + tt;
                const bool hist = t_begin - HALO + tt >= 2;
                const uint32_t h1 = hist ? *(const uint32_t*)(r1 - 2) : 0u, hv = hist ? *(const uint32_t*)(rv - 2) : 0u;
                const float* t1 = ftaps + (d0 + ch) * 3;
                const float* tv = ftaps + (2 * D + d0 + ch) * 3;
                a = feat3(a, h1, t1[0], t1[1], t1[2]);
                c = feat3(c, hv, tv[0], tv[1], tv[2]);
            }
            hu = gate_mul<PRE>(a, c);
        }
        *(u32x4*)(u_lds + ch * URS + tt) = hu;
    }

    u32x4 c1[4], cv[4], c2n[4];      // x1, v, x2 of the step about to be processed
    const u32x4 zero4 = {0, 0, 0, 0};
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        const bool ok = rlive[r4] && t_begin + lane * 8 < L;
        c1[r4] = ok ? ld16<NT>(at(p1[r4], t_begin, lane_b)) : zero4;
        cv[r4] = (PRE && ok) ? ld16<NT>(at(pv[r4], t_begin, lane_b)) : zero4;
        c2n[r4] = (POST && ok) ? ld16<NT>(at(p2[r4], t_begin, lane_b)) : zero4;
    }

    float bz = 0.f;
    if (BIAS != HYENA_BIAS_NONE && (n & 15) < c_live) bz = bias[d0 + (n & 15)];

    // One step.  whole_tag: all sixteen channels of the slab exist and this step and the next lie inside the segment, so
    // no test guards a request or a store.
    auto step = [&](const int64_t ts, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        // u of this step -> LDS
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            if constexpr (FEAT != 0) {
                const u32x4 f1 = feat(c1[r4], car1[r4], fw[0][r4]);
                const u32x4 fv = feat(cv[r4], carv[r4], fw[2][r4]);
                *(u32x4*)(u_lds + (4 * r4 + w) * URS + HALO + lane * 8) = gate_mul<true>(f1, fv);
                __builtin_amdgcn_sched_barrier(0);         // one row at a time: its temporaries are dead before the next starts
            } else {
                *(u32x4*)(u_lds + (4 * r4 + w) * URS + HALO + lane * 8) = gate_mul<PRE>(c1[r4], cv[r4]);
            }
        }
        __syncthreads();

        // prefetch the next step's x1, v, x2 (x2 of this step moves to c2)
        u32x4 c2[4];
        {
            const int64_t tn = ts + TL;
            const bool okt = (tn < t_end) && (tn + lane * 8 < L);
            uint32_t lo = lane_b;
            asm volatile("" : "+v"(lo));          // keeps the compiler from folding it into per-lane row pointers held across the loop
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const bool okn = okt && rlive[r4];
                c2[r4] = c2n[r4];
                if (WHOLE) {
                    c1[r4] = ld16<NT>(at(p1[r4], tn, lo));
                    if (PRE) cv[r4] = ld16<NT>(at(pv[r4], tn, lo));
                    if (POST) c2n[r4] = ld16<NT>(at(p2[r4], tn, lo));
                } else {
                    c1[r4] = okn ? ld16<NT>(at(p1[r4], tn, lo)) : zero4;
                    cv[r4] = (PRE && okn) ? ld16<NT>(at(pv[r4], tn, lo)) : zero4;
                    c2n[r4] = (POST && okn) ? ld16<NT>(at(p2[r4], tn, lo)) : zero4;
                }
            }
        }
        // tail of this step = halo of the next one (read now, written after the MFMA phase)
        const u32x4 tail = *(const u32x4*)(u_lds + (tid >> 4) * URS + TL + (tid & 15) * 8);

        // ---- MFMA phase: wavefront w owns output blocks 2w, 2w+1 (+8 for the upper 16 columns)
        const int c = n & 15, s = n >> 4;
        f32x16 acc0, acc1;
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
        const bf16_t* ub = u_lds + c * URS + 64 * w + 256 * s + 8 * hh;
#pragma unroll
        for (int mm = 0; mm < 12; ++mm) {
            const bf16x8 bf = *(const bf16x8*)(ub + 16 * mm);
            if (mm <= 9 && mm >= m_min) acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[mm <= 9 ? mm : 0], bf, acc0, 0, 0, 0);
            if (mm >= 2 && mm - 2 >= m_min) acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[mm >= 2 ? mm - 2 : 0], bf, acc1, 0, 0, 0);
        }
        // ---- z = bf16(acc [+ D*u]) -> LDS, 16 consecutive samples per lane and tile
#pragma unroll
        for (int tau = 0; tau < 2; ++tau) {
            const int tcol = 64 * w + 32 * tau + 256 * s + 16 * hh;
            const f32x16 acc = tau ? acc1 : acc0;
            u32x4 ua = {0, 0, 0, 0}, ub2 = {0, 0, 0, 0};
            if (BIAS == HYENA_BIAS_GATED_FP32 || BIAS == HYENA_BIAS_GATED_BF16) {
                ua = *(const u32x4*)(u_lds + c * URS + HALO + tcol);
                ub2 = *(const u32x4*)(u_lds + c * URS + HALO + tcol + 8);
            }
            u32x4 z0, z1;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float a0 = acc[2 * j], a1 = acc[2 * j + 1];
                if (BIAS == HYENA_BIAS_GATED_FP32) {
                    const uint32_t uw = j < 4 ? ua[j] : ub2[j - 4];
                    a0 = fmaf(bz, bf_lo(uw), a0);
                    a1 = fmaf(bz, bf_hi(uw), a1);
                }
                if (BIAS == HYENA_BIAS_ADD) {
                    a0 = round_bf(a0) + bz;
                    a1 = round_bf(a1) + bz;
                }
                if (BIAS == HYENA_BIAS_ADD_FP32) {
                    a0 += bz;
                    a1 += bz;
                }
                if (BIAS == HYENA_BIAS_GATED_BF16) {             // bf16 tensor arithmetic: every product and sum rounded
                    const uint32_t uw = j < 4 ? ua[j] : ub2[j - 4];
                    const uint32_t yp = pack_bf2(a0, a1), tp = pack_bf2(bz * bf_lo(uw), bz * bf_hi(uw));
                    a0 = bf_lo(yp) + bf_lo(tp);
                    a1 = bf_hi(yp) + bf_hi(tp);
                }
                const uint32_t p = pack_bf2(a0, a1);
                if (j < 4) z0[j] = p; else z1[j - 4] = p;
            }
            *(u32x4*)(z_lds + c * ZRS + tcol) = z0;
            *(u32x4*)(z_lds + c * ZRS + tcol + 8) = z1;
        }
        __syncthreads();

        *(u32x4*)(u_lds + (tid >> 4) * URS + (tid & 15) * 8) = tail;
        if constexpr (FEAT != 0) {
            // the output gate of this step, outside any test: every wavefront carries every piece on.  (Behind the
            // MFMAs instead, with both accumulators live, it spills 13 registers and measured 1 % slower.)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                c2[r4] = feat(c2[r4], car2[r4], fw[1][r4]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- gate with x2 and store, coalesced
        if (WHOLE || ts + lane * 8 < t_end) {
            uint32_t lo = lane_b;
            asm volatile("" : "+v"(lo));
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                if (!WHOLE && !rlive[r4]) continue;
                const u32x4 zz = *(const u32x4*)(z_lds + (4 * r4 + w) * ZRS + lane * 8);
                u32x4 o = zz;
                if (POST) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[j] = pack_bf2(bf_lo(zz[j]) * bf_lo(c2[r4][j]), bf_hi(zz[j]) * bf_hi(c2[r4][j]));
                }
                st16<NT>((bf16_t*)((char*)(po[r4] + ts) + lo), o);
            }
        }
    };
    // Steps in the middle of a segment take the form without tests.  With a branch around a request or a store the
    // compiler must assume that nothing younger is in flight, and waits for everything at the next use of a prefetched
    // row: the stores of the step before included, a write's whole latency per step.  Counted exactly, that wait leaves
    // the four stores outstanding.  The last step of a segment keeps its tests; the prologue's requests are waited for
    // in full before the first whole step so that its counts start from a known state.
    int64_t ts = t_begin;
    if (c_live == 16 && ts + 2 * TL <= t_end) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0)
        for (; ts + 2 * TL <= t_end; ts += TL) step(ts, std::true_type{});
    }
    for (; ts < t_end; ts += TL) step(ts, std::false_type{});
}

}  // namespace

namespace {
int mr_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* h,
                int taps_reversed, const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L,
                int64_t G, int K, void* stream, const float* ftaps);
}

extern "C" int hyena_mr_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* h,
                            int taps_reversed, const float* bias, int bias_mode, void* out, int64_t B, int64_t D,
                            int64_t L, int64_t G, int K, void* stream) {
    return mr_fwd_impl("hyena_mr_fwd", x1, x2, v, h, taps_reversed, bias, bias_mode, out, B, D, L, G, K, stream, nullptr);
}

extern "C" int hyena_fir_layer_fwd_rows(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                                        const float* feat_taps, int feat_len, const float* h, int taps_reversed,
                                        const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L,
                                        int64_t G, int K, void* stream) {
    const char* who = "hyena_fir_layer_fwd_rows";
    if (!feat_taps) return hyena_fail(HYENA_EINVAL, "%s: feat_taps is required", who);
    if (feat_len != 3) return hyena_fail(HYENA_ENOSUP, "%s: featurizer of %d taps (3)", who, feat_len);
    if (!x1 || !x1->ptr || !x2 || !x2->ptr || !v || !v->ptr)
        return hyena_fail(HYENA_EINVAL, "%s: the three row sets of the projection are required", who);
    if (bias_mode != HYENA_BIAS_NONE && bias_mode != HYENA_BIAS_GATED_FP32)
        return hyena_fail(HYENA_ENOSUP, "%s: bias_mode %d (none or gated float32)", who, bias_mode);
    // Short filters in the short-filter orientation on tensors that stay in the last-level cache: the direct-form
    // kernel (one lane per octet of a row; 52 against 67 us at B = 1, L = 8192, D = 4096, K = 7).  With the featurizer
    // on top that kernel is bound by its vector instructions, so tensors that stream take the matrix-core kernel
    // (367 against 384 us at B = 8).
    const bool resident = 8.0 * (double)B * (double)D * (double)L <= 384e6;
    if (K >= 2 && K <= 8 && bias_mode == HYENA_BIAS_NONE && taps_reversed && h && resident)
        return hyena_se_layer_rows(x1, x2, v, feat_taps, h, out, B, D, L, G, K, stream, who);
    return mr_fwd_impl(who, x1, x2, v, h, taps_reversed, bias, bias_mode, out, B, D, L, G, K, stream, feat_taps);
}

namespace {
int mr_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* h,
                int taps_reversed, const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L,
                int64_t G, int K, void* stream, const float* ftaps) {
    if (!x1 || !x1->ptr || !h || !out) return hyena_fail(HYENA_EINVAL, "%s: x1, h and out are required", who);
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld L=%lld G=%lld", who, (long long)B,
                          (long long)D, (long long)L, (long long)G);
    if (K < 1 || K > 128) return hyena_fail(HYENA_ENOSUP, "%s: K=%d outside 1..128", who, K);
    if (bias_mode < 0 || bias_mode > 4 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "%s: bias_mode %d needs a bias pointer", who, bias_mode);
    if (L % 8 != 0 || !rows_aligned8(x1) || !rows_aligned8(x2) || !rows_aligned8(v) || (((uintptr_t)out) & 15))
        return hyena_fail(HYENA_EALIGN, "%s: L and strides must be multiples of 8, pointers 16-byte aligned", who);
    // the kernels do the channel arithmetic in 32 bits: reject maps and sizes that would wrap or divide by zero
    if (!rows_valid(x1) || !rows_valid(x2) || !rows_valid(v) || B * D >= (1LL << 31) || L / 8 >= (1LL << 31))
        return hyena_fail(HYENA_EINVAL, "%s: B*D, L/8 and the channel map must fit 31 bits", who);
    if (B == 0 || L == 0) return 0;
    const bool pre = v && v->ptr, post = x2 && x2->ptr;

    // Segments along L, chosen by a cost model fitted to measurements on one MI355X: a segment costs its length
    // plus about 160 samples for the halo and the fragment build; segments longer than 2048 samples stream about
    // 5 % slower per doubling (with short ones the blocks of a row set work at many offsets at once, which the
    // memory system serves faster); 768 blocks are resident at a time (3 per CU) and the last round is on average
    // half empty.
    const int64_t rows = B * G * ((D / G + 15) / 16);          // (batch, slab) pairs
    int64_t nseg = 1;
    {
        double best = 0.0;
        for (int64_t sl = 1024; ; sl *= 2) {
            const int64_t c = (L + sl - 1) / sl;
            const double nb = (double)(rows * c);
            double cost = ((double)sl + 160.0) * (nb <= 768.0 ? 1.0 : nb / 768.0 + 0.5);
            for (int64_t x = sl; x > 2048; x /= 2) cost *= 1.05;
            if (best == 0.0 || cost < best) { best = cost; nseg = c; }
            if (sl >= L) break;
        }
    }
    { const int64_t x = hyena_override(HYENA_OV_MR_NSEG); if (x >= 1) nseg = x; }
    int64_t seg_len = (L + nseg - 1) / nseg;
    seg_len = (seg_len + TL - 1) / TL * TL;
    nseg = (L + seg_len - 1) / seg_len;
    const int64_t nblk = rows * nseg;
    if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);

    RowMap m1 = make_rowmap(x1), m2 = make_rowmap(post ? x2 : nullptr), mv = make_rowmap(pre ? v : nullptr);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)nblk);
    const int dg = (int)(D / G);
    bool ok = false;
    // activations larger than the last-level cache stream through it: use non-temporal accesses then
    bool nt = 8.0 * (double)B * (double)D * (double)L > 384e6;
    { const int64_t x = hyena_override(HYENA_OV_MR_NT); if (x >= 0) nt = x != 0; }
    const bool full = K > 98;
#define MR_LAUNCH(P, Q, M, N, F)                                                                              \
    hipLaunchKernelGGL((mr_fir_kernel<P, Q, M, N, F>), grid, dim3(256), 0, s, m1, m2, mv, h, K, taps_reversed, \
                       bias, (bf16_t*)out, D, L, dg, seg_len, (int)nseg, ftaps)
#define MR_CASE(P, Q, M)                                                                                      \
    if (pre == P && post == Q && bias_mode == M) {                                                            \
        if (nt && full) MR_LAUNCH(P, Q, M, true, true);                                                       \
        else if (nt) MR_LAUNCH(P, Q, M, true, false);                                                         \
        else if (full) MR_LAUNCH(P, Q, M, false, true);                                                       \
        else MR_LAUNCH(P, Q, M, false, false);                                                                \
        ok = true;                                                                                            \
    }
#define MR_FEAT(M)                                                                                            \
    if (ftaps && bias_mode == M) {                                                                            \
        if (nt && full) hipLaunchKernelGGL((mr_fir_kernel<true, true, M, true, true, 3>), grid, dim3(256), 0, s, m1, m2, mv, h, K, taps_reversed, bias, (bf16_t*)out, D, L, dg, seg_len, (int)nseg, ftaps);   \
        else if (nt) hipLaunchKernelGGL((mr_fir_kernel<true, true, M, true, false, 3>), grid, dim3(256), 0, s, m1, m2, mv, h, K, taps_reversed, bias, (bf16_t*)out, D, L, dg, seg_len, (int)nseg, ftaps);    \
        else if (full) hipLaunchKernelGGL((mr_fir_kernel<true, true, M, false, true, 3>), grid, dim3(256), 0, s, m1, m2, mv, h, K, taps_reversed, bias, (bf16_t*)out, D, L, dg, seg_len, (int)nseg, ftaps); \
        else hipLaunchKernelGGL((mr_fir_kernel<true, true, M, false, false, 3>), grid, dim3(256), 0, s, m1, m2, mv, h, K, taps_reversed, bias, (bf16_t*)out, D, L, dg, seg_len, (int)nseg, ftaps);         \
        ok = true;                                                                                            \
    }
    if (ftaps) {
        MR_FEAT(HYENA_BIAS_GATED_FP32)
        MR_FEAT(HYENA_BIAS_NONE)
        if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: this bias mode has no featurizer kernel", who);
        return hyena_check_launch(who);
    }
#undef MR_FEAT
    MR_CASE(true, true, HYENA_BIAS_GATED_FP32)
    MR_CASE(true, true, HYENA_BIAS_NONE)
    MR_CASE(true, true, HYENA_BIAS_ADD)
    MR_CASE(false, false, HYENA_BIAS_NONE)
    MR_CASE(false, false, HYENA_BIAS_ADD)
    MR_CASE(false, false, HYENA_BIAS_GATED_FP32)
    MR_CASE(true, true, HYENA_BIAS_ADD_FP32)
    MR_CASE(false, false, HYENA_BIAS_ADD_FP32)
    MR_CASE(true, true, HYENA_BIAS_GATED_BF16)
    MR_CASE(false, false, HYENA_BIAS_GATED_BF16)
#undef MR_CASE
#undef MR_LAUNCH
    if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: this gate/bias combination has no kernel", who);
    return hyena_check_launch(who);
}
}  // namespace
