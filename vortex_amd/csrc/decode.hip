// Cached decode step: FIR over a ring-buffer cache and the modal IIR state
// update, each fused with the gating multiplies.  Both are HBM-bound: the FIR
// step has to read its whole cache once per token, but it writes back one slot
// instead of shifting the cache as vortex/model/engine.py:443-447 does.
#include "common.h"

namespace {

// ---------------------------------------------------------------- fused featurizer step
// Device copy of hyena_proj_step.  The featurizer (short FIR over the 3D projection
// channels, vortex/model/model.py:325-330) is evaluated for exactly the channels a
// lane needs, and the lane that evaluates a channel also writes the new sample into
// that channel's ring slot, so no other lane ever reads a slot that is being replaced.
struct ProjArgs {
    const bf16_t* u;
    int64_t u_bs;
    bf16_t* ring;
    int Rf, pos, C;
    const int* pos_dev;    // when set, the ring position lives in device memory and pos is ignored
    const float* w;        // [Rf+1][C], tap-major
    const float* bias;     // [C] or null
    uint32_t ch_inner, ch_outer, gate_stride, ch_stride;
    int flip;
    __device__ __forceinline__ uint32_t chan(uint32_t gate, uint32_t d) const {
        return (d / ch_inner) * ch_outer + gate * gate_stride + (d % ch_inner) * ch_stride;
    }
    // a device-resident position is reduced mod Rf so that a stale or foreign counter cannot index past the ring
    __device__ __forceinline__ void resolve_pos() {
        if (pos_dev) pos = (int)((uint32_t)*pos_dev % (uint32_t)Rf);
    }
};

// z[j] = bf16( sum_i w[i][c0+j]*slot_i[c0+j] + w[Rf][c0+j]*u[c0+j] (+ bias) ) for 8 consecutive channels.
// RF > 0: the cache depth is known at compile time and every operand (projection row, RF slots, RF+1 tap rows, bias)
// is requested before the first one is used, one memory round trip instead of one per slot.  RF == 0: any depth, one
// slot after the other.  Both add the terms in the same order.
template <int RF>
__device__ __forceinline__ u32x4 proj_step8_n(const ProjArgs& pj, int64_t b, uint32_t c0, float* z) {
    const u32x4 un = *(const u32x4*)(pj.u + b * pj.u_bs + c0);
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    const bf16_t* rb = pj.ring + (b * pj.Rf) * pj.C + c0;
    auto add = [&](const f32x4& t0, const f32x4& t1, const u32x4& q) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] = fmaf(j < 2 ? t0[2 * j] : t1[2 * j - 4], bf_lo(q[j]), acc[2 * j]);
            acc[2 * j + 1] = fmaf(j < 2 ? t0[2 * j + 1] : t1[2 * j - 3], bf_hi(q[j]), acc[2 * j + 1]);
        }
    };
    f32x4 b0 = {0.f, 0.f, 0.f, 0.f}, b1 = {0.f, 0.f, 0.f, 0.f};
    if (RF > 0) {
        constexpr int N = RF > 0 ? RF : 1;
        u32x4 q[N];
        f32x4 t0[N + 1], t1[N + 1];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int s = pj.pos + i;
            if (s >= N) s -= N;
            q[i] = *(const u32x4*)(rb + (int64_t)s * pj.C);
        }
#pragma unroll
        for (int i = 0; i <= N; ++i) {
            t0[i] = *(const f32x4*)(pj.w + (int64_t)i * pj.C + c0);
            t1[i] = *(const f32x4*)(pj.w + (int64_t)i * pj.C + c0 + 4);
        }
        if (pj.bias) {
            b0 = *(const f32x4*)(pj.bias + c0);
            b1 = *(const f32x4*)(pj.bias + c0 + 4);
        }
#pragma unroll
        for (int i = 0; i < N; ++i) add(t0[i], t1[i], q[i]);
        add(t0[N], t1[N], un);
    } else {
        for (int i = 0; i < pj.Rf; ++i) {
            int s = pj.pos + i;
            if (s >= pj.Rf) s -= pj.Rf;
            const u32x4 q = *(const u32x4*)(rb + (int64_t)s * pj.C);
            const f32x4 t0 = *(const f32x4*)(pj.w + (int64_t)i * pj.C + c0);
            const f32x4 t1 = *(const f32x4*)(pj.w + (int64_t)i * pj.C + c0 + 4);
            add(t0, t1, q);
        }
        const f32x4 h0 = *(const f32x4*)(pj.w + (int64_t)pj.Rf * pj.C + c0);
        const f32x4 h1 = *(const f32x4*)(pj.w + (int64_t)pj.Rf * pj.C + c0 + 4);
        add(h0, h1, un);
        if (pj.bias) {
            b0 = *(const f32x4*)(pj.bias + c0);
            b1 = *(const f32x4*)(pj.bias + c0 + 4);
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = round_bf(acc[j] + (j < 4 ? b0[j & 3] : b1[j & 3]));
    return un;                                          // the caller stores it into the oldest slot
}

// The depths short featurizers have (2, 3 and 4 taps) take the one-round-trip form.
__device__ __forceinline__ u32x4 proj_step8(const ProjArgs& pj, int64_t b, uint32_t c0, float* z) {
    if (pj.Rf == 2) return proj_step8_n<2>(pj, b, c0, z);
    if (pj.Rf == 1) return proj_step8_n<1>(pj, b, c0, z);
    if (pj.Rf == 3) return proj_step8_n<3>(pj, b, c0, z);
    return proj_step8_n<0>(pj, b, c0, z);
}

__device__ __forceinline__ void proj_store8(const ProjArgs& pj, int64_t b, uint32_t c0, u32x4 un) {
    *(u32x4*)(pj.ring + ((b * pj.Rf) + pj.pos) * pj.C + c0) = un;
}

// ---------------------------------------------------------------- FIR step
// Block = NSG wavefronts over the same 512 channels; wavefront sg handles cache
// slots sg, sg+NSG, ... so every load instruction reads 1 KiB of one slot row.
// NSG = 8 for deep caches (enough loads in flight to cover HBM latency), 2 for shallow ones.
// Ring layout [B][D/cb][R][cb] with cb = D (plain [B][R][D]) or a multiple of 512: channels contiguous, so the
// slot written back is one coalesced row per batch element and channel block.  With cb = 512 the R slots a block
// reads are one contiguous run of R KiB instead of 1 KiB pieces 2*D bytes apart, which deep caches stream faster.
// FEAT != 0: the gates come from the fused featurizer step (ProjArgs) instead of x1, x2, v.
//
// NBT > 1 (deep caches with a `far` buffer [B][NBT][D] float32): the part of the sum that the cache already
// determines is formed for NBT tokens at a time.  Token counter cnt (ring slot cnt % R); a block's window starts
// when j = (cnt + blockIdx.x + blockIdx.y) % NBT is 0.  Then the block reads its whole cache once and forms, beside
// this token's sum, far[j'] = sum_{i >= j'} w[i - j'] * state_i for j' = 1 .. NBT-1: what the samples cached NOW
// will add to the outputs j' tokens later (i counts from the oldest slot; the j' oldest have dropped out by then).
// The other NBT-1 tokens of the window read far[j] and only the j newest slots: y = far[j] + sum_{k=1..j}
// w[R-k] * (k-th newest) + w[R] * u.  Windows are staggered over the blocks, so every launch moves about 1/NBT of
// the cache.  all_heavy != 0 makes every block rebuild its window from the cache as it stands (the first step on a
// cache, or after anything else wrote to it): a block at position j then forms far[j'] for j' > j over the slots
// that were cached when its window began, sum_{i = j'-j}^{R-1-j} w[i + j - j'] * state_i.
template <bool PRE, bool POST, int BIAS, bool GROUPED, int NSG, int FEAT, int NBT>
__global__ __launch_bounds__(64 * NSG) void fir_step_kernel(const bf16_t* __restrict__ x1, const bf16_t* __restrict__ x2,
                                                       const bf16_t* __restrict__ v, int64_t in_bs, ProjArgs pj,
                                                       bf16_t* __restrict__ ring, int R, int cb, int pos,
                                                       const int* __restrict__ pos_dev, int period,
                                                       float* __restrict__ far, int all_heavy,
                                                       const float* __restrict__ w, const float* __restrict__ bias,
                                                       bf16_t* __restrict__ out, int64_t out_bs, int64_t D, int dg) {
    extern __shared__ float smem[];
    if (pos_dev) pos = (int)((uint32_t)*pos_dev % (uint32_t)period);      // period = R, or lcm(NBT, R) with a far buffer
    const int jw = NBT > 1 ? (int)((uint32_t)(pos + blockIdx.x + blockIdx.y) % (uint32_t)NBT) : 0;   // place in the window
    const bool heavy = NBT == 1 || all_heavy != 0 || jw == 0;
    if (NBT > 1) pos = (int)((uint32_t)pos % (uint32_t)R);
    if (FEAT != 0) pj.resolve_pos();
    const int tid = threadIdx.x, oc = tid & 63, sg = tid >> 6;
    const int64_t dblk = (int64_t)blockIdx.x * 512;
    const int64_t d0 = dblk + oc * 8;
    const int64_t b = blockIdx.y;
    const bool live = d0 < D;
    const int W = R + 1;

    const int ng = GROUPED ? (512 / dg) : 0;
    float* wl = smem + (NBT - 1) * ng;      // [W][ng]  taps of the block's groups, transposed, behind NBT-1 rows of zeros
    float* red = smem + (GROUPED ? (W + NBT - 1) * ng : 0);   // [NSG-1][NBT][2][64][4]
    float* zs = red + (NSG - 1) * NBT * 512;      // [3][512] gates of the block's channels (fused featurizer only)
    const int gl = GROUPED ? (oc * 8) / dg : 0;
    constexpr int UF = 8;                   // cache slots in flight per lane (16, a 127-slot cache in one batch, needs 165 registers: one block per CU, 8 % slower)
    // ring [B][D/cb][R][cb]: the block's 512 channels lie inside one channel block (cb = D is the plain [B][R][D])
    const uint32_t cblk = (uint32_t)d0 / (uint32_t)cb;
    const int64_t roff = ((b * (int64_t)((uint32_t)D / (uint32_t)cb) + cblk) * R) * cb + (d0 - (int64_t)cblk * cb);
    const bf16_t* rb = ring + roff;
    const u32x4 zero4 = {0, 0, 0, 0};

    // The main loop covers the slots that were cached when the block's window began: all R of them, except in a
    // rebuild at place jw of a window, where the jw newest belong to the near part below.
    const int Rl = R - (NBT > 1 ? jw : 0);
    auto load_batch = [&](int i, u32x4* q) {
#pragma unroll
        for (int k = 0; k < UF; ++k) {
            const int ii = i + NSG * k;
            int s = pos + ii;
            if (s >= R) s -= R;
            q[k] = (live && ii < Rl) ? *(const u32x4*)(rb + (int64_t)s * cb) : zero4;
        }
    };
    float acc[NBT][8];
#pragma unroll
    for (int jj = 0; jj < NBT; ++jj)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[jj][c] = 0.f;
    // tap of slot ii for the output jj tokens ahead (jj = 0: this token) is w[ii - jj]; the rows of zeros ahead of the
    // LDS table stand for ii < jj (a slot that has dropped out of the cache by then)
    auto fma_batch = [&](int i, const u32x4* q) {
#pragma unroll
        for (int k = 0; k < UF; ++k) {
            int ii = i + NSG * k;
            if (ii >= R) ii = R - 1;        // the slot was loaded as zeros; any finite tap will do
#pragma unroll
            for (int jj = 0; jj < NBT; ++jj) {
                if (GROUPED) {
                    const float t = wl[(ii - jj) * ng + gl];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        acc[jj][2 * j] = fmaf(t, bf_lo(q[k][j]), acc[jj][2 * j]);
                        acc[jj][2 * j + 1] = fmaf(t, bf_hi(q[k][j]), acc[jj][2 * j + 1]);
                    }
                } else if (live && ii >= jj) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        acc[jj][2 * j] = fmaf(w[(d0 + 2 * j) * W + ii - jj], bf_lo(q[k][j]), acc[jj][2 * j]);
                        acc[jj][2 * j + 1] = fmaf(w[(d0 + 2 * j + 1) * W + ii - jj], bf_hi(q[k][j]), acc[jj][2 * j + 1]);
                    }
                }
            }
        }
    };

    // the first batch of cache reads goes out before the tap table is staged, so HBM is busy from the start
    u32x4 q0[UF];
    if (heavy) load_batch(sg, q0);
    // the output wavefront requests its gates and bias now, so that they arrive with the cache instead of costing
    // a second round trip to memory after the reduction
    u32x4 a1 = zero4, av = zero4, a2 = zero4;
    f32x4 bs0 = {0.f, 0.f, 0.f, 0.f}, bs1 = bs0;
    if (sg == 0 && live) {
        if (FEAT == 0) {
            a1 = *(const u32x4*)(x1 + b * in_bs + d0);
            if (PRE) av = *(const u32x4*)(v + b * in_bs + d0);
            if (POST) a2 = *(const u32x4*)(x2 + b * in_bs + d0);
        }
        if (BIAS != HYENA_BIAS_NONE) {
            bs0 = *(const f32x4*)(bias + d0);
            bs1 = *(const f32x4*)(bias + d0 + 4);
        }
    }
    // and, for the same reason, what the end of the step reads: the taps on the new sample (k = 0) and on the k-th
    // newest slot, those slots (the near part of a window), and inside a window its far sums
    float tk[NBT][GROUPED ? 1 : 8];
    u32x4 qn[NBT > 1 ? NBT - 1 : 1];
    f32x4 f0 = {0.f, 0.f, 0.f, 0.f}, f1 = f0;
#pragma unroll
    for (int k = 0; k < NBT; ++k)
#pragma unroll
        for (int c = 0; c < (GROUPED ? 1 : 8); ++c) tk[k][c] = 0.f;
#pragma unroll
    for (int k = 1; k < NBT; ++k) qn[k - 1] = zero4;
    if (sg == 0 && live) {
        const int64_t gw = GROUPED ? (dblk / dg + gl) * W : 0;
#pragma unroll
        for (int k = 0; k < NBT; ++k) {
            if (k <= jw) {
#pragma unroll
                for (int c = 0; c < (GROUPED ? 1 : 8); ++c) tk[k][c] = GROUPED ? w[gw + R - k] : w[(d0 + c) * W + R - k];
                if (k > 0) {
                    int sl = pos - k;
                    if (sl < 0) sl += R;
                    qn[k - 1] = *(const u32x4*)(rb + (int64_t)sl * cb);
                }
            }
        }
        if (NBT > 1 && !heavy) {
            f0 = *(const f32x4*)(far + ((b * NBT + jw) * D + d0));
            f1 = *(const f32x4*)(far + ((b * NBT + jw) * D + d0 + 4));
        }
    }
    // Fused featurizer: the block's 3 x 512 projection channels are 192 pieces of 8; thread p evaluates piece p
    // (its loads overlap the cache reads above) and leaves the gates in LDS for the wavefront that writes the output.
    if (FEAT != 0) {
        for (int p = tid; p < 192; p += 64 * NSG) {
            // FEAT 3: columns in projection order (3*dl + gate); FEAT 1: gate-major (gate*512 + dl)
            const uint32_t dl0 = FEAT == 3 ? 0 : (uint32_t)(8 * p) & 511;
            const uint32_t ch = FEAT == 3 ? 3 * (uint32_t)dblk + 8 * p : pj.chan((uint32_t)(8 * p) >> 9, (uint32_t)dblk + dl0);
            const bool ok = FEAT == 3 ? 3 * (uint32_t)dblk + 8 * p < 3 * (uint32_t)D : (uint32_t)dblk + dl0 < (uint32_t)D;
            if (ok) {
                float z[8];
                const u32x4 un = proj_step8(pj, b, ch, z);
                proj_store8(pj, b, ch, un);
#pragma unroll
                for (int k = 0; k < 8; ++k) zs[8 * p + k] = z[k];
            }
        }
    }
    float h0[8];                            // taps on the new sample
    if (NBT > 1 && !heavy) {
        // ---- inside a window: far[jw] plus the jw newest slots, all on the output wavefront
        if (FEAT != 0) __syncthreads();     // the gates are in LDS
        if (sg != 0 || !live) return;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[0][c] = c < 4 ? f0[c & 3] : f1[c & 3];
    } else {
        if (GROUPED) {
            const int64_t g0 = dblk / dg;
            const int64_t gmax = (D + dg - 1) / dg;
            for (int e = tid; e < (NBT - 1) * ng; e += 64 * NSG) smem[e] = 0.f;
            if ((W & 3) == 0) {
                for (int e = tid; e < (W / 4) * ng; e += 64 * NSG) {      // groups fastest: conflict-free LDS stores
                    const int i4 = (e / ng) * 4, gl2 = e - (e / ng) * ng;
                    f32x4 t = {0.f, 0.f, 0.f, 0.f};
                    if (g0 + gl2 < gmax) t = *(const f32x4*)(w + (g0 + gl2) * W + i4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) wl[(i4 + k) * ng + gl2] = t[k];
                }
            } else {
                for (int e = tid; e < W * ng; e += 64 * NSG) {
                    const int i = e / ng, gl2 = e - i * ng;
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
            for (int jj = 0; jj < NBT; ++jj)
#pragma unroll
                for (int c = 0; c < 8; ++c)          // 16 B per lane, lanes contiguous
                    red[((((sg - 1) * NBT + jj) * 2 + (c >> 2)) * 64 + oc) * 4 + (c & 3)] = acc[jj][c];
        }
        __syncthreads();          // also orders every read of slot `pos` before its overwrite below
        if (sg != 0 || !live) return;
        constexpr int RED_UNROLL = NBT > 1 ? 1 : NSG - 1;      // with far sums: one wavefront's partial sums at a time
#pragma unroll RED_UNROLL
        for (int k = 0; k < NSG - 1; ++k) {
#pragma unroll
            for (int jj = 0; jj < NBT; ++jj)
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[jj][c] += red[(((k * NBT + jj) * 2 + (c >> 2)) * 64 + oc) * 4 + (c & 3)];
        }
        if (NBT > 1) {
            // what the cache adds to the later tokens of this window
#pragma unroll
            for (int jj = 1; jj < NBT; ++jj) {
                if (jw + jj < NBT) {
                    float* fp = far + ((b * NBT + jw + jj) * D + d0);
                    *(f32x4*)fp = f32x4{acc[jj][0], acc[jj][1], acc[jj][2], acc[jj][3]};
                    *(f32x4*)(fp + 4) = f32x4{acc[jj][4], acc[jj][5], acc[jj][6], acc[jj][7]};
                }
            }
        }
    }
    {
        // taps on the new sample, and (with far sums) the near part: the jw newest slots, which entered the cache
        // after the window's far sums were formed
#pragma unroll
        for (int c = 0; c < 8; ++c) h0[c] = tk[0][GROUPED ? 0 : c];
#pragma unroll
        for (int k = 1; k < NBT; ++k) {
            if (k <= jw) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float t0 = tk[k][GROUPED ? 0 : 2 * j];
                    const float t1 = tk[k][GROUPED ? 0 : 2 * j + 1];
                    acc[0][2 * j] = fmaf(t0, bf_lo(qn[k - 1][j]), acc[0][2 * j]);
                    acc[0][2 * j + 1] = fmaf(t1, bf_hi(qn[k - 1][j]), acc[0][2 * j + 1]);
                }
            }
        }
    }

    if (FEAT != 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float g2[2], g1[2], gv[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int dl = oc * 8 + 2 * j + e;
                g2[e] = FEAT == 3 ? zs[3 * dl] : zs[dl];
                g1[e] = FEAT == 3 ? zs[3 * dl + 1] : zs[512 + dl];
                gv[e] = FEAT == 3 ? zs[3 * dl + 2] : zs[1024 + dl];
            }
            a1[j] = pj.flip ? pack_bf2(g2[0], g2[1]) : pack_bf2(g1[0], g1[1]);
            a2[j] = pj.flip ? pack_bf2(g1[0], g1[1]) : pack_bf2(g2[0], g2[1]);
            av[j] = pack_bf2(gv[0], gv[1]);
        }
    }
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
            float yy = fmaf(h0[c], uu[e], acc[0][c]);
            const float bc = c < 4 ? bs0[c & 3] : bs1[c & 3];
            if (BIAS == HYENA_BIAS_GATED_FP32) yy = fmaf(bc, uu[e], yy);
            if (BIAS == HYENA_BIAS_ADD) yy += bc;
            yy = round_bf(yy);
            if (POST) yy *= (e ? bf_hi(a2[j]) : bf_lo(a2[j]));
            y[e] = yy;
        }
        o[j] = pack_bf2(y[0], y[1]);
    }
    const u32x4 ov = {o[0], o[1], o[2], o[3]};
    *(u32x4*)(out + b * out_bs + d0) = ov;
    const u32x4 uv = {up[0], up[1], up[2], up[3]};
    *(u32x4*)(ring + roff + (int64_t)pos * cb) = uv;
}

// ---------------------------------------------------------------- IIR step
// The floats of modal state that one lane owns, loaded and stored as one vector.
template <int N>
struct alignas(4 * N) StateVec {
    float f[N];
    __device__ __forceinline__ float& operator[](int i) { return f[i]; }
    __device__ __forceinline__ float operator[](int i) const { return f[i]; }
};

// LPB lanes share one channel: each holds 16 bytes of its modal state (4 real or 2 complex
// states; a channel with fewer than 16 bytes of state has one lane), so state traffic is fully
// coalesced.  A lane walks NB batch elements of that channel with the poles and residues held in registers and the NB state loads issued together, which
// puts enough bytes in flight to cover HBM latency.  The residue-weighted sum is reduced with
// xor shuffles inside the lane group.
// FEAT (fused featurizer step): 0 none; 2 lanes 0..2 of a lane group evaluate gates x2, x1, v of their channel
// with scalar loads (any channel map); 1 / 3 the block's first wavefronts evaluate the gates of all its
// channels with 16-byte loads (unit-stride / interleaved map, as in the FIR step) and hand them over in LDS.
//
// WIN > 1: the state is read and written once per window of WIN tokens instead of every token.  With S the
// state before the window's first token t0,  s_{t0+j} = p^(j+1) S + sum_{k<=j} p^k u_{t0+j-k},  so
//   Re sum_s r s_{t0+j} = far[j] + sum_{k<=j} g[k] u_{t0+j-k},   far[j] = Re sum_s r p^(j+1) S,   g[k] = Re sum_s r p^k.
// Windows are staggered over the batch elements, place jw = (cnt + b) % WIN; a block row takes NB batch elements of
// one residue class b % WIN, so that they are at the same place of their windows.  On the first token of its window
// (mode 1) a batch element's blocks fold the inputs of the window before (kept in `hist`, [B][WIN][D] bf16, slot =
// token % WIN) into the stored state, S = p^WIN S' + sum_k p^k u_{t0-1-k}, write it back and form far[0..WIN-1]
// ([B][WIN][D] float32).  On the other tokens (mode 2) nothing of the state or the poles is touched: the work is one
// lane per channel, 256 channels per block, and the rest of the batch element's blocks leave at once.
// `warm` = tokens stepped this way since the stored state was last exact (saturating at WIN): a batch element steps
// the plain way (mode 0) until its first window begins (warm >= jw fails), and a window's first token folds WIN
// pending inputs only if the window before it existed (warm >= WIN).  flush != 0 (mode 3): no token is processed; the
// pending inputs are folded into the state, which is exact afterwards.
struct WinArgs {
    bf16_t* hist;          // [B][WIN][D]
    float* far;            // [B][WIN][D]
    const float* g;        // [G][WIN]
    int cnt;               // token index modulo WIN
    const int* cnt_dev;    // when set, the counter lives in device memory
    int warm, flush;
    // compact != 0: one-dimensional grid of nhb blocks for the batch elements at the head of their window (NB of them
    // per block, nxh blocks of 256 state lanes along the channels) followed by nxl blocks of 256 channels for each of
    // those inside a window; only valid once every window is open (warm >= WIN - 1) and not for a flush
    int compact;
    uint32_t nhb, nxh, nxl;
};

// Sum over the N lanes (a power of two up to 16, aligned) that share a channel, in the order of an xor butterfly: data-
// parallel-primitive operands of the additions themselves (quad swaps, then the mirrored half row / row, whose lanes
// hold the other half's partial sum by then).
template <int CTRL>
__device__ __forceinline__ float dpp_take(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
template <int N>
__device__ __forceinline__ float lane_group_sum(float x) {
    static_assert(N >= 1 && N <= 16 && (N & (N - 1)) == 0, "lane groups of 1, 2, 4, 8 or 16");
    if (N >= 2) x += dpp_take<0xB1>(x);        // quad_perm [1, 0, 3, 2]
    if (N >= 4) x += dpp_take<0x4E>(x);        // quad_perm [2, 3, 0, 1]
    if (N >= 8) x += dpp_take<0x141>(x);       // row_half_mirror
    if (N >= 16) x += dpp_take<0x140>(x);      // row_mirror
    return x;
}

template <int S, bool CPLX, int FEAT, int NB, int WIN>
__global__ __launch_bounds__(256) void iir_step_kernel(const bf16_t* __restrict__ x1, const bf16_t* __restrict__ x2,
                                                       const bf16_t* __restrict__ v, int64_t in_bs, ProjArgs pj,
                                                       float* __restrict__ state, const float* __restrict__ poles,
                                                       const float* __restrict__ residues,
                                                       const float* __restrict__ Dcoef, int d_is_bf16,
                                                       void* __restrict__ out, int out_is_fp32, int64_t out_bs,
                                                       int64_t B, int64_t D, int dg, WinArgs wa) {
    constexpr int FPS = CPLX ? 2 : 1;              // floats per state
    constexpr int VEC = S * FPS >= 4 ? 4 : S * FPS; // floats of state per lane (1 and 2 only where a channel has no more)
    constexpr int LPB = S * FPS / VEC;             // lanes per channel
    using fvec = StateVec<VEC>;
    constexpr int ND = 256 / LPB;                  // channels per block
    constexpr bool VFEAT = FEAT == 1 || FEAT == 3;
    static_assert(WIN <= 1 || (VEC == 4 && FEAT != 2), "windows: 16-byte state pieces, vector featurizer");
    __shared__ float zs[VFEAT ? (WIN > 1 && 3 * 256 > NB * 3 * ND ? 3 * 256 : NB * 3 * ND) : 1];  // [j][gate-major or interleaved][channel]
    if (FEAT != 0) pj.resolve_pos();
    // ---- what this batch element does with this token: 0 plain step, 1 first token of a window, 2 inside a window, 3 flush
    int mode = 0, jw = 0, cnt = 0, npend = 0;
    uint32_t xb = blockIdx.x;                      // block along the channels (256 state lanes, or 256 channels inside a window)
    int64_t brow = blockIdx.y;                     // windows: the batch element of this block
    if (WIN > 1) {
        cnt = wa.cnt_dev ? (int)((uint32_t)*wa.cnt_dev % (uint32_t)WIN) : wa.cnt;
        if (wa.compact) {
            if (blockIdx.x < wa.nhb) {
                const uint32_t hr = blockIdx.x / wa.nxh;
                xb = blockIdx.x - hr * wa.nxh;
                jw = 0;
                brow = ((int64_t)hr * NB) * WIN + (WIN - cnt) % WIN;       // and the NB - 1 next ones of its residue class
            } else {
                const uint32_t e = blockIdx.x - wa.nhb, lr = e / wa.nxl;
                xb = e - lr * wa.nxl;
                jw = 1 + (int)(lr % (uint32_t)(WIN - 1));
                brow = (int64_t)(lr / (uint32_t)(WIN - 1)) * WIN + (jw - cnt + WIN) % WIN;
            }
            if (brow >= B) return;
        } else {
            jw = (int)((uint32_t)(cnt + blockIdx.y) % (uint32_t)WIN);      // the row's residue class decides its place in the window
        }
        if (wa.flush) {
            mode = 3;                              // inputs since the window began: jw of them, or a whole window
            npend = jw > 0 ? (wa.warm >= jw ? jw : 0) : (wa.warm >= WIN ? WIN : 0);
            if (npend == 0) return;                // the stored state is exact already
        } else if (wa.warm >= jw) {
            mode = jw == 0 ? 1 : 2;
            npend = wa.warm >= WIN ? WIN : 0;
        }
    }
    // batch element j of this block row: NB consecutive ones, or (windows; NB > 1 in the compact grid only) NB of one
    // residue class
    auto bj = [&](int j) -> int64_t {
        if (WIN > 1) return brow + (int64_t)j * WIN;
        return (int64_t)blockIdx.y * NB + j;
    };
    if (WIN > 1 && mode == 2) {
        // ---- inside a window: far[jw] and the inputs since the window began; one lane per channel
        const uint32_t dblk = xb * 256;
        if (dblk >= (uint32_t)D) return;
        const uint32_t dch = dblk + threadIdx.x;
        const bool ok = dch < (uint32_t)D;
        const uint32_t dc = ok ? dch : 0;
        const int64_t b = brow;
        if (b >= B) return;
        // everything this token reads besides the gates is requested first, unconditionally (the slots of the window's
        // inputs that are not in use yet are read as well and multiplied away): one round trip for the lot instead of
        // one per term
        const float far_j = (wa.far + (b * WIN + jw) * D)[dc];
        const float dcoef = Dcoef[dc];
        float gk[WIN];
        uint32_t hk[WIN];                          // as loaded; converted at their use, behind the featurizer's requests
        {
            const float* gp = wa.g + (dc / (uint32_t)dg) * (uint32_t)WIN;
#pragma unroll
            for (int k = 0; k < WIN; ++k) gk[k] = gp[k];
#pragma unroll
            for (int k = 1; k < WIN; ++k) {
                int sl = cnt - k;
                if (sl < 0) sl += WIN;
                hk[k] = (wa.hist + (b * WIN + sl) * D)[dc];
            }
        }
        float a, c, gate2;
        if (VFEAT) {
            const int r = threadIdx.x;             // piece r covers zs columns 8r..8r+7 (96 pieces for 3 x 256 channels)
            if (r < 96) {
                const uint32_t dl0 = FEAT == 3 ? 0 : (uint32_t)(8 * r) % 256;
                const uint32_t ch = FEAT == 3 ? 3 * dblk + 8 * r : pj.chan((uint32_t)(8 * r) / 256, dblk + dl0);
                const bool okp = FEAT == 3 ? 3 * dblk + 8 * r < 3 * (uint32_t)D : dblk + dl0 < (uint32_t)D;
                if (okp) {
                    float z[8];
                    const u32x4 un = proj_step8(pj, b, ch, z);
                    proj_store8(pj, b, ch, un);
#pragma unroll
                    for (int k = 0; k < 8; ++k) zs[8 * r + k] = z[k];
                }
            }
            __syncthreads();
            const int dl = threadIdx.x;
            const float g2 = FEAT == 3 ? zs[3 * dl] : zs[dl], g1 = FEAT == 3 ? zs[3 * dl + 1] : zs[256 + dl];
            c = FEAT == 3 ? zs[3 * dl + 2] : zs[512 + dl];
            a = pj.flip ? g2 : g1;
            gate2 = pj.flip ? g1 : g2;
        } else {
            a = bf_to_f((x1 + b * in_bs)[dc]);
            c = bf_to_f((v + b * in_bs)[dc]);
            gate2 = bf_to_f((x2 + b * in_bs)[dc]);
        }
        if (!ok) return;
        const float x1v = round_bf(a * c);
        float part = far_j + gk[0] * x1v;
#pragma unroll
        for (int k = 1; k < WIN; ++k)
        {
            asm volatile("" : "+v"(hk[k]));        // keeps the conversion here, behind the featurizer's requests
            if (k <= jw) part = fmaf(gk[k], __uint_as_float(hk[k] << 16), part);
        }
        float dx = dcoef * x1v;
        if (d_is_bf16) dx = round_bf(dx);
        const float y = gate2 * (part + dx);
        if (out_is_fp32) ((float*)out + b * out_bs)[dc] = y;
        else ((bf16_t*)out + b * out_bs)[dc] = (bf16_t)f_to_bf_bits(y);
        (wa.hist + (b * WIN + cnt) * D)[dc] = (bf16_t)f_to_bf_bits(x1v);
        return;
    }
    const uint32_t idx = xb * 256 + threadIdx.x;                // (channel, lane of the group)
    const int q = (int)(idx % LPB);
    uint32_t d = idx / LPB;
    const bool chan_live = d < (uint32_t)D;
    if (!chan_live) d = 0;
    const uint32_t g = d / (uint32_t)dg;
    // Addresses are a block-uniform row base (batch element; 0 for the rows past the batch, whose lanes store nothing)
    // plus a 32-bit lane offset, so the 64-bit part of the arithmetic is scalar.
    auto bu = [&](int j) -> int64_t { return bj(j) < B ? bj(j) : 0; };
    const int64_t row_floats = D * (int64_t)(S * FPS);
    const uint32_t soff = (d * LPB + q) * VEC;             // this lane's piece of its channel's state inside a row
    fvec st[NB];
    bool live[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        live[j] = chan_live && bj(j) < B;
        st[j] = *(const fvec*)(state + bu(j) * row_floats + soff);
    }
    // the inputs a window's first token (or a flush) folds into the state, newest first: u_{t-1-k}
    float pend[NB][WIN > 1 ? WIN : 1];
    uint32_t pend_raw[NB][WIN > 1 ? WIN : 1];        // as loaded; converted behind the featurizer's requests
    if (WIN > 1 && (mode == 1 || mode == 3)) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int k = 0; k < WIN; ++k) {
                int sl = cnt - 1 - k;
                if (sl < 0) sl += WIN;
                pend_raw[j][k] = (wa.hist + (bu(j) * WIN + sl) * D)[d];          // every slot is requested; the unused
            }                                                                     // ones are dropped further down
    }
    const fvec pp = *(const fvec*)(poles + (g * (uint32_t)(S * FPS) + q * VEC));
    const fvec rr = *(const fvec*)(residues + (g * (uint32_t)(S * FPS) + q * VEC));
    const float dco = mode != 3 ? Dcoef[d] : 0.f;      // a flush has no token: no gates, no output, no Dcoef
    // gates given as vectors, and the window's first filter sample, are requested here with everything above: one
    // round trip for all of a token's operands instead of one per use
    float ga[NB], gc[NB], gg[NB], g0 = 0.f;
    if (WIN > 1 && mode == 1) g0 = wa.g[g * (uint32_t)WIN];
    if (FEAT == 0 && mode != 3) {
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int64_t b = bu(j);
            ga[j] = bf_to_f((x1 + b * in_bs)[d]);
            gc[j] = bf_to_f((v + b * in_bs)[d]);
            gg[j] = bf_to_f((x2 + b * in_bs)[d]);
        }
    }
    // fused featurizer: lanes 0..2 of the group evaluate gates x2, x1, v of every batch element first (their
    // loads overlap), the ring-slot stores follow, and only then the state updates start
    float zf[NB];
    if (mode != 3) {
        if (VFEAT) {
            static_assert(ND % 8 == 0, "whole 8-channel pieces per block");
            constexpr int PPB = 3 * ND / 8;            // 8-channel pieces per batch element
            const uint32_t dblk = xb * ND;
            const int e = threadIdx.x;
            if (e < NB * PPB) {
                const int j = e / PPB, r = e - j * PPB;
                // piece r covers zs columns 8r..8r+7: interleaved order (column = 3*dl + gate) or gate-major (gate*ND + dl)
                const uint32_t dl0 = FEAT == 3 ? 0 : (uint32_t)(8 * r) % ND;
                const uint32_t ch = FEAT == 3 ? 3 * dblk + 8 * r : pj.chan((uint32_t)(8 * r) / ND, dblk + dl0);
                const bool ok = bj(j) < B && (FEAT == 3 ? 3 * dblk + 8 * r < 3 * (uint32_t)D : dblk + dl0 < (uint32_t)D);
                if (ok) {
                    float z[8];
                    const u32x4 un = proj_step8(pj, bj(j), ch, z);
                    proj_store8(pj, bj(j), ch, un);
#pragma unroll
                    for (int k = 0; k < 8; ++k) zs[(j * 3 * ND) + 8 * r + k] = z[k];
                }
            }
            __syncthreads();
        } else if (FEAT == 2) {
            static_assert(FEAT != 2 || LPB >= 4, "the scalar fused featurizer needs three lanes per channel");
            bf16_t un[NB];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                zf[j] = 0.f;
                un[j] = 0;
                if (q < 3) {
                    const int64_t b = bu(j);
                    const uint32_t ch = pj.chan((uint32_t)q, d);
                    const bf16_t* rb = pj.ring + (b * pj.Rf) * pj.C + ch;
                    un[j] = pj.u[b * pj.u_bs + ch];
                    float acc = 0.f;
                    for (int i = 0; i < pj.Rf; ++i) {
                        int s = pj.pos + i;
                        if (s >= pj.Rf) s -= pj.Rf;
                        acc = fmaf(pj.w[(int64_t)i * pj.C + ch], bf_to_f(rb[(int64_t)s * pj.C]), acc);
                    }
                    acc = fmaf(pj.w[(int64_t)pj.Rf * pj.C + ch], bf_to_f(un[j]), acc);
                    if (pj.bias) acc += pj.bias[ch];
                    zf[j] = round_bf(acc);
                }
            }
            if (q < 3) {
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    if (live[j]) pj.ring[((bj(j) * pj.Rf) + pj.pos) * pj.C + pj.chan((uint32_t)q, d)] = un[j];
            }
        }
    }
    // the history slots that hold no pending input were requested with the rest; they are dropped here, behind the
    // featurizer's requests, so that those do not wait for this round trip
    if (WIN > 1 && (mode == 1 || mode == 3)) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int k = 0; k < WIN; ++k)
            {
                // (opaque to the optimizer, which would otherwise convert right behind the load and wait there)
                asm volatile("" : "+v"(pend_raw[j][k]));
                pend[j][k] = k >= npend ? 0.f : __uint_as_float(pend_raw[j][k] << 16);
            }
    }
    // powers of the poles a window needs: pw[m] = p^(m+1), m = 0 .. WIN-1 (state-wise; complex pairs or 4 reals)
    fvec pw[WIN > 1 ? WIN : 1];
    if (WIN > 1 && (mode == 1 || mode == 3)) {
        pw[0] = pp;
#pragma unroll
        for (int m = 1; m < WIN; ++m) {
            if (CPLX) {
#pragma unroll
                for (int k = 0; k < VEC; k += 2) {
                    pw[m][k] = pw[m - 1][k] * pp[k] - pw[m - 1][k + 1] * pp[k + 1];
                    pw[m][k + 1] = pw[m - 1][k] * pp[k + 1] + pw[m - 1][k + 1] * pp[k];
                }
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) pw[m][k] = pw[m - 1][k] * pp[k];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int64_t b = bu(j);
        float a = 0.f, c = 0.f, gate2 = 0.f;
        if (mode == 3) {
        } else if (VFEAT) {
            const int dl = threadIdx.x / LPB;
            const float* zj = zs + j * 3 * ND;
            const float g2 = FEAT == 3 ? zj[3 * dl] : zj[dl], g1 = FEAT == 3 ? zj[3 * dl + 1] : zj[ND + dl];
            c = FEAT == 3 ? zj[3 * dl + 2] : zj[2 * ND + dl];
            a = pj.flip ? g2 : g1;
            gate2 = pj.flip ? g1 : g2;
        } else if (FEAT == 2) {
            const int base = (threadIdx.x & 63) & ~(LPB - 1);
            const float g2 = __shfl(zf[j], base, 64), g1 = __shfl(zf[j], base + 1, 64);
            c = __shfl(zf[j], base + 2, 64);
            a = pj.flip ? g2 : g1;
            gate2 = pj.flip ? g1 : g2;
        } else {
            a = ga[j];
            c = gc[j];
        }
        const float x1v = round_bf(a * c);
        float part = 0.f;
        if (WIN > 1 && mode != 0) {
            // first token of a window (or a flush): fold the pending inputs, S = p^n S' + sum_k p^k u_{t-1-k}
            fvec ns = st[j];
            if (npend > 0) {
#pragma unroll
                for (int m = 0; m < WIN; ++m) {          // p^npend, picked without indexing registers
                    if (m + 1 == npend) {
                        if (CPLX) {
#pragma unroll
                            for (int k = 0; k < VEC; k += 2) {
                                ns[k] = pw[m][k] * st[j][k] - pw[m][k + 1] * st[j][k + 1];
                                ns[k + 1] = pw[m][k] * st[j][k + 1] + pw[m][k + 1] * st[j][k];
                            }
                        } else {
#pragma unroll
                            for (int k = 0; k < VEC; ++k) ns[k] = pw[m][k] * st[j][k];
                        }
                    }
                }
                // + u_{t-1} (p^0) + p u_{t-2} + ...   (pend[j][k] is zero from k = npend on)
#pragma unroll
                for (int k = 0; k < VEC; k += (CPLX ? 2 : 1)) ns[k] += pend[j][0];
#pragma unroll
                for (int m = 1; m < WIN; ++m)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) ns[k] = fmaf(pw[m - 1][k], pend[j][m], ns[k]);
                if (live[j]) *(fvec*)(state + b * row_floats + soff) = ns;
            }
            if (mode == 1) {
                // far[m] = Re sum_s r p^(m+1) S: this lane's states, then the lane group
                float fm[WIN > 1 ? WIN : 1];
#pragma unroll
                for (int m = 0; m < WIN; ++m) {
                    if (CPLX) {
                        float t = 0.f;
#pragma unroll
                        for (int k = 0; k < VEC; k += 2) {
                            const float zr = pw[m][k] * ns[k] - pw[m][k + 1] * ns[k + 1];
                            const float zi = pw[m][k] * ns[k + 1] + pw[m][k + 1] * ns[k];
                            t += rr[k] * zr - rr[k + 1] * zi;
                        }
                        fm[m] = t;
                    } else {
                        fm[m] = (rr[0] * pw[m][0] * ns[0] + rr[1] * pw[m][1] * ns[1]) + (rr[2 % VEC] * pw[m][2 % VEC] * ns[2 % VEC] + rr[3 % VEC] * pw[m][3 % VEC] * ns[3 % VEC]);
                    }
                    fm[m] = lane_group_sum<LPB>(fm[m]);
                }
                if (live[j] && q == 0) {
#pragma unroll
                    for (int m = 1; m < WIN; ++m) (wa.far + (b * WIN + m) * D)[d] = fm[m];
                }
                part = fm[0] + g0 * x1v;
            }
        } else {
            fvec ns;
            if (CPLX) {
                // (pr + i pi)(sr + i si) + x1v, then Re(r*s)
#pragma unroll
                for (int k = 0; k < VEC; k += 2) {
                    ns[k] = fmaf(pp[k], st[j][k], -pp[k + 1] * st[j][k + 1]) + x1v;
                    ns[k + 1] = fmaf(pp[k], st[j][k + 1], pp[k + 1] * st[j][k]);
                }
                if (VEC == 4) part = (rr[0] * ns[0] - rr[1] * ns[1]) + (rr[2] * ns[2] - rr[3] * ns[3]);
                else part = rr[0] * ns[0] - rr[1] * ns[1];
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) ns[k] = fmaf(pp[k], st[j][k], x1v);
                if (VEC == 4) part = (rr[0] * ns[0] + rr[1] * ns[1]) + (rr[2] * ns[2] + rr[3] * ns[3]);
                else if (VEC == 2) part = rr[0] * ns[0] + rr[1] * ns[1];
                else part = rr[0] * ns[0];
            }
            if (live[j]) *(fvec*)(state + b * row_floats + soff) = ns;
            part = lane_group_sum<LPB>(part);
        }
        if (mode != 3 && live[j] && q == 0) {
            float dx = dco * x1v;
            if (d_is_bf16) dx = round_bf(dx);
            const float y = (FEAT != 0 ? gate2 : gg[j]) * (part + dx);
            if (out_is_fp32) ((float*)out + b * out_bs)[d] = y;
            else ((bf16_t*)out + b * out_bs)[d] = (bf16_t)f_to_bf_bits(y);
            // this token's input joins the window's inputs (after every read of the slot it replaces, above)
            if (WIN > 1) (wa.hist + (b * WIN + cnt) * D)[d] = (bf16_t)f_to_bf_bits(x1v);
        }
    }
}

}  // namespace

// Validates a fused-featurizer descriptor and converts it; returns 0 or an error code.
static int make_proj(const hyena_proj_step* p, int64_t D, const char* who, ProjArgs* out) {
    if (!p->u || !p->ring || !p->w) return hyena_fail(HYENA_EINVAL, "%s: proj u, ring, w are required", who);
    if (p->Rf < 1 || p->Rf > 7 || (!p->pos_dev && (p->pos < 0 || p->pos >= p->Rf)))
        return hyena_fail(HYENA_EINVAL, "%s: featurizer cache depth %lld / position %lld", who, (long long)p->Rf,
                          (long long)p->pos);
    const int64_t C = 3 * D;
    if (p->ch_inner <= 0 || p->ch_outer < 0 || p->gate_stride <= 0 || p->ch_stride <= 0 || C >= (1LL << 31))
        return hyena_fail(HYENA_EINVAL, "%s: bad featurizer channel map", who);
    const int64_t last = ((D - 1) / p->ch_inner) * p->ch_outer + 2 * p->gate_stride + ((D - 1) % p->ch_inner) * p->ch_stride;
    if (last >= C) return hyena_fail(HYENA_EINVAL, "%s: featurizer channel map reaches channel %lld of %lld", who,
                                     (long long)last, (long long)C);
    out->u = (const bf16_t*)p->u; out->u_bs = p->u_batch_stride; out->ring = (bf16_t*)p->ring;
    out->Rf = (int)p->Rf; out->pos = p->pos_dev ? 0 : (int)p->pos; out->pos_dev = (const int*)p->pos_dev; out->C = (int)C; out->w = p->w; out->bias = p->bias;
    out->ch_inner = (uint32_t)(p->ch_inner > D ? D : p->ch_inner); out->ch_outer = (uint32_t)p->ch_outer;
    out->gate_stride = (uint32_t)p->gate_stride; out->ch_stride = (uint32_t)p->ch_stride; out->flip = p->flip_x1x2 != 0;
    return 0;
}

// 0: not vectorisable, 1: unit channel stride, 3: interleaved gates
static int proj_vector_mode(const hyena_proj_step* p, int64_t D) {
    const bool al = !(((uintptr_t)p->u | (uintptr_t)p->ring | (uintptr_t)p->w | (uintptr_t)p->bias) & 15) &&
                    p->u_batch_stride % 8 == 0 && D % 8 == 0;
    if (!al) return 0;
    if (p->ch_stride == 1 && p->ch_inner % 8 == 0 && p->ch_outer % 8 == 0 && p->gate_stride % 8 == 0) return 1;
    if (p->ch_stride == 3 && p->gate_stride == 1 && p->ch_inner >= D) return 3;
    return 0;
}

constexpr int FAR_NBT = 3;          // tokens per window of the far sums

static int64_t far_period(int64_t R) {      // lcm(FAR_NBT, R): one counter gives the ring slot (cnt % R) and the window phase (cnt % NBT)
    int64_t a = R, b = FAR_NBT;
    while (b) { const int64_t t = a % b; a = b; b = t; }
    return R / a * FAR_NBT;
}

static int fir_step_launch(const void* x1, const void* x2, const void* v, int64_t in_bs, const hyena_proj_step* proj,
                           void* ring, int64_t R, int64_t cb, int64_t pos, const int32_t* pos_dev, float* far, int rebuild,
                           const float* w, const float* bias,
                           int bias_mode, void* out, int64_t out_bs, int64_t B, int64_t D, int64_t G, void* stream,
                           const char* who) {
    if ((!proj && !x1) || !ring || !w || !out) return hyena_fail(HYENA_EINVAL, "%s: x1, ring, w, out are required", who);
    if (pos_dev) pos = 0;
    const int64_t period = far ? far_period(R) : R;
    if (B < 0 || D <= 0 || G <= 0 || D % G != 0 || R < 1 || R > 4096 || pos < 0 || pos >= period)
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld G=%lld R=%lld pos=%lld", who, (long long)B,
                          (long long)D, (long long)G, (long long)R, (long long)pos);
    if (far && R < 32) return hyena_fail(HYENA_ENOSUP, "%s: the far-sum form is for caches of 32 slots and more", who);
    if (cb != D && (cb <= 0 || cb % 512 != 0 || D % cb != 0))
        return hyena_fail(HYENA_EINVAL, "%s: ring_block %lld must be D or a multiple of 512 that divides D=%lld", who,
                          (long long)cb, (long long)D);
    if (D >= (1LL << 31)) return hyena_fail(HYENA_EINVAL, "%s: D too large", who);
    if (bias_mode < 0 || bias_mode > 2 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "%s: bias_mode %d needs a bias pointer", who, bias_mode);
    if (D % 8 != 0 || in_bs % 8 != 0 || out_bs % 8 != 0 || ((uintptr_t)x1 & 15) || ((uintptr_t)ring & 15) ||
        ((uintptr_t)out & 15) || (x2 && ((uintptr_t)x2 & 15)) || (v && ((uintptr_t)v & 15)) || ((uintptr_t)bias & 15) ||
        ((uintptr_t)far & 15))
        return hyena_fail(HYENA_EALIGN, "%s: D and strides must be multiples of 8, pointers 16-byte aligned", who);
    if (B > 65535) return hyena_fail(HYENA_EINVAL, "%s: B > 65535", who);
    ProjArgs pj = {};
    int feat = 0;
    if (proj) {
        if (int rc = make_proj(proj, D, who, &pj)) return rc;
        feat = proj_vector_mode(proj, D);
        if (!feat) return hyena_fail(HYENA_ENOSUP, "%s: this featurizer channel map / alignment has no fused kernel", who);
        if (bias_mode == HYENA_BIAS_ADD) return hyena_fail(HYENA_ENOSUP, "%s: fused featurizer with an additive bias", who);
    }
    if (B == 0) return 0;
    const int dg = (int)(D / G);
    const bool grouped = (dg % 8 == 0) && (512 % dg == 0);
    if (!grouped && G != D)
        return hyena_fail(HYENA_ENOSUP, "%s: D/G=%d needs per-channel taps (pass G=D)", who, dg);
    const bool pre = proj || v != nullptr, post = proj || x2 != nullptr;
    dim3 grid((unsigned)((D + 511) / 512), (unsigned)B);
    const int nsg = R >= 32 ? 8 : 2;
    const int nbt = far ? FAR_NBT : 1;
    size_t sh = (size_t)(nsg - 1) * nbt * 64 * 8 * sizeof(float) + (grouped ? (size_t)(R + nbt) * (512 / dg) * sizeof(float) : 0) +
                (proj ? 3 * 512 * sizeof(float) : 0);
    if (sh > 160 * 1024) return hyena_fail(HYENA_ENOSUP, "%s: R too large for the LDS tap table", who);
    hipStream_t s = (hipStream_t)stream;
    const bf16_t *p1 = (const bf16_t*)x1, *p2 = (const bf16_t*)x2, *pv = (const bf16_t*)v;
    bool ok = false;
#define FS_GO(P, Q, M, GR, N, F, T)                                                                              \
    hipLaunchKernelGGL((fir_step_kernel<P, Q, M, GR, N, F, T>), grid, dim3(64 * N), sh, s, p1, p2, pv, in_bs, pj, \
                       (bf16_t*)ring, (int)R, (int)cb, (int)pos, (const int*)pos_dev, (int)period, far, rebuild, \
                       w, bias, (bf16_t*)out, out_bs, D, dg)
#define FS_CASE(P, Q, M, F)                                                                                   \
    if (!ok && pre == P && post == Q && bias_mode == M && feat == F) {                                        \
        if (far && grouped) FS_GO(P, Q, M, true, 8, F, FAR_NBT);                                              \
        else if (far) FS_GO(P, Q, M, false, 8, F, FAR_NBT);                                                   \
        else if (grouped && nsg == 8) FS_GO(P, Q, M, true, 8, F, 1);                                          \
        else if (grouped) FS_GO(P, Q, M, true, 2, F, 1);                                                      \
        else if (nsg == 8) FS_GO(P, Q, M, false, 8, F, 1);                                                    \
        else FS_GO(P, Q, M, false, 2, F, 1);                                                                  \
        ok = true;                                                                                            \
    }
    FS_CASE(true, true, HYENA_BIAS_NONE, 0)
    FS_CASE(true, true, HYENA_BIAS_GATED_FP32, 0)
    FS_CASE(false, false, HYENA_BIAS_NONE, 0)
    FS_CASE(false, false, HYENA_BIAS_ADD, 0)
    FS_CASE(false, false, HYENA_BIAS_GATED_FP32, 0)
    FS_CASE(true, true, HYENA_BIAS_ADD, 0)
    FS_CASE(true, true, HYENA_BIAS_NONE, 1)
    FS_CASE(true, true, HYENA_BIAS_GATED_FP32, 1)
    FS_CASE(true, true, HYENA_BIAS_NONE, 3)
    FS_CASE(true, true, HYENA_BIAS_GATED_FP32, 3)
#undef FS_CASE
#undef FS_GO
    if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: this gate/bias combination has no kernel", who);
    return hyena_check_launch(who);
}

extern "C" int hyena_fir_step(const void* x1, const void* x2, const void* v, int64_t in_bs, void* ring, int64_t R,
                              int64_t cb, int64_t pos, const float* w, const float* bias, int bias_mode, void* out,
                              int64_t out_bs, int64_t B, int64_t D, int64_t G, void* stream) {
    return fir_step_launch(x1, x2, v, in_bs, nullptr, ring, R, cb, pos, nullptr, nullptr, 0, w, bias, bias_mode, out, out_bs,
                           B, D, G, stream, "hyena_fir_step");
}

extern "C" int hyena_fir_step_dpos(const void* x1, const void* x2, const void* v, int64_t in_bs, void* ring, int64_t R,
                                   int64_t cb, const int32_t* pos_dev, const float* w, const float* bias, int bias_mode,
                                   void* out, int64_t out_bs, int64_t B, int64_t D, int64_t G, void* stream) {
    if (!pos_dev) return hyena_fail(HYENA_EINVAL, "hyena_fir_step_dpos: pos_dev is required");
    return fir_step_launch(x1, x2, v, in_bs, nullptr, ring, R, cb, 0, pos_dev, nullptr, 0, w, bias, bias_mode, out, out_bs,
                           B, D, G, stream, "hyena_fir_step_dpos");
}

extern "C" int hyena_fir_layer_step(const hyena_proj_step* proj, void* ring, int64_t R, int64_t cb, int64_t pos, const float* w,
                                    const float* bias, int bias_mode, void* out, int64_t out_bs, int64_t B,
                                    int64_t D, int64_t G, void* stream) {
    if (!proj) return hyena_fail(HYENA_EINVAL, "hyena_fir_layer_step: proj is required");
    return fir_step_launch(nullptr, nullptr, nullptr, 0, proj, ring, R, cb, pos, nullptr, nullptr, 0, w, bias, bias_mode, out,
                           out_bs, B, D, G, stream, "hyena_fir_layer_step");
}

extern "C" int hyena_fir_layer_step_dpos(const hyena_proj_step* proj, void* ring, int64_t R, int64_t cb, const int32_t* pos_dev,
                                         const float* w, const float* bias, int bias_mode, void* out, int64_t out_bs,
                                         int64_t B, int64_t D, int64_t G, void* stream) {
    if (!proj || !pos_dev) return hyena_fail(HYENA_EINVAL, "hyena_fir_layer_step_dpos: proj and pos_dev are required");
    return fir_step_launch(nullptr, nullptr, nullptr, 0, proj, ring, R, cb, 0, pos_dev, nullptr, 0, w, bias, bias_mode, out,
                           out_bs, B, D, G, stream, "hyena_fir_layer_step_dpos");
}

extern "C" int64_t hyena_fir_far_period(int64_t R) { return R >= 1 ? far_period(R) : 0; }
extern "C" int64_t hyena_fir_far_bytes(int64_t B, int64_t D) {
    return B >= 0 && D > 0 ? B * FAR_NBT * D * (int64_t)sizeof(float) : 0;
}

extern "C" int hyena_fir_step_far(const void* x1, const void* x2, const void* v, int64_t in_bs, void* ring, int64_t R,
                                  int64_t cb, int64_t cnt, const int32_t* cnt_dev, float* far, int rebuild, const float* w,
                                  const float* bias, int bias_mode, void* out, int64_t out_bs, int64_t B, int64_t D,
                                  int64_t G, void* stream) {
    if (!far) return hyena_fail(HYENA_EINVAL, "hyena_fir_step_far: far is required");
    return fir_step_launch(x1, x2, v, in_bs, nullptr, ring, R, cb, cnt, cnt_dev, far, rebuild != 0, w, bias, bias_mode, out,
                           out_bs, B, D, G, stream, "hyena_fir_step_far");
}

extern "C" int hyena_fir_layer_step_far(const hyena_proj_step* proj, void* ring, int64_t R, int64_t cb, int64_t cnt,
                                        const int32_t* cnt_dev, float* far, int rebuild, const float* w, const float* bias,
                                        int bias_mode, void* out, int64_t out_bs, int64_t B, int64_t D, int64_t G,
                                        void* stream) {
    if (!proj || !far) return hyena_fail(HYENA_EINVAL, "hyena_fir_layer_step_far: proj and far are required");
    return fir_step_launch(nullptr, nullptr, nullptr, 0, proj, ring, R, cb, cnt, cnt_dev, far, rebuild != 0, w, bias, bias_mode,
                           out, out_bs, B, D, G, stream, "hyena_fir_layer_step_far");
}

namespace {
__global__ void ring_advance_kernel(int* __restrict__ pos, const int* __restrict__ depth, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int p = pos[i] + 1;
        pos[i] = p >= depth[i] ? 0 : p;
    }
}
}  // namespace

extern "C" int hyena_ring_advance(int32_t* pos, const int32_t* depth, int64_t n, void* stream) {
    if (!pos || !depth) return hyena_fail(HYENA_EINVAL, "hyena_ring_advance: null pointer");
    if (n < 0 || n > (1 << 24)) return hyena_fail(HYENA_EINVAL, "hyena_ring_advance: bad n=%lld", (long long)n);
    if (n == 0) return 0;
    hipLaunchKernelGGL(ring_advance_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, pos,
                       depth, (int)n);
    return hyena_check_launch("hyena_ring_advance");
}

constexpr int IIR_WIN = 4;          // tokens per window of the windowed modal step
constexpr int IIR_NBH = 2;          // batch elements per block at the head of their window (compact grid, large problems)

struct hyena_iir_window_c {         // hyena_iir_window as the launcher takes it, with the flush flag in its reserved field
    void* hist; float* far; const float* g; int64_t cnt; const int32_t* cnt_dev; int warm; int flush;
};

static bool iir_win_geometry(int64_t B, int64_t D, int64_t S) {
    // built for 16 states (vortex's and the benchmark's size); small problems are launch-bound either way
    return S == 16 && B >= 1 && D % 8 == 0 && B * D >= 65536;
}

static int iir_step_launch(const void* x1, const void* x2, const void* v, int64_t in_bs, const hyena_proj_step* proj,
                           float* state, const float* poles, const float* residues, int is_complex,
                           const float* Dcoef, int d_is_bf16, void* out, int out_is_fp32, int64_t out_bs, int64_t B,
                           int64_t D, int64_t G, int64_t S, const hyena_iir_window_c* win, void* stream, const char* who) {
    const bool flush = win && win->flush;
    if ((!flush && ((!proj && (!x1 || !x2 || !v)) || !Dcoef || !out)) || !state || !poles || !residues)
        return hyena_fail(HYENA_EINVAL, "%s: all pointers are required", who);
    if (B < 0 || D <= 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld G=%lld", who, (long long)B, (long long)D,
                          (long long)G);
    if (S < 1 || S > 32 || (S & (S - 1)))
        return hyena_fail(HYENA_ENOSUP, "%s: state size %lld (powers of two up to 32 supported)", who, (long long)S);
    if (((uintptr_t)state & 15) || ((uintptr_t)poles & 15) || ((uintptr_t)residues & 15))
        return hyena_fail(HYENA_EALIGN, "%s: state, poles, residues must be 16-byte aligned", who);
    WinArgs wa = {};
    if (win) {
        if (!win->hist || (!flush && (!win->far || !win->g)))
            return hyena_fail(HYENA_EINVAL, "%s: the window needs its hist, far and g buffers", who);
        if (!iir_win_geometry(B, D, S))
            return hyena_fail(HYENA_ENOSUP, "%s: the windowed step takes 16 states, D %% 8 == 0 and B*D of 65536 and more; "
                              "use the plain step", who);
        if ((!win->cnt_dev && (win->cnt < 0 || win->cnt >= IIR_WIN)) || win->warm < 0)
            return hyena_fail(HYENA_EINVAL, "%s: window counter %lld / warm %d", who, (long long)win->cnt, win->warm);
        wa.hist = (bf16_t*)win->hist; wa.far = win->far; wa.g = win->g; wa.cnt = win->cnt_dev ? 0 : (int)win->cnt;
        wa.cnt_dev = (const int*)win->cnt_dev; wa.warm = win->warm > IIR_WIN ? IIR_WIN : win->warm; wa.flush = flush;
        wa.compact = !flush && wa.warm >= IIR_WIN - 1;      // every window open: no batch element takes a plain step
    }
    ProjArgs pj = {};
    if (proj) {
        if (int rc = make_proj(proj, D, who, &pj)) return rc;
        if (S * (is_complex ? 2 : 1) < 16)
            return hyena_fail(HYENA_ENOSUP, "%s: fused featurizer with fewer than 16 real / 8 complex states", who);
    }
    if (B == 0) return 0;
    const int dg = (int)(D / G);
    const int lpb = (int)(S * (is_complex ? 2 : 1) >= 4 ? S * (is_complex ? 2 : 1) / 4 : 1);
    if (D * lpb > 0x0fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: D too large", who);   // 32-bit byte offsets inside a row
    // four batch elements per lane when that still leaves a few wavefronts per SIMD; else one.  Windowed form: one
    // (measured: 11.3 / 17.5 us at D = 4096 / 8192 against 15.4 / 19.4 us with four of one residue class b % WIN);
    // its block rows come in groups of WIN, one per residue class
    const int nb = (!win && B >= 4 && B * D * lpb >= 4 * 256 * 1024) ? 4 : 1;
    const int64_t gy = win ? IIR_WIN * (((B + IIR_WIN - 1) / IIR_WIN + nb - 1) / nb) : (B + nb - 1) / nb;
    if (gy > 65535) return hyena_fail(HYENA_EINVAL, "%s: B too large", who);
    dim3 grid((unsigned)((D * lpb + 255) / 256), (unsigned)gy);
    int nbh = 1;
    if (win && wa.compact) {
        const int64_t nrow = (B + IIR_WIN - 1) / IIR_WIN;
        wa.nxh = grid.x;
        wa.nxl = (uint32_t)((D + 255) / 256);
        // one batch element per block while those blocks are all resident at once (8 per CU), two beyond that
        // (measured at B = 64: 9.7 against 10.3 us at D = 4096, 15.0 against 16.4 us at D = 8192)
        nbh = nrow * wa.nxh > 8 * 256 ? IIR_NBH : 1;
        const int64_t nhb = ((nrow + nbh - 1) / nbh) * wa.nxh;
        const int64_t nblk = nhb + nrow * (IIR_WIN - 1) * wa.nxl;
        if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: B*D too large", who);
        wa.nhb = (uint32_t)nhb;
        grid = dim3((unsigned)nblk);
    }
    hipStream_t s = (hipStream_t)stream;
    const bf16_t *p1 = (const bf16_t*)x1, *p2 = (const bf16_t*)x2, *pv = (const bf16_t*)v;
    // fused featurizer: vector form where the channel map and alignment allow it, scalar form otherwise
    const int feat = !proj ? 0 : (proj_vector_mode(proj, D) ? proj_vector_mode(proj, D) : 2);
#define IIR_GO(SS, C, F, N, WN)                                                                                 \
    hipLaunchKernelGGL((iir_step_kernel<SS, C, F, N, WN>), grid, dim3(256), 0, s, p1, p2, pv, in_bs, pj, state, \
                       poles, residues, Dcoef, d_is_bf16, out, out_is_fp32, out_bs, B, D, dg, wa)
    if (win) {
        if (feat == 2)
            return hyena_fail(HYENA_ENOSUP, "%s: the windowed step needs a featurizer channel map with 16-byte pieces", who);
#define IIR_WCASE(C, F) if ((is_complex != 0) == C && feat == F) { if (nbh == IIR_NBH) IIR_GO(16, C, F, IIR_NBH, IIR_WIN); else IIR_GO(16, C, F, 1, IIR_WIN); }
        IIR_WCASE(false, 0) IIR_WCASE(false, 1) IIR_WCASE(false, 3)
        IIR_WCASE(true, 0) IIR_WCASE(true, 1) IIR_WCASE(true, 3)
#undef IIR_WCASE
        return hyena_check_launch(who);
    }
#define IIR_CASE(SS, C, F)                                                                                      \
    if (S == SS && (is_complex != 0) == C && feat == F) { if (nb == 4) IIR_GO(SS, C, F, 4, 1); else IIR_GO(SS, C, F, 1, 1); }
#define IIR_FEATS(SS, C) IIR_CASE(SS, C, 1) IIR_CASE(SS, C, 2) IIR_CASE(SS, C, 3)
    IIR_CASE(1, false, 0) IIR_CASE(2, false, 0) IIR_CASE(4, false, 0)
    IIR_CASE(1, true, 0) IIR_CASE(2, true, 0) IIR_CASE(4, true, 0)
    IIR_CASE(8, false, 0) IIR_CASE(16, false, 0) IIR_CASE(32, false, 0)
    IIR_CASE(8, true, 0) IIR_CASE(16, true, 0) IIR_CASE(32, true, 0)
    IIR_FEATS(16, false) IIR_FEATS(32, false) IIR_FEATS(8, true) IIR_FEATS(16, true) IIR_FEATS(32, true)
#undef IIR_FEATS
#undef IIR_CASE
#undef IIR_GO
    return hyena_check_launch(who);
}

extern "C" int hyena_iir_step(const void* x1, const void* x2, const void* v, int64_t in_bs, float* state,
                              const float* poles, const float* residues, int is_complex, const float* Dcoef,
                              int d_is_bf16, void* out, int out_is_fp32, int64_t out_bs, int64_t B, int64_t D,
                              int64_t G, int64_t S, void* stream) {
    return iir_step_launch(x1, x2, v, in_bs, nullptr, state, poles, residues, is_complex, Dcoef, d_is_bf16, out,
                           out_is_fp32, out_bs, B, D, G, S, nullptr, stream, "hyena_iir_step");
}

extern "C" int hyena_iir_layer_step(const hyena_proj_step* proj, float* state, const float* poles,
                                    const float* residues, int is_complex, const float* Dcoef, int d_is_bf16,
                                    void* out, int out_is_fp32, int64_t out_bs, int64_t B, int64_t D, int64_t G,
                                    int64_t S, void* stream) {
    if (!proj) return hyena_fail(HYENA_EINVAL, "hyena_iir_layer_step: proj is required");
    return iir_step_launch(nullptr, nullptr, nullptr, 0, proj, state, poles, residues, is_complex, Dcoef, d_is_bf16,
                           out, out_is_fp32, out_bs, B, D, G, S, nullptr, stream, "hyena_iir_layer_step");
}

// ---- the windowed modal step (see iir_step_kernel)
static_assert(sizeof(hyena_iir_window) == sizeof(hyena_iir_window_c), "hyena_iir_window layout");

extern "C" int64_t hyena_iir_window_tokens(void) { return IIR_WIN; }
extern "C" int hyena_iir_window_supported(int64_t B, int64_t D, int64_t S, int is_complex) {
    (void)is_complex;
    return D > 0 && iir_win_geometry(B, D, S) ? 1 : 0;
}

extern "C" int hyena_iir_step_win(const void* x1, const void* x2, const void* v, int64_t in_bs, float* state,
                                  const float* poles, const float* residues, int is_complex, const float* Dcoef,
                                  int d_is_bf16, void* out, int out_is_fp32, int64_t out_bs, int64_t B, int64_t D,
                                  int64_t G, int64_t S, const hyena_iir_window* win, void* stream) {
    if (!win) return hyena_fail(HYENA_EINVAL, "hyena_iir_step_win: win is required");
    hyena_iir_window_c w = {win->hist, win->far, win->g, win->cnt, win->cnt_dev, win->warm, 0};
    return iir_step_launch(x1, x2, v, in_bs, nullptr, state, poles, residues, is_complex, Dcoef, d_is_bf16, out,
                           out_is_fp32, out_bs, B, D, G, S, &w, stream, "hyena_iir_step_win");
}

extern "C" int hyena_iir_layer_step_win(const hyena_proj_step* proj, float* state, const float* poles,
                                        const float* residues, int is_complex, const float* Dcoef, int d_is_bf16,
                                        void* out, int out_is_fp32, int64_t out_bs, int64_t B, int64_t D, int64_t G,
                                        int64_t S, const hyena_iir_window* win, void* stream) {
    if (!proj || !win) return hyena_fail(HYENA_EINVAL, "hyena_iir_layer_step_win: proj and win are required");
    hyena_iir_window_c w = {win->hist, win->far, win->g, win->cnt, win->cnt_dev, win->warm, 0};
    return iir_step_launch(nullptr, nullptr, nullptr, 0, proj, state, poles, residues, is_complex, Dcoef, d_is_bf16,
                           out, out_is_fp32, out_bs, B, D, G, S, &w, stream, "hyena_iir_layer_step_win");
}

extern "C" int hyena_iir_window_flush(float* state, const float* poles, const float* residues, int is_complex,
                                      int64_t B, int64_t D, int64_t G, int64_t S, const hyena_iir_window* win,
                                      void* stream) {
    if (!win) return hyena_fail(HYENA_EINVAL, "hyena_iir_window_flush: win is required");
    hyena_iir_window_c w = {win->hist, win->far, win->g, win->cnt, win->cnt_dev, win->warm, 1};
    return iir_step_launch(nullptr, nullptr, nullptr, 0, nullptr, state, poles, residues, is_complex, nullptr, 0, nullptr,
                           0, 0, B, D, G, S, &w, stream, "hyena_iir_window_flush");
}
