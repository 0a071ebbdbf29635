// Channel-last gated FIR (2 <= K <= 128): the Hyena-SE / Hyena-MR operator on
// [B][L][D] tensors, the (batch, seqlen, groups, group_dim) layout of
// vortex/ops/hyena_se/fwd.py:17-43, and, with the featurizer fused in, a whole
// Hyena-SE / MR layer from the dense projection u [B][L][3D] to y [B][L][D]
// (vortex/model/model.py:221-291) with no intermediate in device memory.
//
// Same block-Toeplitz MFMA contraction as mr_fir.hip (ten 32x16 Toeplitz blocks
// per filter group held in registers, u = bf16(x1*v) streamed through the B
// operand), but the block is 64 channels x 128 samples per step so that every
// global access is a full 128-byte line of one time row:
//   global rows (16 B/lane = 8 channels, 4 rows per lane) [-> featurizer FIR in registers]
//   -> u = bf16(x1*v) -> 4x8 register transpose -> LDS [64 ch][256-sample ring]
//   -> B fragments (ds_read_b128) -> MFMA -> z = bf16(acc [+ D*u]) -> LDS [64][128]
//   -> 8x4 register transpose -> * x2 -> global rows.
// Wavefront w of a block contracts channels 16w..16w+15 (one filter group per wavefront).
// The LDS input tile is a two-chunk ring: the chunk written in one step is the
// 128-sample halo of the next, so nothing is copied between steps.
#include <type_traits>

#include "common.h"

namespace {

constexpr int TL = 128;        // samples per step (= halo length)
constexpr int CB = 64;         // channels per block
constexpr int URS = 264;       // u_lds row stride (elements): 528 B = 16 * 33
constexpr int ZRS = 136;       // z_lds row stride (elements): 272 B = 16 * 17

struct ClMap {                 // channel-last operand: (b, t, d) at ptr + b*bs + t*ts + d
    const bf16_t* ptr;
    int64_t bs, ts;
};

struct ProjFwd {               // device copy of hyena_proj_fwd
    const bf16_t* u;
    int64_t bs, ts;
    const float* w;            // [KS][3D], tap-major, oldest tap first
    const float* bias;         // [3D] or null
    uint32_t ch_inner, ch_outer, gate_stride;
    int flip;
    __device__ __forceinline__ uint32_t chan(uint32_t gate, uint32_t d) const {
        return (d / ch_inner) * ch_outer + gate * gate_stride + (d % ch_inner);
    }
};

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) {
    union { u32x4 u; bf16x8 b; } c;
    c.u = x;
    return c.b;
}

// The 16-bit element type of the tensors the gates-given form works on: how a packed pair widens to float, how two
// floats round (to nearest even) into a pair, and the MFMA that contracts such operands.  bfloat16 is what the
// model path uses; float16 serves callers of the (batch, seqlen, groups, group_dim) interface, whose reference
// grid runs in float16 and float32 (vortex/ops/hyena_se/tests/test_fwd.py:25-54).
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;

struct ElBf16 {
    typedef bf16x8 frag;
    static __device__ __forceinline__ float lo(uint32_t w) { return bf_lo(w); }
    static __device__ __forceinline__ float hi(uint32_t w) { return bf_hi(w); }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf2(a, b); }
    static __device__ __forceinline__ float round(float f) { return round_bf(f); }
    static __device__ __forceinline__ frag as_frag(u32x4 x) { return as_bf16x8(x); }
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

struct ElF16 {
    typedef f16x8 frag;
    static __device__ __forceinline__ float lo(uint32_t w) { union { uint32_t u; f16x2_t h; } c; c.u = w; return (float)c.h[0]; }
    static __device__ __forceinline__ float hi(uint32_t w) { union { uint32_t u; f16x2_t h; } c; c.u = w; return (float)c.h[1]; }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        union { uint32_t u; f16x2_t h; } c;
        c.h[0] = (_Float16)a;                    // v_cvt_f16_f32, round to nearest even
        c.h[1] = (_Float16)b;
        return c.u;
    }
    static __device__ __forceinline__ float round(float f) { return (float)(_Float16)f; }
    static __device__ __forceinline__ frag as_frag(u32x4 x) { union { u32x4 u; frag b; } c; c.u = x; return c.b; }
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// 16-bit halves of two dwords: (lo(a), lo(b)) or (hi(a), hi(b)) packed as (first, second)
__device__ __forceinline__ uint32_t pair_lo(uint32_t first, uint32_t second) {
    return __builtin_amdgcn_perm(second, first, 0x05040100u);
}
__device__ __forceinline__ uint32_t pair_hi(uint32_t first, uint32_t second) {
    return __builtin_amdgcn_perm(second, first, 0x07060302u);
}

// element e (0..7) of a packed row of 8 bf16, as float
__device__ __forceinline__ float el(const u32x4& r, int e) { return (e & 1) ? bf_hi(r[e >> 1]) : bf_lo(r[e >> 1]); }

// Featurizer FIR and gates of one lane's 4 rows x 8 operator channels from its three row pieces (raw[i][r]: piece i,
// row r - (KS - 1) relative to the lane's first row; w_lds: the block's taps and bias in lane-piece order):
// bx = bf16(x1*v) and g2 = x2, each as 4 rows of 8 packed channels.
template <int FEAT, int KS>
__device__ __forceinline__ void lane_gates(const u32x4 (&raw)[3][KS + 3], const float* w_lds, int cb, const ProjFwd& pj,
                                           u32x4 (&bx)[4], u32x4 (&g2)[4]) {
    u32x4 zq[3][4];
    int woff = 8 * cb;
    asm volatile("" : "+v"(woff));      // re-read the tap table every step instead of pinning 96 registers
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        float tw[KS][8], bb[8];
#pragma unroll
        for (int k = 0; k <= KS; ++k) {
            const f32x4 t0 = *(const f32x4*)(w_lds + (k * 3 + i) * CB + woff);
            const f32x4 t1 = *(const f32x4*)(w_lds + (k * 3 + i) * CB + woff + 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (k < KS) { tw[k][j] = t0[j]; tw[k][4 + j] = t1[j]; }
                else { bb[j] = t0[j]; bb[4 + j] = t1[j]; }
            }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmaf(tw[k][j], el(raw[i][q + k], j), acc[j]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) zq[i][q][j] = pack_bf2(acc[2 * j], acc[2 * j + 1]);
        }
        if (pj.bias) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    zq[i][q][j] = pack_bf2(bf_lo(zq[i][q][j]) + bb[2 * j], bf_hi(zq[i][q][j]) + bb[2 * j + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);      // one piece at a time: its rows are dead before the next starts
    }
    // rows past the end of the sequence hold bias-only values; they are never stored and never feed a
    // valid output (causality), so they need no masking.  Rows before t = 0 do not exist (ts0 >= 0).
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a1[2], a2[2], av[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int jd = 2 * j + e;
                if (FEAT == 3) {        // channel 3*jd + gate of the lane's 24
                    const int e0 = 3 * jd, e1 = 3 * jd + 1, e2 = 3 * jd + 2;
                    a2[e] = el(zq[e0 >> 3][q], e0 & 7);
                    a1[e] = el(zq[e1 >> 3][q], e1 & 7);
                    av[e] = el(zq[e2 >> 3][q], e2 & 7);
                } else {
                    a2[e] = el(zq[0][q], jd);
                    a1[e] = el(zq[1][q], jd);
                    av[e] = el(zq[2][q], jd);
                }
                if (pj.flip) { const float t = a1[e]; a1[e] = a2[e]; a2[e] = t; }
            }
            bx[q][j] = pack_bf2(a1[0] * av[0], a1[1] * av[1]);
            g2[q][j] = pack_bf2(a2[0], a2[1]);
        }
    }
}

// FEAT: 0 = gates given as three channel-last tensors; 1 = gates from the fused featurizer, unit channel
// stride (plain or head-blocked split); 3 = fused featurizer with interleaved gates (channel 3d+i).
// KS = featurizer taps (FEAT != 0).  AUX = also store y2 (z before the x2 gate) and / or bx = bf16(x1*v).  With the
// featurizer fused in, bx is the cache tail (at most the last K-1 samples): it is copied out of the LDS ring after
// the last step, which keeps the step loop free of the extra stores and their registers.
// MLO = first Toeplitz block that can be non-zero: 0 for any K <= 128, 7 for K <= 17 (lags 0..16 touch only
// blocks 7..9), which leaves three A fragments in registers and five B reads / six MFMAs per step.
// NT = non-temporal accesses for tensors that stream through the last-level cache: the output rows always, the
// input rows only without the fused featurizer (its lanes re-read their neighbours' rows, which must stay cached).
// ET = element traits of the 16-bit tensors (ElBf16, or ElF16 without the featurizer).
// NS = strips of 64 channels per block.  With NS > 1 a block is NS groups of four wavefronts, each working on its own
// strip with its own LDS tiles exactly as a block of the NS = 1 form does; all they share is the two barriers of a
// step, which keeps neighbouring strips of the same time rows in step, so that their requests for adjacent 128-byte
// (384-byte with the featurizer) pieces of a row reach the memory system together.
template <typename ET, bool PRE, bool POST, int BIAS, int FEAT, int KS, bool AUX, int MLO, bool NT, int NS = 1>
__global__ __launch_bounds__(256 * NS, NS == 1 ? 2 : 1) void fir_cl_kernel(ClMap x1, ClMap x2, ClMap v, ProjFwd pj,
                                                        const float* __restrict__ h, int K, int reversed,
                                                        const float* __restrict__ bias, bf16_t* __restrict__ out,
                                                        bf16_t* __restrict__ y2_out, bf16_t* __restrict__ bx_out,
                                                        int64_t bx_from, int64_t L, int64_t D, int dg,
                                                        int64_t seg_len, int nseg, int ndb) {
    static_assert(FEAT == 0 || std::is_same<ET, ElBf16>::value, "the fused featurizer is built for bfloat16");
    constexpr int RF = FEAT ? KS - 1 : 0;          // extra rows a lane reads before its own four
    constexpr int NR = 4 + RF;                     // rows per lane and load piece
    constexpr int NP = (FEAT || (PRE && POST)) ? 3 : (PRE ? 2 : 1);   // load pieces per row
    __shared__ __attribute__((aligned(16))) bf16_t u_lds_all[NS * CB * URS];
    __shared__ __attribute__((aligned(16))) bf16_t z_lds_all[NS * CB * ZRS];
    __shared__ __attribute__((aligned(16))) float w_lds_all[FEAT ? NS * (KS + 1) * 3 * CB : 4];

    const int sub = NS == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));     // this thread's strip
    bf16_t* const u_lds = u_lds_all + sub * CB * URS;
    bf16_t* const z_lds = z_lds_all + sub * CB * ZRS;
    float* const w_lds = w_lds_all + (FEAT ? sub * (KS + 1) * 3 * CB : 0);
    const int tid = threadIdx.x & 255, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bid = blockIdx.x;
    // channel blocks fastest: the blocks resident at one time read neighbouring 128-byte pieces of the same rows.
    // Workgroups are dealt to the 8 XCDs in turn (id mod 8), so every XCD takes every eighth channel block of all
    // row tiles; giving an XCD neighbouring channel blocks (0.457 -> 0.509 ms with the gates given as tensors), whole
    // row tiles (0.488 ms) or an eighth of the block order (0.487 ms) all measured slower.
    // (ndb counts blocks: groups of NS strips; a strip past the last channel runs empty but meets every barrier)
    const uint32_t db = (bid % (uint32_t)ndb) * NS + sub;
    const int seg = (int)((bid / (uint32_t)ndb) % (uint32_t)nseg);
    const int64_t b = bid / ((uint32_t)nseg * (uint32_t)ndb);
    const uint32_t d0 = db * CB;

    // ---- Toeplitz fragments of this wavefront's filter group (see mr_fir.hip for the index algebra)
    const int n = lane & 31, hh = lane >> 5;
    const bool slab_live = d0 + 16 * w < (uint32_t)D;
    const int g = slab_live ? (int)((d0 + 16 * w) / (uint32_t)dg) : 0;
    const int i_time = 16 * ((n >> 2) & 1) + 4 * (n >> 3) + (n & 3);
    typename ET::frag A[10 - MLO];
#pragma unroll
    for (int m = MLO; m < 10; ++m) {
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
            pk[j] = ET::pack2(t[0], t[1]);
        }
        A[m - MLO] = ET::as_frag(pk);
    }

    // ---- this lane's I/O block: rows 4*rb .. 4*rb+3 of the step, channels d0 + 8*cb .. +7
    const int cb = tid & 7, rb = tid >> 3;
    // Inside a 128-sample chunk the samples of channel slab j (16 channels) sit at position t ^ 32*j.  Both LDS
    // row strides are 32 banks modulo 64 per 8 channels, so without this the 8-byte transposed accesses of the
    // lanes cb = 0, 2, 4, 6 (and 1, 3, 5, 7) would fall on the same banks; a slab's own MFMA reads are unaffected.
    const int swz_io = 32 * (cb >> 1), swz_mm = 32 * w;
    const uint32_t dch = d0 + 8 * cb;
    const bool ch_ok = dch < (uint32_t)D;
    // Row pieces are addressed as a block-uniform base (tensor, batch element, piece; the time row is added per step)
    // plus a 32-bit byte offset of the lane (its first row and channels): no 64-bit pointer per lane and piece.  The
    // launcher bounds 128 rows of any operand to 2^32 bytes.
    const bf16_t* pp[NP];
    uint32_t loff[NP];
    int64_t pts;
    if (FEAT == 3) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            pp[i] = pj.u + b * pj.bs + 8 * i;
            loff[i] = ((uint32_t)(4 * rb) * (uint32_t)pj.ts + 3u * dch) * 2u;
        }
        pts = pj.ts;
    } else if (FEAT == 1) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            pp[i] = pj.u + b * pj.bs + (int64_t)i * pj.gate_stride;
            loff[i] = ((uint32_t)(4 * rb) * (uint32_t)pj.ts + pj.chan(0, ch_ok ? dch : 0)) * 2u;
        }
        pts = pj.ts;
    } else {
        pp[0] = x1.ptr + b * x1.bs;
        loff[0] = ((uint32_t)(4 * rb) * (uint32_t)x1.ts + dch) * 2u;
        if (NP >= 2) { pp[1] = v.ptr + b * v.bs; loff[1] = ((uint32_t)(4 * rb) * (uint32_t)v.ts + dch) * 2u; }
        if (NP >= 3) { pp[2] = x2.ptr + b * x2.bs; loff[2] = ((uint32_t)(4 * rb) * (uint32_t)x2.ts + dch) * 2u; }
        pts = 0;
    }
    const int64_t pstr[3] = {FEAT ? pts : x1.ts, FEAT ? pts : v.ts, FEAT ? pts : x2.ts};

    // featurizer taps / bias of this block's channels, in the lane-piece order the loads use
    if (FEAT) {
        for (int e = tid; e < (KS + 1) * 3 * CB; e += 256) {
            const int k = e / (3 * CB), r = e - k * 3 * CB, i = r / CB, dl = r - i * CB;   // piece i, local channel dl
            const uint32_t dd = d0 + dl;
            float val = 0.f;
            if (dd < (uint32_t)D) {
                const uint32_t ch = FEAT == 3 ? 3 * (d0 + (dl & ~7)) + 8 * i + (dl & 7) : pj.chan(i, dd);
                if (k < KS) val = pj.w[(int64_t)k * 3 * D + ch];
                else if (pj.bias) val = pj.bias[ch];
            }
            w_lds[e] = val;
        }
    }

    const int64_t t_begin = (int64_t)seg * seg_len;
    const int64_t t_end = (t_begin + seg_len < L) ? t_begin + seg_len : L;
    if (t_begin >= t_end) return;
    const int64_t ts0 = t_begin > 0 ? t_begin - TL : 0;      // one extra step rebuilds the halo of a later segment
    // a short filter (MLO = 7: K <= 17) only reaches 16 samples back, the featurizer at most 3 more: of the halo
    // step only the last 24 rows are read, the rest stay zero and feed no output of this segment.  Otherwise the
    // whole halo step is read, and with the featurizer fused in also the RF rows ahead of it: the first halo
    // samples are featurizer outputs themselves and need their own history (lag K-1 = 127 reaches sample ts0 + 1).
    const int64_t t_lo = MLO == 7 ? t_begin - 24 : ts0 - RF;

    // zero halo at the sequence start
    if (t_begin == 0) {
        const u32x4 zero4 = {0, 0, 0, 0};
        for (int e = tid; e < CB * (TL / 8); e += 256)
            *(u32x4*)(u_lds + (e >> 4) * URS + TL + (e & 15) * 8) = zero4;
    }
    __syncthreads();           // featurizer table and zeroed halo visible to every wavefront

    u32x4 raw[NP][NR];
    const u32x4 zero4 = {0, 0, 0, 0};
    // whole_tag: every row of the step is inside the segment and every channel of the block exists, so the requests
    // carry no test (and no branch, which lets the compiler count on them when it places its waits)
    auto load_pieces = [&](int64_t ts, int i0, int i1, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        uint32_t lo[NP];                          // (with the featurizer the pieces share one offset)
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            if (FEAT && i > 0) { lo[i] = lo[0]; continue; }
            lo[i] = loff[i];
            asm volatile("" : "+v"(lo[i]));       // keeps the compiler from folding it into per-lane row pointers held across the loop
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t t = ts + 4 * rb + r - RF;
            const bool ok = WHOLE || (ch_ok && t >= t_lo && t >= 0 && t < t_end);
#pragma unroll
            for (int i = 0; i < NP; ++i) if (i >= i0 && i < i1) {
                const u32x4* src = (const u32x4*)((const char*)(pp[i] + (ts + r - RF) * pstr[i]) + lo[i]);
                if (WHOLE) raw[i][r] = (NT && !FEAT) ? __builtin_nontemporal_load(src) : *src;
                else raw[i][r] = ok ? ((NT && !FEAT) ? __builtin_nontemporal_load(src) : *src) : zero4;
            }
        }
    };
    auto load_step = [&](int64_t ts) { load_pieces(ts, 0, NP, std::false_type{}); };
    // Pieces of the next step requested before the MFMA phase (the rest after it).  Without the featurizer all
    // of them travel during the MFMA phase.  With it a lane holds 18 row pieces, which next to all ten A fragments
    // do not fit the register budget of two blocks per CU: one piece goes out early (measured 4 % faster for the
    // medium filter than none; two fit since the output addresses stopped taking registers but measured 7 % slower,
    // and still 1-2 % slower with the steps without tests below).  The short-filter form, with three A fragments, has
    // room for all three: since its middle steps run without tests (counted waits) that is 1.6-2.4 % faster than none,
    // from B*L = 8192 to 131072 rows; before, one piece early had measured the same as none.
    constexpr int NEARLY = FEAT ? (MLO == 0 ? 1 : NP) : NP;
    load_step(ts0);

    float bz = 0.f;
    if (BIAS != HYENA_BIAS_NONE && slab_live) bz = bias[d0 + 16 * w + (n & 15)];

    int cur = 0;                       // ring chunk the current step writes; the other one is its halo
    int64_t ts_last = ts0;
    // One step.  whole_tag: the step computes, all of its rows and of the next step's are inside the segment and every
    // channel of the block exists: no test guards a request or a store then.
    auto step = [&](const int64_t ts, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        ts_last = ts;
        const bool compute = WHOLE || ts >= t_begin;
        // ---- (a) gates of this lane's 4 x 8 block
        u32x4 bx[4], g2[4];
        if constexpr (FEAT != 0) {
            lane_gates<FEAT, KS>(raw, w_lds, cb, pj, bx, g2);
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if constexpr (PRE) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        bx[q][j] = ET::pack2(ET::lo(raw[0][q][j]) * ET::lo(raw[1][q][j]),
                                             ET::hi(raw[0][q][j]) * ET::hi(raw[1][q][j]));
                } else {
                    bx[q] = raw[0][q];
                }
                if constexpr (POST) g2[q] = raw[NP - 1][q];
            }
        }
        // ---- (b) next step's rows (NEARLY pieces of them) are requested now and arrive during the MFMA phase
        __builtin_amdgcn_sched_barrier(0);
        if (WHOLE || ts + TL < t_end) load_pieces(ts + TL, 0, NEARLY, whole_tag);

        // ---- (c) 4 x 8 transpose into the ring chunk `cur`
        {
            bf16_t* ub = u_lds + (8 * cb) * URS + cur * TL + ((4 * rb) ^ swz_io);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                u32x2 t2;
                if (c & 1) { t2[0] = pair_hi(bx[0][c >> 1], bx[1][c >> 1]); t2[1] = pair_hi(bx[2][c >> 1], bx[3][c >> 1]); }
                else       { t2[0] = pair_lo(bx[0][c >> 1], bx[1][c >> 1]); t2[1] = pair_lo(bx[2][c >> 1], bx[3][c >> 1]); }
                *(u32x2*)(ub + c * URS) = t2;
            }
        }
        if (AUX && !FEAT && bx_out && compute && ch_ok) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t t = ts + 4 * rb + q;
                if (t < t_end && t >= bx_from) *(u32x4*)(bx_out + (b * (L - bx_from) + (t - bx_from)) * D + dch) = bx[q];
            }
        }
        __syncthreads();

        // ---- MFMA phase: this wavefront's 16 channels x 128 samples
        const int c = n & 15, s = n >> 4;
        f32x16 acc0, acc1;
        const bf16_t* urow = u_lds + (16 * w + c) * URS;
        if (WHOLE || (compute && slab_live)) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
            const int c0 = 64 * s + 8 * hh + (cur ^ 1) * TL;     // ring position of the halo chunk's first sample
#pragma unroll
            for (int mm = MLO; mm < 12; ++mm) {
                const typename ET::frag bf = ET::as_frag(*(const u32x4*)(urow + (((c0 + 16 * mm) & (2 * TL - 1)) ^ swz_mm)));
                if (mm <= 9) acc0 = ET::mfma(A[mm <= 9 ? mm - MLO : 0], bf, acc0);
                if (mm - 2 >= MLO) acc1 = ET::mfma(A[mm - 2 >= MLO ? mm - 2 - MLO : 0], bf, acc1);
                if ((mm & 3) == 3) __builtin_amdgcn_sched_barrier(0);    // at most four B fragments in registers at a time
            }
        }
        // the rest of the next step's rows go out here, behind the MFMAs and ahead of the epilogue, the barrier and the
        // output stage, which they overlap (the B fragments are dead by now); the short-filter form, with six MFMAs
        // to hide behind, measured 1-2 % better with them behind the barrier
        constexpr bool LATE_BEFORE_EPILOGUE = MLO == 0;
        if (NEARLY < NP && LATE_BEFORE_EPILOGUE) {
            __builtin_amdgcn_sched_barrier(0);
            if (WHOLE || ts + TL < t_end) load_pieces(ts + TL, NEARLY, NP, whole_tag);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (WHOLE || (compute && slab_live)) {
#pragma unroll
            for (int tau = 0; tau < 2; ++tau) {
                const int tcol = 32 * tau + 64 * s + 16 * hh;
                const f32x16 acc = tau ? acc1 : acc0;
                u32x4 ua = {0, 0, 0, 0}, ub2 = {0, 0, 0, 0};
                if (BIAS == HYENA_BIAS_GATED_FP32) {
                    ua = *(const u32x4*)(urow + cur * TL + (tcol ^ swz_mm));
                    ub2 = *(const u32x4*)(urow + cur * TL + (tcol ^ swz_mm) + 8);
                }
                u32x4 z0, z1;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float a0 = acc[2 * j], a1 = acc[2 * j + 1];
                    if (BIAS == HYENA_BIAS_GATED_FP32) {
                        const uint32_t uw = j < 4 ? ua[j] : ub2[j - 4];
                        a0 = fmaf(bz, ET::lo(uw), a0);
                        a1 = fmaf(bz, ET::hi(uw), a1);
                    }
                    if (BIAS == HYENA_BIAS_ADD) {
                        a0 = ET::round(a0) + bz;
                        a1 = ET::round(a1) + bz;
                    }
                    const uint32_t p = ET::pack2(a0, a1);
                    if (j < 4) z0[j] = p; else z1[j - 4] = p;
                }
                *(u32x4*)(z_lds + (16 * w + c) * ZRS + (tcol ^ swz_mm)) = z0;
                *(u32x4*)(z_lds + (16 * w + c) * ZRS + (tcol ^ swz_mm) + 8) = z1;
            }
        }
        __syncthreads();
        if (NEARLY < NP && !LATE_BEFORE_EPILOGUE) {
            __builtin_amdgcn_sched_barrier(0);
            if (WHOLE || ts + TL < t_end) load_pieces(ts + TL, NEARLY, NP, whole_tag);
        }

        // ---- 8 x 4 transpose back, gate with x2, store rows
        if (WHOLE || (compute && ch_ok)) {
            u32x2 zc[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) zc[c] = *(const u32x2*)(z_lds + (8 * cb + c) * ZRS + ((4 * rb) ^ swz_io));
            // the step's first output row as a block-uniform address, the lane's row and channels as a 32-bit byte offset
            // (the launcher bounds 128 rows of D channels to 2^32 bytes): no 64-bit address per lane and row
            bf16_t* const out_step = out + (b * L + ts) * D;
            bf16_t* const y2_step = (AUX && !FEAT && y2_out) ? y2_out + (b * L + ts) * D : nullptr;
            uint32_t lane_row_b = ((uint32_t)(4 * rb) * (uint32_t)D + dch) * 2u;
            const uint32_t row_b = (uint32_t)D * 2u;
            asm volatile("" : "+v"(lane_row_b));      // keeps the compiler from folding it into four per-lane row pointers held (and spilled) across the loop
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t t = ts + 4 * rb + q;
                u32x4 zz;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    zz[j] = (q & 1) ? pair_hi(zc[2 * j][q >> 1], zc[2 * j + 1][q >> 1])
                                    : pair_lo(zc[2 * j][q >> 1], zc[2 * j + 1][q >> 1]);
                if (WHOLE || t < t_end) {
                    if (AUX && !FEAT && y2_out) *(u32x4*)((char*)y2_step + (lane_row_b + q * row_b)) = zz;
                    u32x4 o = zz;
                    if (POST) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            o[j] = ET::pack2(ET::lo(zz[j]) * ET::lo(g2[q][j]), ET::hi(zz[j]) * ET::hi(g2[q][j]));
                    }
                    u32x4* const dst = (u32x4*)((char*)out_step + (lane_row_b + q * row_b));
                    if (NT) __builtin_nontemporal_store(o, dst);
                    else *dst = o;
                }
            }
        }
        cur ^= 1;
    };
    // The steps in the middle of a segment take the form without tests: with a branch around a request or a store the
    // compiler has to assume that nothing younger is in flight and waits for everything at the next use of a row piece,
    // the stores of the step before included; counted exactly, that wait leaves the four stores outstanding.  The steps
    // at either end (the halo step, the last two) keep their tests, and the state handed to the first whole step is made
    // known by an explicit wait for everything.  Measured at the config-2 / config-1 shapes: fused Hyena-MR layer 0.506 ->
    // 0.488-0.490 ms, fused Hyena-SE layer 55.6 -> 52.5-53.1 us; with the gates given as tensors 0.4546 -> 0.4585 ms
    // (all of the next step's rows go out at once there, on top of the stores; 0.4568 ms with them held back behind the
    // barrier), so that form keeps its tests.
    int64_t ts = ts0;
    if (!AUX && FEAT != 0 && d0 + CB <= (uint32_t)D) {
        for (; ts < t_begin; ts += TL) step(ts, std::false_type{});
        if (ts + 2 * TL <= t_end) {
            __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0)
            for (; ts + 2 * TL <= t_end; ts += TL) step(ts, std::true_type{});
        }
    }
    for (; ts < t_end; ts += TL) step(ts, std::false_type{});

    // ---- cache tail from the ring: chunk cur ^ 1 holds samples ts_last .. ts_last + 127, chunk cur the 128 before
    if (AUX && FEAT && bx_out && t_end == L) {
        const int ntail = (int)(L - bx_from);                        // <= K - 1 <= 127 (checked by the launcher)
        for (int e = tid; e < ntail * (CB / 8); e += 256) {
            const int ti = e >> 3, oc = e & 7;
            const int rel = (int)(bx_from + ti - (ts_last - TL));    // 1 .. 255
            const int chunk = rel >= TL ? (cur ^ 1) : cur, pos = rel & (TL - 1);
            if (d0 + 8 * oc < (uint32_t)D) {
                u32x4 o;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int c0 = 8 * oc + 2 * j, c1 = c0 + 1;      // both in slab (8*oc) >> 4
                    const int p = chunk * TL + (pos ^ (32 * (oc >> 1)));
                    o[j] = (uint32_t)u_lds[c0 * URS + p] | ((uint32_t)u_lds[c1 * URS + p] << 16);
                }
                *(u32x4*)(bx_out + (b * (int64_t)ntail + ti) * D + d0 + 8 * oc) = o;
            }
        }
    }
}

// Featurizer and gates for the sequence-major operators (Hyena-LI): u [B][L][3D] in, xv = bf16(x1*v) and x2 out as
// [B][D][Lout] rows (Lout = L + pad, the first `pad` columns zero).  One block takes 64 operator channels x 256
// output columns: the lanes evaluate the featurizer on their 4 rows x 8 channels as in fir_cl_kernel (two passes of
// 128 rows), transpose into two LDS tiles [64 ch][256 columns] and the block stores 512-byte runs of each channel
// row; a block walks several consecutive tiles, the first row pieces of the next one requested before the stores.
// Blocks with neighbouring ids take neighbouring channel strips of the same rows.  Plain (cached) stores: the
// neighbouring runs of a row written by the next tiles merge in the cache (measured 3-8 % faster than streaming stores).
constexpr int GT = 256;        // output columns per block
constexpr int GRS = 264;       // row stride (elements) of the transposed tiles: 528 B = 16 * 33

template <int FEAT, int KS>
__global__ __launch_bounds__(256, 2) void proj_gates_kernel(ProjFwd pj, bf16_t* __restrict__ xv_out,
                                                            bf16_t* __restrict__ x2_out, int64_t L, int64_t Lout,
                                                            int64_t out_rs, int pad, int64_t D, int ndb, int nchunk,
                                                            int ntpb) {
    constexpr int RF = KS - 1, NR = 4 + RF;
    __shared__ __attribute__((aligned(16))) bf16_t xv_t[CB * GRS];
    __shared__ __attribute__((aligned(16))) bf16_t x2_t[CB * GRS];
    __shared__ __attribute__((aligned(16))) float w_lds[(KS + 1) * 3 * CB];
    const int tid = threadIdx.x;
    const uint32_t bid = blockIdx.x;
    // Workgroups are dealt to the 8 XCDs in turn (id mod 8): XCD x takes the x-th eighth of the channel blocks of a row
    // tile, neighbouring strips, so that its L2 fetches 3 KB runs of each row (D = 4096) instead of every eighth 384-byte
    // piece: 2.27 -> 2.18 ms at the config-3 shape.  (The same order made fir_cl_kernel slower: 0.457 -> 0.509 ms with
    // the gates given as tensors.)
    uint32_t db = bid % (uint32_t)ndb;
    if ((ndb & 7) == 0) db = (db & 7u) * ((uint32_t)ndb >> 3) + (db >> 3);
    const uint32_t chunk = (bid / (uint32_t)ndb) % (uint32_t)nchunk;      // ntpb consecutive tiles along the columns
    const int64_t b = bid / ((uint32_t)ndb * (uint32_t)nchunk);
    const uint32_t d0 = db * CB;
    const int64_t c_begin = (int64_t)chunk * ntpb * GT;
    const int64_t c_end = c_begin + (int64_t)ntpb * GT < Lout ? c_begin + (int64_t)ntpb * GT : Lout;
    if (c_begin >= c_end) return;

    const int cb = tid & 7, rb = tid >> 3;
    const int swz_io = 32 * (cb >> 1);                     // as in fir_cl_kernel: keeps the 8-byte transposed writes off each other's banks
    const uint32_t dch = d0 + 8 * cb;
    const bool ch_ok = dch < (uint32_t)D;
    const bf16_t* pp[3];
#pragma unroll
    for (int i = 0; i < 3; ++i)
        pp[i] = FEAT == 3 ? pj.u + b * pj.bs + 3 * (int64_t)dch + 8 * i : pj.u + b * pj.bs + pj.chan(i, ch_ok ? dch : 0);

    const u32x4 zero4 = {0, 0, 0, 0};
    // the 18 (21) row pieces of one pass of 128 columns starting at column cs; rows past either end read as zero
    // whole_tag: every row of the pass exists and so does every channel of the block; the requests carry no test then
    auto load_pass = [&](int64_t cs, u32x4 (&raw)[3][NR], auto whole_tag) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t t = cs + 4 * rb + r - RF - pad;  // input sample of this row
            const bool ok = WHOLE || (ch_ok && t >= 0 && t < L);
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                if (WHOLE) raw[i][r] = *(const u32x4*)(pp[i] + t * pj.ts);
                else raw[i][r] = ok ? *(const u32x4*)(pp[i] + t * pj.ts) : zero4;
            }
        }
    };
    u32x4 raw[3][NR];
    load_pass(c_begin, raw, std::false_type{});            // travels while the tap table is staged

    for (int e = tid; e < (KS + 1) * 3 * CB; e += 256) {   // taps / bias of the block's channels in lane-piece order
        const int k = e / (3 * CB), r = e - k * 3 * CB, i = r / CB, dl = r - i * CB;
        const uint32_t dd = d0 + dl;
        float val = 0.f;
        if (dd < (uint32_t)D) {
            const uint32_t ch = FEAT == 3 ? 3 * (d0 + (dl & ~7)) + 8 * i + (dl & 7) : pj.chan(i, dd);
            if (k < KS) val = pj.w[(int64_t)k * 3 * D + ch];
            else if (pj.bias) val = pj.bias[ch];
        }
        w_lds[e] = val;
    }
    __syncthreads();

    // featurizer, gates and the 4 x 8 transposes of one pass into half `half` of the two tiles
    auto gate_pass = [&](int64_t cs, int half, const u32x4 (&raw)[3][NR]) __attribute__((always_inline)) {
        u32x4 bx[4], g2[4];
        lane_gates<FEAT, KS>(raw, w_lds, cb, pj, bx, g2);
        if (cs < pad) {                                    // the padding columns stay zero, bias or not
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (cs + 4 * rb + q < pad) { bx[q] = zero4; g2[q] = zero4; }
        }
        bf16_t* xb = xv_t + (8 * cb) * GRS + half * TL + ((4 * rb) ^ swz_io);
        bf16_t* gb = x2_t + (8 * cb) * GRS + half * TL + ((4 * rb) ^ swz_io);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            u32x2 t2, t3;
            if (c & 1) {
                t2[0] = pair_hi(bx[0][c >> 1], bx[1][c >> 1]); t2[1] = pair_hi(bx[2][c >> 1], bx[3][c >> 1]);
                t3[0] = pair_hi(g2[0][c >> 1], g2[1][c >> 1]); t3[1] = pair_hi(g2[2][c >> 1], g2[3][c >> 1]);
            } else {
                t2[0] = pair_lo(bx[0][c >> 1], bx[1][c >> 1]); t2[1] = pair_lo(bx[2][c >> 1], bx[3][c >> 1]);
                t3[0] = pair_lo(g2[0][c >> 1], g2[1][c >> 1]); t3[1] = pair_lo(g2[2][c >> 1], g2[3][c >> 1]);
            }
            *(u32x2*)(xb + c * GRS) = t2;
            *(u32x2*)(gb + c * GRS) = t3;
        }
    };

    const int l32 = tid & 31, r8 = tid >> 5;
    const int tcol = 8 * l32;
    // One tile.  whole_tag: this tile and the next lie inside the block's columns, all their input rows exist and so does
    // every channel of the block: no test guards a request or a store then.
    auto tile_step = [&](const int64_t c0, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        const bool second = WHOLE || c0 + TL < c_end, next = WHOLE || c0 + GT < c_end;
        gate_pass(c0, 0, raw);
        if (second) {
            load_pass(c0 + TL, raw, whole_tag);
            gate_pass(c0 + TL, 1, raw);
        }
        if (next) load_pass(c0 + GT, raw, whole_tag);      // travels during the stores
        __syncthreads();
        // ---- stores: 32 lanes cover the 512 bytes of one channel row, 8 rows per round, xv then x2
        const int64_t col = c0 + tcol;
        auto store_round = [&](int rnd) __attribute__((always_inline)) {
            const int rr = rnd * 8 + r8, ch = rr & (CB - 1);
            if (!WHOLE && d0 + ch >= (uint32_t)D) return;
            const bf16_t* tile = rr < CB ? xv_t : x2_t;
            const u32x4 o = *(const u32x4*)(tile + ch * GRS + (tcol & TL) + ((tcol & (TL - 1)) ^ (32 * (ch >> 4))));
            *(u32x4*)((rr < CB ? xv_out : x2_out) + (b * D + d0 + ch) * out_rs + col) = o;
        };
        if constexpr (WHOLE) {
#pragma unroll
            for (int rnd = 0; rnd < 2 * CB / 8; ++rnd) store_round(rnd);       // straight-line: the sixteen stores are counted
        } else if (col < Lout) {
#pragma unroll 4
            for (int rnd = 0; rnd < 2 * CB / 8; ++rnd) store_round(rnd);
        }
        if (next) __syncthreads();                         // the tiles are free again
    };
    // Tiles in the middle of the block's run take the form without tests (see fir_cl_kernel: with a branch around a
    // request or a store the compiler waits for everything in flight, the stores of the tile before included, at the
    // next use of a row piece); the first tile of the sequence, whose first rows do not exist, and a run's last two keep
    // their tests.
    int64_t c0 = c_begin;
    if (KS <= 3 && d0 + CB <= (uint32_t)D) {              // (with four taps the second copy of the step does not fit the registers)
        for (; c0 < c_end && c0 < pad + RF; c0 += GT) tile_step(c0, std::false_type{});
        if (c0 + 2 * GT <= c_end) {
            __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0): a known state for the counted waits
#pragma unroll 1
            for (; c0 + 2 * GT <= c_end; c0 += GT) tile_step(c0, std::true_type{});
        }
    }
#pragma unroll 1
    for (; c0 < c_end; c0 += GT) tile_step(c0, std::false_type{});
}

// the float16 traits where that form exists (no featurizer), bfloat16 otherwise (the launcher refuses float16 there)
template <int FEAT> using F16For = typename std::conditional<FEAT == 0, ElF16, ElBf16>::type;

struct LaunchArgs {
    ClMap x1, x2, v;
    ProjFwd pj;
    int feat, ks;
    bool pre, post;
    bool f16;                  // float16 tensors (gates given, no featurizer); bfloat16 otherwise
};

static int fir_cl_launch(const LaunchArgs& a, const float* h, int taps_reversed, const float* bias, int bias_mode,
                         void* out, void* y2_out, void* bx_out, int64_t bx_from, int64_t B, int64_t L, int64_t D,
                         int64_t G, int K, void* stream, const char* who) {
    if (!h || !out) return hyena_fail(HYENA_EINVAL, "%s: h and out are required", who);
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0 || D >= (1LL << 24))
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld L=%lld G=%lld", who, (long long)B, (long long)D,
                          (long long)L, (long long)G);
    if (K < 1 || K > 128) return hyena_fail(HYENA_ENOSUP, "%s: K=%d outside 1..128", who, K);
    if ((D / G) % 16 != 0)
        return hyena_fail(HYENA_ENOSUP, "%s: D/G=%lld must be a multiple of 16", who, (long long)(D / G));
    if (bias_mode < 0 || bias_mode > 4 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "%s: bias_mode %d needs a bias pointer", who, bias_mode);
    if (bias_mode > HYENA_BIAS_GATED_FP32)
        return hyena_fail(HYENA_ENOSUP, "%s: bias_mode %d is built for the sequence-major kernels only", who, bias_mode);
    if (bx_out && (bx_from < 0 || bx_from > L)) return hyena_fail(HYENA_EINVAL, "%s: bx_from outside 0..L", who);
    if (a.f16 && a.feat) return hyena_fail(HYENA_ENOSUP, "%s: the fused featurizer takes bfloat16 only", who);
    if (bx_out && a.feat && L - bx_from > K - 1)
        return hyena_fail(HYENA_ENOSUP, "%s: with the featurizer fused, bx is the cache tail (at most K-1 = %d samples)",
                          who, K - 1);
    if ((((uintptr_t)out | (uintptr_t)y2_out | (uintptr_t)bx_out) & 15))
        return hyena_fail(HYENA_EALIGN, "%s: outputs must be 16-byte aligned", who);
    if (B == 0 || L == 0) return 0;

    // Segments along L.  512 blocks are resident at a time (2 per CU); pick the segment count whose block
    // count fills whole rounds of 512 best, charging each segment its extra halo step: 128 samples, or about a
    // third of that for the short-filter variant, which reads only the last 24 rows of it.
    const bool aux = y2_out || bx_out;
    const bool shortk = K <= 17 && a.pre && bias_mode == HYENA_BIAS_NONE;
    const double halo_cost = shortk ? 40.0 : (double)TL;
    // Strips of 64 channels per block (see the kernel): three with the gates given, two with the featurizer fused in
    // (its registers allow two wavefronts per SIMD), for bfloat16 launches without intermediates on tensors that stream
    // through the last-level cache.  Measured against one strip per block on tensors of 0.5 to 8.6 GB (D = 1024 .. 8192,
    // rows of 8192 .. 262144 samples, 7 and 128 taps): 3-14 % less time with the gates given, 1-11 % for the fused layers;
    // tensors that stay in the cache lose 2-11 %, as do rows shorter than 4096 samples in the fused form.
    const bool streams = 8.0 * (double)B * (double)D * (double)L > 384e6;
    const int ns_form = a.feat ? 2 : 3;
    const bool ns_able = !(y2_out || bx_out) && !a.f16 && (D + CB - 1) / CB >= 2 * ns_form;   // (the float16 kernels are built for one strip per block only)
    int ns = (ns_able && streams && L >= 4096) ? ns_form : 1;
    { const int64_t x = hyena_override(HYENA_OV_CL_NS); if (x >= 1) ns = (x > 1 && ns_able) ? ns_form : 1; }
    const int64_t ndb = ((D + CB - 1) / CB + ns - 1) / ns;       // blocks along the channels
    const int64_t rows = B * ndb;
    int64_t nseg = 1;
    {
        const int64_t max_seg = (L + 1023) / 1024 < 64 ? (L + 1023) / 1024 : 64;
        double best = -1.0;
        for (int64_t c = 1; c <= (max_seg < 1 ? 1 : max_seg); ++c) {
            const int64_t sl = ((L + c - 1) / c + TL - 1) / TL * TL;
            const int64_t nb = rows * ((L + sl - 1) / sl);
            const int64_t resident = ns == 1 ? 512 : 256;
            const double fill = (double)nb / (double)((nb + resident - 1) / resident * resident);
            const double score = fill * (double)sl / ((double)sl + halo_cost);
            if (score > best + 1e-9) { best = score; nseg = c; }
        }
    }
    { const int64_t x = hyena_override(HYENA_OV_CL_NSEG); if (x >= 1) nseg = x; }
    int64_t seg_len = (L + nseg - 1) / nseg;
    seg_len = (seg_len + TL - 1) / TL * TL;
    nseg = (L + seg_len - 1) / seg_len;
    const int64_t nblk = rows * nseg;
    if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);

    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)nblk);
    const int dg = (int)(D / G);
    // tensors larger than the last-level cache stream through it: non-temporal accesses then
    bool nt = streams;
    { const int64_t x = hyena_override(HYENA_OV_CL_NT); if (x >= 0) nt = x != 0; }
    bool ok = false;
#define CL_GO_NS(T, P, Q, M, F, KSV, AX, ML, N, NSV)                                                                 \
    hipLaunchKernelGGL((fir_cl_kernel<T, P, Q, M, F, KSV, AX, ML, N, NSV>), grid, dim3(256 * NSV), 0, s, a.x1, a.x2, a.v, \
                       a.pj, h, K, taps_reversed, bias, (bf16_t*)out, (bf16_t*)y2_out, (bf16_t*)bx_out, bx_from, L, D, \
                       dg, seg_len, (int)nseg, (int)ndb)
// several strips per block: bfloat16 without intermediates only (three strips with the gates given, two with the featurizer)
#define CL_GO_T(T, P, Q, M, F, KSV, AX, ML, N)                                                                       \
    do {                                                                                                             \
        if constexpr (!(AX) && std::is_same<T, ElBf16>::value) {                                                     \
            if (ns > 1) { CL_GO_NS(T, P, Q, M, F, KSV, false, ML, N, ((F) == 0 ? 3 : 2)); break; }                   \
        }                                                                                                            \
        CL_GO_NS(T, P, Q, M, F, KSV, AX, ML, N, 1);                                                                  \
    } while (0)
// float16 only exists for the form with the gates given as tensors (F == 0)
#define CL_GO(P, Q, M, F, KSV, AX, ML, N)                                                                         \
    do {                                                                                                          \
        if (a.f16) CL_GO_T(F16For<F>, P, Q, M, F, KSV, AX, ML, N);                                                \
        else CL_GO_T(ElBf16, P, Q, M, F, KSV, AX, ML, N);                                                         \
    } while (0)
#define CL_CASE(P, Q, M, F, KSV)                                                                                  \
    if (!ok && a.pre == P && a.post == Q && bias_mode == M && a.feat == F && (F == 0 || a.ks == KSV)) {           \
        if (aux && shortk) CL_GO(P, Q, M, F, KSV, true, (P && M == HYENA_BIAS_NONE) ? 7 : 0, false);              \
        else if (aux) CL_GO(P, Q, M, F, KSV, true, 0, false);                                                     \
        else if (shortk && nt) CL_GO(P, Q, M, F, KSV, false, (P && M == HYENA_BIAS_NONE) ? 7 : 0, true);          \
        else if (shortk) CL_GO(P, Q, M, F, KSV, false, (P && M == HYENA_BIAS_NONE) ? 7 : 0, false);               \
        else if (nt) CL_GO(P, Q, M, F, KSV, false, 0, true);                                                      \
        else CL_GO(P, Q, M, F, KSV, false, 0, false);                                                             \
        ok = true;                                                                                                \
    }
    CL_CASE(true, true, HYENA_BIAS_NONE, 0, 3)
    CL_CASE(true, true, HYENA_BIAS_GATED_FP32, 0, 3)
    CL_CASE(true, true, HYENA_BIAS_ADD, 0, 3)
    CL_CASE(false, false, HYENA_BIAS_NONE, 0, 3)
    CL_CASE(false, false, HYENA_BIAS_ADD, 0, 3)
    CL_CASE(false, false, HYENA_BIAS_GATED_FP32, 0, 3)
    CL_CASE(true, true, HYENA_BIAS_NONE, 1, 3)
    CL_CASE(true, true, HYENA_BIAS_GATED_FP32, 1, 3)
    CL_CASE(true, true, HYENA_BIAS_NONE, 3, 3)
    CL_CASE(true, true, HYENA_BIAS_GATED_FP32, 3, 3)
    CL_CASE(true, true, HYENA_BIAS_NONE, 1, 4)
    CL_CASE(true, true, HYENA_BIAS_GATED_FP32, 1, 4)
    CL_CASE(true, true, HYENA_BIAS_NONE, 3, 4)
    CL_CASE(true, true, HYENA_BIAS_GATED_FP32, 3, 4)
#undef CL_CASE
#undef CL_GO
#undef CL_GO_T
#undef CL_GO_NS
    if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: this gate / bias / featurizer-length combination has no kernel", who);
    return hyena_check_launch(who);
}

// Validates a prefill featurizer descriptor and fills the launch arguments (feat = 1: unit channel stride, 3: interleaved)
static int make_proj_fwd(const hyena_proj_fwd* proj, int64_t D, const char* who, LaunchArgs& a) {
    if (!proj || !proj->u || !proj->w) return hyena_fail(HYENA_EINVAL, "%s: proj, proj->u, proj->w are required", who);
    if (proj->Ks != 3 && proj->Ks != 4)
        return hyena_fail(HYENA_ENOSUP, "%s: featurizer length %d (3 or 4 supported)", who, proj->Ks);
    if (D <= 0 || D % 8 != 0 || ((uintptr_t)proj->u & 15) || proj->u_batch_stride % 8 != 0 ||
        proj->u_time_stride % 8 != 0)
        return hyena_fail(HYENA_EALIGN, "%s: D and strides must be multiples of 8, u 16-byte aligned", who);
    if (proj->ch_inner <= 0 || proj->ch_outer < 0 || proj->gate_stride <= 0)
        return hyena_fail(HYENA_EINVAL, "%s: bad featurizer channel map", who);
    if (proj->u_time_stride < 0 || proj->u_time_stride >= (1LL << 24) || D >= (1LL << 24))
        return hyena_fail(HYENA_EINVAL, "%s: u_time_stride and D must lie below 2^24 (32-bit byte offsets inside a step)", who);
    a.pj.u = (const bf16_t*)proj->u; a.pj.bs = proj->u_batch_stride; a.pj.ts = proj->u_time_stride;
    a.pj.w = proj->w; a.pj.bias = proj->bias;
    a.pj.ch_inner = (uint32_t)(proj->ch_inner > D ? D : proj->ch_inner); a.pj.ch_outer = (uint32_t)proj->ch_outer;
    a.pj.gate_stride = (uint32_t)proj->gate_stride; a.pj.flip = proj->flip_x1x2 != 0;
    if (proj->ch_stride == 3 && proj->gate_stride == 1 && proj->ch_inner >= D) a.feat = 3;
    else if (proj->ch_stride == 1 && proj->ch_inner % 8 == 0 && proj->ch_outer % 8 == 0 && proj->gate_stride % 8 == 0) {
        a.feat = 1;
        const int64_t last = ((D - 1) / proj->ch_inner) * proj->ch_outer + 2 * proj->gate_stride + (D - 1) % proj->ch_inner;
        if (last >= 3 * D) return hyena_fail(HYENA_EINVAL, "%s: featurizer channel map reaches channel %lld of %lld", who,
                                             (long long)last, (long long)(3 * D));
    } else return hyena_fail(HYENA_ENOSUP, "%s: this featurizer channel map has no fused kernel", who);
    a.ks = proj->Ks; a.pre = true; a.post = true;
    return 0;
}

static bool cl_ok(const hyena_cl* c) {
    return c && c->ptr && !((uintptr_t)c->ptr & 15) && c->batch_stride % 8 == 0 && c->time_stride % 8 == 0;
}
// the kernels address a lane's rows with 32-bit byte offsets inside a 128-row step
static bool cl_stride_ok(const hyena_cl* c) { return c->time_stride >= 0 && c->time_stride < (1LL << 24); }

}  // namespace

extern "C" int hyena_fir_cl_fwd(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h,
                                int taps_reversed, const float* bias, int bias_mode, void* out, void* y2_out,
                                void* bx_out, int64_t bx_from, int64_t B, int64_t L, int64_t D, int64_t G, int K,
                                void* stream) {
    const char* who = "hyena_fir_cl_fwd";
    if (!x1 || !x1->ptr) return hyena_fail(HYENA_EINVAL, "%s: x1 is required", who);
    const bool pre = v && v->ptr, post = x2 && x2->ptr;
    if (pre != post) return hyena_fail(HYENA_ENOSUP, "%s: pass both gates v and x2, or neither", who);
    if (!cl_ok(x1) || (pre && (!cl_ok(v) || !cl_ok(x2))) || D % 8 != 0)
        return hyena_fail(HYENA_EALIGN, "%s: D and strides must be multiples of 8, pointers 16-byte aligned", who);
    if (!cl_stride_ok(x1) || (pre && (!cl_stride_ok(v) || !cl_stride_ok(x2))))
        return hyena_fail(HYENA_EINVAL, "%s: time strides must lie in 0 .. 2^24 - 1 elements", who);
    LaunchArgs a = {};
    a.x1 = {(const bf16_t*)x1->ptr, x1->batch_stride, x1->time_stride};
    if (pre) {
        a.v = {(const bf16_t*)v->ptr, v->batch_stride, v->time_stride};
        a.x2 = {(const bf16_t*)x2->ptr, x2->batch_stride, x2->time_stride};
    }
    a.feat = 0; a.ks = 3; a.pre = pre; a.post = post;
    return fir_cl_launch(a, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D, G, K, stream, who);
}

extern "C" int hyena_fir_cl_fwd_dtype(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v, const float* h,
                                      int taps_reversed, const float* bias, int bias_mode, void* out, void* y2_out,
                                      void* bx_out, int64_t bx_from, int64_t B, int64_t L, int64_t D, int64_t G, int K,
                                      int dtype, void* stream) {
    const char* who = "hyena_fir_cl_fwd_dtype";
    if (dtype == HYENA_DTYPE_BF16 && K <= 128)
        return hyena_fir_cl_fwd(x1, x2, v, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D, G, K,
                                stream);
    if (dtype != HYENA_DTYPE_BF16 && dtype != HYENA_DTYPE_F16 && dtype != HYENA_DTYPE_F32)
        return hyena_fail(HYENA_EINVAL, "%s: unknown dtype %d", who, dtype);
    if (!x1 || !x1->ptr || !h || !out) return hyena_fail(HYENA_EINVAL, "%s: x1, h and out are required", who);
    const bool pre = v && v->ptr, post = x2 && x2->ptr;
    if (pre != post) return hyena_fail(HYENA_ENOSUP, "%s: pass both gates v and x2, or neither", who);
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0 || D >= (1LL << 24))
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld L=%lld G=%lld", who, (long long)B, (long long)D,
                          (long long)L, (long long)G);
    if (K < 1 || K > (1 << 20)) return hyena_fail(HYENA_ENOSUP, "%s: K=%d outside 1..2^20", who, K);
    if (bias_mode < 0 || bias_mode > 4 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "%s: bias_mode %d needs a bias pointer", who, bias_mode);
    if (bx_out && (bx_from < 0 || bx_from > L)) return hyena_fail(HYENA_EINVAL, "%s: bx_from outside 0..L", who);
    const uintptr_t esz = dtype == HYENA_DTYPE_F32 ? 4 : 2;
    auto el_ok = [&](const hyena_cl* c) { return ((uintptr_t)c->ptr & (esz - 1)) == 0 && c->time_stride >= 0; };
    if (!el_ok(x1) || (pre && (!el_ok(v) || !el_ok(x2))) ||
        (((uintptr_t)out | (uintptr_t)y2_out | (uintptr_t)bx_out) & (esz - 1)))
        return hyena_fail(HYENA_EALIGN, "%s: pointers must be aligned to the element size, time strides non-negative", who);
    if (B == 0 || L == 0) return 0;
    // float16: the MFMA form where its shape and alignment rules hold
    if (dtype == HYENA_DTYPE_F16 && K <= 128 && (D / G) % 16 == 0 && D % 8 == 0 && bias_mode <= HYENA_BIAS_GATED_FP32 && cl_ok(x1) &&
        cl_stride_ok(x1) && (!pre || (cl_ok(v) && cl_ok(x2) && cl_stride_ok(v) && cl_stride_ok(x2))) &&
        !(((uintptr_t)out | (uintptr_t)y2_out | (uintptr_t)bx_out) & 15)) {
        LaunchArgs a = {};
        a.x1 = {(const bf16_t*)x1->ptr, x1->batch_stride, x1->time_stride};
        if (pre) {
            a.v = {(const bf16_t*)v->ptr, v->batch_stride, v->time_stride};
            a.x2 = {(const bf16_t*)x2->ptr, x2->batch_stride, x2->time_stride};
        }
        a.feat = 0; a.ks = 3; a.pre = pre; a.post = post; a.f16 = true;
        return fir_cl_launch(a, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D, G, K, stream, who);
    }
    return hyena_fir_cl_direct(x1, x2, v, h, taps_reversed, bias, bias_mode, out, y2_out, bx_out, bx_from, B, L, D, G, K,
                               dtype, stream, who);
}

extern "C" int hyena_fir_layer_fwd(const hyena_proj_fwd* proj, const float* h, int taps_reversed, const float* bias,
                                   int bias_mode, void* out, void* bx_out, int64_t bx_from, int64_t B, int64_t L,
                                   int64_t D, int64_t G, int K, void* stream) {
    const char* who = "hyena_fir_layer_fwd";
    LaunchArgs a = {};
    if (int rc = make_proj_fwd(proj, D, who, a)) return rc;
    if (bias_mode == HYENA_BIAS_ADD) return hyena_fail(HYENA_ENOSUP, "%s: additive inner bias", who);
    return fir_cl_launch(a, h, taps_reversed, bias, bias_mode, out, nullptr, bx_out, bx_from, B, L, D, G, K, stream, who);
}

extern "C" int hyena_featurizer_gates_fwd(const hyena_proj_fwd* proj, void* xv_out, void* x2_out, int64_t out_row_stride,
                                          int64_t B, int64_t L, int64_t D, int front_pad, void* stream) {
    const char* who = "hyena_featurizer_gates_fwd";
    if (!xv_out || !x2_out) return hyena_fail(HYENA_EINVAL, "%s: both outputs are required", who);
    if (B < 0 || L < 0 || D >= (1LL << 30)) return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld L=%lld D=%lld", who,
                                                               (long long)B, (long long)L, (long long)D);
    if (front_pad < 0 || front_pad > 7) return hyena_fail(HYENA_EINVAL, "%s: front_pad %d outside 0..7", who, front_pad);
    LaunchArgs a = {};
    if (int rc = make_proj_fwd(proj, D, who, a)) return rc;
    const int64_t Lout = L > 0 ? L + front_pad : 0;
    if (Lout % 8 != 0 || out_row_stride % 8 != 0 || (((uintptr_t)xv_out | (uintptr_t)x2_out) & 15))
        return hyena_fail(HYENA_EALIGN, "%s: L + front_pad and out_row_stride must be multiples of 8, outputs 16-byte aligned", who);
    if (out_row_stride < Lout) return hyena_fail(HYENA_EINVAL, "%s: out_row_stride %lld below the %lld columns of a row", who,
                                                 (long long)out_row_stride, (long long)Lout);
    if (B == 0 || L == 0) return 0;
    const int64_t ndb = (D + CB - 1) / CB, ntt = (Lout + GT - 1) / GT;
    // consecutive tiles per block (the tap table is staged once, the next tile's rows travel during the stores): as
    // many as leave about four rounds of resident blocks (512 at a time), at most 4 (measured flat from 2 to 8)
    int64_t ntpb = B * ndb * ntt / 2048;
    ntpb = ntpb < 1 ? 1 : (ntpb > 4 ? 4 : ntpb);
    { const int64_t x = hyena_override(HYENA_OV_CL_NSEG); if (x >= 1) ntpb = (ntt + x - 1) / x; }
    const int64_t nchunk = (ntt + ntpb - 1) / ntpb;
    if (B * ndb * nchunk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);
    dim3 grid((unsigned)(B * ndb * nchunk));
    hipStream_t s = (hipStream_t)stream;
#define PG_GO(F, KSV)                                                                                              \
    hipLaunchKernelGGL((proj_gates_kernel<F, KSV>), grid, dim3(256), 0, s, a.pj, (bf16_t*)xv_out, (bf16_t*)x2_out, L, \
                       Lout, out_row_stride, front_pad, D, (int)ndb, (int)nchunk, (int)ntpb)
    if (a.feat == 3 && a.ks == 3) PG_GO(3, 3);
    else if (a.feat == 3) PG_GO(3, 4);
    else if (a.ks == 3) PG_GO(1, 3);
    else PG_GO(1, 4);
#undef PG_GO
    return hyena_check_launch(who);
}
