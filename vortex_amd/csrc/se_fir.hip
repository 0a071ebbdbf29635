// Hyena-SE: gated causal depthwise short FIR, direct form, HBM-bound.
//
// One lane owns 8 consecutive samples of one (batch, channel) row: three 16-byte
// loads (x1, v, x2), one 16-byte store.  The K-1 samples a lane needs from
// before its octet come from the neighbouring lane through a wavefront shuffle;
// only lane 0 of a wavefront (or the first octet of a row) touches memory again
// for them.  Accumulation is fp32; the two roundings to bf16 are where
// vortex/model/engine.py:159 and :208 put them.
#include "common.h"

namespace {

template <bool NT>
__device__ __forceinline__ u32x4 ld16(const bf16_t* p) {
    return NT ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
}

// Three-tap featurizer FIR on one octet of a raw projection row; hw holds the two samples ahead of it.  fp32 FMAs,
// oldest sample first, one rounding to bf16: the arithmetic of the other featurizer kernels.
__device__ __forceinline__ u32x4 feat3(const u32x4 cc, const uint32_t hw, const float (&w)[3]) {
    float rr[10];
    rr[0] = bf_lo(hw);
    rr[1] = bf_hi(hw);
#pragma unroll
    for (int j = 0; j < 4; ++j) { rr[2 + 2 * j] = bf_lo(cc[j]); rr[3 + 2 * j] = bf_hi(cc[j]); }
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float f0 = fmaf(w[2], rr[2 * j + 2], fmaf(w[1], rr[2 * j + 1], fmaf(w[0], rr[2 * j], 0.f)));
        const float f1 = fmaf(w[2], rr[2 * j + 3], fmaf(w[1], rr[2 * j + 2], fmaf(w[0], rr[2 * j + 1], 0.f)));
        o[j] = pack_bf2(f0, f1);
    }
    return o;
}

// FEAT = 3: the rows are the raw projection of the layer, stored sequence-major; the three-tap featurizer FIR of
// vortex/model/model.py:233-246 (vortex/model/engine.py:188-223 with gate = False) runs on the lane's octets first.
// Its two samples of history are the last dword of the lane to the left (a wavefront shift); lane 0 of a wavefront
// fetches them, and those of the octet it reloads for the inner filter's halo, from memory.
template <int K, bool PRE, bool POST, int BIAS, bool ROWU, bool NT, int FEAT = 0>
__global__ __launch_bounds__(256) void se_fir_kernel(RowMap x1, RowMap x2, RowMap v,
                                                     const float* __restrict__ taps,
                                                     const float* __restrict__ bias,
                                                     bf16_t* __restrict__ out,
                                                     int64_t D, int64_t L, int dg, int dg_shift,
                                                     int64_t octs_per_row, int64_t total_octs,
                                                     const float* __restrict__ ftaps) {
    static_assert(FEAT == 0 || (FEAT == 3 && PRE && POST), "featurizer: three taps, all three gates");
    constexpr int H = K - 1;                 // halo samples
    constexpr int HD = (H + 1) / 2;          // halo dwords taken from the previous lane
    // all index arithmetic in 32 bits: the host checks that B*D and L/8 fit
    uint32_t row, oct;
    uint32_t b, d;
    // Workgroups are dealt to the 8 XCDs in turn (linear id mod 8).  For tensors that stream through the caches XCD x
    // takes the x-th eighth of the blocks in memory order, so that each XCD walks one contiguous part of the tensors.
    uint32_t gx = blockIdx.x, gy = blockIdx.y, gz = blockIdx.z;
    if (NT) {
        const uint32_t nb = gridDim.x * gridDim.y * gridDim.z;         // the host bounds the block count to 2^31
        if ((nb & 7u) == 0) {
            uint32_t lid = gx + gridDim.x * (gy + gridDim.y * gz);
            lid = (lid & 7u) * (nb >> 3) + (lid >> 3);
            gx = lid % gridDim.x;
            lid /= gridDim.x;
            gy = lid % gridDim.y;
            gz = lid / gridDim.y;
        }
    }
    if (ROWU) {                              // a block never straddles rows: grid = (blocks per row, D, B)
        d = gy;
        b = gz;
        row = b * (uint32_t)D + d;
        oct = gx * 256u + threadIdx.x;
    } else {
        const uint64_t idx = (uint64_t)gx * 256u + threadIdx.x;
        row = (uint32_t)(idx / (uint32_t)octs_per_row);
        oct = (uint32_t)(idx - (uint64_t)row * (uint32_t)octs_per_row);
    }
    const bool active = ROWU ? true : ((uint64_t)row * (uint64_t)octs_per_row + oct < (uint64_t)total_octs);
    if (!active) { row = 0; oct = 0; }
    if (!ROWU) { b = row / (uint32_t)D; d = row - b * (uint32_t)D; }
    const int64_t t0 = (int64_t)oct * 8;
    // dg_shift >= 0: D/G is a power of two and the group index is a shift
    const int g = dg_shift >= 0 ? (int)(d >> dg_shift) : (int)(d / (uint32_t)dg);

    float w[K];
#pragma unroll
    for (int k = 0; k < K; ++k) w[k] = taps[g * K + k];

    const bf16_t* p1 = x1.row(b, d) + t0;
    const bf16_t* pvv = PRE ? v.row(b, d) + t0 : nullptr;
    u32x4 a1 = ld16<NT>(p1);
    u32x4 av = {0, 0, 0, 0}, a2 = {0, 0, 0, 0};
    if (PRE) av = ld16<NT>(pvv);
    const bf16_t* p2 = POST ? x2.row(b, d) + t0 : nullptr;
    if (POST) a2 = ld16<NT>(p2);
    // lane 0 of a wavefront cannot get its halo from a neighbour: it reloads the previous octet, and
    // the reload is issued here, together with the main loads, so that its latency is not exposed
    const int lane = threadIdx.x & 63;
    const bool reload = (lane == 0) && (oct != 0);
    u32x4 h1 = {0, 0, 0, 0}, hv = {0, 0, 0, 0};
    uint32_t g1 = 0, gv = 0, g2 = 0, gg1 = 0, ggv = 0;      // FEAT, lane 0: the dwords ahead of this octet and of the reloaded one
    if (reload) {
        h1 = *(const u32x4*)(p1 - 8);
        if (PRE) hv = *(const u32x4*)(pvv - 8);
        if constexpr (FEAT != 0) {
            g1 = h1[3];
            gv = hv[3];
            g2 = *(const uint32_t*)(p2 - 2);
            if (oct > 1) { gg1 = *(const uint32_t*)(p1 - 10); ggv = *(const uint32_t*)(pvv - 10); }
        }
    }
    if constexpr (FEAT != 0) {
        float f1w[3], fvw[3], f2w[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            f1w[k] = ftaps[(int64_t)d * 3 + k];
            f2w[k] = ftaps[((int64_t)D + d) * 3 + k];
            fvw[k] = ftaps[((int64_t)2 * D + d) * 3 + k];
        }
        // history of this octet: the left neighbour's last dword; lane 0 keeps what it fetched, the first octet of a
        // row has none (a wavefront may straddle rows when blocks do)
        uint32_t q1 = (uint32_t)__builtin_amdgcn_update_dpp((int)g1, (int)a1[3], 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
        uint32_t qv = (uint32_t)__builtin_amdgcn_update_dpp((int)gv, (int)av[3], 0x138, 0xf, 0xf, false);
        uint32_t q2 = (uint32_t)__builtin_amdgcn_update_dpp((int)g2, (int)a2[3], 0x138, 0xf, 0xf, false);
        if (oct == 0) { q1 = 0; qv = 0; q2 = 0; }
        a1 = feat3(a1, q1, f1w);
        av = feat3(av, qv, fvw);
        a2 = feat3(a2, q2, f2w);
        if (reload) {
            h1 = feat3(h1, gg1, f1w);
            hv = feat3(hv, ggv, fvw);
        }
    }

    // u = bf16(x1*v), kept both as floats and as packed bf16 pairs
    float u[8];
    uint32_t pk[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (PRE) pk[j] = pack_bf2(bf_lo(a1[j]) * bf_lo(av[j]), bf_hi(a1[j]) * bf_hi(av[j]));
        else pk[j] = a1[j];
        u[2 * j] = bf_lo(pk[j]);
        u[2 * j + 1] = bf_hi(pk[j]);
    }

    // halo: last HD dwords of the previous lane's octet (zeros at the start of a row)
    uint32_t hp[HD];
#pragma unroll
    for (int j = 0; j < HD; ++j) {
        const int q = 4 - HD + j;
        hp[j] = __shfl_up(pk[q], 1, 64);
        if (lane == 0 || oct == 0) {
            hp[j] = 0;
            if (reload) hp[j] = PRE ? pack_bf2(bf_lo(h1[q]) * bf_lo(hv[q]), bf_hi(h1[q]) * bf_hi(hv[q])) : h1[q];
        }
    }

    // ext = [K-1 halo samples | 8 own samples]
    float ext[H + 8];
#pragma unroll
    for (int i = 0; i < H; ++i) {
        const int e = 2 * HD - H + i;                      // element inside hp[] (skip one if H is odd)
        ext[i] = (e & 1) ? bf_hi(hp[e >> 1]) : bf_lo(hp[e >> 1]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) ext[H + i] = u[i];

    float bz = 0.f;
    if (BIAS != HYENA_BIAS_NONE) bz = bias[d];

    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float z[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int i = 2 * j + e;
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < K; ++k) acc = fmaf(w[k], ext[i + k], acc);
            if (BIAS == HYENA_BIAS_GATED_FP32) acc = fmaf(bz, u[i], acc);
            if (BIAS == HYENA_BIAS_ADD_FP32) acc += bz;
            z[e] = acc;
        }
        uint32_t zp = pack_bf2(z[0], z[1]);                      // z = bf16(conv), one conversion per pair
        if (BIAS == HYENA_BIAS_ADD) zp = pack_bf2(bf_lo(zp) + bz, bf_hi(zp) + bz);
        if (BIAS == HYENA_BIAS_GATED_BF16) {                     // bf16 tensor arithmetic: every product and sum rounded
            const uint32_t tp = pack_bf2(bz * u[2 * j], bz * u[2 * j + 1]);
            zp = pack_bf2(bf_lo(zp) + bf_lo(tp), bf_hi(zp) + bf_hi(tp));
        }
        o[j] = POST ? pack_bf2(bf_lo(zp) * bf_lo(a2[j]), bf_hi(zp) * bf_hi(a2[j])) : zp;
    }
    if (active) {
        u32x4 ov = {o[0], o[1], o[2], o[3]};
        if (NT) __builtin_nontemporal_store(ov, (u32x4*)(out + (int64_t)row * L + t0));
        else *(u32x4*)(out + (int64_t)row * L + t0) = ov;
    }
}

template <int K, bool PRE, bool POST, int BIAS, int FEAT = 0>
void launch_k(bool rowu, bool nt, dim3 grid, hipStream_t s, RowMap x1, RowMap x2, RowMap v, const float* taps,
              const float* bias, bf16_t* out, int64_t D, int64_t L, int dg, int64_t opr, int64_t tot,
              const float* ftaps = nullptr) {
    int dg_shift = -1;
    if ((dg & (dg - 1)) == 0) { dg_shift = 0; while ((1 << dg_shift) < dg) ++dg_shift; }
#define SE_GO(R, N) hipLaunchKernelGGL((se_fir_kernel<K, PRE, POST, BIAS, R, N, FEAT>), grid, dim3(256), 0, s, x1, x2, v, \
                                      taps, bias, out, D, L, dg, dg_shift, opr, tot, ftaps)
    if (rowu && nt) SE_GO(true, true);
    else if (rowu) SE_GO(true, false);
    else if (nt) SE_GO(false, true);
    else SE_GO(false, false);
#undef SE_GO
}

template <int K>
bool launch_gates(bool pre, bool post, int bias_mode, bool rowu, bool nt, dim3 grid, hipStream_t s, RowMap x1, RowMap x2,
                  RowMap v, const float* taps, const float* bias, bf16_t* out, int64_t D, int64_t L, int dg,
                  int64_t opr, int64_t tot) {
#define SE_CASE(P, Q, M)                                                                                    \
    if (pre == P && post == Q && bias_mode == M) {                                                          \
        launch_k<K, P, Q, M>(rowu, nt, grid, s, x1, x2, v, taps, bias, out, D, L, dg, opr, tot);                \
        return true;                                                                                        \
    }
    SE_CASE(true, true, HYENA_BIAS_NONE)
    SE_CASE(false, false, HYENA_BIAS_NONE)
    SE_CASE(false, false, HYENA_BIAS_ADD)
    SE_CASE(true, true, HYENA_BIAS_ADD)
    SE_CASE(true, true, HYENA_BIAS_GATED_FP32)
    SE_CASE(true, false, HYENA_BIAS_NONE)
    SE_CASE(false, true, HYENA_BIAS_NONE)
    SE_CASE(false, false, HYENA_BIAS_GATED_FP32)
    SE_CASE(true, true, HYENA_BIAS_ADD_FP32)
    SE_CASE(false, false, HYENA_BIAS_ADD_FP32)
    SE_CASE(true, true, HYENA_BIAS_GATED_BF16)
    SE_CASE(false, false, HYENA_BIAS_GATED_BF16)
#undef SE_CASE
    return false;
}

}  // namespace

namespace {
int se_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* taps,
                const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K,
                void* stream, const float* ftaps);
}

extern "C" int hyena_se_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* taps,
                            const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L, int64_t G,
                            int K, void* stream) {
    return se_fwd_impl("hyena_se_fwd", x1, x2, v, taps, bias, bias_mode, out, B, D, L, G, K, stream, nullptr);
}

// The short-filter form of hyena_fir_layer_fwd_rows (2 <= K <= 8, no inner bias): arguments as there, taps in the
// short-filter orientation (taps[g][K-1] on the current sample), already validated for the featurizer part.
int hyena_se_layer_rows(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* feat_taps,
                        const float* taps, void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K, void* stream,
                        const char* who) {
    return se_fwd_impl(who, x1, x2, v, taps, nullptr, HYENA_BIAS_NONE, out, B, D, L, G, K, stream, feat_taps);
}

namespace {
int se_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* taps,
                const float* bias, int bias_mode, void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K,
                void* stream, const float* ftaps) {
    if (!x1 || !x1->ptr || !taps || !out) return hyena_fail(HYENA_EINVAL, "%s: x1, taps and out are required", who);
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld L=%lld G=%lld", who, (long long)B,
                          (long long)D, (long long)L, (long long)G);
    if (K < 2 || K > 8) return hyena_fail(HYENA_ENOSUP, "%s: K=%d outside 2..8 (use hyena_mr_fwd)", who, K);
    if (bias_mode < 0 || bias_mode > 4 || (bias_mode != HYENA_BIAS_NONE && !bias))
        return hyena_fail(HYENA_EINVAL, "%s: bias_mode %d needs a bias pointer", who, bias_mode);
    if (L % 8 != 0 || !rows_aligned8(x1) || !rows_aligned8(x2) || !rows_aligned8(v) || (((uintptr_t)out) & 15))
        return hyena_fail(HYENA_EALIGN, "%s: L and strides must be multiples of 8, pointers 16-byte aligned", who);
    const bool pre = v && v->ptr, post = x2 && x2->ptr;
    if (!rows_valid(x1) || !rows_valid(x2) || !rows_valid(v) || B * D >= (1LL << 31) || L / 8 >= (1LL << 31))
        return hyena_fail(HYENA_EINVAL, "%s: B*D, L/8 and the channel map must fit 31 bits", who);
    if (B == 0 || L == 0) return 0;
    const int64_t opr = L / 8, tot = B * D * opr;
    const bool rowu = (opr % 256 == 0) && D <= 65535 && B <= 65535;
    // activations larger than the last-level cache stream through it: non-temporal accesses then
    bool nt = 8.0 * (double)B * (double)D * (double)L > 384e6;
    { const int64_t x = hyena_override(HYENA_OV_SE_NT); if (x >= 0) nt = x != 0; }
    const int64_t nblk = (tot + 255) / 256;
    if (nblk > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);
    dim3 grid((unsigned)nblk);
    if (rowu) grid = dim3((unsigned)(opr / 256), (unsigned)D, (unsigned)B);
    hipStream_t s = (hipStream_t)stream;
    RowMap m1 = make_rowmap(x1), m2 = make_rowmap(post ? x2 : nullptr), mv = make_rowmap(pre ? v : nullptr);
    const int dg = (int)(D / G);
    bf16_t* o = (bf16_t*)out;
    bool ok = false;
    if (ftaps) {
        switch (K) {
#define SE_F(KK) case KK: launch_k<KK, true, true, HYENA_BIAS_NONE, 3>(rowu, nt, grid, s, m1, m2, mv, taps, bias, o, D, L, dg, opr, tot, ftaps); ok = true; break;
            SE_F(2) SE_F(3) SE_F(4) SE_F(5) SE_F(6) SE_F(7) SE_F(8)
#undef SE_F
        }
        if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: no short-filter featurizer kernel for K=%d", who, K);
        return hyena_check_launch(who);
    }
    switch (K) {
#define SE_K(KK) case KK: ok = launch_gates<KK>(pre, post, bias_mode, rowu, nt, grid, s, m1, m2, mv, taps, bias, o, D, L, dg, opr, tot); break;
        SE_K(2) SE_K(3) SE_K(4) SE_K(5) SE_K(6) SE_K(7) SE_K(8)
#undef SE_K
    }
    if (!ok) return hyena_fail(HYENA_ENOSUP, "%s: this gate/bias combination has no kernel", who);
    return hyena_check_launch(who);
}
}  // namespace
