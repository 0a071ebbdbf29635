// Hyena-LI prefill: long gated convolution with an implicit modal filter
// h[t] = Re sum_s r_s p_s^t, computed in one pass over L as a chunked modal scan:
//
//   chunk c (128 samples):  y_c = T * u_c  +  Pout * X_c ,   X_{c+1} = p^128 (.) X_c + Pin * u_c
//
//   T    [128 x 128]  lower-triangular Toeplitz of the filter head h[0..127]
//   Pin  [2S  x 128]  (Re, Im) of p_s^(127-j): the chunk's contribution to the state
//   Pout [128 x 2S ]  (Re, -Im) of r_s p_s^(i+1): what the incoming state adds to sample i
//   X_c  [2S]         complex modal state after the samples before chunk c
//
// All three contractions run on v_mfma_f32_16x16x32_bf16 with fp32 accumulation.  To keep the
// fp32 long-convolution output within 1e-4 of an fp32 evaluation, every fp32 coefficient is
// split into two bf16 terms (hi + lo) and the state, which is not bf16-exact, is split as well
// (hi*hi + hi*lo + lo*hi); the inputs u = bf16(x1*v) are exact.  The recurrence itself is carried
// in fp32 registers.  The final X is the decode state of vortex/model/engine.py:525-559 for free.
//
// Work decomposition: a WAVEFRONT owns CPW channels of one filter group and walks the whole
// sequence alone.  With CPW = 4 a step is 512 samples (4 chunks) and the 16 MFMA columns are
// 4 channels x 4 chunks; the 64 lanes hold the 4 x 16 complex states of the scan, one each.
// With CPW = 1 (filter groups narrower than 4 channels, e.g. one filter per channel) a step is
// 2048 samples of one channel and the 16 columns are its 16 chunks; each of the four lane rows
// scans one 512-sample piece from a zero state and the pieces are joined with two lane-row swaps
// (v_permlane16_swap, v_permlane32_swap).  Either way one B fragment
// serves every column of the step.  Nothing is shared between wavefronts: there is no
// block barrier anywhere, only the in-order LDS pipe of the wavefront itself, and the four
// wavefronts of a CU drift apart and cover each other's memory latency.  Global traffic is
// coalesced 16 B per lane (1 KiB per row and instruction), prefetched PF steps ahead in registers,
// and goes through buffer descriptors whose range check stands in for every bounds test.
#include <mutex>
#include <type_traits>

#include "common.h"

namespace {

constexpr int TL = 512;        // samples per step
constexpr int C = 128;         // chunk
constexpr int S = 16;          // modal state size (poles per group)
constexpr int R2 = 2 * S;      // real rows of the state, row 2*pole + (0: Re, 1: Im)

// per-wavefront LDS slices (elements)
constexpr int CHS = 160;                 // chunk stride inside a row: 128 samples + 64 B pad
constexpr int URS = 4 * CHS + 8;         // row stride 648 elements = 1296 B (odd multiple of 16 B)
constexpr int LRS = R2 + 4;              // row of chunk contributions: 32 floats + 16 B pad
constexpr int XRS = R2 + 8;              // row of split states: 32 bf16 + 16 B pad
constexpr int WAVE_LDS_BYTES = 2 * 4 * URS * 2 + 16 * LRS * 4 + 2 * 16 * XRS * 2;   // u, z, l, xh, xl

// The 48 MFMA A-operand fragments a wavefront keeps in registers (bf16 hi / lo terms, 16 B per lane each):
//   [ 0.. 7] Toeplitz hi, index 2*delta + ib    [ 8..15] Toeplitz lo      (delta = 0..3 superblocks back)
//   [16..23] Pout hi, index 2*Sigma + ib        [24..31] Pout lo
//   [32..39] Pin  hi, index 4*mu + kappa        [40..47] Pin  lo
constexpr int FR_T = 0, FR_PO = 16, FR_PI = 32, N_FRAG = 48;
// Workspace per group (floats), evaluated in double by the plan kernel.  Every power of a pole the fragments
// need is one fp32 complex product of a coarse and a fine table entry, p^(16a+b) = P16[a] * P1[b]:
constexpr int WS_ZPAD = 32;                        // zeros ahead of the head: lags -31..-1 read as 0 without a test
constexpr int WS_HEAD = WS_ZPAD;                   // [128]        filter head h[0..127]
constexpr int WS_P16 = WS_HEAD + C;                // [16][9][2]   p^(16a), a = 0..8  (a = 8: the chunk factor p^128)
constexpr int WS_P1 = WS_P16 + S * 9 * 2;          // [16][16][2]  p^b
constexpr int WS_R1 = WS_P1 + S * 16 * 2;          // [16][16][2]  r * p^b
constexpr int WS_END = WS_R1 + S * 16 * 2;
constexpr int WS_GROUP = 1536;                     // 1472 used; 6 KB, a whole number of 16-byte lane loads
static_assert(WS_END <= WS_GROUP, "workspace layout");

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) {
    union { u32x4 u; bf16x8 b; } c;
    c.u = x;
    return c.b;
}

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

// LDS traffic of one wavefront is in order in hardware; this only stops the compiler from moving
// LDS accesses of different lanes across the hand-off points.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sample (inside a 32-sample superblock) that MFMA row m of half-block ib stands for.  Feeding the
// A rows in this order makes lane quad q of the 16x16 accumulators own samples 8q..8q+7.
__device__ __forceinline__ int li_sample(int ib, int m) { return 8 * (m >> 2) + 4 * ib + (m & 3); }

// ------------------------------------------------------------------ plan kernel
// One block per group; coefficients evaluated in double from the fp32 parameters.
__global__ __launch_bounds__(256) void li_plan_kernel(const float* __restrict__ log_poles,   // [G][S][2]
                                                      const float* __restrict__ residues,    // [G][S][2]
                                                      float* __restrict__ ws,
                                                      int sr) {                              // modes given, <= S
    const int g = blockIdx.x, tid = threadIdx.x;
    float* w = ws + (size_t)g * WS_GROUP;
    const float* lp = log_poles + (size_t)g * sr * 2;
    const float* rs = residues + (size_t)g * sr * 2;
    // p^k = exp(k*lr) * (cos(k*th), sin(k*th)); the modes past sr are p = 1 with residue 0, which add nothing
    auto ppow = [&](int s, int k, double& re, double& im) {
        if (s >= sr) { re = 1.0; im = 0.0; return; }
        const double m = exp((double)k * (double)lp[2 * s]);
        const double a = (double)k * (double)lp[2 * s + 1];
        re = m * cos(a);
        im = m * sin(a);
    };
    if (tid < WS_ZPAD) w[tid] = 0.f;
    if (tid < C) {                                  // filter head h[0..127]
        double acc = 0.0;
        for (int s = 0; s < sr; ++s) {
            double re, im;
            ppow(s, tid, re, im);
            acc += (double)rs[2 * s] * re - (double)rs[2 * s + 1] * im;
        }
        w[WS_HEAD + tid] = (float)acc;
    }
    for (int e = tid; e < S * 9; e += 256) {        // coarse powers
        const int s = e / 9, a = e - 9 * s;
        double re, im;
        ppow(s, 16 * a, re, im);
        w[WS_P16 + 2 * e] = (float)re;
        w[WS_P16 + 2 * e + 1] = (float)im;
    }
    {                                               // fine powers, plain and times the residue: 256 threads = 16 x 16
        const int s = tid >> 4, b = tid & 15;
        double re, im;
        ppow(s, b, re, im);
        w[WS_P1 + 2 * tid] = (float)re;
        w[WS_P1 + 2 * tid + 1] = (float)im;
        const double rr = s < sr ? rs[2 * s] : 0.f, ri = s < sr ? rs[2 * s + 1] : 0.f;
        w[WS_R1 + 2 * tid] = (float)(rr * re - ri * im);
        w[WS_R1 + 2 * tid + 1] = (float)(rr * im + ri * re);
    }
    for (int e = WS_END + tid; e < WS_GROUP; e += 256) w[e] = 0.f;
}

// (hi, lo) bf16 split of eight fp32 coefficients into two A-operand fragments
__device__ __forceinline__ void li_split(const float* val, u32x4& ph, u32x4& pl) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = val[2 * j], b = val[2 * j + 1];
        const float ah = round_bf(a), bh = round_bf(b);
        ph[j] = (__float_as_uint(ah) >> 16) | (__float_as_uint(bh) & 0xffff0000u);
        pl[j] = pack_bf2(a - ah, b - bh);
    }
}

// ------------------------------------------------------------------ main kernel
struct LiArgs {
    RowMap x1, x2, v;
    const float* ws;          // plan workspace
    const float* Dcoef;       // [D] or null
    bf16_t* out;              // [B][D][L]
    float* y32;               // optional [B][D][L] fp32 convolution output (before any rounding)
    float* state_out;         // optional [B][D][sr][2]
    int sr;                   // modes the caller has (<= S)
    int64_t D, L;
    int dg;
    int d_is_bf16;
    int64_t nquads;           // B * D / 4 wavefront-sized work items
    uint32_t xchunk;          // blocks an XCD takes in one run (0: plain block order)
    const float* ftaps;       // FEAT: featurizer taps [3: x1, x2, v][D][FEAT], oldest sample first
};

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0)

// COOP: the four wavefronts of a block share one work item (CPW channels) and take consecutive pieces of a step
// four times as long, so that a block reads 4 KiB (CPW = 4) or 16 KiB (CPW = 1) of each row in one go and a quarter
// as many rows are in flight on the chip: long rows stream faster that way.  The modal state crosses the
// wavefronts through LDS once per step (one block barrier); everything else stays private to a wavefront.
//
// FEAT = 3: the rows are the raw projection of the layer, sequence-major, and the three-tap featurizer FIR of
// vortex/model/model.py:233-246 (engine.py:188-223 with gate = False) runs on every 16-byte piece at the moment the
// step consumes it: a lane needs the two samples ahead of its eight, which are the last dword of the lane to its
// left (a wavefront shift) or, for lane 0, of lane 63 of the piece before it in time, carried in a scalar register.
// The products and their order are those of the other featurizer kernels (fp32 FMAs, oldest sample first, one
// rounding to bf16), so the gates are bit-identical to theirs.  Lone wavefronts only: a cooperating wavefront's
// predecessor piece belongs to another wavefront.
template <bool PRE, bool POST, bool NT, int PF, int DMODE, bool Y32, int CPW, bool COOP, int FEAT = 0>
__global__ __launch_bounds__(256, 1) void li_kernel(LiArgs a) {
    static_assert(CPW == 4 || CPW == 1, "4 channels x 512 samples or 1 channel x 2048 samples per step");
    static_assert(!COOP || CPW == 4, "the cooperative form is built for four channels per work item");
    static_assert(FEAT == 0 || (FEAT == 3 && PRE && POST && !COOP && !Y32), "featurizer: three taps, all three gates, lone wavefronts");
    constexpr int TLW = TL * (4 / CPW);                        // samples of one channel per step and wavefront
    constexpr int STEP = COOP ? 4 * TLW : TLW;                 // distance between two steps of one wavefront
    constexpr int NROW = CPW == 4 ? 4 : 1;                     // distinct rows per stream
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[4 * WAVE_LDS_BYTES];
    __shared__ float2 e_sh[COOP ? 2 * 4 * 64 : 1];             // [step parity][wavefront][lane] piece end states
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups are dealt to the 8 XCDs in turn (id mod 8).  An XCD takes runs of xchunk consecutive blocks (by
    // default one run: the x-th eighth of the rows), so that it walks contiguous parts of the tensors instead of every
    // eighth row group of all of them: 1.64 -> 1.52-1.56 ms at B = 1, L = 262144, D = 4096 with 256 filter groups,
    // 1.62 -> 1.58 ms with one filter per channel.
    uint32_t xbid = blockIdx.x;
    if (a.xchunk) {
        const uint32_t r = xbid >> 3;
        xbid = (r / a.xchunk) * 8u * a.xchunk + (xbid & 7u) * a.xchunk + r % a.xchunk;
    }
    const int64_t quad = COOP ? (int64_t)xbid : (int64_t)xbid * 4 + w;   // CPW channels of one batch element
    if (quad >= a.nquads) return;                              // whole wavefront leaves (never with COOP: no barrier is skipped)
    const uint32_t qpb = (uint32_t)(a.D / CPW);
    const int64_t b = (uint32_t)quad / qpb;
    const int64_t d0 = (int64_t)((uint32_t)quad % qpb) * CPW;
    const int g = (int)((uint32_t)d0 / (uint32_t)a.dg);
    const float* ws = a.ws + (size_t)g * WS_GROUP;
    // The kernel walks a virtual row of Lv = L + pad samples, a whole number of chunks, whose first pad samples
    // are zeros ahead of the real row: zero history in front of a causal filter changes no output, and the last
    // chunk then ends exactly on sample L-1, so the scan's state after it is the decode state as it stands.
    const int64_t L = a.L;
    const int pad = (int)((C - L % C) % C);                    // multiple of 8 (L is), < 128
    const int64_t Lv = L + pad;
    const int64_t woff = COOP ? (int64_t)w * TLW : 0;          // this wavefront's piece inside a step
    const int64_t Lw = Lv - woff;                              // the virtual row as this wavefront sees it (may be <= 0)
    const int64_t lo = pad - woff;                             // positions below lo (first wavefront, first chunk) are padding

    unsigned char* lds = lds_all + w * WAVE_LDS_BYTES;
    bf16_t* u_w = (bf16_t*)lds;                                // [4][URS]
    bf16_t* z_w = u_w + 4 * URS;                               // [4][URS]
    float* l_w = (float*)(z_w + 4 * URS);                      // [4 chunks][4 ch][LRS]
    bf16_t* xh_w = (bf16_t*)(l_w + 16 * LRS);                  // [4][4][XRS]
    bf16_t* xl_w = xh_w + 16 * XRS;

    // ---- the group's coefficient table is requested first; rows requested behind it arrive after it (loads
    // return in order) and travel while the fragments are being built
    constexpr int TQ = COOP ? (WS_GROUP / 4 + 255) / 256 : WS_GROUP / 4 / 64;
    f32x4 tq[TQ];
#pragma unroll
    for (int i = 0; i < TQ; ++i) {
        const int e = COOP ? tid + 256 * i : i * 64 + lane;
        tq[i] = (!COOP || e < WS_GROUP / 4) ? ((const f32x4*)ws)[e] : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- coalesced layout: lane moves samples 8*lane..8*lane+7 of each of the 4 rows
    const int lofs = lane * 8 + 32 * (lane >> 4);              // position inside a padded LDS row
    // Rows are addressed through buffer descriptors (base = sample 0 of the row, range = its L samples): a request
    // outside the row reads zeros and a store outside it is dropped by the address unit, so no access of the main
    // loop sits under a branch or a predicate, neither the padding ahead of sample 0 nor the tail behind sample
    // L-1 nor the pieces of a step that do not exist, and the compiler can count exactly how many younger requests
    // may still be in flight when a register stage is consumed.  An access is out of range when its per-lane offset
    // is >= range - scalar offset (unsigned): the per-lane offset carries everything that can be negative (lane,
    // piece, padding), the scalar offset the time, which is kept >= 0 by moving one step into the lane offset.
    __amdgpu_buffer_rsrc_t r1[NROW], rv[PRE ? NROW : 1], r2[POST ? NROW : 1], ro[NROW];
    const int range = (int)(L * 2);                            // bytes (the launcher keeps rows below 2 GiB)
#pragma unroll
    for (int r = 0; r < NROW; ++r) {
        const int64_t d = d0 + r;
        r1[r] = __builtin_amdgcn_make_buffer_rsrc((void*)a.x1.row(b, d), 0, range, 0x00020000);
        if constexpr (PRE) rv[r] = __builtin_amdgcn_make_buffer_rsrc((void*)a.v.row(b, d), 0, range, 0x00020000);
        if constexpr (POST) r2[r] = __builtin_amdgcn_make_buffer_rsrc((void*)a.x2.row(b, d), 0, range, 0x00020000);
        ro[r] = __builtin_amdgcn_make_buffer_rsrc((void*)(a.out + (b * a.D + d) * L), 0, range, 0x00020000);
    }
    // LDS row r is channel d0 + r (CPW = 4) or the r-th 512-sample piece of channel d0 (CPW = 1)
    auto roff = [](int r) -> int64_t { return CPW == 4 ? 0 : (int64_t)TL * r; };
    auto rrow = [](int r) { return CPW == 4 ? r : 0; };
    constexpr uint32_t STEP2 = (uint32_t)STEP * 2u;
    // byte offset of this lane's piece of row r at row time t = STEP (virtual position -> real sample: minus lo)
    const uint32_t vo0 = (uint32_t)(((int)lane * 8 - (int)lo + STEP) * 2);
    auto vo = [&](int r) -> uint32_t { return vo0 + (uint32_t)(roff(r) * 2); };
    // row time t -> (what to take off the lane offset, scalar offset): t >= STEP in the main loop
    auto ld_at = [&](const __amdgpu_buffer_rsrc_t& rs, int r, int64_t t) -> u32x4 {     // t >= STEP
        return __builtin_amdgcn_raw_buffer_load_b128(rs, vo(r), (uint32_t)(t - STEP) * 2u, NT ? 2 : 0);
    };
    auto ld_any = [&](const __amdgpu_buffer_rsrc_t& rs, int r, int64_t t) -> u32x4 {    // t >= 0
        const uint32_t back = t >= STEP ? 0u : STEP2, so = t >= STEP ? (uint32_t)(t - STEP) * 2u : 0u;
        return __builtin_amdgcn_raw_buffer_load_b128(rs, vo(r) - back, so, NT ? 2 : 0);
    };
    auto st_any = [&](const __amdgpu_buffer_rsrc_t& rs, int r, int64_t t, u32x4 val) {  // any t; t < 0: dropped
        const uint32_t back = t >= STEP ? 0u : STEP2;
        const uint32_t so = t >= STEP ? (uint32_t)(t - STEP) * 2u : (t >= 0 ? 0u : 0xFFFFFFFFu);
        __builtin_amdgcn_raw_buffer_store_b128(val, rs, vo(r) - back, so, NT ? 2 : 0);
    };
    u32x4 c1[PF][4], cv[PRE ? PF : 1][4], c2[POST ? PF : 1][4];      // register stages (absent gates take none)
    auto request_rows = [&]() {
#pragma unroll
        for (int p = 0; p < PF; ++p)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t t = (int64_t)p * STEP;
                c1[p][r] = ld_any(r1[rrow(r)], r, t);
                if constexpr (PRE) cv[p][r] = ld_any(rv[rrow(r)], r, t);
                if constexpr (POST) c2[p][r] = ld_any(r2[rrow(r)], r, t);
            }
    };
    // With four channels per wavefront the rows are requested before the fragment build and travel during it
    // (measured 5 % faster at L = 8192..32768).  With one channel per wavefront the same order measured 1-3 %
    // slower on rows up to 8192 samples and 1-2 % faster from 131072 on; there the rows are requested after the build.
    constexpr bool ROWS_FIRST = CPW == 4;
    if (ROWS_FIRST) request_rows();

    // ---- A fragments, built from the group's 6 KB coefficient table and pinned in registers.  The table and,
    // with COOP, the finished fragments pass through LDS rows that the main loop only uses afterwards: a lone
    // wavefront stages the table in its own slice and builds all 48 fragments; cooperating wavefronts stage one
    // table for the block, build a quarter of the fragments each and read the rest from LDS.
    // 16x16x32 A operand: lane holds row m = lane & 15, k = 8*(lane >> 4) + e, e = 0..7.
    bf16x8 Th[8], Tl[8], Poh[8], Pol[8], Pih[8], Pil[8];
    float pcr, pci;                                            // p^128 of this lane's pole (lane & 15)
    {
        float* tb = COOP ? (float*)lds_all : (float*)lds;
        u32x4* fb = (u32x4*)(lds_all + WS_GROUP * 4);           // COOP: [48 fragments][64 lanes]
        static_assert(WS_GROUP * 4 <= 2 * 4 * URS * 2, "coefficient table must fit the u / z rows");
        static_assert(WS_GROUP * 4 + N_FRAG * 64 * 16 <= 4 * WAVE_LDS_BYTES, "table and fragments must fit the block's LDS");
#pragma unroll
        for (int i = 0; i < TQ; ++i) {
            const int e = COOP ? tid + 256 * i : i * 64 + lane;
            if (!COOP || e < WS_GROUP / 4) ((f32x4*)tb)[e] = tq[i];
        }
        if (COOP) __syncthreads(); else wave_sync();
        const int m = lane & 15, qa = lane >> 4;
        pcr = tb[WS_P16 + 2 * (9 * m + 8)];
        pci = tb[WS_P16 + 2 * (9 * m + 8) + 1];
        const float2* t16 = (const float2*)(tb + WS_P16);
        const float2* t1 = (const float2*)(tb + WS_P1);
        const float2* tr = (const float2*)(tb + WS_R1);
        u32x4 th[N_FRAG];
        float val[8];
        auto mine = [&](int f) { return !COOP || (f & 3) == w; };      // which fragment pairs this wavefront builds
#pragma unroll
        for (int f = 0; f < 8; ++f) {               // Toeplitz: rows of (superblock Sigma, half ib) x inputs of block J
            if (!mine(f)) continue;
            const int delta = f >> 1, ib = f & 1;   // delta = Sigma - J
            // lag = 32*delta + sample - (8*qa + k) lies in -31..127; the zeros ahead of the head stand for lag < 0
            const float* hp = tb + WS_HEAD + 32 * delta + li_sample(ib, m) - 8 * qa;
#pragma unroll
            for (int k = 0; k < 8; ++k) val[k] = hp[-k];
            li_split(val, th[FR_T + f], th[FR_T + 8 + f]);
        }
        // Pout: output sample i of (Sigma, ib) x state rows 8*qa + k hold Re / -Im of r * p^(i+1).  The exponent is
        // e = 32*Sigma + 4*ib + eb with eb = 1..28 per lane, so its table indices are (e >> 4) = 2*Sigma + hi and
        // (e & 15) = lo with hi, lo fixed per (lane, ib): one address per lane, the rest are immediate offsets.
        {
            const int eb = li_sample(0, m) + 1;
#pragma unroll
            for (int ib = 0; ib < 2; ++ib) {
                const int hi = (eb + 4 * ib) >> 4, lo = (eb + 4 * ib) & 15;
                const float2* pa0 = t16 + (4 * qa) * 9 + hi;
                float2 rb[4];
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) rb[kk] = tr[(4 * qa + kk) * 16 + lo];
#pragma unroll
                for (int Sg = 0; Sg < 4; ++Sg) {
                    const int f = 2 * Sg + ib;
                    if (!mine(f)) continue;
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        const float2 pa = pa0[kk * 9 + 2 * Sg];
                        val[2 * kk] = pa.x * rb[kk].x - pa.y * rb[kk].y;
                        val[2 * kk + 1] = -(pa.x * rb[kk].y + pa.y * rb[kk].x);
                    }
                    li_split(val, th[FR_PO + f], th[FR_PO + 8 + f]);
                }
            }
        }
        // Pin: state row 16*mu + m x inputs 32*kappa + 8*qa + k hold Re or Im (row parity) of p^(127 - j).  With
        // e = 127 - 32*kappa - 8*qa - k the coarse index (e >> 4) = 7 - (qa >> 1) - 2*kappa does not depend on k and the
        // fine one (e & 15) = 15 - 8*(qa & 1) - k not on kappa (no borrow for k = 0..7).
        {
            const bool im_row = m & 1;
#pragma unroll
            for (int mu = 0; mu < 2; ++mu) {
                const int s = 8 * mu + (m >> 1);
                const float2* pb0 = t1 + s * 16 + 15 - 8 * (qa & 1);
                const float2* pa0 = t16 + s * 9 + 7 - (qa >> 1);
                float2 pb[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) pb[k] = pb0[-k];
#pragma unroll
                for (int kp = 0; kp < 4; ++kp) {
                    const int f = 4 * mu + kp;
                    if (!mine(f)) continue;
                    const float2 pa = pa0[-2 * kp];
                    // Re = pa.x*pb.x - pa.y*pb.y, Im = pa.y*pb.x + pa.x*pb.y
                    const float ca = im_row ? pa.y : pa.x, cb = im_row ? pa.x : -pa.y;
#pragma unroll
                    for (int k = 0; k < 8; ++k) val[k] = ca * pb[k].x + cb * pb[k].y;
                    li_split(val, th[FR_PI + f], th[FR_PI + 8 + f]);
                }
            }
        }
        if (COOP) {
#pragma unroll
            for (int g3 = 0; g3 < 3; ++g3)
#pragma unroll
                for (int f = 0; f < 8; ++f)
                    if (mine(f)) {
                        fb[(16 * g3 + f) * 64 + lane] = th[16 * g3 + f];
                        fb[(16 * g3 + 8 + f) * 64 + lane] = th[16 * g3 + 8 + f];
                    }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < N_FRAG; ++i) th[i] = fb[i * 64 + lane];
        }
#pragma unroll
        for (int i = 0; i < N_FRAG; ++i) asm volatile("" : "+a"(th[i]));     // fragments live in accumulation registers: only the MFMAs read them
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            Th[q] = as_bf16x8(th[FR_T + q]);   Tl[q] = as_bf16x8(th[FR_T + 8 + q]);
            Poh[q] = as_bf16x8(th[FR_PO + q]); Pol[q] = as_bf16x8(th[FR_PO + 8 + q]);
            Pih[q] = as_bf16x8(th[FR_PI + q]); Pil[q] = as_bf16x8(th[FR_PI + 8 + q]);
        }
        // the LDS rows used here are free for the main loop from here on
        if (COOP) __syncthreads(); else wave_sync();
    }
    if (!ROWS_FIRST) request_rows();

    // MFMA-side lane geometry: column n = channel c + 4 * chunk s, k / row quad q
    const int n = lane & 15, q = lane >> 4;
    const int c = n & 3, s = n >> 2;
    // scan-side lane geometry: one complex state per lane
    // (sq: the lane row, which is the channel with CPW = 4 and the 512-sample piece of the step with CPW = 1)
    const int sq = lane >> 4, sc = CPW == 4 ? sq : 0, sp = lane & 15;
    float Xr = 0.f, Xi = 0.f;
    float Xfr = 0.f, Xfi = 0.f;                                // state after the chunk that holds sample L-1
    bool have_final = !COOP && CPW == 4;                       // otherwise only the wavefront / lane row whose piece holds sample L-1
    float dco = 0.f;
    if (a.Dcoef) dco = a.Dcoef[d0 + (CPW == 4 ? c : 0)];
    float X0r = 0.f, X0i = 0.f;                                // COOP, CPW = 1: state at the start of the step
    float ppr = pcr, ppi = pci;                                // COOP: p^TLW, one wavefront's piece
    if (COOP) {
#pragma unroll
        for (int k = 1; k < 16 / CPW; ++k) { const float t = ppr * pcr - ppi * pci; ppi = ppr * pci + ppi * pcr; ppr = t; }
    }
    // CPW = 1: powers of the pole that carry a state over one, two and four 512-sample pieces, and over the pieces
    // ahead of this lane row's own (p^0, p^512, p^1024, p^1536)
    float p4r = 1.f, p4i = 0.f, p8r = 1.f, p8i = 0.f, p16r = 1.f, p16i = 0.f, mqr = 1.f, mqi = 0.f;
    if constexpr (CPW == 1) {
        auto sqr = [](float& r, float& i) { const float t = r * r - i * i; i = 2.f * r * i; r = t; };
        p4r = pcr; p4i = pci;
        sqr(p4r, p4i); sqr(p4r, p4i);                          // p^512
        p8r = p4r; p8i = p4i; sqr(p8r, p8i);                   // p^1024
        p16r = p8r; p16i = p8i; sqr(p16r, p16i);               // p^2048
        const float p12r = p8r * p4r - p8i * p4i, p12i = p8r * p4i + p8i * p4r;
        mqr = sq == 0 ? 1.f : sq == 1 ? p4r : sq == 2 ? p8r : p12r;
        mqi = sq == 0 ? 0.f : sq == 1 ? p4i : sq == 2 ? p8i : p12i;
    }

    // ---- FEAT: taps of this wavefront's channels (wave-uniform, kept in scalar registers) and the carried dwords
    constexpr int NCH = CPW == 4 ? 4 : 1;                      // distinct channels, and carry chains, per stream
    float fw[FEAT ? 3 : 1][NCH][3];
    uint32_t car1[NCH], carv[NCH], car2[NCH];                  // last two raw samples of the piece consumed before
#pragma unroll
    for (int r = 0; r < NCH; ++r) {
        car1[r] = carv[r] = car2[r] = 0u;                      // the row starts behind zeros
        if constexpr (FEAT != 0) {
#pragma unroll
            for (int i = 0; i < 3; ++i)
#pragma unroll
                for (int k = 0; k < 3; ++k)
                    fw[i][r][k] = __uint_as_float((uint32_t)__builtin_amdgcn_readfirstlane(
                        (int)__float_as_uint(a.ftaps[((int64_t)i * a.D + d0 + r) * 3 + k])));
        }
    }
    auto feat = [&](const u32x4 cc, uint32_t& carry, const float (&wt)[3]) __attribute__((always_inline)) -> u32x4 {
        // samples -2, -1: lane l takes the last dword of lane l-1, lane 0 keeps `carry`
        const uint32_t hw = (uint32_t)__builtin_amdgcn_update_dpp((int)carry, (int)cc[3], 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
        carry = (uint32_t)__builtin_amdgcn_readlane((int)cc[3], 63);
        float rr[10];
        rr[0] = bf_lo(hw);
        rr[1] = bf_hi(hw);
#pragma unroll
        for (int j = 0; j < 4; ++j) { rr[2 + 2 * j] = bf_lo(cc[j]); rr[3 + 2 * j] = bf_hi(cc[j]); }
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float f0 = fmaf(wt[2], rr[2 * j + 2], fmaf(wt[1], rr[2 * j + 1], fmaf(wt[0], rr[2 * j], 0.f)));
            const float f1 = fmaf(wt[2], rr[2 * j + 3], fmaf(wt[1], rr[2 * j + 2], fmaf(wt[0], rr[2 * j + 1], 0.f)));
            o[j] = pack_bf2(f0, f1);
        }
        return o;
    };
    auto chain = [](int r) { return CPW == 4 ? r : 0; };       // CPW = 1: the four pieces of a step follow each other in time

    // FEAT with four channels per wavefront: u = bf16(f(x1) * f(v)) of the step held by register stage p (row time
    // ts) is formed one step ahead, behind the Toeplitz MFMAs of the step before, so that the featurizer's vector
    // instructions run in their shadow; it waits in registers until its step writes it to LDS, and the stage is
    // refilled with step ts + PF*STEP at once (1.87 -> 1.80 ms at B = 1, L = 262144, D = 4096 with 256 filters).  With
    // one channel per wavefront the same order needs a register stage less and measured 11 % slower (2.04 against
    // 1.83 ms): that form runs its featurizer at the top of the step.
    constexpr bool EARLY = FEAT != 0 && CPW == 4;
    u32x4 un[EARLY ? 4 : 1];
    auto prepare_u = [&](const int p, const int64_t ts) __attribute__((always_inline)) {
        if constexpr (EARLY) {
            const int64_t tn = ts + (int64_t)PF * STEP;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const u32x4 f1 = feat(c1[p][r], car1[chain(r)], fw[0][chain(r)]);
                const u32x4 fv = feat(cv[p][r], carv[chain(r)], fw[2][chain(r)]);
                un[r] = gate_mul<true>(f1, fv);
                c1[p][r] = ld_at(r1[rrow(r)], r, tn);
                cv[p][r] = ld_at(rv[rrow(r)], r, tn);
            }
        }
    };

    // One step.  No memory access is conditional: what lies outside the row is handled by the buffer descriptors.
    auto step = [&](const int p, const int64_t ts) __attribute__((always_inline)) {
        const int pp = (p + PF - 1) % PF;                      // register stage of the previous step
        const int64_t tn = ts + (int64_t)PF * STEP;            // step that reuses this register stage

        // u = bf16(x1*v) of this step -> LDS; refill the stage with step ts + PF*STEP
        if constexpr (EARLY) {
            // formed one step ahead (prepare_u, in the shadow of the step before): only the LDS write is left here
#pragma unroll
            for (int r = 0; r < 4; ++r) *(u32x4*)(u_w + r * URS + lofs) = un[r];
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if constexpr (FEAT != 0) {
                    const u32x4 f1 = feat(c1[p][r], car1[chain(r)], fw[0][chain(r)]);
                    const u32x4 fv = feat(cv[p][r], carv[chain(r)], fw[2][chain(r)]);
                    *(u32x4*)(u_w + r * URS + lofs) = gate_mul<true>(f1, fv);
                    __builtin_amdgcn_sched_barrier(0);         // one row at a time: its temporaries are dead before the next starts
                } else if constexpr (PRE) *(u32x4*)(u_w + r * URS + lofs) = gate_mul<true>(c1[p][r], cv[p][r]);
                else *(u32x4*)(u_w + r * URS + lofs) = c1[p][r];
            }
            // (the scheduler would move these requests, and what waits on the registers they overwrite, far from
            // here and run out of registers: pin the group)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                c1[p][r] = ld_at(r1[rrow(r)], r, tn);
                if constexpr (PRE) cv[p][r] = ld_at(rv[rrow(r)], r, tn);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        wave_sync();

        // B fragments: column (c, s) x inputs 32*J + 8*q.. of its chunk; shared by every MFMA below
        bf16x8 bu[4];
#pragma unroll
        for (int J = 0; J < 4; ++J) bu[J] = *(const bf16x8*)(u_w + c * URS + s * CHS + 32 * J + 8 * q);
        // z of the previous step, coalesced layout
        u32x4 zz[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) zz[r] = *(const u32x4*)(z_w + r * URS + lofs);

        // ---- state-in: L[32 x 16 cols] = Pin[32 x 128] * u
        f32x4 l0 = {0, 0, 0, 0}, l1 = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            l0 = MFMA16(Pih[k], bu[k], l0);
            l1 = MFMA16(Pih[4 + k], bu[k], l1);
            l0 = MFMA16(Pil[k], bu[k], l0);
            l1 = MFMA16(Pil[4 + k], bu[k], l1);
        }
        {   // lane (column n, quad q) holds state rows 4q..4q+3 of each half
            float* lp = l_w + n * LRS + 4 * q;                 // row index s*4 + c == n  (n = c + 4s)
            *(f32x4*)lp = l0;
            *(f32x4*)(lp + 16) = l1;
        }

        // ---- Toeplitz: superblock Sigma (32 samples) x half ib, inputs J <= Sigma
        f32x4 acc[4][2];
#pragma unroll
        for (int Sg = 0; Sg < 4; ++Sg)
#pragma unroll
            for (int ib = 0; ib < 2; ++ib) {
                f32x4 t = {0, 0, 0, 0};
#pragma unroll
                for (int J = 0; J <= Sg; ++J) {
                    t = MFMA16(Th[2 * (Sg - J) + ib], bu[J], t);
                    t = MFMA16(Tl[2 * (Sg - J) + ib], bu[J], t);
                }
                acc[Sg][ib] = t;
            }

        if constexpr (EARLY) prepare_u((p + 1) % PF, ts + STEP);

        // ---- deferred output of the previous step: gate with x2, store, refill its x2 stage
        {
            const int64_t ts_out = ts - STEP, t_refill = ts - STEP + (int64_t)PF * STEP;
            u32x4 o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                o[r] = zz[r];
                if constexpr (POST) {
                    u32x4 g2 = c2[pp][r];
                    if constexpr (FEAT != 0) {
                        // the first step has no output behind it: its stage holds a later piece, which is consumed,
                        // and carried on, when its own turn comes
                        if (ts_out >= 0) g2 = feat(c2[pp][r], car2[chain(r)], fw[1][chain(r)]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[r][j] = pack_bf2(bf_lo(zz[r][j]) * bf_lo(g2[j]), bf_hi(zz[r][j]) * bf_hi(g2[j]));
                }
            }
            // (in the first step of a row ts_out < 0: the store is dropped, and with FEAT the refill asks again
            // for the piece the stage already holds)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                st_any(ro[rrow(r)], r, ts_out, o[r]);
                if constexpr (POST) c2[pp][r] = ld_at(r2[rrow(r)], r, t_refill);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        wave_sync();

        // ---- scan over the chunks of the step in time order: lane = (lane row sq, pole sp).
        // Column n = c + 4s sits in row n of l_w / x*_w, and a lane row walks the four chunks s = 0..3 of its c = sq:
        // the four chunks of the step of its channel (CPW = 4), or the sq-th 512-sample piece of the one channel's
        // step (CPW = 1), whose entering state comes from the lane rows before it.
        {
            constexpr int NK = 4;
            float lr[NK], li[NK];
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int row = k * 4 + sq;
                const float2 t = *(const float2*)(l_w + row * LRS + 2 * sp);
                lr[k] = t.x;
                li[k] = t.y;
            }
            float nX0r = 0.f, nX0i = 0.f;
            if constexpr (CPW == 1) {
                // What a piece adds to the state (its end state from a zero start), gathered over the four lane rows
                // with two lane-row swaps: a wavefront-wide exchange in the vector ALU, no trip through LDS.
                float er = 0.f, ei = 0.f;
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const float nr = fmaf(pcr, er, fmaf(-pci, ei, lr[k]));
                    ei = fmaf(pcr, ei, fmaf(pci, er, li[k]));
                    er = nr;
                }
                // v_permlane16_swap of a register with itself: [0] holds rows (0, 0, 2, 2), [1] rows (1, 1, 3, 3)
                const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(er), __float_as_uint(er), false, false);
                const auto i16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(ei), __float_as_uint(ei), false, false);
                const float ar = __uint_as_float(r16[0]), ai = __uint_as_float(i16[0]);
                const float br = __uint_as_float(r16[1]), bi = __uint_as_float(i16[1]);
                // pieces (0, 1) and (2, 3) joined: rows (c01, c01, c23, c23)
                const float cr = fmaf(p4r, ar, fmaf(-p4i, ai, br)), ci = fmaf(p4r, ai, fmaf(p4i, ar, bi));
                // v_permlane32_swap: [0] holds rows (0, 1, 0, 1), [1] rows (2, 3, 2, 3)
                const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(cr), __float_as_uint(cr), false, false);
                const auto i32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(ci), __float_as_uint(ci), false, false);
                const float c01r = __uint_as_float(r32[0]), c01i = __uint_as_float(i32[0]);
                const float c23r = __uint_as_float(r32[1]), c23i = __uint_as_float(i32[1]);
                // state entering piece sq: X0 pushed through the pieces before it plus what those pieces added
                //   sq 0: X0    1: p^512 X0 + e0    2: p^1024 X0 + c01    3: p^1536 X0 + p^512 c01 + e2
                // (selected, not multiplied by 0 / 1: what later pieces hold never reaches an earlier one)
                float xr = mqr * X0r - mqi * X0i, xi = mqr * X0i + mqi * X0r;
                const float tr = (sq & 1) ? p4r * c01r - p4i * c01i : c01r;
                const float ti = (sq & 1) ? p4r * c01i + p4i * c01r : c01i;
                xr += (sq & 2) ? tr : 0.f;
                xi += (sq & 2) ? ti : 0.f;
                xr += (sq & 1) ? ar : 0.f;
                xi += (sq & 1) ? ai : 0.f;
                Xr = xr;
                Xi = xi;
                // state after the step, the same in every lane row
                nX0r = fmaf(p16r, X0r, fmaf(-p16i, X0i, fmaf(p8r, c01r, fmaf(-p8i, c01i, c23r))));
                nX0i = fmaf(p16r, X0i, fmaf(p16i, X0r, fmaf(p8r, c01i, fmaf(p8i, c01r, c23i))));
            }
            if (COOP) {
                // what this piece adds to the state (its end state from a zero start) goes to the other wavefronts;
                // the state entering the piece is the block's state X0 pushed through the pieces before it
                float er = 0.f, ei = 0.f;
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const float nr = fmaf(pcr, er, fmaf(-pci, ei, lr[k]));
                    ei = fmaf(pcr, ei, fmaf(pci, er, li[k]));
                    er = nr;
                }
                const int par = (int)((ts / STEP) & 1);
                e_sh[(par * 4 + w) * 64 + lane] = make_float2(er, ei);
                __syncthreads();
                float xr = X0r, xi = X0i;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float2 e = e_sh[(par * 4 + j) * 64 + lane];
                    if (j == w) { Xr = xr; Xi = xi; }
                    const float nr = fmaf(ppr, xr, fmaf(-ppi, xi, e.x));
                    xi = fmaf(ppr, xi, fmaf(ppi, xr, e.y));
                    xr = nr;
                }
                X0r = xr;
                X0i = xi;
            }
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int row = k * 4 + sq;
                const uint32_t xh = pack_bf2(Xr, Xi);
                const int o = row * XRS + 2 * sp;
                *(uint32_t*)(xh_w + o) = xh;
                *(uint32_t*)(xl_w + o) = pack_bf2(Xr - bf_lo(xh), Xi - bf_hi(xh));
                const float nr = fmaf(pcr, Xr, fmaf(-pci, Xi, lr[k]));
                const float ni = fmaf(pcr, Xi, fmaf(pci, Xr, li[k]));
                Xr = nr;
                Xi = ni;
                {                                              // this chunk covers te - 128 .. te - 1
                    const int64_t te = ts + (int64_t)C * ((CPW == 4 ? k : 4 * sq + k) + 1);
                    if (te >= Lw && te - C < Lw) { Xfr = Xr; Xfi = Xi; have_final = true; }
                }
            }
            if constexpr (CPW == 1) { X0r = nX0r; X0i = nX0i; }
        }
        wave_sync();

        // ---- state-out: acc += Pout[rows x 32] * X[32 x cols], three bf16 products
        {
            const bf16x8 xh = *(const bf16x8*)(xh_w + n * XRS + 8 * q);     // row s*4 + c == n
            const bf16x8 xl = *(const bf16x8*)(xl_w + n * XRS + 8 * q);
#pragma unroll
            for (int Sg = 0; Sg < 4; ++Sg)
#pragma unroll
                for (int ib = 0; ib < 2; ++ib) {
                    f32x4 t = acc[Sg][ib];
                    t = MFMA16(Poh[2 * Sg + ib], xh, t);
                    t = MFMA16(Poh[2 * Sg + ib], xl, t);
                    t = MFMA16(Pol[2 * Sg + ib], xh, t);
                    acc[Sg][ib] = t;
                }
        }

        // ---- epilogue -> LDS.  lane (column (c, s), quad q) owns samples 32*Sigma + 8q .. +7 of chunk s
        //   DMODE 1: y = bf16(conv); z = bf16(y + bf16(D*u))   (bf16 tensors, vortex/model/engine.py:352-353)
        //   DMODE 0: y = bf16(conv); z = bf16(y + D*u)          (float32 D)
        //   DMODE 2: z = bf16(conv + D*u)                       (one rounding)
#pragma unroll
        for (int Sg = 0; Sg < 4; ++Sg) {
            const int tl = 32 * Sg + 8 * q;                     // inside the chunk
            if (Y32) {
                const int64_t t0 = ts + roff(c) + C * s + tl;
                if (t0 < Lw && t0 >= lo) {
                    float* yp = a.y32 + (b * a.D + d0 + (CPW == 4 ? c : 0)) * L + woff + t0 - pad;
                    *(f32x4*)yp = acc[Sg][0];
                    *(f32x4*)(yp + 4) = acc[Sg][1];
                }
            }
            const u32x4 uu = *(const u32x4*)(u_w + c * URS + s * CHS + tl);
            u32x4 z;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 av = acc[Sg][j >> 1];
                const float a0 = av[2 * (j & 1)], a1 = av[2 * (j & 1) + 1];
                const float u0 = bf_lo(uu[j]), u1 = bf_hi(uu[j]);
                if (DMODE == 2) {
                    z[j] = pack_bf2(fmaf(dco, u0, a0), fmaf(dco, u1, a1));
                } else {
                    const uint32_t yp = pack_bf2(a0, a1);
                    if (DMODE == 1) {
                        const uint32_t tp = pack_bf2(dco * u0, dco * u1);
                        z[j] = pack_bf2(bf_lo(yp) + bf_lo(tp), bf_hi(yp) + bf_hi(tp));
                    } else {
                        z[j] = pack_bf2(fmaf(dco, u0, bf_lo(yp)), fmaf(dco, u1, bf_hi(yp)));
                    }
                }
            }
            *(u32x4*)(z_w + c * URS + s * CHS + tl) = z;
        }
        // the wave_sync after the next step's u write orders these z writes before their coalesced reads
    };

    // Rotations of PF steps while a whole rotation lies inside the block's row (Lv, not Lw: with COOP every wavefront
    // runs every step and meets every barrier), then the steps that are left.  Steps may ask for pieces behind the
    // end of the row (they read zeros) and the first one stores nothing.
    if constexpr (EARLY) prepare_u(0, 0);
    int64_t ts = 0;
    for (; ts + (int64_t)(PF - 1) * STEP < Lv; ts += (int64_t)PF * STEP) {
#pragma unroll
        for (int p = 0; p < PF; ++p) step(p, ts + (int64_t)p * STEP);
    }
#pragma unroll
    for (int p = 0; p < PF - 1; ++p)
        if (ts + (int64_t)p * STEP < Lv) step(p, ts + (int64_t)p * STEP);
    {   // output of the last step
        const int64_t ts_last = ((Lv + STEP - 1) / STEP - 1) * STEP;
        wave_sync();
        const int pl = (int)((ts_last / STEP) % PF);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32x4 zz = *(const u32x4*)(z_w + r * URS + lofs);
            u32x4 o = zz;
            if constexpr (POST) {
                u32x4 x2v = c2[0][r];
#pragma unroll
                for (int p = 1; p < PF; ++p)
                    if (p == pl) x2v = c2[p][r];
                if constexpr (FEAT != 0) x2v = feat(x2v, car2[chain(r)], fw[1][chain(r)]);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    o[j] = pack_bf2(bf_lo(zz[j]) * bf_lo(x2v[j]), bf_hi(zz[j]) * bf_hi(x2v[j]));
            }
            st_any(ro[rrow(r)], r, ts_last, o);
        }
    }

    if (a.state_out && have_final) {
        // the last chunk of the virtual row ends on sample L-1: the scan's state after it is the decode state
        if (sp < a.sr) {                                       // CPW = 1: the lane row whose piece ended the row
            float* sp_ = a.state_out + ((b * a.D + d0 + sc) * a.sr + sp) * 2;
            sp_[0] = Xfr;
            sp_[1] = Xfi;
        }
    }
}

}  // namespace

extern "C" int64_t hyena_li_plan_bytes(int64_t G, int64_t S_) {
    if (G <= 0 || S_ < 1 || S_ > S) return 0;
    return (int64_t)G * WS_GROUP * (int64_t)sizeof(float);
}

extern "C" int hyena_li_plan(const float* log_poles, const float* residues, int64_t G, int64_t S_, void* workspace,
                             void* stream) {
    if (!log_poles || !residues || !workspace) return hyena_fail(HYENA_EINVAL, "hyena_li_plan: null pointer");
    if (G <= 0 || G > 0x7fffffff) return hyena_fail(HYENA_EINVAL, "hyena_li_plan: bad G=%lld", (long long)G);
    if (S_ < 1 || S_ > S) return hyena_fail(HYENA_ENOSUP, "hyena_li_plan: state size %lld (1..16)", (long long)S_);
    if (((uintptr_t)workspace) & 15) return hyena_fail(HYENA_EALIGN, "hyena_li_plan: workspace must be 16-byte aligned");
    hipLaunchKernelGGL(li_plan_kernel, dim3((unsigned)G), dim3(256), 0, (hipStream_t)stream, log_poles, residues,
                       (float*)workspace, (int)S_);
    return hyena_check_launch("hyena_li_plan");
}

namespace {
int li_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const void* workspace,
                const float* Dcoef, int d_is_bf16, void* out, float* y_conv_fp32, float* state_out,
                int64_t B, int64_t D, int64_t L, int64_t G, int64_t S_, void* stream, bool check_only,
                const float* ftaps = nullptr);
}

extern "C" int hyena_li_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const void* workspace,
                            const float* Dcoef, int d_is_bf16, void* out, float* y_conv_fp32, float* state_out,
                            int64_t B, int64_t D, int64_t L, int64_t G, int64_t S_, void* stream) {
    return li_fwd_impl("hyena_li_fwd", x1, x2, v, workspace, Dcoef, d_is_bf16, out, y_conv_fp32, state_out, B, D, L, G,
                       S_, stream, false);
}

extern "C" int hyena_li_layer_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const float* feat_taps,
                                  int feat_len, const void* workspace, const float* Dcoef, int d_is_bf16, void* out,
                                  float* state_out, int64_t B, int64_t D, int64_t L, int64_t G, int64_t S_, void* stream) {
    const char* who = "hyena_li_layer_fwd";
    if (!feat_taps) return hyena_fail(HYENA_EINVAL, "%s: feat_taps is required", who);
    if (feat_len != 3) return hyena_fail(HYENA_ENOSUP, "%s: featurizer of %d taps (3)", who, feat_len);
    if (!x1 || !x1->ptr || !x2 || !x2->ptr || !v || !v->ptr)
        return hyena_fail(HYENA_EINVAL, "%s: the three row sets of the projection are required", who);
    return li_fwd_impl(who, x1, x2, v, workspace, Dcoef, d_is_bf16, out, nullptr, state_out, B, D, L, G, S_, stream,
                       false, feat_taps);
}

// ------------------------------------------------------------------ the form that allocates nothing
// The coefficient tables live in a file-scope device array instead of a caller-owned workspace.  Host code
// must not use the array's name as an address: each device holds its own copy, whose address is looked up
// once per device (hipGetSymbolAddress with that device current) and kept.
namespace {
constexpr int64_t LI_STATIC_MAX_GROUPS = 8192;                 // 48 MiB per device, held until the process ends: the
                                                               // largest filter bank of the reference's configurations
                                                               // (hcl_filter_groups: 8192, configs/evo2-40b-8k.yml)
constexpr int LI_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[LI_STATIC_MAX_GROUPS * WS_GROUP];
std::mutex g_scratch_mu;
float* g_scratch_ptr[LI_STATIC_MAX_DEVICES] = {};

int li_scratch_for_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hyena_fail((int)e, "hyena_li_fwd_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= LI_STATIC_MAX_DEVICES)
        return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd_static: device index %d (0..%d)", dev, LI_STATIC_MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return hyena_fail(e != hipSuccess ? (int)e : HYENA_EINVAL, "hyena_li_fwd_static: hipGetSymbolAddress: %s",
                              hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" int hyena_li_fwd_static(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                                   const float* log_poles, const float* residues, const float* Dcoef, int d_is_bf16,
                                   void* out, float* y_conv_fp32, float* state_out, int64_t B, int64_t D, int64_t L,
                                   int64_t G, int64_t S_, void* stream) {
    if (!log_poles || !residues) return hyena_fail(HYENA_EINVAL, "hyena_li_fwd_static: log_poles and residues are required");
    if (G <= 0) return hyena_fail(HYENA_EINVAL, "hyena_li_fwd_static: bad G=%lld", (long long)G);
    if (G > LI_STATIC_MAX_GROUPS)
        return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd_static: %lld filter groups exceed the static table of %lld; use "
                          "hyena_li_plan + hyena_li_fwd with a caller-owned workspace", (long long)G,
                          (long long)LI_STATIC_MAX_GROUPS);
    if (S_ < 1 || S_ > S) return hyena_fail(HYENA_ENOSUP, "hyena_li_fwd_static: state size %lld (1..16)", (long long)S_);
    float* ws = nullptr;
    if (int rc = li_scratch_for_current_device(&ws)) return rc;
    // every argument check of the main launch runs before anything is enqueued
    if (int rc = li_fwd_impl("hyena_li_fwd_static", x1, x2, v, ws, Dcoef, d_is_bf16, out, y_conv_fp32, state_out, B, D,
                             L, G, S_, stream, true))
        return rc;
    if (B == 0 || L == 0) return 0;
    // the plan kernel rewrites the whole table of each of the G groups, so nothing of an earlier call survives in
    // the part this call reads
    hipLaunchKernelGGL(li_plan_kernel, dim3((unsigned)G), dim3(256), 0, (hipStream_t)stream, log_poles, residues, ws,
                       (int)S_);
    if (int rc = hyena_check_launch("hyena_li_fwd_static (tables)")) return rc;
    return li_fwd_impl("hyena_li_fwd_static", x1, x2, v, ws, Dcoef, d_is_bf16, out, y_conv_fp32, state_out, B, D, L, G,
                       S_, stream, false);
}

namespace {
int li_fwd_impl(const char* who, const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v, const void* workspace,
                const float* Dcoef, int d_is_bf16, void* out, float* y_conv_fp32, float* state_out,
                int64_t B, int64_t D, int64_t L, int64_t G, int64_t S_, void* stream, bool check_only,
                const float* ftaps) {
    if (!x1 || !x1->ptr || !workspace || !out)
        return hyena_fail(HYENA_EINVAL, "%s: x1, workspace and out are required", who);
    if (B < 0 || D <= 0 || L < 0 || G <= 0 || D % G != 0)
        return hyena_fail(HYENA_EINVAL, "%s: bad sizes B=%lld D=%lld L=%lld G=%lld", who, (long long)B,
                          (long long)D, (long long)L, (long long)G);
    if (S_ < 1 || S_ > S) return hyena_fail(HYENA_ENOSUP, "%s: state size %lld (1..16)", who, (long long)S_);
    if (L % 8 != 0 || !rows_aligned8(x1) || !rows_aligned8(x2) || !rows_aligned8(v) || (((uintptr_t)out) & 15) ||
        (((uintptr_t)y_conv_fp32) & 15) || (((uintptr_t)workspace) & 15))
        return hyena_fail(HYENA_EALIGN, "%s: L and strides must be multiples of 8, pointers 16-byte aligned", who);
    if (d_is_bf16 < 0 || d_is_bf16 > 2) return hyena_fail(HYENA_EINVAL, "%s: d_is_bf16 must be 0, 1 or 2", who);
    // the kernel does the channel arithmetic in 32 bits: reject maps and sizes that would wrap or divide by zero
    if (!rows_valid(x1) || !rows_valid(x2) || !rows_valid(v) || B * D >= (1LL << 31))
        return hyena_fail(HYENA_EINVAL, "%s: B*D and the channel map must fit 31 bits", who);
    // rows are addressed through 32-bit byte offsets inside a buffer descriptor
    if (L > (1LL << 30) - (1LL << 16))
        return hyena_fail(HYENA_ENOSUP, "%s: rows of L=%lld samples (up to 2^30 - 2^16)", who, (long long)L);
    const bool pre = v && v->ptr, post = x2 && x2->ptr;
    if (pre && !post) return hyena_fail(HYENA_ENOSUP, "%s: v without x2 (pass both, x2 alone with x1 holding x1*v, or neither)", who);
    if (ftaps && (!pre || !post || y_conv_fp32))
        return hyena_fail(HYENA_EINVAL, "%s: the featurizer form takes all three projection row sets and no float32 output", who);
    if (B == 0 || L == 0) return 0;
    // Work decomposition (measured on B*D = 1024 .. 8192 rows, L = 8192 .. 524288):
    //  * rows of 65536 samples or more: one channel per wavefront, 2048 samples per step.  A wavefront then reads
    //    4 KiB of its row in one go, which the memory system serves 4-9 % faster than four rows 1 KiB at a time.
    //  * shorter rows: four channels of one filter per wavefront, 512 samples per step (a quarter of the scan
    //    links and fragment builds) - as lone wavefronts when there are enough of them to fill the chip, in the
    //    cooperative form (one block per four channels, four times as many blocks) when there are not.
    //  * long gated rows with four channels per filter: the cooperative form again (its four wavefronts read
    //    consecutive pieces of the same four rows; 1-4 % faster than one channel per wavefront from 65536 samples
    //    on, e.g. 1.61 against 1.64-1.65 ms with three gate streams and 1.25 against 1.29 ms on x1*v rows at L = 262144).
    const bool can4 = (D / G) % 4 == 0;
    const bool long_coop = can4 && L >= 65536 && post && !ftaps;      // the featurizer form runs lone wavefronts only
    int cpw = (can4 && (L < 65536 || long_coop)) ? 4 : 1;    // channels per wavefront (they share one filter)
    // featurizer form (lone wavefronts only): four channels per wavefront on rows below 65536 samples when that
    // still gives every SIMD a wavefront (B = 1, D = 4096: 61 against 88 us at L = 8192, 430 against 413 us at
    // L = 65536, 1.67 against 1.59 ms at L = 262144; D = 1024, L = 16384: 102 against 36 us)
    if (ftaps) cpw = (can4 && L < 65536 && B * (D / 4) >= 1024) ? 4 : 1;
    { const int64_t x = hyena_override(HYENA_OV_LI_CPW); if (x == 1) cpw = 1; else if (x == 4 && can4) cpw = 4; }
    const int64_t nquads = B * (D / cpw);
    bool coop = cpw == 4 && (nquads <= 512 || long_coop);
    { const int64_t x = hyena_override(HYENA_OV_LI_COOP); if (x >= 0) coop = cpw == 4 && x != 0; }
    if (ftaps) coop = false;
    const int64_t nblk = coop ? nquads : (nquads + 3) / 4;
    if (nquads > 0x7fffffffLL) return hyena_fail(HYENA_EINVAL, "%s: problem too large for one launch", who);
    if (check_only) return 0;
    LiArgs a;
    a.x1 = make_rowmap(x1);
    a.x2 = make_rowmap(post ? x2 : nullptr);
    a.v = make_rowmap(pre ? v : nullptr);
    a.ws = (const float*)workspace;
    a.Dcoef = Dcoef;
    a.out = (bf16_t*)out;
    a.y32 = y_conv_fp32;
    a.state_out = state_out;
    a.sr = (int)S_;
    a.D = D;
    a.L = L;
    a.dg = (int)(D / G);
    a.d_is_bf16 = d_is_bf16;
    a.nquads = nquads;
    a.ftaps = ftaps;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)nblk);
    bool nt = 8.0 * (double)B * (double)D * (double)L > 384e6;
    { const int64_t x = hyena_override(HYENA_OV_LI_NT); if (x >= 0) nt = x != 0; }
    // DMODE and Y32 are compile-time so that the hot loop carries no uniform branches.  The fp32
    // side output is a verification path: it always uses cached accesses.
    const int dmode = d_is_bf16;
    const bool y32 = y_conv_fp32 != nullptr;
    if (y32) nt = false;
    {
        // runs of blocks per XCD: a whole eighth of the grid unless pinned; a run length that does not tile the grid
        // falls back to the plain order.  One channel per wavefront on tensors that stay in the last-level cache
        // measured 5 % faster in the plain order (B = 1, L = 8192, one filter per channel: 88.9 against 93.9 us).
        int64_t c = (nblk % 8 == 0 && !(cpw == 1 && !nt)) ? nblk / 8 : 0;
        const int64_t x = hyena_override(HYENA_OV_LI_XCD);
        if (x >= 0) c = (x > 0 && nblk % (8 * x) == 0) ? x : 0;
        a.xchunk = (uint32_t)c;
    }
// prefetch depth in steps: two with four channels per wavefront (three measured the same: 1.528 ms either way in
// the cooperative form, 1.615 against 1.618 ms for lone wavefronts, 1.708 against 1.702 ms with the featurizer
// inside, at B = 1, L = 262144, D = 4096).  One channel per wavefront: three (two measured 1.569 against 1.576 ms),
// two on x1*v rows.
#define LI_LAUNCH(P, Q, N, M, Y)                                                                           \
    do {                                                                                                   \
        if (cpw == 4 && coop) hipLaunchKernelGGL((li_kernel<P, Q, N, 2, M, Y, 4, true>), grid, dim3(256), 0, s, a);   \
        else if (cpw == 4) hipLaunchKernelGGL((li_kernel<P, Q, N, 2, M, Y, 4, false>), grid, dim3(256), 0, s, a);     \
        else hipLaunchKernelGGL((li_kernel<P, Q, N, (P != Q) ? 2 : 3, M, Y, 1, false>), grid, dim3(256), 0, s, a);    \
    } while (0)
#define LI_M(P, Q, N, Y) do { if (dmode == 1) LI_LAUNCH(P, Q, N, 1, Y); else if (dmode == 2) LI_LAUNCH(P, Q, N, 2, Y); else LI_LAUNCH(P, Q, N, 0, Y); } while (0)
#define LI_N(P, Q) do { if (y32) LI_M(P, Q, false, true); else if (nt) LI_M(P, Q, true, false); else LI_M(P, Q, false, false); } while (0)
#define LI_F(N, M)                                                                                          \
    do {                                                                                                   \
        if (cpw == 4) hipLaunchKernelGGL((li_kernel<true, true, N, 2, M, false, 4, false, 3>), grid, dim3(256), 0, s, a);   \
        else hipLaunchKernelGGL((li_kernel<true, true, N, 3, M, false, 1, false, 3>), grid, dim3(256), 0, s, a);             \
    } while (0)
#define LI_FM(N) do { if (dmode == 1) LI_F(N, 1); else if (dmode == 2) LI_F(N, 2); else LI_F(N, 0); } while (0)
    if (ftaps) { if (nt) LI_FM(true); else LI_FM(false); }
    else if (pre && post) LI_N(true, true);
    else if (post) LI_N(false, true);          // x1 already holds bf16(x1*v) (hyena_featurizer_gates_fwd)
    else LI_N(false, false);
#undef LI_FM
#undef LI_F
#undef LI_N
#undef LI_M
#undef LI_LAUNCH
    return hyena_check_launch(who);
}
}  // namespace
