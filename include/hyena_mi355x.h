/* C ABI of libhyena_mi355x.so: hand-written gfx950 kernels for the Hyena
 * operator hot path (Hyena-SE / MR / LI prefill and the cached decode step).
 *
 * Conventions (they mirror the reference's own native launcher,
 * vortex/ops/conv/csrc/step_fir.cu:94-109, and its pybind glue,
 * vortex/ops/conv/csrc/causal_conv1d.cpp:139-225):
 *   - plain pointers, 64-bit sizes, a hipStream_t passed as void*;
 *   - inputs are borrowed, outputs and state are caller-allocated device memory;
 *   - a NULL optional pointer means "absent";
 *   - every call only enqueues work on `stream` (no sync, no allocation, no host threads);
 *   - return 0 on success, a negative HYENA_E* for a rejected argument,
 *     a positive hipError_t if the launch failed; hyena_last_error_string()
 *     describes the last failure on the calling thread.
 * All activation tensors are bfloat16.  Filters, biases, poles are float32.
 */
#ifndef HYENA_MI355X_H
#define HYENA_MI355X_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HYENA_EINVAL  (-1)   /* bad shape / size / enum                         */
#define HYENA_EALIGN  (-2)   /* pointer or stride not aligned as required       */
#define HYENA_ENOSUP  (-3)   /* valid request this build has no kernel for      */

/* One gate operand of the [B, 3D, L] projection, seen as D rows of L samples.
 * Channel d of batch b starts at
 *   ptr + b*batch_stride + ((d / ch_inner)*ch_outer + d % ch_inner)*row_stride
 * (all in elements).  A plain `u.split(D, dim=1)` has ch_inner = D; the
 * head-blocked column_split of vortex/model/utils.py:41-85 has
 * ch_inner = head_dim, ch_outer = 3*head_dim.  Samples of a row are contiguous. */
typedef struct hyena_rows {
    const void* ptr;
    int64_t batch_stride;
    int64_t row_stride;
    int64_t ch_inner;
    int64_t ch_outer;
} hyena_rows;

enum hyena_bias_mode {
    HYENA_BIAS_NONE = 0,
    HYENA_BIAS_ADD = 1,         /* z = bf16(bf16(conv) + bias[d])      vortex/model/engine.py:222-223 */
    HYENA_BIAS_GATED_FP32 = 2,  /* z = bf16(conv + bias[d]*u) in fp32  vortex/model/engine.py:78      */
    /* the two below: hyena_se_fwd and hyena_mr_fwd only */
    HYENA_BIAS_ADD_FP32 = 3,    /* z = bf16(conv + bias[d]), one rounding: F.conv1d with float32 weights and its
                                   own bias argument, vortex/ops/hyena_se/interface.py:236-243 */
    HYENA_BIAS_GATED_BF16 = 4   /* z = bf16(bf16(conv) + bf16(bias[d]*u)): bf16 tensor arithmetic after the
                                   convolution was cast, vortex/model/engine.py:208-221, :352-353 */
};

const char* hyena_version(void);
const char* hyena_last_error_string(void);

/* Launch-shape override, for tests and tuning sweeps; no counterpart in the reference.  The launchers choose
 * segment counts, cached / non-temporal accesses and work decompositions from the problem size; this pins one of
 * those choices process-wide until it is reset with a negative value.  Nothing is read from the environment.
 *   "mr_nseg", "cl_nseg"                       segments along L of hyena_mr_fwd, hyena_fir_cl_fwd / layer_fwd
 *                                               (cl_nseg also: blocks along L per channel strip in hyena_featurizer_gates_fwd)
 *   "li_xcd"                                    hyena_li_fwd: consecutive row groups an XCD takes in one run (0 = blocks in
 *                                               plain order, every eighth to one XCD; default a whole eighth of the rows)
 *   "se_nt", "mr_nt", "li_nt", "cl_nt"         0 = cached, 1 = non-temporal global accesses
 *   "li_cpw"                                    1 / 4 = channels per wavefront in hyena_li_fwd (4 needs D/G % 4 == 0)
 *   "li_coop"                                   0 / 1 = lone / cooperating wavefronts in hyena_li_fwd
 *   "cl_ns"                                     1 = one 64-channel strip per block in hyena_fir_cl_fwd / layer_fwd, 2 or
 *                                               more = the form with several strips per block wherever it exists
 *   "cl_f32_mfma"                               float32 tensors in hyena_fir_cl_fwd_dtype: 0 = always the direct form,
 *                                               1 / 2 = the matrix-core form with one tile per block / blocks that walk
 *                                               a ring of tiles, wherever the matrix-core form applies
 * Returns 0, or HYENA_EINVAL for an unknown name. */
int hyena_set_launch_override(const char* name, int64_t value);

/* Hyena-SE: gated causal depthwise short FIR (2 <= K <= 8), direct form.
 * Replaces HyenaInferenceEngine.parallel_fir, K < 128 branch
 * (vortex/model/engine.py:131-260, body :188-232):
 *   u = bf16(x1*v)            (u = x1 when v == NULL)
 *   z[t] = bf16( sum_k taps[g][k] * u[t-(K-1)+k] )   fp32 accumulate, zero left pad,
 *                                                    taps[g][K-1] on the current sample
 *   z = bias rule (enum above), out = bf16(x2*z)     (out = z when x2 == NULL)
 * taps: [G][K] float32, group g covers channels g*D/G .. (g+1)*D/G-1
 * (repeat_interleave of vortex/model/model.py:261-262).  out: [B][D][L] bf16, contiguous. */
int hyena_se_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                 const float* taps, const float* bias, int bias_mode,
                 void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K,
                 void* stream);

/* Featurizer short FIR (2 <= K <= 8) over the C = 3D channels of the input projection,
 * fused with the [B][L][C] -> [B][C][L] layout change.  Replaces parallel_fir with
 * gate=False, dim_last=True (vortex/model/engine.py:188-223; call site
 * vortex/model/model.py:233-246; native precedent: the channel-last kernel
 * vortex/ops/conv/csrc/causal_conv1d_fwd.cu:210):
 *   z[b][c][t] = bf16( sum_k taps[g(c)][k] * u[b][t-(K-1)+k][c] )   (+ bias[c], rounded again)
 * u: bf16, channels contiguous, sample t of batch b at u + b*u_batch_stride + t*u_time_stride.
 * taps: [G][K] float32 (G = C for vortex's per-channel short filter).  out: [B][C][L] bf16.
 * interleave3 != 0 also applies the channel de-interleave of vortex/model/utils.py:26-38
 * (input channel 3j+i is written to output row i*C/3 + j).
 * front_pad (0..7) makes sequence lengths that are not a multiple of 8 usable by the sequence-major
 * kernels: out is [B][C][L + front_pad] with front_pad leading zero columns (L + front_pad % 8 == 0).
 * Zero samples ahead of a causal filter with zero history change nothing, so the operators run on
 * L + front_pad samples and the caller drops the first front_pad outputs. */
int hyena_featurizer_fwd(const void* u, int64_t u_batch_stride, int64_t u_time_stride,
                         const float* taps, const float* bias, int interleave3, void* out,
                         int64_t B, int64_t L, int64_t C, int64_t G, int K, int front_pad, void* stream);

/* Hyena-MR: gated causal depthwise FIR with 2 <= K <= 128 as a chunked,
 * block-Toeplitz contraction on bf16 MFMA with fp32 accumulation.
 * Replaces parallel_fir, K >= 128 branch + fftconv_func
 * (vortex/model/engine.py:174-187, :38-83); algorithm after the two-pass
 * Toeplitz form of vortex/ops/hyena_se/ref_fwd.py:216-266:
 *   u = bf16(x1*v);  y[t] = sum_k h[g][k] * u[t-k]   (true convolution, h[g][0] on the current sample)
 *   z = bias rule;   out = bf16(x2*z)
 * With taps_reversed != 0 the filter is read in the SE orientation instead
 * (h[g][K-1] on the current sample).  L and strides must be multiples of 8.  The 16 channels of an MFMA
 * tile share one filter, so groups of D/G = 16, 32, ... channels use the matrix cores fully; other group
 * sizes run with partly filled tiles (D/G = 15: 94 %, one filter per channel: 6 %).  out: [B][D][L] bf16. */
int hyena_mr_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                 const float* h, int taps_reversed, const float* bias, int bias_mode,
                 void* out, int64_t B, int64_t D, int64_t L, int64_t G, int K,
                 void* stream);

/* Hyena-LI: long gated convolution with an implicit modal filter, one pass over L
 * as a chunked modal scan on bf16 MFMA (split-precision, fp32 accumulate and state).
 * Replaces HyenaInferenceEngine.parallel_iir (vortex/model/engine.py:262-404),
 * the filter materialisation HyenaCascade.compute_filter (vortex/model/model.py:390-398)
 * and the state prefill prefill_via_modal_fft (vortex/model/engine.py:525-559):
 *   h[g][t] = Re sum_s r[g][s] * exp(t * log_p[g][s])          (never materialised)
 *   x1v = bf16(x1*v);  y = conv(h, x1v) in fp32;  out = bf16((bf16(y) + Dcoef*x1v) * x2)
 *   state_out[b][d][s] = sum_j p^(L-1-j) x1v[b][d][j]          (complex, (re, im) pairs)
 *
 * hyena_li_plan turns the modal parameters into a 6 KB per-group coefficient table, evaluated in double on
 * the device: the filter head h[0..127] and coarse and fine powers of every pole (p^(16a), p^b, r*p^b).
 * Each wavefront of hyena_li_fwd expands its group's table once into the MFMA operand fragments it keeps in
 * registers.  log_poles and residues are [G][S][2] float32 (re, im) pairs; real poles have im = 0.  The caller
 * owns the workspace: hyena_li_plan_bytes(G, S) bytes of device memory, reusable until the parameters change.
 * S is 1..16 (fewer than 16 modes are filled up with poles of residue zero inside the table).
 *
 * hyena_li_fwd: L and strides must be multiples of 8, L at most 2^30 - 2^16 (rows are addressed with 32-bit byte
 * offsets; HYENA_ENOSUP beyond); any D/G (groups of a multiple of 4 channels are fastest).  Nothing outside the
 * B*D rows of L samples is read or written.
 * y_conv_fp32 (optional, [B][D][L]) receives the fp32 convolution before any rounding;
 * state_out (optional, [B][D][S][2] float32) the modal state after the last sample.
 * d_is_bf16 selects the rounding of z = y + Dcoef*x1v: 1 = bf16(bf16(y) + bf16(Dcoef*x1v)), what
 * bf16 tensors give in vortex/model/engine.py:352-353; 0 = bf16(bf16(y) + Dcoef*x1v), a float32
 * Dcoef; 2 = bf16(y + Dcoef*x1v), a single rounding (cheaper, within one bf16 ulp of mode 1).
 * v == NULL with x2 given: x1 already holds x1v = bf16(x1*v) (what hyena_featurizer_gates_fwd writes), 6 instead of 8
 * bytes per sample; v == x2 == NULL: the ungated convolution of x1. */
int64_t hyena_li_plan_bytes(int64_t G, int64_t S);
int hyena_li_plan(const float* log_poles, const float* residues, int64_t G, int64_t S,
                  void* workspace, void* stream);
int hyena_li_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                 const void* workspace, const float* Dcoef, int d_is_bf16,
                 void* out, float* y_conv_fp32, float* state_out,
                 int64_t B, int64_t D, int64_t L, int64_t G, int64_t S, void* stream);

/* A whole Hyena-LI layer in one pass over a projection that is stored sequence-major: the featurizer FIR
 * (HyenaCascade.parallel_forward's first parallel_fir call, vortex/model/model.py:233-246, i.e.
 * vortex/model/engine.py:188-223 with gate = False), the split into x2 | x1 | v with or without `interleave` /
 * column_split (vortex/model/model.py:250-252, vortex/model/utils.py:26-85) and parallel_iir with its state prefill
 * (vortex/model/engine.py:283-353, :525-559), 6 bytes read and 2 written per (batch, channel, sample):
 *   f_i[t] = bf16(w_i[d][0]*p_i[t-2] + w_i[d][1]*p_i[t-1] + w_i[d][2]*p_i[t])     i = x1, x2, v; p_i = the rows given
 *   out    = hyena_li_fwd on (x1, x2, v) = (f_x1, f_x2, f_v)
 * x1, x2, v describe rows of the RAW projection p [B][3D][L] (L contiguous) -- what the producing GEMM writes when it
 * is asked for the transposed product; the reference permutes its [B][L][3D] projection to this shape itself before
 * the convolution (engine.py:189-190), so the values and their order along L are the same.  Channel maps: plain split
 * rows i*D + d (ch_inner = ch_outer = D), head-blocked split (ch_inner = head_dim, ch_outer = 3*head_dim), interleaved
 * rows 3*d + i (ch_inner = 1, ch_outer = 3, ptr advanced by i rows).  feat_taps: [3][D][feat_len] float32, the
 * featurizer weight rows of the x1, x2 and v row of every operator channel, oldest sample first (F.conv1d's weight
 * order); feat_len must be 3; no featurizer bias.  Gates are bit-identical to hyena_featurizer_fwd /
 * hyena_featurizer_gates_fwd, outputs and state to hyena_li_fwd on those gates in the same work decomposition.
 * The featurizer cache of a following decode is the last feat_len-1 samples of the projection itself. */
int hyena_li_layer_fwd(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                       const float* feat_taps, int feat_len, const void* workspace, const float* Dcoef,
                       int d_is_bf16, void* out, float* state_out,
                       int64_t B, int64_t D, int64_t L, int64_t G, int64_t S, void* stream);

/* A whole Hyena-SE / MR layer in one pass over a projection that is stored sequence-major: the featurizer FIR
 * (vortex/model/model.py:233-246, vortex/model/engine.py:188-223 with gate = False), the split under any channel map
 * (vortex/model/model.py:250-252, vortex/model/utils.py:26-85) and the gated inner FIR of hyena_mr_fwd
 * (vortex/model/model.py:268-291, vortex/model/engine.py:131-260), 6 bytes read and 2 written per sample:
 *   f_i[t] = bf16(w_i[d][0]*p_i[t-2] + w_i[d][1]*p_i[t-1] + w_i[d][2]*p_i[t])     i = x1, x2, v; p_i = the rows given
 *   out    = hyena_mr_fwd on (x1, x2, v) = (f_x1, f_x2, f_v)        any 1 <= K <= 128, on the matrix cores
 * Rows, channel maps and feat_taps as in hyena_li_layer_fwd.  bias_mode: HYENA_BIAS_NONE or HYENA_BIAS_GATED_FP32.
 * Bit-identical to hyena_featurizer_fwd followed by hyena_mr_fwd.  out: [B][D][L] bf16.  The inner FIR cache of a
 * following decode (the last K-1 values of bf16(f_x1 * f_v)) is not written; callers form it from the tail of the
 * projection (hyena_featurizer_fwd on the last K+1 samples). */
int hyena_fir_layer_fwd_rows(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                             const float* feat_taps, int feat_len, const float* h, int taps_reversed,
                             const float* bias, int bias_mode, void* out,
                             int64_t B, int64_t D, int64_t L, int64_t G, int K, void* stream);

/* hyena_li_plan + hyena_li_fwd in a form that allocates nothing and takes no workspace.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory or keep a workspace alive -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The coefficient tables go into a static device
 * array inside the library (6 KB per filter group; at most 8192 groups = 48 MiB, which each GPU the library runs
 * on holds until the process ends); more groups are refused with HYENA_ENOSUP.  The tables are rebuilt from
 * log_poles / residues ([G][S][2] float32) on every call, on `stream`, ahead of the main launch.  Same arguments,
 * arithmetic and results as hyena_li_fwd otherwise.  Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (different streams, or threads) race; calls on one stream are ordered and safe. */
int hyena_li_fwd_static(const hyena_rows* x1, const hyena_rows* x2, const hyena_rows* v,
                        const float* log_poles, const float* residues, const float* Dcoef, int d_is_bf16,
                        void* out, float* y_conv_fp32, float* state_out,
                        int64_t B, int64_t D, int64_t L, int64_t G, int64_t S, void* stream);

/* Decode FIR step on a ring-buffer cache.  Replaces HyenaInferenceEngine.step_fir
 * (vortex/model/engine.py:406-449; native precedent vortex/ops/conv/csrc/step_fir.cu:13-109)
 * fused with the caller's gates (vortex/model/model.py:352, :359):
 *   u = bf16(x1*v)                       (u = x1 when v == NULL)
 *   y = w[g][R]*u + sum_{i<R} w[g][i]*state_i      state_i = i-th oldest cached input
 *   y = y + bias[d]*u (bias_mode GATED_FP32) | y + bias[d] (ADD) ; y = bf16(y)
 *   out = bf16(y*x2)                     (out = y when x2 == NULL)
 *   the oldest slot is overwritten with u.
 * ring: [B][D/ring_block][R][ring_block] bf16, slot (pos+i) % R holds the i-th oldest input, so the
 * caller passes pos and afterwards uses (pos+1) % R.  ring_block = D is the plain [B][R][D]
 * cache; ring_block = 512 (any multiple of 512 that divides D) keeps the R slots of 512 channels
 * in one contiguous run, which a cache of 127 slots streams 6 % (D = 4096) to 20 % (D = 8192) faster.
 * w: [G][R+1] float32, the taps already sliced/flipped as engine.py:421-425 does, oldest first.
 * x1, x2, v, out: [B][D] bf16 with the given batch strides (elements). */
int hyena_fir_step(const void* x1, const void* x2, const void* v, int64_t in_batch_stride,
                   void* ring, int64_t R, int64_t ring_block, int64_t pos,
                   const float* w, const float* bias, int bias_mode,
                   void* out, int64_t out_batch_stride,
                   int64_t B, int64_t D, int64_t G, void* stream);

/* Decode modal IIR step.  Replaces HyenaInferenceEngine.step_iir
 * (vortex/model/engine.py:451-467):
 *   x1v = bf16(x1*v); state = p*state + x1v; y = x2*(Re sum_s r_s*state_s + Dcoef*x1v)
 * state: [B][D][S] float32 (is_complex == 0) or [B][D][S][2] (re, im) float32, updated in place.
 * poles (already exponentiated) and residues: [G][S] or [G][S][2] float32.
 * Dcoef: [D] float32; d_is_bf16 != 0 rounds Dcoef*x1v to bf16 as a bf16 parameter does.
 * out: [B][D] bf16 (out_is_fp32 == 0) or float32.  S is a power of two up to 32. */
int hyena_iir_step(const void* x1, const void* x2, const void* v, int64_t in_batch_stride,
                   float* state, const float* poles, const float* residues, int is_complex,
                   const float* Dcoef, int d_is_bf16,
                   void* out, int out_is_fp32, int64_t out_batch_stride,
                   int64_t B, int64_t D, int64_t G, int64_t S, void* stream);

/* The featurizer's own decode step (vortex/model/model.py:325-330: step_fir on the 3D-channel
 * projection with the short filter, then interleave / split, model.py:332-343), described so that a
 * layer step can evaluate it on the fly and the gates x2, x1, v never pass through device memory:
 *   z[c] = bf16( sum_{i<Rf} w[i][c]*slot_i[c] + w[Rf][c]*u[c] (+ bias[c]) ),  slot (pos) <- u
 * Gate i (0: x2, 1: x1, 2: v) of operator channel d is z at channel
 *   (d / ch_inner)*ch_outer + i*gate_stride + (d % ch_inner)*ch_stride
 * plain split: ch_inner = D, gate_stride = D, ch_stride = 1; head-blocked column_split
 * (vortex/model/utils.py:41-85): ch_inner = gate_stride = head_dim, ch_outer = 3*head_dim, ch_stride = 1;
 * interleave (utils.py:26-38) followed by the plain split: ch_inner = D, gate_stride = 1, ch_stride = 3.
 * flip_x1x2 != 0 swaps gates 0 and 1 (vortex/model/engine.py:160-161). */
typedef struct hyena_proj_step {
    const void* u;            /* [B][3D] bf16: this token's projection, channels contiguous        */
    int64_t u_batch_stride;   /* elements                                                          */
    void* ring;               /* [B][Rf][3D] bf16 featurizer cache; slot (pos+i) % Rf = i-th oldest */
    int64_t Rf, pos;          /* the caller advances pos to (pos+1) % Rf after the call            */
    const float* w;           /* [Rf+1][3D] float32, tap-major, oldest tap first                   */
    const float* bias;        /* [3D] float32 or NULL                                              */
    int64_t ch_inner, ch_outer, gate_stride, ch_stride;
    int flip_x1x2;
    const int32_t* pos_dev;   /* NULL, or the ring position in device memory (then pos is ignored)  */
} hyena_proj_step;

/* hyena_fir_step / hyena_iir_step with the featurizer step of the same layer fused in: one launch per
 * Hyena layer and token.  Same arithmetic as the featurizer's hyena_fir_step (bias rule ADD) followed by
 * the gated step; the featurizer cache slot and the inner cache / state are both updated.
 * hyena_fir_layer_step needs one of the three channel maps listed above, 16-byte aligned pointers and
 * head_dim % 8 == 0; it takes bias_mode NONE or GATED_FP32.  hyena_iir_layer_step takes any map; it
 * needs at least 16 real or 8 complex states. */
int hyena_fir_layer_step(const hyena_proj_step* proj,
                         void* ring, int64_t R, int64_t ring_block, int64_t pos,
                         const float* w, const float* bias, int bias_mode,
                         void* out, int64_t out_batch_stride,
                         int64_t B, int64_t D, int64_t G, void* stream);
int hyena_iir_layer_step(const hyena_proj_step* proj,
                         float* state, const float* poles, const float* residues, int is_complex,
                         const float* Dcoef, int d_is_bf16,
                         void* out, int out_is_fp32, int64_t out_batch_stride,
                         int64_t B, int64_t D, int64_t G, int64_t S, void* stream);

/* Ring positions in device memory, for callers that replay a recorded token step (a HIP graph) and so cannot
 * change a scalar argument between tokens.  No counterpart in the reference, whose caches have no position
 * (vortex/model/engine.py:443-447 shifts the whole cache each token).  The _dpos forms read the position of the
 * inner cache from *pos_dev (reduced mod R); hyena_proj_step.pos_dev does the same for the featurizer cache in
 * every layer step.  hyena_ring_advance moves n positions on by one slot, pos[i] = (pos[i] + 1) % depth[i]:
 * one launch per token for all the rings of a model, after the layer steps of that token. */
int hyena_fir_step_dpos(const void* x1, const void* x2, const void* v, int64_t in_batch_stride,
                        void* ring, int64_t R, int64_t ring_block, const int32_t* pos_dev,
                        const float* w, const float* bias, int bias_mode,
                        void* out, int64_t out_batch_stride,
                        int64_t B, int64_t D, int64_t G, void* stream);
int hyena_fir_layer_step_dpos(const hyena_proj_step* proj,
                              void* ring, int64_t R, int64_t ring_block, const int32_t* pos_dev,
                              const float* w, const float* bias, int bias_mode,
                              void* out, int64_t out_batch_stride,
                              int64_t B, int64_t D, int64_t G, void* stream);
int hyena_ring_advance(int32_t* pos, const int32_t* depth, int64_t n, void* stream);

/* FIR step on a deep cache (R >= 32) that reads about a third of the cache per token.  No counterpart in the
 * reference, which reads (and rewrites) the whole cache every token (vortex/model/engine.py:427-447); same result up
 * to the order of the float32 sums.  The part of a later token's sum that the cache already determines is formed
 * three tokens at a time and kept in `far` ([B][3][D] float32, hyena_fir_far_bytes(B, D) bytes, contents owned by
 * these calls): a block of 512 channels reads its whole cache on every third token (staggered over the blocks) and
 * far[j] plus the j newest slots on the others.  `far` depends on the taps: one buffer per (cache, w) pair.
 * cnt: token counter in [0, hyena_fir_far_period(R)) (the ring slot is cnt % R; the caller moves on to
 * (cnt + 1) % period), or cnt_dev != NULL: the counter in device memory (hyena_ring_advance with depth = period).
 * rebuild != 0: every block rebuilds its far sums from the cache as it stands; pass it on the first step and
 * after anything else (hyena_fir_step, a prefill) has written to the cache.  Other arguments as hyena_fir_step /
 * hyena_fir_layer_step. */
int64_t hyena_fir_far_period(int64_t R);
int64_t hyena_fir_far_bytes(int64_t B, int64_t D);
int hyena_fir_step_far(const void* x1, const void* x2, const void* v, int64_t in_batch_stride,
                       void* ring, int64_t R, int64_t ring_block, int64_t cnt, const int32_t* cnt_dev,
                       float* far, int rebuild,
                       const float* w, const float* bias, int bias_mode,
                       void* out, int64_t out_batch_stride,
                       int64_t B, int64_t D, int64_t G, void* stream);
int hyena_fir_layer_step_far(const hyena_proj_step* proj,
                             void* ring, int64_t R, int64_t ring_block, int64_t cnt, const int32_t* cnt_dev,
                             float* far, int rebuild,
                             const float* w, const float* bias, int bias_mode,
                             void* out, int64_t out_batch_stride,
                             int64_t B, int64_t D, int64_t G, void* stream);

/* Modal IIR step that reads and writes the state once per window of hyena_iir_window_tokens() (4) tokens instead of
 * every token.  No counterpart in the reference (vortex/model/engine.py:451-467 updates the state per token); same
 * outputs up to float32 rounding.  With S the state before a window's first token t0,
 *   Re sum_s r s_{t0+j} = far[j] + sum_{k<=j} g[k] u_{t0+j-k},  far[j] = Re sum_s r p^(j+1) S,  g[k] = Re sum_s r p^k:
 * on the first token of a window the kernel folds the window before into the stored state and forms far[]; on the
 * other tokens it reads neither state nor poles.  Windows are staggered over the batch elements.  The caller owns
 *   hist [B][W][D] bf16 (the last W inputs x1*v; contents owned by these calls), far [B][W][D] float32,
 *   g [G][W] float32 (from the caller: g[k] = Re sum_s residues * poles^k), W = hyena_iir_window_tokens(),
 * counts tokens in cnt = token % W (or cnt_dev: the counter in device memory, advanced with hyena_ring_advance,
 * depth W) and passes warm = the number of tokens stepped with these calls since `state` was last exact (0 on the
 * first call; anything >= W means "W or more").  Between two windows the `state` tensor lags the tokens by up to W
 * inputs; hyena_iir_window_flush (called with cnt = the counter of the NEXT token, i.e. advanced past the last step, and
 * the current warm) folds them in; afterwards go on counting cnt as before and restart warm at 0.  Flush before
 * anything else reads the state.  Available for 16 states, 16-byte aligned gates with D % 8 == 0, and (in the layer step) the featurizer
 * maps that have a vector form (hyena_iir_window_supported); other cases return HYENA_ENOSUP: use hyena_iir_step. */
typedef struct hyena_iir_window {
    void* hist;
    float* far;
    const float* g;
    int64_t cnt;
    const int32_t* cnt_dev;
    int warm;
    int reserved;                /* 0 */
} hyena_iir_window;
int64_t hyena_iir_window_tokens(void);
int hyena_iir_window_supported(int64_t B, int64_t D, int64_t S, int is_complex);
int hyena_iir_step_win(const void* x1, const void* x2, const void* v, int64_t in_batch_stride,
                       float* state, const float* poles, const float* residues, int is_complex,
                       const float* Dcoef, int d_is_bf16,
                       void* out, int out_is_fp32, int64_t out_batch_stride,
                       int64_t B, int64_t D, int64_t G, int64_t S, const hyena_iir_window* win, void* stream);
int hyena_iir_layer_step_win(const hyena_proj_step* proj,
                             float* state, const float* poles, const float* residues, int is_complex,
                             const float* Dcoef, int d_is_bf16,
                             void* out, int out_is_fp32, int64_t out_batch_stride,
                             int64_t B, int64_t D, int64_t G, int64_t S, const hyena_iir_window* win, void* stream);
int hyena_iir_window_flush(float* state, const float* poles, const float* residues, int is_complex,
                           int64_t B, int64_t D, int64_t G, int64_t S, const hyena_iir_window* win, void* stream);

/* Channel-last operand [B][L][D]: element (b, t, d) at ptr + b*batch_stride + t*time_stride + d (elements).
 * This is the (batch, seqlen, groups, group_dim) layout of vortex/ops/hyena_se/fwd.py:17-43 with D = groups*group_dim. */
typedef struct hyena_cl {
    const void* ptr;
    int64_t batch_stride;
    int64_t time_stride;
} hyena_cl;

/* Gated causal FIR (1 <= K <= 128) on channel-last tensors, block-Toeplitz MFMA contraction.
 * Replaces two_pass_fwd_grouped (vortex/ops/hyena_se/fwd.py:17-290; kernels fwd_kernels.py:631-794) and the
 * layout handling of inner_hyena_se_ref (vortex/ops/hyena_se/interface.py:272-397):
 *   bx = bf16(x1*v);  y2[t] = bias rule( sum_k h[g][k]*bx[t-k] );  out = bf16(x2*y2)
 * (x1 = B, v = x, x2 = C in the reference's naming; v == x2 == NULL gives the ungated FIR.)
 * h: [G][K] float32, h[g][0] on the current sample unless taps_reversed.  D/G % 16 == 0, D % 8 == 0.
 * out: [B][L][D] bf16 contiguous.  Optional outputs, the intermediates fwd.py:23-25 can return:
 *   y2_out [B][L][D]: the convolution before the x2 gate;
 *   bx_out [B][L-bx_from][D]: rows t >= bx_from of bx (bx_from = 0: all of it; bx_from = L-(K-1): the FIR
 *   cache a decode step continues from, vortex/model/engine.py:255-258). */
int hyena_fir_cl_fwd(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v,
                     const float* h, int taps_reversed, const float* bias, int bias_mode,
                     void* out, void* y2_out, void* bx_out, int64_t bx_from,
                     int64_t B, int64_t L, int64_t D, int64_t G, int K, void* stream);

/* Element types of hyena_fir_cl_fwd_dtype. */
enum hyena_dtype {
    HYENA_DTYPE_BF16 = 0,
    HYENA_DTYPE_F16 = 1,
    HYENA_DTYPE_F32 = 2
};

/* hyena_fir_cl_fwd for the element types the reference's own parity grid of this operator runs in
 * (vortex/ops/hyena_se/tests/test_fwd.py:25-54 and tests/test_two_pass_ref.py:17-51: float16 and float32 tensors of
 * shape (batch, seqlen, groups, group_dim), checked against gcg_fwd_ref_corrected, vortex/ops/hyena_se/ref_fwd.py:80-127).
 * x1, x2, v, out, y2_out, bx_out hold elements of `dtype`; strides in elements; h and bias stay float32.
 *   HYENA_DTYPE_BF16: exactly hyena_fir_cl_fwd for K <= 128; longer filters (vortex/model/engine.py:174-187 takes any
 *                     length through its FFT, :339-349 any long_fir_threshold) run the direct form below with the
 *                     roundings of bfloat16 tensor arithmetic.
 *   HYENA_DTYPE_F16:  the same MFMA kernel on float16 operands (v_mfma_f32_32x32x16_f16; taps rounded to float16,
 *                     bx = f16(x1*v), y2 = f16(conv), out = f16(x2*y2): the roundings of float16 tensor arithmetic)
 *                     when D/G % 16 == 0, D % 8 == 0 and the operands are 16-byte aligned with strides % 8 == 0;
 *                     any other shape runs a direct-form kernel with the same roundings and float32 taps.
 *   HYENA_DTYPE_F32:  direct form, float32 operands and accumulation, nothing rounded below float32; any D/G.
 * The direct form takes every bias mode (the "bf16" in their names reads as "element type") and any K >= 1 (filters
 * beyond 128 taps in blocks of 128 lags, in every element type); the MFMA form takes the bias modes of hyena_fir_cl_fwd
 * and 1 <= K <= 128. */
int hyena_fir_cl_fwd_dtype(const hyena_cl* x1, const hyena_cl* x2, const hyena_cl* v,
                           const float* h, int taps_reversed, const float* bias, int bias_mode,
                           void* out, void* y2_out, void* bx_out, int64_t bx_from,
                           int64_t B, int64_t L, int64_t D, int64_t G, int K, int dtype, void* stream);

/* The featurizer of a Hyena layer at prefill (vortex/model/model.py:233-252: short FIR over the 3D channels
 * of the dense projection, then interleave / split), described so that hyena_fir_layer_fwd can evaluate it on
 * the fly:  z[t][c] = bf16( sum_k w[k][c]*u[t-(Ks-1)+k][c] )  (then + bias[c], rounded again).
 * Gate i (0: x2, 1: x1, 2: v) of operator channel d is z at channel
 *   (d / ch_inner)*ch_outer + i*gate_stride + (d % ch_inner)*ch_stride      (maps as in hyena_proj_step). */
typedef struct hyena_proj_fwd {
    const void* u;              /* [B][L][3D] bf16, channels contiguous */
    int64_t u_batch_stride, u_time_stride;
    const float* w;             /* [Ks][3D] float32, tap-major, w[Ks-1] on the current sample */
    const float* bias;          /* [3D] float32 or NULL */
    int Ks;                     /* 3 or 4 */
    int flip_x1x2;
    int64_t ch_inner, ch_outer, gate_stride, ch_stride;
} hyena_proj_fwd;

/* Featurizer and gates of a Hyena-LI layer at prefill in one launch: the featurizer FIR over the projection
 * u [B][L][3D] (vortex/model/engine.py:188-223), interleave / split (vortex/model/model.py:251-252,
 * engine.py:300-310) and x1v = x1*v (engine.py:312), written as the two row tensors hyena_li_fwd reads:
 *   xv_out [B][D][L + front_pad] = bf16(x1*v),  x2_out [B][D][L + front_pad] = x2   (bf16; the first front_pad
 * columns are zero: front_pad = -L % 8 makes any L usable).  Rows are out_row_stride elements apart (a multiple of 8,
 * at least L + front_pad; the columns beyond are not written): rows a power of two apart stream more slowly in the
 * scan that follows, a stride a few KB off one avoids that.  The three gate tensors [B][3D][L] of
 * hyena_featurizer_fwd are never written: 10 instead of 12 bytes per (channel, sample) here and 6 instead of 8 in
 * hyena_li_fwd (v = NULL).  Channel maps and Ks as hyena_fir_layer_fwd; others return HYENA_ENOSUP. */
int hyena_featurizer_gates_fwd(const hyena_proj_fwd* proj, void* xv_out, void* x2_out, int64_t out_row_stride,
                               int64_t B, int64_t L, int64_t D, int front_pad, void* stream);

/* A whole Hyena-SE / Hyena-MR layer at prefill in one launch: featurizer FIR, split, x1*v gate, inner FIR,
 * bias rule (NONE or GATED_FP32), x2 gate; u [B][L][3D] in, out [B][L][D], nothing in between touches device
 * memory.  Replaces the two parallel_fir calls of vortex/model/model.py:233-291.  bx_out / bx_from as above, but
 * here bx is the cache tail only: L - bx_from may not exceed K - 1 (it is copied out of the kernel's LDS ring after
 * the last step). */
int hyena_fir_layer_fwd(const hyena_proj_fwd* proj,
                        const float* h, int taps_reversed, const float* bias, int bias_mode,
                        void* out, void* bx_out, int64_t bx_from,
                        int64_t B, int64_t L, int64_t D, int64_t G, int K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HYENA_MI355X_H */
