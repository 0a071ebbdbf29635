"""CPU oracle for the Hyena operator hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain PyTorch on the CPU, the arithmetic of the
reference's Hyena operator path (vortex/model/engine.py and its callers),
including every dtype rounding point.  It is the checker for the HIP kernels:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import it.  Nothing in the product package may call into this file.

Each function cites the reference file:line it follows (paths relative to the
reference checkout).  The reference is Python/torch, so the restatement is
Python/torch too; torch's own conv1d / fft are the library routines the
reference itself calls.

How each function is pinned (see tests/test_oracle_*.py):
  se_fir / parallel_fir(K<128) : brute-force O(L*K) float64 loops, impulse
                                 response, and the two-pass Toeplitz identity
                                 held by the reference's test_two_pass_ref.py
  mr_fir / parallel_fir(K>=128): ref_fftconv of the reference's
                                 test/test_forward.py:13-23 restated, direct
                                 float64 convolution, equality with se_fir on
                                 the flipped filter, impulse response
  modal_filter                 : closed forms h[0]=sum(r), geometric series sum
  parallel_iir / modal state   : FFT path == explicit recurrence (the identity
                                 asserted by the reference's
                                 test/test_prefill.py:85-229)
  toeplitz / correction        : known-answer arange filter of
                                 vortex/ops/hyena_se/tests/test_toeplitz.py
  causal_conv1d_ref /
  inner_hyena_se_ref           : float64 brute-force loops (bias inside the single
                                 rounding, gated bias), a hand-computed rounding
                                 known answer, and the impulse response, which
                                 shows the striped filter-to-channel map
  step_fir / step_iir          : no reference test touches these ("parity
                                 unpinned" by the reference's own tests); they
                                 are pinned here by prefill-vs-decode
                                 consistency and the closed-form recurrence,
                                 plus the committed golden vectors in
                                 tests/golden/ when present.
  prefill_direct_recurrence_ref: the literal loop of engine.py:473-504 (bf16
                                 state, in-place lanes, lane-0 output): three
                                 hand-computed three-step cases, and equality
                                 with the plain recurrence where its quirks
                                 cannot act (real poles, float32 activations)
  OracleCascade                : prefill of L+n tokens == prefill of L tokens +
                                 n one-token calls (outputs and caches) over SE /
                                 MR / LI x split x interleave x x1-x2 flip, and
                                 an index known answer (which projection channel
                                 acts as x2 / x1 / v on either branch)
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# layout glue  (vortex/model/utils.py:26-85)
# --------------------------------------------------------------------------

def interleave(z):
    """De-interleave stride-3 channels into [x1 | x2 | v] blocks.

    vortex/model/utils.py:26-38: channels 0::3, 1::3, 2::3 are concatenated
    along the channel axis (axis 1 for [B, 3D, L], last axis for [B, 3D]).
    """
    if z.dim() == 3:
        return torch.cat([z[:, 0::3], z[:, 1::3], z[:, 2::3]], dim=1)
    return torch.cat([z[..., 0::3], z[..., 1::3], z[..., 2::3]], dim=-1)


def column_split(x, num_heads, head_size):
    """Head-blocked split of 3D channels into (x2, x1, v).

    vortex/model/utils.py:41-85: channels are viewed as
    [num_heads, 3*head_size]; the first/second/third head_size of each head go
    to x2/x1/v.  Works for [B, 3D] and [B, 3D, L].
    """
    if x.dim() == 2:
        xr = x.reshape(x.shape[0], num_heads, 3 * head_size)
        parts = [xr[..., i * head_size:(i + 1) * head_size].reshape(x.shape[0], -1) for i in range(3)]
    else:
        xr = x.reshape(x.shape[0], num_heads, 3 * head_size, x.shape[2])
        parts = [
            xr[:, :, i * head_size:(i + 1) * head_size].reshape(x.shape[0], -1, x.shape[-1]) for i in range(3)
        ]
    return parts[0], parts[1], parts[2]


def split_gates(u, dims, column_split_hyena=False, flip_x1x2=False):
    """(x2, x1, v) from the [B, 3D, L] (or [B, 3D]) projection.

    vortex/model/engine.py:150-158 and :283-310.
    """
    hidden, n_heads, head_dim = dims[0], dims[1], dims[2]
    if column_split_hyena:
        x2, x1, v = column_split(u, n_heads, head_dim)
    else:
        x2, x1, v = u.split([hidden, hidden, hidden], dim=1)
    if flip_x1x2:
        x1, x2 = x2, x1
    return x2, x1, v


# --------------------------------------------------------------------------
# prefill FIR  (vortex/model/engine.py:131-260)
# --------------------------------------------------------------------------

def short_fir_fp32(u, weight, fir_length):
    """fp32 depthwise cross-correlation with left zero padding.

    vortex/model/engine.py:197-204: conv1d on fp32 copies, padding K-1,
    groups = channel count, truncated to the first L outputs.  weight is
    [D, 1, K]; weight[..., K-1] multiplies the current sample.
    """
    L = u.shape[-1]
    return F.conv1d(
        u.to(torch.float32), weight.to(torch.float32), bias=None, stride=1,
        padding=fir_length - 1, groups=u.shape[1],
    )[..., :L]


def fft_causal_conv_fp32(u, k):
    """Causal convolution y[t] = sum_j k[j] u[t-j] through a length-2L FFT.

    vortex/model/engine.py:50-73 (non-bidirectional branch).  u: [B, D, L]
    fp32, k: [D, 1, Lk] or [D, Lk] fp32.
    """
    L = u.shape[-1]
    n = 2 * L
    k_f = torch.fft.rfft(k, n=n) / n
    k_f = k_f.squeeze()
    if u.dim() > k_f.dim():
        k_f = k_f.unsqueeze(0)
    u_f = torch.fft.rfft(u.to(k.dtype), n=n)
    return torch.fft.irfft(u_f * k_f, n=n, norm="forward")[..., :L]


def fftconv_with_bias(u, k, D):
    """engine.py:38-83: fft conv, then `+ u * D[:, None]` in fp32, cast to u.dtype."""
    y = fft_causal_conv_fp32(u, k)
    out = y + u * D.unsqueeze(-1)
    return out.to(u.dtype)


def parallel_fir(
    u, weight, bias, L=None, dims=None, groups=None, gated_bias=False,
    column_split_hyena=False, dim_last=True, fir_length=3, gate=False,
    want_state=False, padding_mask=None, flip_x1x2=False,
):
    """Restatement of HyenaInferenceEngine.parallel_fir (engine.py:131-260).

    Returns (z, fir_state) with z in [B, D, L] layout.  `want_state` stands
    for `inference_params is not None` (engine.py:255-258).
    """
    x2 = None
    if gate:
        x2, x1, v = split_gates(u, dims, column_split_hyena, flip_x1x2)
        u = x1 * v                                   # engine.py:159, input dtype
    if fir_length >= 128:
        # engine.py:174-187.  The fp32 upcast, FFT conv, fp32 bias add, then
        # two casts back to the input dtype.
        z = fftconv_with_bias(u.to(torch.float32), weight[:, :, : u.shape[-1]].to(torch.float32), bias)
        z = z.to(u.dtype)
    else:
        if dim_last:
            u = u.permute(0, 2, 1)
        z = short_fir_fp32(u, weight, fir_length).to(u.dtype)     # engine.py:197-208
        if bias is not None:                                       # engine.py:219-223
            z = z + bias[None, :, None] * u if gated_bias else z + bias[None, :, None]
    if isinstance(padding_mask, torch.Tensor):                     # engine.py:226-227
        z = z * padding_mask[:, None]
    if gate:
        z = x2 * z                                                 # engine.py:232
    state = u[..., -fir_length + 1:] if want_state else None      # engine.py:255-258
    return z, state


def se_fir(x2, x1, v, h_groups, fir_length=None):
    """Hyena-SE gated short FIR on explicit gates.

    Same arithmetic as parallel_fir(gate=True, K<128) after the split:
    u = bf16(x1*v); z = bf16(corr_K(u)); out = bf16(x2*z).  h_groups is
    [G, 1, K]; it is expanded with repeat_interleave(D/G) as in
    vortex/model/model.py:261-262.
    """
    D = x1.shape[1]
    K = h_groups.shape[-1] if fir_length is None else fir_length
    w = h_groups.repeat_interleave(D // h_groups.shape[0], 0)
    u = x1 * v
    z = short_fir_fp32(u, w, K).to(u.dtype)
    return x2 * z, u[..., -K + 1:]


def mr_fir(x2, x1, v, h_groups, D_bias):
    """Hyena-MR gated medium FIR (true convolution through FFT) on explicit gates.

    parallel_fir(gate=True, K>=128): u = bf16(x1*v); y = fftconv(u, h);
    z = bf16(y + u*D) ; out = bf16(x2*z).  (engine.py:174-187, :38-83, :232)
    """
    Dch = x1.shape[1]
    w = h_groups.repeat_interleave(Dch // h_groups.shape[0], 0)
    u = x1 * v
    z = fftconv_with_bias(u.to(torch.float32), w[:, :, : u.shape[-1]].to(torch.float32), D_bias.to(torch.float32))
    z = z.to(u.dtype)
    K = h_groups.shape[-1]
    return x2 * z, u[..., -K + 1:]


# --------------------------------------------------------------------------
# modal filter and Hyena-LI prefill  (model.py:377-398, engine.py:262-404)
# --------------------------------------------------------------------------

def modal_filter(log_poles, residues, L, dtype=None):
    """h[g, t] = Re sum_s residues[g, s] * exp(log_poles[g, s, 0] * t), t < L.

    vortex/model/model.py:390-398 (real parameters).  Complex parameters use
    the same expression and the real part is taken, matching
    `(residues * poles**t).real.sum(1)` of model.py:847.  Returns [1, G, L].
    `dtype=torch.float64/complex128` evaluates the same formula in double.
    """
    t = torch.arange(L, device=log_poles.device)[None, None]
    if dtype is not None:
        cdt = dtype
        if log_poles.is_complex():
            cdt = torch.complex128 if dtype == torch.float64 else torch.complex64
        log_poles, residues = log_poles.to(cdt), residues.to(cdt)
    h = (residues[..., None] * (log_poles * t).exp()).sum(1)[None]
    return h.real if h.is_complex() else h


def long_conv_fp32(x1v, h):
    """engine.py:331-337: fp32 FFT long convolution, returns (y_fp32, X_s)."""
    L = x1v.shape[-1]
    n = 2 * L
    H = torch.fft.rfft(h.to(torch.float32), n=n) / n
    X_s = torch.fft.fft(x1v.to(torch.float32), n=n)
    X = X_s[..., : H.shape[-1]]
    y = torch.fft.irfft(X * H, n=n, norm="forward")[..., :L]
    return y, X_s


def modal_state_fft(X_s, log_poles, L, hidden, groups, keep_complex=False):
    """engine.py:525-559: modal state after L tokens through the FFT of p^t.

    state[b, d, s] = sum_j p^(L-1-j) x1v[b, d, j].  The reference casts the
    complex result to float32, i.e. drops the imaginary part (engine.py:559);
    keep_complex=True returns the complex state (needed for complex poles).
    """
    n = 2 * L
    t = torch.arange(L)[None, None]
    lp = log_poles.to(torch.complex64 if log_poles.is_complex() else torch.float32)
    state_s = (lp * t).exp()                                     # [G, S, L]
    state_S = torch.fft.fft(state_s, n=n)[None]                  # [1, G, S, 2L]
    if groups > 1:
        state_S = state_S.repeat_interleave(hidden // groups, 1)
    state = torch.fft.ifft(X_s[..., None, :] * state_S, n=n)[..., L - 1]
    if keep_complex:
        return state
    return state.real.to(torch.float32)


def modal_state_closed_form(x1v, log_poles, dtype=torch.float64):
    """Textbook form of the same state: sum_j p^(L-1-j) u[j], in double."""
    L = x1v.shape[-1]
    cdt = torch.complex128 if log_poles.is_complex() else dtype
    lp = log_poles.to(cdt)[..., 0]                               # [G, S]
    G = lp.shape[0]
    Dch = x1v.shape[1]
    lp = lp.repeat_interleave(Dch // G, 0)                       # [D, S]
    e = torch.arange(L - 1, -1, -1, dtype=torch.float64)
    w = (lp[..., None] * e).exp()                                # [D, S, L]
    return torch.einsum("dsl,bdl->bds", w, x1v.to(cdt))


def truncated_fir(x1v, h, threshold):
    """The long_fir_threshold branch of parallel_iir (engine.py:339-349): the first `threshold` samples of the
    materialised filter h [1, D, L], cast to the activations' dtype, applied with F.conv1d and padding
    threshold-1.  conv1d is a cross-correlation, so tap h[threshold-1] lands on the current sample and h[0] on
    the oldest one: y[t] = sum_j h[threshold-1-j] * x1v[t-j], computed in the activations' dtype."""
    assert h.shape[0] == 1, "batch size must be 1 for long_fir_threshold"
    w = h[0][:, None][..., :threshold]
    L = x1v.shape[-1]
    return F.conv1d(x1v, w.to(dtype=x1v.dtype), stride=1, groups=x1v.shape[1], padding=w.shape[-1] - 1)[..., :L]


def parallel_iir(
    z_pre, h, D, L, poles, residues, dims, column_split_hyena=False,
    flip_x1x2=False, want_state=False, keep_complex_state=False, return_fp32_conv=False,
    long_fir_threshold=None,
):
    """Restatement of HyenaInferenceEngine.parallel_iir: the default FFT branch and the truncated-FIR branch.

    engine.py:283-353 and :379-404.  Returns (y [B, L, D], state or None[,
    y_conv_fp32]).  Cast order: y = bf16(conv); out = (y + x1v*D)*x2 in the
    tensors' own dtypes.  With long_fir_threshold the reference has no spectrum to prefill the state from
    (engine.py:380-392 reads X_s, which that branch never assigns), so the branch only exists without a cache.
    """
    hidden, _, _, state_size, groups = dims
    x2, x1, v = split_gates(z_pre, dims, column_split_hyena, flip_x1x2)
    x1v = x1 * v
    if long_fir_threshold is not None:
        assert not want_state, "the reference cannot prefill the modal state on this branch"
        y = truncated_fir(x1v, h, long_fir_threshold).to(x1v.dtype)
        y = (y + x1v * D.unsqueeze(-1)) * x2
        return (y.permute(0, 2, 1), None)
    y32, X_s = long_conv_fp32(x1v, h)
    y = y32.to(x1v.dtype)
    y = (y + x1v * D.unsqueeze(-1)) * x2
    state = None
    if want_state:
        state = modal_state_fft(X_s, poles, L, hidden, groups, keep_complex=keep_complex_state)
    out = (y.permute(0, 2, 1), state)
    if return_fp32_conv:
        out = out + (y32,)
    return out


def li_prefill(x2, x1, v, log_poles, residues, D_bias, want_state=True):
    """Hyena-LI on explicit gates with grouped (possibly complex) poles.

    Filter per group from modal_filter, expanded over the group's channels;
    conv as engine.py:331-337; gating as engine.py:352-353.  Returns
    (out [B, D, L], y_conv_fp32 [B, D, L], state [B, D, S] complex or real).
    """
    B, Dch, L = x1.shape
    G = log_poles.shape[0]
    h = modal_filter(log_poles, residues, L)[0]                  # [G, L]
    h = h.repeat_interleave(Dch // G, 0)[None]                   # [1, D, L]
    x1v = x1 * v
    y32, X_s = long_conv_fp32(x1v, h)
    y = y32.to(x1v.dtype)
    out = (y + x1v * D_bias.unsqueeze(-1)) * x2
    state = None
    if want_state:
        state = modal_state_closed_form(x1v, log_poles)
        state = state.to(torch.complex64) if state.is_complex() else state.to(torch.float32)
    return out, y32, state


def prefill_direct_recurrence(x1v, log_poles, residues):
    """Explicit modal recurrence  s_t = p s_{t-1} + u_t,  y_t = Re sum r s_t, in double.

    The mathematics that engine.py:473-504 is meant to evaluate (true complex
    product, exact state), NOT that loop's own arithmetic, which differs in three
    ways (see prefill_direct_recurrence_ref below).  Used as the independent check
    of the FFT path.  Returns (y [B, D, L] float64, final state [B, D, S]).
    """
    B, Dch, L = x1v.shape
    G = log_poles.shape[0]
    cplx = log_poles.is_complex() or residues.is_complex()
    dt = torch.complex128 if cplx else torch.float64
    p = log_poles.to(dt)[..., 0].exp().repeat_interleave(Dch // G, 0)[None]   # [1, D, S]
    r = residues.to(dt).repeat_interleave(Dch // G, 0)[None]
    s = torch.zeros(B, Dch, p.shape[-1], dtype=dt)
    y = torch.zeros(B, Dch, L, dtype=torch.float64)
    xu = x1v.to(dt)
    for i in range(L):
        s = p * s + xu[:, :, i, None]
        acc = (r * s).sum(-1)
        y[:, :, i] = acc.real if cplx else acc
    return y, s


def prefill_direct_recurrence_ref(x1v, poles, residues):
    """Restatement of HyenaInferenceEngine.prefill_via_direct_recurrence as it is written (engine.py:473-504).

    x1v [B, D, L] in the activations' dtype; poles and residues [D, S, 1, 2] with (re, im) lanes (the poles
    themselves: this branch never exponentiates).  What the loop does, which the mathematics would not:
      * the state is created as `0 * x1v_[:, :, 0]` (engine.py:487) and so has the activations' dtype: with bf16
        activations it is rounded to bf16 after every update, and so is the output row (engine.py:488);
      * the real lane is overwritten first and the imaginary lane then reads the NEW real lane
        (engine.py:498-499), which is not the complex product unless the poles are real;
      * the output keeps lane 0 of the lane-wise product residues * state summed over the modes
        (engine.py:500), i.e. sum_s r_re * s_re without the - r_im * s_im term.
    Returns (output [B, D, L] in x1v.dtype, state [B, D, S, 2] float32) -- the state is what the reference
    stores in inference_params.state_dict (engine.py:502).
    """
    B, Dch, L = x1v.shape
    S = poles.shape[1]
    lanes = x1v[..., None, None].repeat(1, 1, 1, S, 2)         # [B, D, L, S, 2]
    lanes[..., 1] = 0
    state = 0 * lanes[:, :, 0]                                 # [B, D, S, 2], activations' dtype
    out = 0 * lanes[:, :, :, 0, 0]                             # [B, D, L]
    p = poles[:, :, 0][None]                                   # [1, D, S, 2]
    r = residues[:, :, 0][None].repeat(B, 1, 1, 1)             # [B, D, S, 2]
    for i in range(L):
        state[..., 0] = p[..., 0] * state[..., 0] - p[..., 1] * state[..., 1] + lanes[:, :, i, :, 0]
        state[..., 1] = p[..., 0] * state[..., 1] + p[..., 1] * state[..., 0] + lanes[:, :, i, :, 1]
        out[:, :, i] = torch.sum(r * state, dim=-2)[..., 0]
    return out, state.to(torch.float32)


# --------------------------------------------------------------------------
# decode steps  (engine.py:406-467)
# --------------------------------------------------------------------------

def step_fir(u, fir_state, weight, bias=None, gated_bias=False, flip_filter=False):
    """Restatement of HyenaInferenceEngine.step_fir (engine.py:406-449).

    u: [B, D]; fir_state: [B, D, cache] oldest-first; weight: [D, 1, K].
    Returns (y in u.dtype, new state in float32).
    """
    w = weight.squeeze()
    cache = fir_state.shape[-1]
    K = w.shape[-1]
    if flip_filter:
        w = w.flip(-1)[..., -cache - 1:].unsqueeze(0)
    else:
        w = w[..., : cache + 1].unsqueeze(0)
    in_dtype = u.dtype
    w = w.to(torch.float32)
    uf = u.to(torch.float32)
    st = fir_state.to(torch.float32)
    y = w[..., -1] * uf + torch.sum(st * w[..., :-1], dim=-1)
    if bias is not None:
        b = bias.to(torch.float32)
        y = y + b * uf if gated_bias else y + b
    if cache < K - 1:
        st = torch.cat([st, uf[..., None]], dim=-1)
    else:
        st = torch.roll(st, -1, dims=2)
        st[..., -1] = uf
    return y.to(in_dtype), st


def step_iir(x2, x1, v, D, residues, log_poles, iir_state):
    """Restatement of HyenaInferenceEngine.step_iir (engine.py:451-467).

    x2, x1, v: [B, D]; log_poles [G, S, 1], residues [G, S] with G == D or 1
    (broadcast); iir_state [B, D, S].  Complex parameters give a complex y;
    callers take its real part.
    """
    x1v = x1 * v
    p = torch.exp(log_poles)[..., 0][None]
    r = residues[None]
    iir_state = p * iir_state + x1v[..., None]
    res = torch.sum(r * iir_state, dim=-1)
    y = x2 * (res + D * x1v)
    return y, iir_state


# --------------------------------------------------------------------------
# two-pass chunked Toeplitz form  (vortex/ops/hyena_se/utils.py, ref_fwd.py)
# --------------------------------------------------------------------------

def toeplitz(hf, size):
    """T[g, i, j] = hf[g, i-j] for 0 <= i-j < K, else 0  (hyena_se/utils.py:5-25)."""
    g, K = hf.shape
    i = torch.arange(size)[:, None]
    j = torch.arange(size)[None, :]
    lag = i - j
    ok = (lag >= 0) & (lag < K)
    T = torch.zeros(g, size, size, dtype=hf.dtype)
    T[:, ok] = hf[:, lag[ok]]
    return T


def correction_toeplitz(hf, size):
    """T^[g, i, j] = hf[g, i+size-j] for j >= i and i+size-j < K  (utils.py:38-51)."""
    g, K = hf.shape
    i = torch.arange(size)[:, None]
    j = torch.arange(size)[None, :]
    lag = i + size - j
    ok = (j >= i) & (lag < K)
    T = torch.zeros(g, size, size, dtype=hf.dtype)
    T[:, ok] = hf[:, lag[ok]]
    return T


def gcg_fwd_ref(x, B, C, h):
    """Gate-conv-gate reference in the (b, l, g, dg) layout, input dtype throughout.

    vortex/ops/hyena_se/ref_fwd.py:80-127: Bx = B*x; depthwise conv1d with
    h.repeat_interleave(dg), padding K-1, first L outputs; C * y.
    """
    bs, l, g, dg = x.shape
    K = h.shape[-1]
    Bx = (B * x).permute(0, 2, 3, 1).reshape(bs, g * dg, l)
    w = h.repeat_interleave(dg, dim=0)
    y = F.conv1d(Bx, w, groups=g * dg, stride=1, padding=K - 1)[..., :l]
    y = y.reshape(bs, g, dg, l).permute(0, 3, 1, 2)
    return C * y


def gcg_two_pass_chunked(x, B, C, h, chunk):
    """Two-pass chunked Toeplitz algorithm (ref_fwd.py:216-266).

    Per chunk c: y_c = T @ Bx_c + T^ @ Bx_{c-1} with T, T^ built from the
    flipped filter; out = C * y.
    """
    b, l, g, dg = x.shape
    n = l // chunk
    hf = h.flip(-1)[:, 0]
    Bx = (B * x).reshape(b, n, chunk, g, dg).permute(0, 1, 3, 2, 4)   # b n g chunk dg
    T = toeplitz(hf, chunk).to(x.dtype)
    Th = correction_toeplitz(hf, chunk).to(x.dtype)
    y = torch.matmul(T, Bx)
    prev = torch.roll(Bx, 1, dims=1)
    prev[:, 0] = 0
    y = y + torch.matmul(Th, prev)
    y = y.permute(0, 1, 3, 2, 4).reshape(b, l, g, dg)
    return C * y


def causal_conv1d_ref(x, weight, bias=None, apply_gated_bias=False):
    """vortex/ops/hyena_se/interface.py:207-244 with activation=None.

    x [B, D, L], weight [D, K]; computed in weight.dtype, cast back to x.dtype.
    """
    dt = x.dtype
    x = x.to(weight.dtype)
    L = x.shape[-1]
    Dch, K = weight.shape
    gb = None
    if apply_gated_bias:
        gb, bias = bias, None
    out = F.conv1d(x, weight.unsqueeze(1), bias, padding=K - 1, groups=Dch)[..., :L]
    if apply_gated_bias:
        out = out + x * gb
    return out.to(dt)


def reshape_inputs(x, k, q, num_groups, input_layout):
    """vortex/ops/hyena_se/interface.py:272-319 for inner_layout == "bdl" (the only inner layout the
    reference's inner_hyena_se_ref accepts, interface.py:370): to [B, D, L], channel d = g*dg + j."""
    def one(t):
        if input_layout == "bdl":
            return t
        if input_layout == "blgdg":                       # rearrange "b l g dg -> b (g dg) l"
            b, l, g, dg = t.shape
            assert g == num_groups, "number of groups in feature groups and filter must match"
            return t.permute(0, 2, 3, 1).reshape(b, g * dg, l)
        if input_layout == "bgdgl":                       # rearrange "b g d l -> b (g d) l"
            b, g, dg, l = t.shape
            assert g == num_groups, "number of groups in feature groups and filter must match"
            return t.reshape(b, g * dg, l)
        raise NotImplementedError("input_layout must be bdl, blgdg or bgdgl")
    return one(x), one(k), one(q)


def reshape_outputs(y, num_groups, output_layout):
    """vortex/ops/hyena_se/interface.py:322-339 for inner_layout == "bdl"."""
    b, d, l = y.shape
    if output_layout == "bdl":
        return y
    if output_layout == "bld":
        return y.permute(0, 2, 1)
    if output_layout == "blgdg":                          # rearrange "b (g dg) l -> b l g dg"
        return y.reshape(b, num_groups, d // num_groups, l).permute(0, 3, 1, 2)
    raise NotImplementedError("output_layout must be bld, bdl or blgdg")


def inner_hyena_se_ref(x, k, q, h, bias=None, input_layout="bdl", output_layout="bdl", apply_gated_bias=False,
                       kernel_path="unfused_gcg_fast"):
    """vortex/ops/hyena_se/interface.py:342-397: y = q * causal_conv1d(k * x) with h (g, 1, K).

    Filters are assigned to channels with `h.squeeze(1).repeat(d // g, 1)` (interface.py:375-376): channel c
    uses filter c % g -- striped, unlike the repeat_interleave (blocked) map of the model path and of
    gcg_fwd_ref.  With g == d the reference leaves h as [d, 1, K], which its own causal_conv1d_ref cannot
    unpack (`dim, width = weight.shape`, interface.py:231); the squeeze is the evident intent and is done here.
    The K <= 4 shortcut of kernel_path "unfused_gcg_fast" (interface.py:380-381) calls the causal_conv1d CUDA
    extension, which is not part of this oracle: it accumulates conv + bias in float32 and rounds once
    (vortex/ops/conv/csrc/causal_conv1d_fwd.cu:108-120), i.e. causal_conv1d_ref with float32 weights, which is
    what runs here for it.  It takes no gated bias.
    """
    num_groups = h.shape[0]
    x, k, q = reshape_inputs(x, k, q, num_groups, input_layout)
    assert k.shape == q.shape == x.shape, "feature groups must have the same shape"
    b, d, l = x.shape
    h = h.squeeze(1)
    if num_groups != d:
        h = h.repeat(d // num_groups, 1)
    kx = k * x
    if kernel_path == "unfused_gcg_fast" and h.shape[-1] <= 4:
        y = causal_conv1d_ref(kx, h.float(), bias=None if bias is None else bias.float())
    else:
        y = causal_conv1d_ref(kx, h, bias=bias, apply_gated_bias=apply_gated_bias)
    return reshape_outputs(q * y, num_groups, output_layout)


# --------------------------------------------------------------------------
# engine-shaped wrapper so that parity tests read like calls into the reference
# --------------------------------------------------------------------------

@dataclass
class OracleCache:
    """Counterpart of vortex/model/cache.py:31-61 (dicts keyed by layer index)."""
    fir_state_dict: dict = field(default_factory=dict)
    fir_inner_state_dict: dict = field(default_factory=dict)
    state_dict: dict = field(default_factory=dict)
    seqlen_offset: int = 0


class OracleEngine:
    """Duck-type of HyenaInferenceEngine backed by the functions above."""

    def __init__(self, layer_idx=None, hyena_flip_x1x2=False):
        self.layer_idx = layer_idx
        self.hyena_flip_x1x2 = hyena_flip_x1x2

    def parallel_fir(self, fir_fn, u, weight, bias, L, dims, groups=None, gated_bias=False,
                     column_split_hyena=False, dim_last=True, fir_length=3, gate=False,
                     inference_params=None, prefill_mode=None, padding_mask=None):
        return parallel_fir(u, weight, bias, L, dims, groups, gated_bias, column_split_hyena,
                            dim_last, fir_length, gate, inference_params is not None,
                            padding_mask, self.hyena_flip_x1x2)

    def parallel_iir(self, z_pre, h, D, L, poles, residues, t, dims, layer_idx,
                     inference_params=None, prefill_style="fft", fftconv_fn=None,
                     padding_mask=None, use_flashfft=False, column_split_hyena=False,
                     long_fir_threshold=None):
        y, state = parallel_iir(z_pre, h, D, L, poles, residues, dims, column_split_hyena,
                                self.hyena_flip_x1x2, inference_params is not None,
                                keep_complex_state=poles.is_complex(), long_fir_threshold=long_fir_threshold)
        if inference_params is not None:
            inference_params.state_dict[layer_idx] = state
        return y

    def step_fir(self, u, fir_state, weight, bias=None, gated_bias=False, flip_filter=False):
        return step_fir(u, fir_state, weight, bias, gated_bias, flip_filter)

    def step_iir(self, x2, x1, v, D, residues, poles, iir_state, iir_groups=1):
        if iir_groups > 1:
            raise NotImplementedError
        return step_iir(x2, x1, v, D, residues, poles, iir_state)


# --------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations (seeded on the CPU)
# --------------------------------------------------------------------------

def make_gates(B, D, L, seed=0, dtype=torch.bfloat16):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return tuple(torch.randn(B, D, L, generator=g).to(dtype) for _ in range(3))   # x2, x1, v


def make_se_filter(G, K=7, seed=100):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(G, 1, K, generator=g) / math.sqrt(K)


def make_mr_filter(G, K=128, seed=200):
    g = torch.Generator(device="cpu").manual_seed(seed)
    w = torch.randn(G, 1, K, generator=g) / math.sqrt(K)
    a = 0.01 + 0.09 * torch.rand(G, 1, 1, generator=g)
    return w * torch.exp(-a * torch.arange(K)[None, None])


def make_modal_complex(G, S=16, seed=300, pmin=0.9, pmax=0.9999):
    """Complex poles |p|~U(pmin,pmax), arg~U(0,pi); residues ~CN(0,1). log_poles [G,S,1] complex64."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    mag = pmin + (pmax - pmin) * torch.rand(G, S, generator=g, dtype=torch.float64)
    ang = math.pi * torch.rand(G, S, generator=g, dtype=torch.float64)
    log_poles = torch.complex(mag.log(), ang).to(torch.complex64)[..., None]
    res = torch.complex(torch.randn(G, S, generator=g), torch.randn(G, S, generator=g)) / math.sqrt(2.0)
    return log_poles, res.to(torch.complex64)


def make_modal_real(G, S=16, seed=400, pmin=0.9, pmax=0.9999):
    """Real poles in vortex's own parametrisation: log_poles [G,S,1] fp32 (<0), residues [G,S] fp32."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    mag = pmin + (pmax - pmin) * torch.rand(G, S, generator=g, dtype=torch.float64)
    return mag.log().to(torch.float32)[..., None], torch.randn(G, S, generator=g)


# --------------------------------------------------------------------------
# the operator module's call sequence  (vortex/model/model.py:214-398)
# --------------------------------------------------------------------------

class OracleCascade:
    """Restatement of HyenaCascade.forward on top of any engine with the four
    HyenaInferenceEngine methods (the oracle's or the product's), so that a parity
    test drives both through the same call sequence.

    params: dict with short_filter_weight [3D,1,Ks], short_filter_bias or None, and either
    h [G,1,K] (+ D [hidden] when K >= 128) or log_poles [G,S,1], residues [G,S], D [hidden].
    """

    def __init__(self, engine, params, hidden, n_heads, groups, layer_idx=0, fir_inner_filter_length=None,
                 column_split_hyena=False, interleave=False, state_size=16, long_fir_threshold=None,
                 hyena_flip_x1x2=None):
        self.long_fir_threshold = long_fir_threshold            # model.py:185
        # model.py:141 and :159 read the same config key into the module and into its engine
        self.hyena_flip_x1x2 = getattr(engine, "hyena_flip_x1x2", False) if hyena_flip_x1x2 is None else hyena_flip_x1x2
        self.engine, self.p = engine, params
        self.hidden, self.n_heads, self.groups = hidden, n_heads, groups
        self.layer_idx, self.K = layer_idx, fir_inner_filter_length
        self.column_split_hyena, self.interleave, self.state_size = column_split_hyena, interleave, state_size
        self.Ks = params["short_filter_weight"].shape[-1]

    def forward(self, u, inference_params=None, padding_mask=None):
        # model.py:214-219
        if inference_params is not None and self.layer_idx in inference_params.fir_state_dict.keys():
            return self.sequential_forward(u, inference_params)
        return self.parallel_forward(u, inference_params, padding_mask)

    def parallel_forward(self, u, inference_params=None, padding_mask=None):
        # model.py:221-316
        p, L = self.p, u.shape[1]
        dims = (self.hidden, self.n_heads, self.hidden // self.n_heads, self.state_size, self.groups)
        z_pre, fir_state = self.engine.parallel_fir(
            F.conv1d, u, p["short_filter_weight"], p.get("short_filter_bias"), L, dims=dims, gate=False,
            column_split_hyena=self.column_split_hyena, fir_length=self.Ks, inference_params=inference_params,
            padding_mask=padding_mask, dim_last=True)
        if inference_params:
            inference_params.fir_state_dict[self.layer_idx] = fir_state
        if self.interleave:
            z_pre = interleave(z_pre)
        if self.K is None:
            h = modal_filter(p["log_poles"].to(u.device), p["residues"].to(u.device), L)     # model.py:390-398
            h = h.to(u.device)
        else:
            h = p["h"]
        if self.groups > 1:
            h = h.repeat_interleave(self.hidden // self.groups, 0)                          # model.py:261-262
        if self.K is not None:
            y, inner = self.engine.parallel_fir(
                F.conv1d, z_pre, h, p.get("D"), L, dims=dims, gate=True, gated_bias=self.K >= 128, dim_last=False,
                column_split_hyena=self.column_split_hyena, fir_length=self.K, inference_params=inference_params,
                padding_mask=padding_mask, groups=self.groups)
            y = y.permute(0, 2, 1)
            if inference_params:
                inference_params.fir_inner_state_dict[self.layer_idx] = inner
        else:
            y = self.engine.parallel_iir(
                z_pre, h, p["D"], L, t=None, poles=p["log_poles"], residues=p["residues"], dims=dims,
                inference_params=inference_params, layer_idx=self.layer_idx, prefill_style="fft",
                use_flashfft=False, fftconv_fn=None, column_split_hyena=self.column_split_hyena,
                long_fir_threshold=self.long_fir_threshold, padding_mask=padding_mask)
        return y, inference_params

    def sequential_forward(self, u, inference_params):
        # model.py:318-375
        p = self.p
        if u.dim() > 2:
            u = u[:, -1]
        z_pre, fir_state = self.engine.step_fir(u, inference_params.fir_state_dict[self.layer_idx],
                                                weight=p["short_filter_weight"], bias=p.get("short_filter_bias"))
        inference_params.fir_state_dict[self.layer_idx] = fir_state
        if self.interleave:
            z_pre = interleave(z_pre)
        hd = self.hidden // self.n_heads
        x2, x1, v = (column_split(z_pre, self.n_heads, hd) if self.column_split_hyena
                     else z_pre.split([self.hidden] * 3, dim=1))
        if self.hyena_flip_x1x2:                                                            # model.py:342-343
            x1, x2 = x2, x1
        if self.K is not None:
            h = p["h"].repeat_interleave(self.hidden // self.groups, 0) if self.groups > 1 else p["h"]
            y, inner = self.engine.step_fir(x1 * v, inference_params.fir_inner_state_dict[self.layer_idx], weight=h,
                                            bias=p.get("D"), flip_filter=self.K >= 128, gated_bias=self.K >= 128)
            y = y * x2
            inference_params.fir_inner_state_dict[self.layer_idx] = inner
        else:
            y, st = self.engine.step_iir(x2, x1, v, p["D"], p["residues"], p["log_poles"],
                                         inference_params.state_dict[self.layer_idx], iir_groups=1)
            inference_params.state_dict[self.layer_idx] = st
            if y.is_complex():          # complex poles (not in vortex, where parameters are real): keep Re
                y = y.real
        y = y.to(dtype=u.dtype)
        return y[:, None], inference_params
