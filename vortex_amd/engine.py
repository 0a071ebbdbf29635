"""Drop-in replacement for vortex's HyenaInferenceEngine, backed by the gfx950 kernels.

Same four methods, argument names and return conventions as
vortex/model/engine.py:112-467, so that `block.filter.engine = HyenaInferenceEngine(...)`
switches a vortex HyenaCascade to the HIP path with no other source change.
Everything here runs on the GPU through the C ABI; there is no PyTorch fallback
for the convolutions, and CPU tensors are rejected.
"""
import weakref

import torch

from . import ops
from ._lib import HYENA_BIAS_ADD, HYENA_BIAS_GATED_BF16, HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE

IIR_PREFILL_MODES = ["recurrence", "modal-fft", "hybrid-modal-recurrence", "modal-scan", "canonical-fft",
                     "iir-fir-caching"]


_GROUPED_OK = {}     # id(weight) -> (weakref, version, groups, verdict): the row-equality check runs once per parameter version


def _rows_constant_in_groups(weight, w, D, groups):
    """Whether a [D, K] tap table repeats each row D/groups times (what repeat_interleave of a [G, 1, K] filter bank
    gives, vortex/model/model.py:261-262).  One device reduction and host read per parameter version, cached."""
    hit = _GROUPED_OK.get(id(weight))
    if hit is not None and hit[0]() is weight and hit[1] == weight._version and hit[2] == groups:
        return hit[3]
    ok = bool((w.reshape(groups, D // groups, -1) == w.reshape(groups, D // groups, -1)[:, :1]).all())
    if len(_GROUPED_OK) > 256:
        _GROUPED_OK.clear()
    _GROUPED_OK[id(weight)] = (weakref.ref(weight), weight._version, groups, ok)
    return ok


def _group_taps(weight, D, groups):
    """[D, 1, K] or [G, 1, K] -> [G', K] float32 taps for the kernels.

    vortex hands the engine a [G, 1, K] filter bank expanded with repeat_interleave to [D, 1, K] together with
    `groups` (vortex/model/model.py:261-286); its own conv1d ignores `groups` and filters per channel
    (vortex/model/engine.py:203).  The expanded table is folded back to [G, K] only when its rows really are
    constant inside each group (checked once per parameter version); distinct per-channel rows run per channel."""
    w = weight.detach().reshape(weight.shape[0], -1)
    rows = w.shape[0]
    if groups is not None and rows == D and groups < D and D % groups == 0 and _rows_constant_in_groups(weight, w, D, groups):
        w = w[:: D // groups]
    return w.to(torch.float32).contiguous()


def _same_tensor(hit, t):
    """Cache guard: the cached entry was built from this very tensor object at this version."""
    return hit is not None and hit[0]() is t and hit[1] == t._version


class HyenaInferenceEngine:
    def __init__(self, fir_fn=None, iir_prefill_style="modal-fft", layer_idx=None,
                 ground_truth_activations_path=None, print_activations=False, hyena_flip_x1x2=False) -> None:
        self.fir_fn = fir_fn
        assert iir_prefill_style in IIR_PREFILL_MODES, f"iir_prefill_style must be one of {IIR_PREFILL_MODES}"
        self.iir_prefill_style = iir_prefill_style
        self.layer_idx = layer_idx
        self.low_mem_mode = False
        self.ground_truth_activations_path = ground_truth_activations_path
        self.print_activations = print_activations
        self.hyena_flip_x1x2 = hyena_flip_x1x2
        self._plan_hit = None        # (weakref poles, version, weakref residues, version, kind, ModalPlan)
        self._poles_hit = None       # (weakref log-poles, version, exponentiated poles)

    # ------------------------------------------------------------------ prefill FIR
    def parallel_fir(self, fir_fn, u, weight, bias, L, dims, groups=None, gated_bias=False,
                     column_split_hyena=False, dim_last=True, fir_length=3, gate=False,
                     inference_params=None, prefill_mode=None, padding_mask=None):
        """vortex/model/engine.py:131-260.  Returns (z [B, D, L], fir_state or None)."""
        if fir_fn is not None and fir_fn is not torch.nn.functional.conv1d:
            raise NotImplementedError("custom fir_fn callables (deprecated in vortex) are not supported")
        if u.dtype != torch.bfloat16:
            raise TypeError(f"the gfx950 Hyena kernels take bfloat16 activations, got {u.dtype}")
        K = fir_length
        if gate:
            hidden, n_heads, head_dim = dims[0], dims[1], dims[2]
            if dim_last:
                raise NotImplementedError("gated FIR expects the [B, 3D, L] layout (dim_last=False)")
            B, _, L = u.shape
            hd = head_dim if column_split_hyena else None
            up, pad = ops.front_pad8(u)                 # a copy only for lengths / strides the kernels cannot take
            L += pad
            r2, r1, rv = (ops.rows_of_projection(up, hidden, i, hd) for i in range(3))
            if self.hyena_flip_x1x2:
                r1, r2 = r2, r1
            D = hidden
            taps = _group_taps(weight, D, groups)
            if taps.shape[1] > 128:
                # longer than any MFMA kernel is built for: the direct-form kernel on the gates as tensors, with the
                # arithmetic of the K >= 128 branch (engine.py:174-187: true convolution, fp32 `+ D*u`) or of the
                # short branch (cross-correlation, bias after the cast) by K, as below
                z2, x1t, vt = self._gate_views(u, hidden, hd)
                if K >= 128:
                    mode = HYENA_BIAS_NONE if bias is None else HYENA_BIAS_GATED_FP32
                    z = ops.fir_fwd_long(x1t, z2, vt, taps[:, :L], bias=ops._f32(bias), bias_mode=mode)
                else:
                    mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_BF16 if gated_bias else HYENA_BIAS_ADD)
                    z = ops.fir_fwd_long(x1t, z2, vt, taps, bias=ops._f32(bias), bias_mode=mode, taps_reversed=True)
                state = (x1t[..., -(K - 1):] * vt[..., -(K - 1):]) if inference_params is not None else None
                if isinstance(padding_mask, torch.Tensor):
                    z = z * padding_mask[:, None].to(z.dtype)
                return z, state
            if K >= 128:
                # true convolution with the fp32 `+ D*u` term (engine.py:174-187, :78)
                mode = HYENA_BIAS_NONE if bias is None else HYENA_BIAS_GATED_FP32
                z = ops.fir_fwd_rows(r1, r2, rv, taps, B, D, L, taps.shape[1], device=u.device,
                                     bias=ops._f32(bias), bias_mode=mode, taps_reversed=False, force_mfma=True)
            else:
                if bias is not None and bias.dtype != torch.bfloat16:
                    raise NotImplementedError("a float32 bias promotes the short-FIR output to float32 in vortex; "
                                              "only bfloat16 (or no) bias is supported")
                # after the cast of the convolution: z + bias*u or z + bias in bf16 tensor arithmetic (engine.py:218-223)
                mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_BF16 if gated_bias else HYENA_BIAS_ADD)
                z = ops.fir_fwd_rows(r1, r2, rv, taps, B, D, L, taps.shape[1], device=u.device,
                                     bias=ops._f32(bias), bias_mode=mode, taps_reversed=True)
            if pad:
                z = z[..., pad:]
            state = None
            if inference_params is not None:
                x1, v = self._gate_tails(u, hidden, hd, K - 1)
                state = x1 * v
        else:
            if bias is not None and bias.dtype != torch.bfloat16:
                raise NotImplementedError("a float32 short-filter bias promotes the output to float32 in vortex; "
                                          "only bfloat16 (or no) bias is supported")
            if dim_last:
                B, L, C = u.shape
                taps = _group_taps(weight, C, groups)
                pad = (-L) % 8
                z = ops.featurizer_fwd(u, taps, bias, front_pad=pad)       # [B, C, L + pad], fused transpose
                if pad:
                    z = z[..., pad:]
                ut = u.permute(0, 2, 1)
            else:
                B, C, L = u.shape
                taps = _group_taps(weight, C, groups)
                mode = HYENA_BIAS_NONE if bias is None else HYENA_BIAS_ADD
                up, pad = ops.front_pad8(u)
                z = ops.fir_fwd_rows(ops.rows_of(up), None, None, taps, B, C, L + pad, taps.shape[1], device=u.device,
                                     bias=ops._f32(bias), bias_mode=mode, taps_reversed=True)
                if pad:
                    z = z[..., pad:]
                ut = u
            state = ut[..., -K + 1:] if inference_params is not None else None
        if isinstance(padding_mask, torch.Tensor):
            z = z * padding_mask[:, None].to(z.dtype)      # 0/1 masks commute exactly with the gate
        return z, state

    def _gate_views(self, u, hidden, head_dim):
        """(x2, x1, v) views of the [B, 3D, L] projection (vortex/model/engine.py:150-158), flip applied."""
        if head_dim is None:
            x2, x1, v = u.split([hidden, hidden, hidden], dim=1)
        else:
            ur = u.reshape(u.shape[0], -1, 3, head_dim, u.shape[-1])
            x2, x1, v = (ur[:, :, i].reshape(u.shape[0], hidden, u.shape[-1]) for i in range(3))
        if self.hyena_flip_x1x2:
            x1, x2 = x2, x1
        return x2, x1, v

    def _gate_tails(self, u, hidden, head_dim, n):
        t = u[..., -n:]
        if head_dim is None:
            x2, x1, v = t.split([hidden, hidden, hidden], dim=1)
        else:
            tr = t.reshape(t.shape[0], -1, 3, head_dim, t.shape[-1])
            x2, x1, v = (tr[:, :, i].reshape(t.shape[0], hidden, t.shape[-1]) for i in range(3))
        if self.hyena_flip_x1x2:
            x1, x2 = x2, x1
        return x1, v

    # ------------------------------------------------------------------ prefill IIR
    def _plan(self, poles, residues, kind="log", build=None):
        """ModalPlan of (poles, residues), rebuilt when either tensor object or its version changes.  Keyed on the
        objects themselves (weak references), not on addresses, which the allocator reuses."""
        h = self._plan_hit
        if h is not None and h[0]() is poles and h[1] == poles._version and h[2]() is residues \
                and h[3] == residues._version and h[4] == kind:
            return h[5]
        plan = build() if build is not None else ops.ModalPlan(poles, residues)
        self._plan_hit = (weakref.ref(poles), poles._version, weakref.ref(residues), residues._version, kind, plan)
        return plan

    def parallel_iir(self, z_pre, h, D, L, poles, residues, t, dims, layer_idx, inference_params=None,
                     prefill_style="fft", fftconv_fn=None, padding_mask=None, use_flashfft=False,
                     column_split_hyena=False, long_fir_threshold=None):
        """vortex/model/engine.py:262-404.  `h` (the materialised filter) is not read: the kernel works
        from `poles` (log-poles) and `residues` directly.  Returns y [B, L, D]; writes the modal state
        into inference_params.state_dict[layer_idx].  With long_fir_threshold (engine.py:339-349) the first
        `threshold` samples of `h`, rounded to bf16, run as a per-channel FIR in the orientation F.conv1d gives
        them there (h[threshold-1] on the current sample); up to 128 taps, and, as in the reference, without a
        cache to prefill."""
        if z_pre.dtype != torch.bfloat16:
            raise TypeError(f"the gfx950 Hyena kernels take bfloat16 activations, got {z_pre.dtype}")
        hidden, n_heads, head_dim = dims[0], dims[1], dims[2]
        B, _, L = z_pre.shape
        hd = head_dim if column_split_hyena else None
        zp, pad = ops.front_pad8(z_pre)
        r2, r1, rv = (ops.rows_of_projection(zp, hidden, i, hd) for i in range(3))
        if self.hyena_flip_x1x2:
            r1, r2 = r2, r1
        if long_fir_threshold is not None:
            if inference_params is not None:
                raise NotImplementedError("long_fir_threshold with a cache: the reference has no state prefill on "
                                          "this branch (vortex/model/engine.py:380-392 reads an unassigned X_s)")
            T = min(int(long_fir_threshold), h.shape[-1])
            assert h.shape[0] == 1, "batch size must be 1 for long_fir_threshold"
            taps = h[0][:, :T].to(torch.bfloat16).to(torch.float32).contiguous()       # [D, T], bf16-rounded
            # (bf16(y) + x1v*D) in the tensors' own dtype (engine.py:351-353): bf16 arithmetic with a bf16 D
            mode = HYENA_BIAS_GATED_BF16 if D.dtype == torch.bfloat16 else HYENA_BIAS_GATED_FP32
            if T > 128:     # beyond the MFMA kernel's filter length: direct form on the gates as tensors
                x2t, x1t, vt = self._gate_views(z_pre, hidden, hd)
                out = ops.fir_fwd_long(x1t, x2t, vt, taps, bias=ops._f32(D), bias_mode=mode, taps_reversed=True)
                return out.permute(0, 2, 1)
            out = ops.fir_fwd_rows(r1, r2, rv, taps, B, hidden, L + pad, T, device=z_pre.device, bias=ops._f32(D),
                                   bias_mode=mode, taps_reversed=True, force_mfma=True)
            if pad:
                out = out[..., pad:]
            return out.permute(0, 2, 1)
        want_state = inference_params is not None
        if want_state and prefill_style == "recurrence":
            return self._prefill_recurrence(r1, r2, rv, D, poles, residues, B, hidden, L, pad, z_pre.device,
                                            inference_params, layer_idx)
        if want_state and prefill_style != "fft":
            raise NotImplementedError(f"prefill_style {prefill_style!r}")          # engine.py:395-396
        plan = self._plan(poles, residues)
        out, _, state = ops.li_fwd_rows(r1, r2, rv, plan, D, B, hidden, L + pad, device=z_pre.device,
                                        want_state=want_state)
        if want_state:
            inference_params.state_dict[layer_idx] = state
        if pad:
            out = out[..., pad:]
        return out.permute(0, 2, 1)

    def _prefill_recurrence(self, r1, r2, rv, D, poles, residues, B, hidden, L, pad, device, inference_params,
                            layer_idx):
        """prefill_style == "recurrence" (vortex/model/engine.py:314-321, :473-504).  On this branch the reference
        takes the poles themselves (not their logarithms) and the residues as [D, S, 1, 2] tensors of (re, im)
        lanes, one filter per channel, and leaves the state as [B, D, S, 2] float32.  The same chunked scan runs it:
        the recurrence s_t = p s_{t-1} + u_t is what the kernel evaluates anyway.  Deviations, all on the side of
        the mathematics: the state is carried in float32 (the reference's `0 * x1v_` makes it bf16 and rounds it
        every step), the complex product is the true one (the reference's in-place lane update feeds the new real
        lane into the imaginary one), and y = sum_s r_re * s_re as the reference forms it (its `[..., 0]` of the
        lane-wise product drops r_im * s_im).  With real poles -- the only kind vortex's own parameters give --
        these coincide with the FFT prefill."""
        if poles.dim() != 4 or poles.shape[-1] != 2 or residues.shape != poles.shape or poles.shape[0] != hidden:
            raise ValueError("prefill_style='recurrence' takes poles and residues of shape [D, state, 1, 2] (re, im)")
        def build():
            p = torch.view_as_complex(poles.detach()[:, :, 0].to(torch.float32).contiguous())        # [D, S]
            # log p; a pole of exactly zero gets e^-100, which is zero in float32 from the first power on
            logp = torch.complex(p.abs().clamp_min(1e-43).log().clamp_min(-100.0), torch.angle(p))
            res = torch.complex(residues.detach()[:, :, 0, 0].to(torch.float32), torch.zeros_like(p.real))
            return ops.ModalPlan(logp, res)

        plan = self._plan(poles, residues, "rec", build)
        out, _, state = ops.li_fwd_rows(r1, r2, rv, plan, D, B, hidden, L + pad, device=device, want_state=True)
        inference_params.state_dict[layer_idx] = torch.view_as_real(state).contiguous()               # [B, D, S, 2]
        if pad:
            out = out[..., pad:]
        return out.permute(0, 2, 1)

    # ------------------------------------------------------------------ decode
    def step_fir(self, u, fir_state, weight, bias=None, gated_bias=False, flip_filter=False):
        """vortex/model/engine.py:406-449.  `fir_state` is the reference's [B, D, cache] tensor
        (oldest first) on the first call and the FirRing this method returned afterwards."""
        w = weight.detach().reshape(weight.shape[0], -1).to(torch.float32)
        K = w.shape[-1]
        if not isinstance(fir_state, ops.FirRing):
            fir_state = ops.FirRing.from_reference(fir_state)
        cache = fir_state.shape[-1]
        taps = (w.flip(-1)[..., -cache - 1:] if flip_filter else w[..., : cache + 1]).contiguous()
        if cache < K - 1:
            # short prompt: vortex grows the cache by one sample per step (engine.py:443-444)
            if cache == 0:
                raise NotImplementedError("decode from an empty FIR cache is not supported")
            ref = fir_state.reference_order(torch.bfloat16)
            y = ops.fir_step(u, fir_state, taps, bias=bias, gated_bias=gated_bias)
            return y, ops.FirRing.from_reference(torch.cat([ref, u[..., None].to(ref.dtype)], dim=-1))
        y = ops.fir_step(u, fir_state, taps, bias=bias, gated_bias=gated_bias)
        return y, fir_state

    def step_iir(self, x2, x1, v, D, residues, poles, iir_state, iir_groups=1):
        """vortex/model/engine.py:451-467.  The state is updated in place and returned; y is float32
        as torch promotion makes it in the reference."""
        if iir_groups > 1:
            raise NotImplementedError
        if _same_tensor(self._poles_hit, poles):
            p = self._poles_hit[2]
        else:
            p = torch.exp(poles.detach())[..., 0].contiguous()
            self._poles_hit = (weakref.ref(poles), poles._version, p)
        if not iir_state.is_contiguous():
            iir_state = iir_state.contiguous()
        y = ops.iir_step(x1, x2, v, iir_state, p, residues.detach(), D, out_dtype=torch.float32)
        return y, iir_state
