"""The Hyena operator module on the gfx950 kernels: counterpart of vortex's HyenaCascade.

Reproduces the call sequence of vortex/model/model.py:125-398 (featurizer FIR ->
interleave -> split -> inner operator; prefill when the layer has no cached state,
one-token decode afterwards) but hands the kernels what they want directly: grouped
filters without repeat_interleave, modal parameters without a materialised filter,
ring-buffer FIR caches, and the modal state emitted by the prefill kernel itself.
Cache containers mirror vortex/model/cache.py:31-61.
"""
from dataclasses import dataclass, field

import torch
import torch.nn as nn

from . import ops
from ._lib import HYENA_BIAS_ADD, HYENA_BIAS_GATED_BF16, HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE


@dataclass
class HyenaCascadeIIRInferenceParams:
    """vortex/model/cache.py:31-44."""
    fir_filter_length: int = 3
    state_dim: int = 16
    seqlen_offset: int = 0
    fir_state_dict: dict = field(default_factory=dict)
    state_dict: dict = field(default_factory=dict)

    def reset(self):
        self.fir_filter_length, self.state_dim, self.seqlen_offset = 3, 16, 0


@dataclass
class HyenaCascadeFIRInferenceParams:
    """vortex/model/cache.py:47-61."""
    fir_filter_length: int = 3
    fir_inner_filter_length: int = 4
    seqlen_offset: int = 0
    fir_inner_state_dict: dict = field(default_factory=dict)
    fir_state_dict: dict = field(default_factory=dict)
    state_dict: dict = field(default_factory=dict)

    def reset(self):
        self.fir_filter_length, self.fir_inner_filter_length, self.seqlen_offset = 3, 4, 0


def _ring(tail, depth, flipped=False):
    """FirRing of `depth` slots from the channel-last tail [B, n <= depth, C] of a prompt.

    A prompt shorter than the filter leaves the oldest slots zero and records how many are real (`valid`).
    With the flipped (Hyena-MR) tap slicing of vortex/model/engine.py:421-422 the reference's growing cache is
    exactly this zero history.  With the plain slicing (:424-425) it is not: the reference then puts tap
    `cache` on the new sample; _grown_taps reproduces that while the cache fills up."""
    n = tail.shape[1]
    if n < depth:
        tail = torch.cat([tail.new_zeros(tail.shape[0], depth - n, tail.shape[2]), tail], dim=1)
    ring = ops.FirRing(tail.contiguous(), 0)
    ring.valid = depth if flipped else n
    return ring


def _grown_taps(w, valid):
    """Taps [G, R+1] (oldest first) the reference applies to a cache holding `valid` < R samples with the plain
    slicing weight[..., :valid+1] (vortex/model/engine.py:424-425): tap i on the i-th oldest real sample, tap
    `valid` on the new one.  Laid out for a full-depth ring whose R - valid oldest slots are zero."""
    R = w.shape[1] - 1
    t = torch.zeros_like(w)
    t[:, R - valid:R] = w[:, :valid]
    t[:, R] = w[:, valid]
    return t


def _cfg(config, key, default=None):
    v = config.get(key, default) if hasattr(config, "get") else getattr(config, key, default)
    return default if v is None else v


def project_sequence_major(weight, x):
    """The dense projection x [B, L, H] -> [B, L, C] with weight [C, H] (no bias), computed as W x^T so that the GEMM
    writes [B, C, L] with the samples contiguous; returned as the [B, L, C] view of that memory.  Same values as
    F.linear(x, weight) up to the GEMM's own summation order.  One plain 2-D product per batch element (torch.matmul
    on the broadcast pair measured twice as slow)."""
    B, L, _ = x.shape
    weight, x = weight.detach(), x.detach()         # forward only: the products are written in place
    p = torch.empty(B, weight.shape[0], L, dtype=x.dtype, device=x.device)
    for b in range(B):
        torch.mm(weight, x[b].t(), out=p[b])
    return p.transpose(1, 2)


class SequenceMajorProjection(nn.Module):
    """Stands in for the `projections` linear layer of a Hyena block (vortex/model/model.py:487-490 calls it on the
    normalised input): the same projection, stored sequence-major for prefills, so that a Hyena-LI cascade behind it
    runs featurizer, gates and scan in one launch.  Decode tokens, prompts that are not a whole number of 8-sample
    pieces, biased layers and anything that is not a plain linear layer on the GPU go through the wrapped layer
    unchanged.  The wrapped layer keeps its parameters (and their names under `.linear`)."""

    def __init__(self, linear):
        super().__init__()
        self.linear = linear

    @property
    def weight(self):
        return self.linear.weight

    @property
    def bias(self):
        return getattr(self.linear, "bias", None)

    def forward(self, x):
        lin = self.linear
        if (isinstance(lin, nn.Linear) and lin.bias is None and x.dim() == 3 and x.is_cuda and x.shape[1] > 1
                and x.shape[1] % 8 == 0 and x.dtype == lin.weight.dtype):
            return project_sequence_major(lin.weight, x)
        return lin(x)


def use_hip_filters(model, sequence_major_projections=False):
    """Replaces the `filter` of every Hyena block of a vortex model (an object with `.blocks`, each Hyena block
    holding its HyenaCascade as `.filter`, vortex/model/model.py:523-575) by its counterpart on the HIP kernels.
    sequence_major_projections=True also wraps the `projections` layer of the Hyena-LI blocks in a
    SequenceMajorProjection, so that their prefill runs in one launch.  Returns the number of blocks switched."""
    n = 0
    for block in model.blocks:
        f = getattr(block, "filter", None)
        if f is not None and hasattr(f, "short_filter_weight") and not isinstance(f, HyenaCascade):
            block.filter = HyenaCascade.from_vortex(f)
            n += 1
        f = getattr(block, "filter", None)
        proj = getattr(block, "projections", None)
        if (sequence_major_projections and isinstance(f, HyenaCascade) and f._can_fuse_gates_layer()
                and isinstance(proj, nn.Linear) and proj.bias is None):
            block.projections = SequenceMajorProjection(proj)
    return n


class HyenaCascade(nn.Module):
    """Parameters and forward of one Hyena operator (SE / MR when fir_inner_filter_length is set, LI otherwise).

    Parameter names and shapes follow vortex/model/model.py:152-210 so that vortex state
    dicts load: short_filter_weight [3D, 1, Ks], short_filter_bias [3D] (optional),
    h [G, 1, K] + D [hidden] (MR only) for FIR layers, log_poles [G, S, 1] + residues [G, S] + D
    for modal layers.  log_poles / residues may be complex64.
    """

    def __init__(self, config, layer_idx, hyena_filter_groups=None, fir_inner_filter_length=None,
                 complex_modal=False):
        super().__init__()
        self.config, self.layer_idx = config, layer_idx
        self.hidden_size = config["hidden_size"] if isinstance(config, dict) else config.hidden_size
        D = self.hidden_size
        self.hyena_filter_groups = hyena_filter_groups or D
        self.state_size = _cfg(config, "state_size", 16)
        self.num_attention_heads = _cfg(config, "num_attention_heads", 1)
        self.hidden_size_per_attention_head = D // self.num_attention_heads
        self.column_split_hyena = _cfg(config, "column_split_hyena", True)
        self.hyena_flip_x1x2 = _cfg(config, "hyena_flip_x1x2", False)
        self.interleave = _cfg(config, "interleave", False)
        self.short_filter_length = _cfg(config, "short_filter_length", 3)
        self.long_fir_threshold = _cfg(config, "long_fir_threshold", None)      # vortex/model/model.py:185
        self.fir_inner_filter_length = fir_inner_filter_length
        self.short_filter_weight = nn.Parameter(torch.randn(3 * D, 1, self.short_filter_length))
        self.short_filter_bias = nn.Parameter(torch.randn(3 * D)) if _cfg(config, "short_filter_bias", False) else None
        G = self.hyena_filter_groups
        if fir_inner_filter_length:
            self.h = nn.Parameter(torch.randn(G, 1, fir_inner_filter_length))
            self.D = nn.Parameter(torch.zeros(D)) if fir_inner_filter_length >= 128 else None
        else:
            dt = torch.complex64 if complex_modal else torch.float32
            self.log_poles = nn.Parameter(torch.randn(G, self.state_size, 1, dtype=dt))
            self.residues = nn.Parameter(torch.randn(G, self.state_size, dtype=dt))
            self.D = nn.Parameter(torch.zeros(D))
            self.h = None
        self.t = None
        self._plan = None
        self._decode = None
        self.fuse_decode = True        # one launch per decode step where the fused layer-step kernels apply
        # decode, opt-in: the modal state is read and written once per four tokens (ops.IirStepper windowed);
        # inference_params.state_dict then lags the tokens by up to four inputs until flush_decode_state().
        # Off by default: the reference leaves the state current after every token (vortex/model/model.py:362-372)
        self.window_decode_state = False
        self.fuse_prefill = True       # one launch per SE / MR prefill where the fused layer kernel applies
        self._f32_cache = {}

    @classmethod
    def from_vortex(cls, ref):
        """A module on the HIP kernels with the configuration and the parameters (shared storage, not copied) of a
        vortex HyenaCascade instance (vortex/model/model.py:125-210)."""
        complex_modal = getattr(ref, "log_poles", None) is not None and ref.log_poles.is_complex()
        new = cls(ref.config, ref.layer_idx, hyena_filter_groups=ref.hyena_filter_groups,
                  fir_inner_filter_length=ref.fir_inner_filter_length, complex_modal=complex_modal)
        for name in ("short_filter_weight", "short_filter_bias", "h", "D", "log_poles", "residues"):
            p = getattr(ref, name, None)
            if p is not None and not isinstance(p, nn.Parameter):
                p = nn.Parameter(p, requires_grad=False)
            setattr(new, name, p)
        return new

    # ------------------------------------------------------------------
    def forward(self, u, inference_params=None, padding_mask=None, *args, **kwargs):
        if inference_params is not None and self.layer_idx in inference_params.fir_state_dict.keys():
            return self.sequential_forward(u, inference_params)
        return self.parallel_forward(u, inference_params, padding_mask)

    def _rows(self, z_pre):
        D = self.hidden_size
        hd = self.hidden_size_per_attention_head if self.column_split_hyena else None
        r2, r1, rv = (ops.rows_of_projection(z_pre, D, i, hd) for i in range(3))
        if self.hyena_flip_x1x2:
            r1, r2 = r2, r1
        return r1, r2, rv

    def _split(self, z):
        """(x2, x1, v) views of a [B, 3D] or [B, 3D, R] tensor, as vortex/model/model.py:336-343."""
        D, hd = self.hidden_size, self.hidden_size_per_attention_head
        if self.column_split_hyena:
            zr = z.reshape(z.shape[0], -1, 3, hd, *z.shape[2:])
            x2, x1, v = (zr[:, :, i].reshape(z.shape[0], D, *z.shape[2:]) for i in range(3))
        else:
            x2, x1, v = z.split([D, D, D], dim=1)
        if self.hyena_flip_x1x2:
            x1, x2 = x2, x1
        return x2, x1, v

    def _f32_param(self, name, shape=None):
        """float32 contiguous copy of a (possibly bf16) parameter, rebuilt only when the parameter changes."""
        p = getattr(self, name)
        if p is None:
            return None
        key = (id(p), p.data_ptr(), p._version, p.dtype)
        hit = self._f32_cache.get(name)
        if hit is None or hit[0] != key:
            t = p.detach().to(torch.float32)
            hit = (key, (t.reshape(shape) if shape is not None else t).contiguous())
            self._f32_cache[name] = hit
        return hit[1]

    def update_time(self, L, device):
        """vortex/model/model.py:377-388: the cached time vector [1, 1, L]."""
        t = getattr(self, "t", None)
        if t is None or t.shape[-1] < L or t.device != torch.device(device):
            self.t = torch.arange(L, device=device)[None, None]
        else:
            self.t = t[..., :L]

    def compute_filter(self, L, device):
        """vortex/model/model.py:390-398: the materialised modal filter h [1, G, L] in float32 (the real part for
        complex parameters) with the float32 parameters.  The kernels never need it (they work from the poles and
        residues); it is here for callers that inspect or export the filter."""
        self.update_time(L, device)
        filter_dtype = torch.float32
        cdt = torch.complex64 if self.log_poles.is_complex() else filter_dtype
        residues, log_poles = self.residues.to(cdt), self.log_poles.to(cdt)
        h = (residues[..., None] * (log_poles * self.t).exp()).sum(1)[None]
        return (h.real if h.is_complex() else h), filter_dtype, log_poles, residues

    def modal_plan(self):
        key = (id(self.log_poles), id(self.residues), self.log_poles._version, self.residues._version,
               self.log_poles.data_ptr(), self.residues.data_ptr())
        if self._plan is None or self._plan[0] != key:
            self._plan = (key, ops.ModalPlan(self.log_poles, self.residues))
        return self._plan[1]

    def parallel_forward(self, u, inference_params=None, padding_mask=None):
        """Prefill: u [B, L, 3D] bf16 -> y [B, L, D] bf16 (vortex/model/model.py:221-316)."""
        masked = isinstance(padding_mask, torch.Tensor)
        B, L, C = u.shape
        D, Ks = self.hidden_size, self.short_filter_length
        caching = inference_params is not None
        if not masked and self.fuse_prefill and self._can_fuse_prefill(u, L, caching):
            return self._fused_prefill(u, inference_params), inference_params
        if not masked and self.fuse_prefill and self._can_scan_projection_rows(u):
            return self._modal_prefill_from_rows(u, inference_params), inference_params
        if not masked and self.fuse_prefill and self._can_filter_projection_rows(u):
            return self._fir_prefill_from_rows(u, inference_params), inference_params
        if not masked and self.fuse_prefill and self._can_fuse_gates(u):
            return self._modal_prefill_from_projection(u, inference_params), inference_params
        w = self._f32_param("short_filter_weight", (C, Ks))
        # the sequence-major kernels take multiples of 8 samples: other lengths run behind -L % 8 zero samples
        pad, L_true = (-L) % 8, L
        L += pad
        z_pre = ops.featurizer_fwd(u, w, self._f32_param("short_filter_bias"), interleave=self.interleave,
                                   front_pad=pad)
        if masked:      # rare path (padded batches): the 0/1 mask of vortex/model/engine.py:226-227 through torch
            mask = torch.nn.functional.pad(padding_mask, (pad, 0))[:, None].to(z_pre.dtype)
            z_pre = z_pre * mask
        r1, r2, rv = self._rows(z_pre)
        K = self.fir_inner_filter_length
        if K:
            taps = self._f32_param("h", (self.h.shape[0], K))
            if K > 128:     # no MFMA kernel for such filters: the direct-form kernel on the gates as tensors
                x2t, x1t, vt = self._split(z_pre)
                y = ops.fir_fwd_long(x1t, x2t, vt, taps[:, :L], bias=self._f32_param("D"), bias_mode=HYENA_BIAS_GATED_FP32)
            elif K >= 128:
                y = ops.fir_fwd_rows(r1, r2, rv, taps, B, D, L, K, device=u.device, bias=self._f32_param("D"),
                                     bias_mode=HYENA_BIAS_GATED_FP32, taps_reversed=False, force_mfma=True)
            else:
                y = ops.fir_fwd_rows(r1, r2, rv, taps, B, D, L, K, device=u.device, taps_reversed=True)
            if masked:
                y = y * mask     # a 0/1 mask on the convolution commutes with the x2 gate
        elif self.long_fir_threshold is not None:
            # vortex/model/engine.py:339-349: the first `threshold` samples of the modal filter as a bf16 FIR, with
            # the last of them on the current sample (F.conv1d correlates); the reference cannot prefill a cache here
            if caching:
                raise NotImplementedError("long_fir_threshold with a cache: the reference has no state prefill on "
                                          "this branch (vortex/model/engine.py:380-392 reads an unassigned X_s)")
            T = min(int(self.long_fir_threshold), L_true)
            with torch.no_grad():
                h = self.compute_filter(T, u.device)[0][0]
            taps = h.to(torch.bfloat16).to(torch.float32).contiguous()                     # [G, T]
            # (bf16(y) + x1v*D) in the tensors' own dtype (engine.py:351-353): bf16 arithmetic with a bf16 D
            mode = HYENA_BIAS_GATED_BF16 if self.D.dtype == torch.bfloat16 else HYENA_BIAS_GATED_FP32
            if T > 128:     # beyond the MFMA kernel's filter length: the direct-form kernel on the gates as tensors
                x2t, x1t, vt = self._split(z_pre)
                y = ops.fir_fwd_long(x1t, x2t, vt, taps, bias=self._f32_param("D"), bias_mode=mode, taps_reversed=True)
            else:
                y = ops.fir_fwd_rows(r1, r2, rv, taps, B, D, L, T, device=u.device, bias=self._f32_param("D"),
                                     bias_mode=mode, taps_reversed=True, force_mfma=True)
        else:
            y, _, state = ops.li_fwd_rows(r1, r2, rv, self.modal_plan(), self.D, B, D, L, device=u.device,
                                          want_state=caching)
            if caching:
                inference_params.state_dict[self.layer_idx] = state
        if caching:
            # the channel-last tail of u is already the ring layout [B, R, 3D]
            inference_params.fir_state_dict[self.layer_idx] = _ring(u[:, max(L_true - (Ks - 1), 0):], Ks - 1)
            if K:
                _, x1, v = self._split(z_pre[..., max(L - (K - 1), pad):])
                inference_params.fir_inner_state_dict[self.layer_idx] = _ring((x1 * v).permute(0, 2, 1), K - 1,
                                                                              flipped=K >= 128)
            self._drop_decode()
        if pad:
            y = y[..., pad:]
        return y.permute(0, 2, 1), inference_params

    def _channel_map(self):
        return ops.gate_channel_map(self.hidden_size, interleave=self.interleave,
                                    head_dim=self.hidden_size_per_attention_head if self.column_split_hyena else None)

    def _can_fuse_prefill(self, u, L, caching):
        """Whether hyena_fir_layer_fwd covers this layer: an SE / MR layer with a 3- or 4-tap featurizer, a closed
        channel map, 16-channel filter groups and an aligned projection."""
        K, D, hd = self.fir_inner_filter_length, self.hidden_size, self.hidden_size_per_attention_head
        if not K or K > 128 or self.short_filter_length not in (3, 4) or self._channel_map() is None:
            return False
        if (D // self.hyena_filter_groups) % 16 or D % 8 or (self.column_split_hyena and hd % 8):
            return False
        return u.stride(2) == 1 and u.stride(1) % 8 == 0 and u.stride(0) % 8 == 0 and u.data_ptr() % 16 == 0

    def _can_fuse_gates(self, u):
        """Whether hyena_featurizer_gates_fwd covers this layer: a Hyena-LI layer (modal filter, no truncated-FIR
        branch) with a 3- or 4-tap featurizer, a closed channel map and an aligned projection."""
        D, hd = self.hidden_size, self.hidden_size_per_attention_head
        if not self._can_fuse_gates_layer() or self.short_filter_length not in (3, 4):
            return False
        if D % 8 or (self.column_split_hyena and hd % 8):
            return False
        return u.stride(2) == 1 and u.stride(1) % 8 == 0 and u.stride(0) % 8 == 0 and u.data_ptr() % 16 == 0

    def _can_scan_projection_rows(self, u):
        """Whether hyena_li_layer_fwd covers this call: a Hyena-LI layer with a three-tap featurizer without bias and a
        closed channel map, whose projection u [B, L, 3D] is stored sequence-major (the [B, 3D, L] product the
        projection GEMM writes when asked for it transposed, handed over as `p.transpose(1, 2)`), a whole number of
        8-sample pieces long."""
        return self._can_fuse_gates_layer() and self._rows_layout_ok(u)

    def _rows_layout_ok(self, u):
        B, L, C = u.shape
        return (self.short_filter_length == 3 and self.short_filter_bias is None and self._channel_map() is not None
                and L % 8 == 0 and L > 1 and C > 1 and u.stride(1) == 1 and u.stride(2) % 8 == 0
                and u.stride(0) % 8 == 0 and u.data_ptr() % 16 == 0)

    def _can_filter_projection_rows(self, u):
        """Whether hyena_fir_layer_fwd_rows covers this call: a Hyena-SE / MR layer (inner filter of at most 128 taps)
        whose projection is stored sequence-major, under the conditions of _can_scan_projection_rows, and a prompt
        long enough to fill the inner cache from its own tail."""
        K = self.fir_inner_filter_length
        return bool(K) and K <= 128 and self._rows_layout_ok(u) and u.shape[1] >= K + 1

    def _feat_rows_taps(self, chan, C, Ks):
        """Featurizer weight rows [3, D, Ks] of the (x1, x2, v) row of every operator channel (flip applied)."""
        key = ("feat_rows", id(self.short_filter_weight), self.short_filter_weight.data_ptr(),
               self.short_filter_weight._version, self.hyena_flip_x1x2)
        hit = self._f32_cache.get("wf_rows")
        if hit is None or hit[0] != key:
            w = self._f32_param("short_filter_weight", (C, Ks))
            t2, t1, tv = w[chan[0]], w[chan[1]], w[chan[2]]
            if self.hyena_flip_x1x2:
                t1, t2 = t2, t1
            hit = (key, torch.stack([t1, t2, tv]).contiguous())
            self._f32_cache["wf_rows"] = hit
        return hit[1]

    def _fir_prefill_from_rows(self, u, inference_params):
        """Hyena-SE / MR prefill in one launch from a sequence-major projection: featurizer, split, gates and the
        inner FIR on the matrix cores (vortex/model/model.py:233-291)."""
        B, L, C = u.shape
        D, Ks, K = self.hidden_size, self.short_filter_length, self.fir_inner_filter_length
        caching = inference_params is not None
        mr = K >= 128
        p = u.transpose(1, 2)                                                       # [B, 3D, L], samples contiguous
        (q2, q1, qv), chan = ops.projection_rows(
            p, D, interleave=self.interleave,
            head_dim=self.hidden_size_per_attention_head if self.column_split_hyena else None)
        ft = self._feat_rows_taps(chan, C, Ks)
        if self.hyena_flip_x1x2:
            q1, q2 = q2, q1
        y = ops.fir_layer_fwd_rows(q1, q2, qv, ft, self._f32_param("h", (self.h.shape[0], K)), B, D, L, K,
                                   device=u.device, bias=self._f32_param("D") if mr else None,
                                   bias_mode=HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE, taps_reversed=not mr)
        if caching:
            inference_params.fir_state_dict[self.layer_idx] = _ring(u[:, L - (Ks - 1):], Ks - 1)
            # the inner cache is the last K-1 values of bf16(x1*v): the featurizer kernel on the prompt's tail (its
            # first Ks-1 outputs lack their history and are dropped)
            n = K - 1 + Ks - 1
            z = ops.featurizer_fwd(u[:, L - n:].contiguous(), self._f32_param("short_filter_weight", (C, Ks)), None,
                                   interleave=self.interleave, front_pad=(-n) % 8)
            _, x1, v = self._split(z[..., z.shape[-1] - (K - 1):])
            inference_params.fir_inner_state_dict[self.layer_idx] = _ring((x1 * v).permute(0, 2, 1), K - 1, flipped=mr)
            self._drop_decode()
        return y.permute(0, 2, 1)

    def _can_fuse_gates_layer(self):
        """A Hyena-LI layer (modal filter, no truncated-FIR branch) with a closed channel map."""
        if self.fir_inner_filter_length or self.long_fir_threshold is not None:
            return False
        return self._channel_map() is not None

    def _modal_prefill_from_rows(self, u, inference_params):
        """Hyena-LI prefill in one launch from a sequence-major projection: featurizer, split, gates and the modal
        scan (vortex/model/model.py:233-252, :295-312), 6 bytes read and 2 written per (batch, channel, sample)."""
        B, L, C = u.shape
        D, Ks = self.hidden_size, self.short_filter_length
        caching = inference_params is not None
        p = u.transpose(1, 2)                                                       # [B, 3D, L], samples contiguous
        (q2, q1, qv), chan = ops.projection_rows(
            p, D, interleave=self.interleave,
            head_dim=self.hidden_size_per_attention_head if self.column_split_hyena else None)
        ft = self._feat_rows_taps(chan, C, Ks)
        if self.hyena_flip_x1x2:
            q1, q2 = q2, q1
        y, state = ops.li_layer_fwd_rows(q1, q2, qv, ft, self.modal_plan(), self.D, B, D, L, device=u.device,
                                         want_state=caching)
        if caching:
            inference_params.state_dict[self.layer_idx] = state
            inference_params.fir_state_dict[self.layer_idx] = _ring(u[:, max(L - (Ks - 1), 0):], Ks - 1)
            self._drop_decode()
        return y.permute(0, 2, 1)

    def _featurizer_taps_t(self, C, Ks):
        key = ("short_filter_weight_t", id(self.short_filter_weight), self.short_filter_weight.data_ptr(),
               self.short_filter_weight._version)
        hit = self._f32_cache.get("wf_t")
        if hit is None or hit[0] != key:
            hit = (key, self._f32_param("short_filter_weight", (C, Ks)).t().contiguous())
            self._f32_cache["wf_t"] = hit
        return hit[1]

    def _modal_prefill_from_projection(self, u, inference_params):
        """Hyena-LI prefill in two launches: featurizer + split + x1*v (rows xv, x2), then the modal scan."""
        B, L, C = u.shape
        D, Ks = self.hidden_size, self.short_filter_length
        caching = inference_params is not None
        pad = (-L) % 8
        xv, x2 = ops.featurizer_gates_fwd(u, self._featurizer_taps_t(C, Ks), self._f32_param("short_filter_bias"),
                                          self._channel_map(), flip_x1x2=self.hyena_flip_x1x2, front_pad=pad)
        y, _, state = ops.li_fwd_rows(ops.rows_of(xv), ops.rows_of(x2), None, self.modal_plan(), self.D, B, D, L + pad,
                                      device=u.device, want_state=caching)
        if caching:
            inference_params.state_dict[self.layer_idx] = state
            inference_params.fir_state_dict[self.layer_idx] = _ring(u[:, max(L - (Ks - 1), 0):], Ks - 1)
            self._drop_decode()
        if pad:
            y = y[..., pad:]
        return y.permute(0, 2, 1)

    def _fused_prefill(self, u, inference_params):
        """u [B, L, 3D] -> y [B, L, D] in one launch; with a cache object also the two FIR caches."""
        B, L, C = u.shape
        K, Ks = self.fir_inner_filter_length, self.short_filter_length
        wf_t = self._featurizer_taps_t(C, Ks)
        mr = K >= 128
        taps = self._f32_param("h", (self.h.shape[0], K))
        caching = inference_params is not None
        res = ops.fir_layer_fwd(u, wf_t, self._f32_param("short_filter_bias"), self._channel_map(), taps,
                                bias=self._f32_param("D") if mr else None,
                                bias_mode=HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE, taps_reversed=not mr,
                                flip_x1x2=self.hyena_flip_x1x2, bx_from=max(L - (K - 1), 0) if caching else None)
        if not caching:
            return res
        y, bx = res
        inference_params.fir_state_dict[self.layer_idx] = _ring(u[:, max(L - (Ks - 1), 0):], Ks - 1)
        inference_params.fir_inner_state_dict[self.layer_idx] = _ring(bx, K - 1, flipped=mr)
        self._drop_decode()
        return y

    # ------------------------------------------------------------------
    def _decode_plan(self, inference_params):
        """Binds the decode kernels to this layer's caches once per generation."""
        i = self.layer_idx
        ring = inference_params.fir_state_dict[i]
        if self._decode is not None and self._decode["ring"] is ring:
            return self._decode
        self._drop_decode()          # bound to another cache object: leave that one's state complete first
        C, Ks, D = 3 * self.hidden_size, self.short_filter_length, self.hidden_size
        dev = ring.buf.device
        d = {"ring": ring}
        d["feat"] = ops.FirStepper(ring, self.short_filter_weight.detach().reshape(C, Ks), bias=self.short_filter_bias,
                                   gated=False)
        if self.interleave:
            j = torch.arange(C, device=dev)
            d["perm"] = (j % (C // 3)) * 3 + j // (C // 3)      # output row r = i*C/3 + j'  <-  channel 3j' + i
        K = self.fir_inner_filter_length
        if K:
            taps = self.h.detach().reshape(self.h.shape[0], K)
            taps = taps if K < 128 else taps.flip(-1)           # oldest tap first (engine.py:421-425)
            d["inner"] = ops.FirStepper(inference_params.fir_inner_state_dict[i], taps.contiguous(),
                                        bias=self.D if K >= 128 else None, gated_bias=K >= 128)
        else:
            st = inference_params.state_dict[i]
            poles = torch.exp(self.log_poles.detach())[..., 0].contiguous()
            d["inner"] = ops.IirStepper(st, poles, self.residues.detach(), self.D.detach(),
                                        windowed=self.window_decode_state)
        d["layer"] = self._fused_step(ring, d["inner"])
        self._decode = d
        return d

    def _fused_step(self, ring, inner):
        """The one-launch layer step, or None where the fused kernels do not apply (then three launches are used)."""
        cmap = self._channel_map()
        Ks, hd = self.short_filter_length, self.hidden_size_per_attention_head
        fir = isinstance(inner, ops.FirStepper)
        if cmap is None or Ks < 2 or Ks > 8 or self.hidden_size % 8:
            return None
        if fir and (inner.mode == HYENA_BIAS_ADD or (self.column_split_hyena and hd % 8)):
            return None
        if not fir and inner.S * (2 if inner.cplx else 1) < 16:      # the fused kernel needs three lanes per channel
            return None
        return ops.LayerStepper(ring, self.short_filter_weight.detach().reshape(3 * self.hidden_size, Ks),
                                self.short_filter_bias, cmap, inner, flip_x1x2=self.hyena_flip_x1x2)

    def _drop_decode(self):
        """Unbinds the decode kernels from the caches they were bound to.  A windowed modal stepper holds the last
        inputs of its open windows itself, so its state tensor is brought up to date first: whoever owns that cache
        object (another sequence served by this module in turn) finds it complete."""
        inner = (self._decode or {}).get("inner")
        if isinstance(inner, ops.IirStepper) and inner.pos_dev is None:
            inner.flush()
        self._decode = None

    def flush_decode_state(self):
        """Brings inference_params.state_dict[layer_idx] up to the last token (the windowed modal step lets it lag by up
        to four inputs); call it before reading or saving the state during decode.  No-op otherwise."""
        inner = (self._decode or {}).get("inner")
        if isinstance(inner, ops.IirStepper):
            inner.flush()

    def _growing_step(self, u, d):
        """Decode step while a cache still holds fewer samples than its filter needs (prompt shorter than the
        filter): the reference's tap slicing for that case, with tap tables rebuilt per step."""
        B, D = u.shape[0], self.hidden_size

        def fir(stepper, x1, x2, v, out):
            ring = stepper.ring
            valid, R = getattr(ring, "valid", stepper.R), stepper.R
            if valid < R:
                # tap tables that change from token to token: the whole-cache step (far sums carry the taps of the
                # token that formed them into the next two outputs)
                full = stepper.w
                stepper.w = _grown_taps(full, valid)
                stepper(x1, x2, v, out, far=False)
                stepper.w = full
                ring.valid = valid + 1
            else:
                stepper(x1, x2, v, out)

        z_pre = torch.empty(B, 3 * D, dtype=torch.bfloat16, device=u.device)
        fir(d["feat"], u.contiguous(), None, None, z_pre)
        if self.interleave:
            z_pre = z_pre[:, d["perm"]]
        x2, x1, v = (t.contiguous() for t in self._split(z_pre))
        y = torch.empty(B, D, dtype=torch.bfloat16, device=u.device)
        if self.fir_inner_filter_length:
            fir(d["inner"], x1, x2, v, y)
        else:
            d["inner"](x1, x2, v, y)
        return y[:, None]

    def sequential_forward(self, u, inference_params):
        """Decode: u [B, 3D] or [B, 1, 3D] bf16 -> y [B, 1, D] (vortex/model/model.py:318-375)."""
        if u.dim() > 2:
            u = u[:, -1]
        if u.shape[1] > 1 and u.stride(1) != 1:      # a token cut from a sequence-major projection: the step kernels
            u = u.contiguous()                        # take contiguous channels (a copy of 6*D bytes per batch element)
        d = self._decode_plan(inference_params)
        B = u.shape[0]
        rings = [d["ring"]] + ([d["inner"].ring] if self.fir_inner_filter_length else [])
        if any(getattr(r, "valid", r.R) < r.R for r in rings):
            return self._growing_step(u, d), inference_params
        if self.fuse_decode and d["layer"] is not None and u.stride(1) == 1 and u.stride(0) % 8 == 0 and u.data_ptr() % 16 == 0:
            y = torch.empty(B, self.hidden_size, dtype=torch.bfloat16, device=u.device)
            d["layer"](u, y)
            return y[:, None], inference_params
        z_pre = torch.empty(B, 3 * self.hidden_size, dtype=torch.bfloat16, device=u.device)
        d["feat"](u, None, None, z_pre)
        if self.interleave:
            z_pre = z_pre[:, d["perm"]]
        x2, x1, v = self._split(z_pre)
        if self.column_split_hyena:
            x2, x1, v = x2.contiguous(), x1.contiguous(), v.contiguous()
        y = torch.empty(B, self.hidden_size, dtype=torch.bfloat16, device=u.device)
        d["inner"](x1, x2, v, y)
        return y[:, None], inference_params
