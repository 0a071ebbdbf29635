"""Tensor-level wrappers over the C ABI: shape/dtype checks, row descriptors, stream.

Every function enqueues on torch's current stream and returns torch tensors that
it allocated; nothing here computes on the CPU or through PyTorch operators.
"""
import ctypes

import torch

from . import _lib
from ._lib import HYENA_BIAS_ADD, HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE, Cl, ProjFwd, ProjStep, Rows

_CL_DTYPES = {torch.bfloat16: _lib.HYENA_DTYPE_BF16, torch.float16: _lib.HYENA_DTYPE_F16, torch.float32: _lib.HYENA_DTYPE_F32}


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("vortex_amd operators run on the GPU only (got a CPU tensor); there is no CPU fallback")


def _strides(t):
    """Strides of a tensor with those of size-one dimensions (which torch leaves arbitrary) replaced by the dense
    values, so that the alignment checks of the C entry points see what a larger tensor of that layout would have."""
    st, dense = list(t.stride()), 1
    for i in range(t.dim() - 1, -1, -1):
        if t.shape[i] == 1:
            st[i] = dense
        dense = max(dense, st[i] * t.shape[i])
    return st


def rows_of(t):
    """Row descriptor of a [B, D, L] bf16 tensor whose samples are contiguous."""
    if t is None:
        return None
    if t.dtype != torch.bfloat16:
        raise TypeError(f"expected bfloat16 gates, got {t.dtype}")
    if t.dim() != 3 or (t.shape[2] > 1 and t.stride(2) != 1):
        raise ValueError("expected a [B, D, L] tensor with contiguous samples")
    B, D, L = t.shape
    bs, rs, _ = _strides(t)
    return Rows(t.data_ptr(), bs, rs, D, D)


def rows_of_projection(u, hidden, which, head_dim=None):
    """Row descriptor of gate `which` (0, 1, 2) inside a [B, 3*hidden, L] projection.

    head_dim=None is the plain split of vortex/model/engine.py:156; otherwise the
    head-blocked column split of vortex/model/utils.py:41-85.
    """
    if u.dtype != torch.bfloat16 or u.dim() != 3 or u.stride(2) != 1:
        raise ValueError("expected a [B, 3D, L] bfloat16 tensor with contiguous samples")
    if u.shape[1] != 3 * hidden or (head_dim is not None and (head_dim <= 0 or hidden % head_dim)):
        # the descriptors address rows up to 3*hidden - 1: anything else would read outside the tensor
        raise ValueError(f"a [B, {3 * hidden}, L] projection and a head_dim that divides {hidden} are required "
                         f"(got {tuple(u.shape)}, head_dim={head_dim})")
    es = u.element_size()
    if head_dim is None:
        return Rows(u.data_ptr() + which * hidden * u.stride(1) * es, u.stride(0), u.stride(1), hidden, hidden)
    return Rows(u.data_ptr() + which * head_dim * u.stride(1) * es, u.stride(0), u.stride(1), head_dim, 3 * head_dim)


def _ref(r):
    return ctypes.byref(r) if r is not None else None


def _f32(t, shape=None):
    if t is None:
        return None
    t = t.detach()
    if t.dtype != torch.float32 or not t.is_contiguous():
        t = t.to(torch.float32).contiguous()
    return t


def front_pad8(t):
    """Makes a [B, D, L] bf16 tensor usable by the sequence-major kernels: (tensor, pad).

    The kernels move 8 samples (16 bytes) per lane, so rows must start 16-byte aligned and hold a multiple
    of 8 samples.  A tensor that already does is returned as is (pad = 0); otherwise it is copied behind
    pad = -L % 8 zero columns.  Zero samples ahead of a causal filter with zero history change neither the
    later outputs nor the final modal state, so callers run on L + pad samples and drop the first pad outputs.
    """
    B, D, L = t.shape
    pad = (-L) % 8
    st = _strides(t)
    if pad == 0 and st[2] == 1 and st[1] % 8 == 0 and st[0] % 8 == 0 and t.data_ptr() % 16 == 0:
        return t, 0
    buf = torch.empty((B, D, L + pad), dtype=t.dtype, device=t.device)
    if pad:
        buf[..., :pad] = 0
    buf[..., pad:] = t
    return buf, pad


def _bias_mode(bias, gated, fp32_gated):
    if bias is None:
        return HYENA_BIAS_NONE
    if gated:
        if not fp32_gated:
            raise NotImplementedError("gated bias after the bf16 rounding (short-FIR branch) has no kernel")
        return HYENA_BIAS_GATED_FP32
    return HYENA_BIAS_ADD


def fir_fwd_rows(x1r, x2r, vr, taps, B, D, L, K, *, device, bias=None, bias_mode=HYENA_BIAS_NONE,
                 taps_reversed=False, force_mfma=False, out=None):
    """Shared launcher of the prefill FIR kernels on row descriptors.

    taps [G, K] float32.  taps_reversed=False means the convolution orientation
    (taps[:, 0] on the current sample); True means the short-filter orientation of
    vortex (taps[:, K-1] on the current sample).
    """
    taps = _f32(taps)
    G = taps.shape[0]
    if out is None:
        out = torch.empty((B, D, L), dtype=torch.bfloat16, device=device)
    if out.numel() == 0:
        return out
    L_ = _lib.lib()
    if K <= 8 and not force_mfma:
        if not taps_reversed:
            taps = taps.flip(-1).contiguous()
        rc = L_.hyena_se_fwd(_ref(x1r), _ref(x2r), _ref(vr), _ptr(taps), _ptr(bias), bias_mode, _ptr(out),
                             B, D, L, G, K, _stream())
        _lib.check(rc, "hyena_se_fwd")
    else:
        rc = L_.hyena_mr_fwd(_ref(x1r), _ref(x2r), _ref(vr), _ptr(taps), int(taps_reversed), _ptr(bias), bias_mode,
                             _ptr(out), B, D, L, G, K, _stream())
        _lib.check(rc, "hyena_mr_fwd")
    return out


def fir_layer_fwd_rows(x1r, x2r, vr, feat_taps, taps, B, D, L, K, *, device, bias=None, bias_mode=HYENA_BIAS_NONE,
                       taps_reversed=False, out=None):
    """hyena_fir_layer_fwd_rows: a whole Hyena-SE / MR layer in one pass over the rows of a raw sequence-major
    projection -- the three-tap featurizer FIR on every piece as it is read, then the gated FIR of fir_fwd_rows on the
    matrix cores (any K <= 128).  feat_taps [3, D, 3] float32: the featurizer weight rows of the x1, x2 and v row of
    every operator channel, oldest sample first.  Returns out [B, D, L] bf16."""
    taps = _f32(taps)
    G = taps.shape[0]
    if out is None:
        out = torch.empty((B, D, L), dtype=torch.bfloat16, device=device)
    if out.numel() == 0:
        return out
    if feat_taps.dtype != torch.float32 or not feat_taps.is_contiguous() or tuple(feat_taps.shape) != (3, D, 3):
        raise ValueError("feat_taps must be a contiguous float32 [3, D, 3] tensor")
    rc = _lib.lib().hyena_fir_layer_fwd_rows(_ref(x1r), _ref(x2r), _ref(vr), _ptr(feat_taps), 3, _ptr(taps),
                                             int(taps_reversed), _ptr(bias), bias_mode, _ptr(out), B, D, L, G, K,
                                             _stream())
    _lib.check(rc, "hyena_fir_layer_fwd_rows")
    return out


def _cl_of(t, dtype=torch.bfloat16):
    """hyena_cl of a [B, L, D] tensor of `dtype` with contiguous channels (any batch / time stride)."""
    if t is None:
        return None
    if t.dtype != dtype or t.dim() != 3 or (t.shape[2] > 1 and t.stride(2) != 1):
        raise ValueError(f"expected a [B, L, D] {dtype} tensor with contiguous channels")
    bs, ts, _ = _strides(t)
    return Cl(t.data_ptr(), bs, ts)


def fir_cl_fwd(x1, x2, v, taps, *, bias=None, bias_mode=HYENA_BIAS_NONE, taps_reversed=False, want_y2=False,
               want_bx=False, bx_from=0, out=None):
    """Gated FIR on channel-last [B, L, D] tensors: out = x2 * conv(taps, x1*v), 1 <= K <= 128.

    bfloat16 tensors (the model path) and float16 tensors run the MFMA kernel (filter groups of a multiple of 16
    channels); float32 tensors, and float16 shapes the MFMA kernel does not cover, run a direct-form kernel
    (hyena_fir_cl_fwd_dtype).  All tensors share x1's dtype, which is also the dtype of the results.
    taps [G, K] float32, convolution orientation unless taps_reversed.  Returns out, or (out, y2, bx) when an
    intermediate is requested (y2: the convolution before the x2 gate; bx: rows bx_from.. of x1*v in that dtype).
    """
    _need_cuda(x1, x2, v, taps)
    dt = x1.dtype
    if dt not in _CL_DTYPES:
        raise TypeError(f"channel-last FIR takes bfloat16, float16 or float32 tensors, got {dt}")
    taps = _f32(taps)
    G, K = taps.shape
    B, L, D = x1.shape
    if out is None:
        out = torch.empty((B, L, D), dtype=dt, device=x1.device)
    elif out.dtype != dt or not out.is_contiguous():
        raise ValueError("out must be contiguous and of the inputs' dtype")
    y2 = torch.empty_like(out) if want_y2 else None
    bx = torch.empty((B, L - bx_from, D), dtype=dt, device=x1.device) if want_bx else None
    if out.numel():
        c1, c2, cv = _cl_of(x1, dt), _cl_of(x2, dt), _cl_of(v, dt)
        if dt == torch.bfloat16 and K <= 128:
            rc = _lib.lib().hyena_fir_cl_fwd(_ref(c1), _ref(c2), _ref(cv), _ptr(taps), int(taps_reversed), _ptr(_f32(bias)),
                                             bias_mode, _ptr(out), _ptr(y2), _ptr(bx), bx_from, B, L, D, G, K, _stream())
        else:
            rc = _lib.lib().hyena_fir_cl_fwd_dtype(_ref(c1), _ref(c2), _ref(cv), _ptr(taps), int(taps_reversed),
                                                   _ptr(_f32(bias)), bias_mode, _ptr(out), _ptr(y2), _ptr(bx), bx_from,
                                                   B, L, D, G, K, _CL_DTYPES[dt], _stream())
        _lib.check(rc, "hyena_fir_cl_fwd")
    return (out, y2, bx) if (want_y2 or want_bx) else out


def fir_fwd_long(x1, x2, v, taps, *, bias=None, bias_mode=HYENA_BIAS_NONE, taps_reversed=False):
    """Gated FIR with more than 128 taps on [B, D, L] bf16 gates (views welcome): out [B, D, L].

    No MFMA kernel is built for such filters (none of the reference's configurations has one); they run the
    direct-form channel-last kernel (hyena_fir_cl_fwd_dtype) between two layout changes through torch."""
    cl = lambda t: None if t is None else t.transpose(1, 2).contiguous()
    y = fir_cl_fwd(cl(x1), cl(x2), cl(v), taps, bias=bias, bias_mode=bias_mode, taps_reversed=taps_reversed)
    return y.transpose(1, 2).contiguous()


def fir_layer_fwd(u, feat_w, feat_bias, channel_map, taps, *, bias=None, bias_mode=HYENA_BIAS_NONE,
                  taps_reversed=False, flip_x1x2=False, bx_from=None, out=None):
    """A whole Hyena-SE / MR layer at prefill in one launch: u [B, L, 3D] bf16 -> out [B, L, D] bf16.

    feat_w [Ks, 3D] float32 (tap-major, last row on the current sample), feat_bias [3D] or None, channel_map from
    gate_channel_map().  bx_from: also return rows bx_from.. of bf16(x1*v), the inner FIR cache of a decode step
    (at most the last K-1 rows: L - bx_from <= K - 1).
    """
    _need_cuda(u, feat_w, taps)
    if u.dtype != torch.bfloat16 or u.dim() != 3 or u.stride(2) != 1:
        raise ValueError("expected a [B, L, 3D] bfloat16 projection with contiguous channels")
    taps = _f32(taps)
    G, K = taps.shape
    B, L, C = u.shape
    D = C // 3
    feat_w, feat_bias = _f32(feat_w), _f32(feat_bias)
    if feat_w.shape[1] != C:
        raise ValueError("feat_w must be [Ks, 3D] (tap-major)")
    ci, co, gs, cs = channel_map
    if out is None:
        out = torch.empty((B, L, D), dtype=torch.bfloat16, device=u.device)
    bx = torch.empty((B, L - bx_from, D), dtype=torch.bfloat16, device=u.device) if bx_from is not None else None
    if out.numel():
        pj = ProjFwd(u.data_ptr(), _strides(u)[0], _strides(u)[1], feat_w.data_ptr(),
                     feat_bias.data_ptr() if feat_bias is not None else None, feat_w.shape[0], int(flip_x1x2),
                     ci, co, gs, cs)
        rc = _lib.lib().hyena_fir_layer_fwd(ctypes.byref(pj), _ptr(taps), int(taps_reversed), _ptr(_f32(bias)),
                                            bias_mode, _ptr(out), _ptr(bx), bx_from or 0, B, L, D, G, K, _stream())
        _lib.check(rc, "hyena_fir_layer_fwd")
    return out if bx_from is None else (out, bx)


def featurizer_gates_fwd(u, feat_w, feat_bias, channel_map, *, flip_x1x2=False, front_pad=0, row_pad=0):
    """Featurizer, split and x1*v of a Hyena-LI layer in one launch: u [B, L, 3D] bf16 -> (xv, x2), each
    [B, D, L + front_pad] bf16 with xv = bf16(x1*v): the rows li_fwd_rows reads as (x1r=rows_of(xv), x2r=rows_of(x2),
    vr=None).  feat_w [Ks, 3D] float32 tap-major, feat_bias [3D] or None, channel_map from gate_channel_map().
    row_pad (a multiple of 8): the rows of the two results are L + front_pad + row_pad elements apart (views of wider
    buffers), e.g. to keep long rows from lying a power of two apart."""
    _need_cuda(u, feat_w)
    if u.dtype != torch.bfloat16 or u.dim() != 3 or u.stride(2) != 1:
        raise ValueError("expected a [B, L, 3D] bfloat16 projection with contiguous channels")
    B, L, C = u.shape
    D = C // 3
    feat_w, feat_bias = _f32(feat_w), _f32(feat_bias)
    if feat_w.shape[1] != C:
        raise ValueError("feat_w must be [Ks, 3D] (tap-major)")
    ci, co, gs, cs = channel_map
    Lout = L + front_pad if L else 0
    xv = torch.empty((B, D, Lout + row_pad), dtype=torch.bfloat16, device=u.device)[..., :Lout]
    x2 = torch.empty((B, D, Lout + row_pad), dtype=torch.bfloat16, device=u.device)[..., :Lout]
    if xv.numel():
        pj = ProjFwd(u.data_ptr(), _strides(u)[0], _strides(u)[1], feat_w.data_ptr(),
                     feat_bias.data_ptr() if feat_bias is not None else None, feat_w.shape[0], int(flip_x1x2),
                     ci, co, gs, cs)
        rc = _lib.lib().hyena_featurizer_gates_fwd(ctypes.byref(pj), _ptr(xv), _ptr(x2), Lout + row_pad, B, L, D,
                                                   front_pad, _stream())
        _lib.check(rc, "hyena_featurizer_gates_fwd")
    return xv, x2


def hyena_se_fwd(x1, x2, v, h, bias=None, *, force_mfma=False):
    """Hyena-SE prefill: out = bf16(x2 * bf16(corr_K(bf16(x1*v)))) on [B, D, L] bf16 gates.

    h: [G, 1, K] or [G, K] float32 in vortex's short-filter orientation (h[..., K-1]
    multiplies the current sample; vortex/model/engine.py:197-204).  Returns [B, D, L] bf16.
    """
    _need_cuda(x1, x2, v, h)
    B, D, L = x1.shape
    taps = _f32(h).reshape(h.shape[0], -1)
    K = taps.shape[1]
    b = _f32(bias)
    (x1, pad), (x2, _), (v, _) = front_pad8(x1), front_pad8(x2), front_pad8(v)
    out = fir_fwd_rows(rows_of(x1), rows_of(x2), rows_of(v), taps, B, D, L + pad, K, device=x1.device, bias=b,
                       bias_mode=_bias_mode(b, False, False), taps_reversed=True, force_mfma=force_mfma)
    return out[..., pad:] if pad else out


def hyena_mr_fwd(x1, x2, v, h, D_bias=None):
    """Hyena-MR prefill: out = bf16(x2 * bf16(conv(h, u) + D*u)), u = bf16(x1*v).

    h: [G, 1, K] or [G, K] float32, true-convolution orientation (h[..., 0] on the
    current sample; vortex/model/engine.py:174-187).  D_bias: [D] or None.
    """
    _need_cuda(x1, x2, v, h)
    B, D, L = x1.shape
    taps = _f32(h).reshape(h.shape[0], -1)
    K = taps.shape[1]
    b = _f32(D_bias)
    if K > 128:
        return fir_fwd_long(x1, x2, v, taps, bias=b, bias_mode=_bias_mode(b, True, True))
    (x1, pad), (x2, _), (v, _) = front_pad8(x1), front_pad8(x2), front_pad8(v)
    out = fir_fwd_rows(rows_of(x1), rows_of(x2), rows_of(v), taps, B, D, L + pad, K, device=x1.device, bias=b,
                       bias_mode=_bias_mode(b, True, True), taps_reversed=False, force_mfma=True)
    return out[..., pad:] if pad else out


def featurizer_fwd(u, taps, bias=None, interleave=False, front_pad=0):
    """Featurizer short FIR on the channel-last projection: u [B, L, C] bf16 -> z [B, C, L + front_pad] bf16.

    taps: [G, K] float32 in vortex's short-filter orientation (taps[:, K-1] on the current
    sample), G = C or a divisor of C.  bias: [C] or None (added after the bf16 rounding of the
    convolution, vortex/model/engine.py:208-223).  interleave=True also applies
    vortex/model/utils.py:26-38 (channels 0::3 | 1::3 | 2::3) while writing.  front_pad = -L % 8 leading zero
    columns make a length that is not a multiple of 8 usable by the sequence-major kernels (see front_pad8).
    """
    _need_cuda(u, taps)
    if u.dtype != torch.bfloat16 or u.dim() != 3 or u.stride(2) != 1:
        raise ValueError("expected a [B, L, C] bfloat16 tensor with contiguous channels")
    B, L, C = u.shape
    taps = _f32(taps)
    out = torch.empty((B, C, L + front_pad), dtype=torch.bfloat16, device=u.device)
    if out.numel() == 0:
        return out
    b = _f32(bias)
    rc = _lib.lib().hyena_featurizer_fwd(_ptr(u), _strides(u)[0], _strides(u)[1], _ptr(taps), _ptr(b), int(interleave), _ptr(out),
                                         B, L, C, taps.shape[0], taps.shape[1], front_pad, _stream())
    _lib.check(rc, "hyena_featurizer_fwd")
    return out


class ModalPlan:
    """Device-side coefficient tables of one modal filter bank (see hyena_li_plan)."""

    def __init__(self, log_poles, residues):
        _need_cuda(log_poles, residues)
        lp = log_poles.detach().reshape(log_poles.shape[0], -1)
        rs = residues.detach().reshape(residues.shape[0], -1)
        self.G, self.S = lp.shape
        self.is_complex = lp.is_complex() or rs.is_complex()

        def pairs(t):
            t = t.to(torch.complex64) if not t.is_complex() else t.to(torch.complex64)
            return torch.view_as_real(t.contiguous()).contiguous()

        self._lp, self._rs = pairs(lp), pairs(rs)
        nbytes = _lib.lib().hyena_li_plan_bytes(self.G, self.S)
        if nbytes <= 0:
            raise NotImplementedError(f"modal state size {self.S} is not supported (1..16)")
        self.workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=lp.device)
        rc = _lib.lib().hyena_li_plan(_ptr(self._lp), _ptr(self._rs), self.G, self.S, _ptr(self.workspace), _stream())
        _lib.check(rc, "hyena_li_plan")


def li_fwd_rows(x1r, x2r, vr, plan, Dcoef, B, D, L, *, device, want_state=False, want_fp32=False, out=None,
                single_rounding=False):
    if out is None:
        out = torch.empty((B, D, L), dtype=torch.bfloat16, device=device)
    y32 = torch.empty((B, D, L), dtype=torch.float32, device=device) if want_fp32 else None
    state = torch.zeros((B, D, plan.S, 2), dtype=torch.float32, device=device) if want_state else None
    if out.numel() == 0:
        if state is not None:
            state = torch.view_as_complex(state) if plan.is_complex else state[..., 0].contiguous()
        return out, y32, state
    dco = _f32(Dcoef)
    d_is_bf16 = 2 if single_rounding else int(Dcoef is None or Dcoef.dtype == torch.bfloat16)
    rc = _lib.lib().hyena_li_fwd(_ref(x1r), _ref(x2r), _ref(vr), _ptr(plan.workspace), _ptr(dco), d_is_bf16,
                                 _ptr(out), _ptr(y32), _ptr(state), B, D, L, plan.G, plan.S, _stream())
    _lib.check(rc, "hyena_li_fwd")
    if state is not None:
        state = torch.view_as_complex(state) if plan.is_complex else state[..., 0].contiguous()
    return out, y32, state


def projection_rows(p, hidden, *, interleave=False, head_dim=None):
    """Row descriptors (x2, x1, v) of a raw sequence-major projection p [B, 3*hidden, L] under the channel maps of
    vortex/model/utils.py:26-85, and the projection channel of every (gate, operator channel) as an int64 tensor
    [3, hidden] in the same (x2, x1, v) order.  interleave: projection channel 3*d + i; head_dim: the head-blocked
    column split; neither: the plain split i*hidden + d.  interleave with head_dim has no closed map (ValueError)."""
    if interleave and head_dim is not None:
        raise ValueError("interleave combined with column_split has no closed channel map")
    if p.dtype != torch.bfloat16 or p.dim() != 3 or p.stride(2) != 1:
        raise ValueError("expected a [B, 3D, L] bfloat16 tensor with contiguous samples")
    if p.shape[1] != 3 * hidden or (head_dim is not None and (head_dim <= 0 or hidden % head_dim)):
        raise ValueError(f"a [B, {3 * hidden}, L] projection and a head_dim that divides {hidden} are required "
                         f"(got {tuple(p.shape)}, head_dim={head_dim})")
    d = torch.arange(hidden, device=p.device)
    if interleave:
        es = p.element_size()
        rows = tuple(Rows(p.data_ptr() + i * p.stride(1) * es, p.stride(0), p.stride(1), 1, 3) for i in range(3))
        chan = torch.stack([3 * d + i for i in range(3)])
    elif head_dim is not None:
        rows = tuple(rows_of_projection(p, hidden, i, head_dim) for i in range(3))
        chan = torch.stack([(d // head_dim) * 3 * head_dim + d % head_dim + i * head_dim for i in range(3)])
    else:
        rows = tuple(rows_of_projection(p, hidden, i) for i in range(3))
        chan = torch.stack([d + i * hidden for i in range(3)])
    return rows, chan


def li_layer_fwd_rows(x1r, x2r, vr, feat_taps, plan, Dcoef, B, D, L, *, device, want_state=False, out=None,
                      single_rounding=False):
    """hyena_li_layer_fwd: featurizer FIR, gates and the modal scan in one pass over the rows of a raw sequence-major
    projection.  feat_taps [3, D, 3] float32: the featurizer weight rows of the x1, x2 and v row of every operator
    channel.  Returns (out [B, D, L] bf16, state or None) as li_fwd_rows does."""
    if out is None:
        out = torch.empty((B, D, L), dtype=torch.bfloat16, device=device)
    state = torch.zeros((B, D, plan.S, 2), dtype=torch.float32, device=device) if want_state else None
    if out.numel():
        if feat_taps.dtype != torch.float32 or not feat_taps.is_contiguous() or tuple(feat_taps.shape) != (3, D, 3):
            raise ValueError("feat_taps must be a contiguous float32 [3, D, 3] tensor")
        dco = _f32(Dcoef)
        d_is_bf16 = 2 if single_rounding else int(Dcoef is None or Dcoef.dtype == torch.bfloat16)
        rc = _lib.lib().hyena_li_layer_fwd(_ref(x1r), _ref(x2r), _ref(vr), _ptr(feat_taps), 3, _ptr(plan.workspace),
                                           _ptr(dco), d_is_bf16, _ptr(out), _ptr(state), B, D, L, plan.G, plan.S,
                                           _stream())
        _lib.check(rc, "hyena_li_layer_fwd")
    if state is not None:
        state = torch.view_as_complex(state) if plan.is_complex else state[..., 0].contiguous()
    return out, state


def hyena_li_fwd(x1, x2, v, log_poles, residues, D_bias=None, *, plan=None, want_state=False, want_fp32=False,
                 single_rounding=False):
    """Hyena-LI prefill on [B, D, L] bf16 gates with grouped modal parameters.

    log_poles [G, S, 1] (or [G, S]) and residues [G, S], float32 or complex64
    (vortex/model/model.py:202-209, :390-398).  Returns (out [B, D, L] bf16,
    y_conv fp32 or None, state [B, D, S] or None); the state is complex64 for complex
    poles and float32 for real ones (the real part, as vortex/model/engine.py:559 keeps).
    Pass a ModalPlan to reuse the coefficient tables between calls.  single_rounding=True computes
    z = bf16(conv + D*x1v) with one rounding instead of the three of the reference's bf16 tensor
    arithmetic (fewer vector instructions; within one bf16 ulp of the default).
    """
    _need_cuda(x1, x2, v, log_poles, residues)
    B, D, L = x1.shape
    if plan is None:
        plan = ModalPlan(log_poles, residues)
    (x1, pad), (x2, _), (v, _) = front_pad8(x1), front_pad8(x2), front_pad8(v)
    out, y32, state = li_fwd_rows(rows_of(x1), rows_of(x2), rows_of(v), plan, D_bias, B, D, L + pad, device=x1.device,
                                  want_state=want_state, want_fp32=want_fp32, single_rounding=single_rounding)
    if pad:
        out, y32 = out[..., pad:], (y32[..., pad:] if y32 is not None else None)
    return out, y32, state


class FirRing:
    """Ring-buffer FIR cache of R slots over D channels (bf16) plus the index of its oldest slot.

    Holds the same samples as the reference's [B, D, R] oldest-first fir_state
    (vortex/model/engine.py:414, :443-447); reference_order() returns that view.

    Built from the slots as a [B, R, D] tensor.  `buf` is the device layout [B, D/block, R, block]: block = D is
    that tensor itself (a view, so a caller's tensor is updated in place); block = 512 keeps the R slots of 512
    channels in one contiguous run, which the step kernel streams faster from deep caches.  block=None picks 512
    for caches of 32 slots and more whose D is a multiple of 512, and D otherwise.
    """

    def __init__(self, slots, pos=0, block=None):
        if slots.dtype != torch.bfloat16 or slots.dim() != 3:
            raise TypeError(f"the cache slots must be a [B, R, D] bfloat16 tensor, got {tuple(slots.shape)} {slots.dtype}")
        B, R, D = slots.shape
        if not 0 <= pos < max(R, 1):
            raise ValueError(f"oldest-slot index {pos} outside 0..{R - 1}")
        if block is None:
            block = 512 if (R >= 32 and D % 512 == 0 and D > 512) else D
        if block != D and (block % 512 or D % block):
            raise ValueError(f"block {block} must be D or a multiple of 512 that divides D={D}")
        self.B, self.R, self.D, self.block = B, R, D, block
        if block == D:
            self.buf = slots.contiguous().view(B, 1, R, D)
        else:
            self.buf = slots.reshape(B, R, D // block, block).permute(0, 2, 1, 3).contiguous()
        self.pos = pos              # oldest slot; with a far-sum stepper bound, a token counter modulo `period`
        self.period = R             # (then the oldest slot is pos % R)
        self.far_owner = None       # the FirStepper whose far sums are in step with this cache, if any
        self.pos_dev = None         # int32 [1] device tensor once a RingClock owns the position (then pos is stale)

    @classmethod
    def from_reference(cls, fir_state, block=None):
        """fir_state: [B, D, R] oldest-first (any float dtype holding bf16-exact values)."""
        return cls(fir_state.to(torch.bfloat16).permute(0, 2, 1).contiguous(), 0, block)

    @property
    def shape(self):   # what engine.step_fir reads as cache size: shape[-1]
        return torch.Size((self.B, self.D, self.R))

    def slots(self):
        """The slots as [B, R, D] in storage order (slot `pos` is the oldest); a view for block = D."""
        return self.buf.permute(0, 2, 1, 3).reshape(self.B, self.R, self.D)

    def reference_order(self, dtype=torch.float32):
        pos = self.pos if self.pos_dev is None else int(self.pos_dev.item())
        idx = (torch.arange(self.R, device=self.buf.device) + pos) % self.R
        return self.slots().index_select(1, idx).permute(0, 2, 1).to(dtype)


def fir_step(x1, ring, w, *, x2=None, v=None, bias=None, gated_bias=False):
    """One decode step of a FIR over its ring cache, fused with the gates.

    x1 (and x2, v): [B, D] bf16.  w: [G, R+1] float32, oldest tap first, the last
    column on the new sample.  Updates `ring` in place and returns y [B, D] bf16.
    """
    _need_cuda(x1, ring.buf, w)
    B, D = x1.shape
    R = ring.R
    if ring.D != D:
        raise ValueError(f"cache over {ring.D} channels, gates over {D}")
    w = _step_taps(w, D)
    G = w.shape[0]
    if w.shape[1] != R + 1:
        raise ValueError(f"taps have {w.shape[1]} columns, cache depth {R} needs {R + 1}")
    for t in (x1, x2, v):
        if t is not None and (t.dtype != torch.bfloat16 or t.stride(1) != 1 or t.stride(0) != x1.stride(0)):
            raise ValueError("gates must be bf16 [B, D] with unit channel stride and equal batch strides")
    out = torch.empty((B, D), dtype=torch.bfloat16, device=x1.device)
    b = _f32(bias)
    mode = HYENA_BIAS_NONE if b is None else (HYENA_BIAS_GATED_FP32 if gated_bias else HYENA_BIAS_ADD)
    if ring.pos_dev is not None:                # the position is on a RingClock, which also advances it
        ring.far_owner = None
        rc = _lib.lib().hyena_fir_step_dpos(_ptr(x1), _ptr(x2), _ptr(v), x1.stride(0), _ptr(ring.buf), R, ring.block,
                                            _ptr(ring.pos_dev), _ptr(w), _ptr(b), mode, _ptr(out), out.stride(0),
                                            B, D, G, _stream())
        _lib.check(rc, "hyena_fir_step_dpos")
        return out
    rc = _lib.lib().hyena_fir_step(_ptr(x1), _ptr(x2), _ptr(v), x1.stride(0), _ptr(ring.buf), R, ring.block,
                                   ring.pos % R, _ptr(w), _ptr(b), mode, _ptr(out), out.stride(0), B, D, G, _stream())
    _lib.check(rc, "hyena_fir_step")
    ring.pos = (ring.pos + 1) % ring.period
    ring.far_owner = None           # a stepper with far sums bound to this cache has to rebuild them
    return out


def iir_step(x1, x2, v, state, poles, residues, Dcoef, *, out_dtype=torch.bfloat16):
    """One decode step of the modal IIR, fused with the gates; `state` is updated in place.

    state: [B, D, S] float32 or complex64.  poles (exponentiated) and residues:
    [G, S] of the same kind.  Dcoef: [D] bf16 or float32 (its dtype selects the
    rounding of Dcoef*x1v, as torch promotion does in vortex/model/engine.py:465).
    """
    _need_cuda(x1, x2, v, state, poles, residues, Dcoef)
    B, D = x1.shape
    cplx = state.is_complex()
    if not state.is_contiguous():
        raise ValueError("state must be contiguous")
    S = state.shape[-1]

    def flat(t):
        t = t.detach()
        if cplx:
            t = torch.view_as_real(t.to(torch.complex64).contiguous())
        return _f32(t)

    p, r = flat(poles), flat(residues)
    G = poles.shape[0]
    st = torch.view_as_real(state) if cplx else state
    if st.dtype != torch.float32:
        raise TypeError("state must be float32 or complex64")
    out = torch.empty((B, D), dtype=out_dtype, device=x1.device)
    dco = _f32(Dcoef)
    rc = _lib.lib().hyena_iir_step(_ptr(x1), _ptr(x2), _ptr(v), x1.stride(0), _ptr(st), _ptr(p), _ptr(r), int(cplx),
                                   _ptr(dco), int(Dcoef.dtype == torch.bfloat16), _ptr(out),
                                   int(out_dtype == torch.float32), out.stride(0), B, D, G, S, _stream())
    _lib.check(rc, "hyena_iir_step")
    return out


def _step_taps(w, D):
    """Taps [G, R+1] in the form hyena_fir_step takes: shared by groups of 8, 16, ... 512 channels (a divisor of
    512), or one row per channel; other group sizes are expanded to per-channel rows here."""
    w = _f32(w)
    G = w.shape[0]
    dg = D // G
    if G != D and not (dg % 8 == 0 and 512 % dg == 0):
        w = w.repeat_interleave(dg, 0).contiguous()
    return w


class FirStepper:
    """A decode FIR step with every argument except the gates bound once (low host overhead).

    far_sums (default: caches of 32 slots and more): the step reads about a third of the cache per token by
    forming, three tokens at a time, what the cached samples add to the next outputs (hyena_fir_step_far; same result up
    to the order of the float32 sums).  The stepper owns the far-sum buffer, which belongs to this (cache, taps) pair;
    if anything else steps the cache in between, the next call rebuilds it."""

    def __init__(self, ring, w, bias=None, gated_bias=False, gated=True, far_sums=None):
        _need_cuda(ring.buf, w)
        self.ring, self.bias = ring, _f32(bias)
        self.R, self.D = ring.R, ring.D
        self.w = _step_taps(w, self.D)
        self.G = self.w.shape[0]
        if self.w.shape[1] != self.R + 1:
            raise ValueError(f"taps have {self.w.shape[1]} columns, cache depth {self.R} needs {self.R + 1}")
        self.mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_FP32 if gated_bias else HYENA_BIAS_ADD)
        self.gated = gated
        L = _lib.lib()
        self._fn, self._fn_dpos, self._fn_far = L.hyena_fir_step, L.hyena_fir_step_dpos, L.hyena_fir_step_far
        if far_sums is None:
            far_sums = self.R >= 32
        self.far = None
        if far_sums:
            if self.R < 32:
                raise ValueError("far sums are for caches of 32 slots and more")
            if ring.pos_dev is not None:
                raise RuntimeError("bind the stepper before the cache goes on a RingClock")
            self.far = torch.empty(L.hyena_fir_far_bytes(ring.B, self.D) // 4, dtype=torch.float32, device=ring.buf.device)
            ring.period = L.hyena_fir_far_period(self.R)

    def far_rebuild(self):
        """1 when this call has to rebuild the far sums (first step, or something else stepped the cache); claims the cache."""
        if self.ring.far_owner is self:
            return 0
        self.ring.far_owner = self
        return 1

    def __call__(self, x1, x2, v, out, far=True):
        """far=False: this token reads the whole cache even if the stepper keeps far sums (which the next far step
        then rebuilds); for callers that change `w` between tokens."""
        B = x1.shape[0]
        ring = self.ring
        dpos = ring.pos_dev is not None
        if self.far is not None and far:
            rc = self._fn_far(
                x1.data_ptr(), x2.data_ptr() if self.gated else None, v.data_ptr() if self.gated else None,
                x1.stride(0), ring.buf.data_ptr(), self.R, ring.block, 0 if dpos else ring.pos,
                ring.pos_dev.data_ptr() if dpos else None, self.far.data_ptr(), self.far_rebuild(), self.w.data_ptr(),
                self.bias.data_ptr() if self.bias is not None else None, self.mode, out.data_ptr(),
                out.stride(0), B, self.D, self.G, torch.cuda.current_stream().cuda_stream)
        else:
            ring.far_owner = None
            rc = (self._fn_dpos if dpos else self._fn)(
                x1.data_ptr(), x2.data_ptr() if self.gated else None, v.data_ptr() if self.gated else None,
                x1.stride(0), ring.buf.data_ptr(), self.R, ring.block,
                ring.pos_dev.data_ptr() if dpos else ring.pos % self.R,
                self.w.data_ptr(), self.bias.data_ptr() if self.bias is not None else None, self.mode, out.data_ptr(),
                out.stride(0), B, self.D, self.G, torch.cuda.current_stream().cuda_stream)
        if rc:
            _lib.check(rc, "hyena_fir_step")
        if not dpos:
            ring.pos = (ring.pos + 1) % ring.period
        return out


class IirStepper:
    """A decode modal-IIR step with the state and modal parameters bound once.

    windowed=True (16 states; otherwise ignored): the state tensor is read and written once per window of four tokens
    instead of every token (hyena_iir_step_win; same outputs up to float32 rounding).  Between windows the state
    tensor lags the tokens by up to four inputs: call flush() before anything else reads it.  The stepper then also
    counts tokens (`pos`, `period`, `pos_dev`), so it can go on a RingClock like a cache."""

    def __init__(self, state, poles, residues, Dcoef, windowed=False):
        _need_cuda(state, poles, residues, Dcoef)
        self.cplx = state.is_complex()
        flat = (lambda t: _f32(torch.view_as_real(t.detach().to(torch.complex64).contiguous()))) if self.cplx \
            else (lambda t: _f32(t.detach()))
        self.state = state
        self.st = torch.view_as_real(state) if self.cplx else state
        self.p, self.r = flat(poles), flat(residues)
        self.dco, self.d_is_bf16 = _f32(Dcoef), int(Dcoef.dtype == torch.bfloat16)
        self.G, self.S = poles.shape[0], state.shape[-1]
        self.D = state.shape[1]
        L = _lib.lib()
        self._fn = L.hyena_iir_step
        self.win = None
        self.pos_dev, self._recorded, self.warm = None, False, 0
        B = state.shape[0]
        if windowed and L.hyena_iir_window_supported(B, self.D, self.S, int(self.cplx)):
            W = L.hyena_iir_window_tokens()
            dev = state.device
            pk = poles.detach().to(torch.complex128 if self.cplx else torch.float64)
            rk = residues.detach().to(pk.dtype)
            g = torch.stack([(rk * pk ** k).real.sum(-1) if self.cplx else (rk * pk ** k).sum(-1) for k in range(W)], -1)
            self._g = g.to(torch.float32).contiguous()
            self._hist = torch.zeros(B, W, self.D, dtype=torch.bfloat16, device=dev)
            self._far = torch.zeros(B, W, self.D, dtype=torch.float32, device=dev)
            self.win = _lib.IirWindow(self._hist.data_ptr(), self._far.data_ptr(), self._g.data_ptr(), 0, None, 0, 0)
            self._wref = ctypes.byref(self.win)
            self._fn_win, self._fn_flush = L.hyena_iir_step_win, L.hyena_iir_window_flush
            self.pos, self.period, self.pos_dev, self.warm = 0, W, None, 0
            self._recorded = False      # a stream capture has taken a step of this stepper (with `warm` baked in)

    def _window(self):
        """The window descriptor for this call; advances the host-side counters."""
        w = self.win
        if self.pos_dev is not None:
            # a recorded step replays this call with `warm` frozen: every window has to be open by then
            if torch.cuda.is_current_stream_capturing():
                if self.warm < self.period:
                    raise RuntimeError(f"step {self.period} tokens eagerly before recording the windowed modal step")
                self._recorded = True
            w.cnt, w.cnt_dev = 0, self.pos_dev.data_ptr()
        else:
            w.cnt, w.cnt_dev = self.pos, None
            self.pos = (self.pos + 1) % self.period
        w.warm = self.warm
        self.warm = min(self.warm + 1, self.period)
        return self._wref

    def __call__(self, x1, x2, v, out):
        B = x1.shape[0]
        stream = torch.cuda.current_stream().cuda_stream
        if self.win is not None:
            rc = self._fn_win(x1.data_ptr(), x2.data_ptr(), v.data_ptr(), x1.stride(0), self.st.data_ptr(),
                              self.p.data_ptr(), self.r.data_ptr(), int(self.cplx), self.dco.data_ptr(), self.d_is_bf16,
                              out.data_ptr(), int(out.dtype == torch.float32), out.stride(0), B, self.D, self.G, self.S,
                              self._window(), stream)
        else:
            rc = self._fn(x1.data_ptr(), x2.data_ptr(), v.data_ptr(), x1.stride(0), self.st.data_ptr(), self.p.data_ptr(),
                          self.r.data_ptr(), int(self.cplx), self.dco.data_ptr(), self.d_is_bf16, out.data_ptr(),
                          int(out.dtype == torch.float32), out.stride(0), B, self.D, self.G, self.S, stream)
        if rc:
            _lib.check(rc, "hyena_iir_step")
        return out

    def flush(self):
        """Folds the inputs of the open windows into the state tensor, which is exact afterwards (no-op for the plain
        stepper).  The next steps start new windows."""
        if self.win is None or self.warm == 0:
            return
        if self._recorded and self.pos_dev is not None:
            # the recorded launch has "every window open" in its arguments; after a flush it would fold inputs into
            # the state that the flush has folded already
            raise RuntimeError("a recorded token step replays this stepper with its windows open: release the "
                               "recording (RingClock.release / RecordedDecodeStep.release) before flushing, and "
                               "record again after at least `period` eager steps")
        w = self.win
        w.cnt, w.cnt_dev = (0, self.pos_dev.data_ptr()) if self.pos_dev is not None else (self.pos, None)
        w.warm = self.warm
        rc = self._fn_flush(self.st.data_ptr(), self.p.data_ptr(), self.r.data_ptr(), int(self.cplx), self.state.shape[0],
                            self.D, self.G, self.S, self._wref, torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "hyena_iir_window_flush")
        self.warm = 0

    def unwindow(self):
        """Back to the plain step (after a flush): for callers whose launch has no windowed form."""
        self.flush()
        self.win = None


def gate_channel_map(hidden, *, interleave=False, head_dim=None):
    """(ch_inner, ch_outer, gate_stride, ch_stride) of hyena_proj_step for a [.., 3*hidden] projection.

    interleave: vortex/model/utils.py:26-38 then the plain split; head_dim: the head-blocked
    column_split of utils.py:41-85.  The two together have no closed channel map (returns None).
    """
    if interleave and head_dim is not None:
        return None
    if interleave:
        return hidden, 0, 1, 3
    if head_dim is not None:
        return head_dim, 3 * head_dim, head_dim, 1
    return hidden, 0, hidden, 1


class LayerStepper:
    """One launch per Hyena layer and token: featurizer step, split, gates and the inner FIR / IIR step.

    feat_ring: FirRing over the 3D projection channels; feat_w [3D, Rf+1] (oldest tap first), feat_bias [3D] or None.
    inner: a FirStepper or IirStepper already bound to the layer's inner cache / modal state.
    """

    def __init__(self, feat_ring, feat_w, feat_bias, channel_map, inner, flip_x1x2=False):
        _need_cuda(feat_ring.buf, feat_w)
        self.ring, self.inner = feat_ring, inner
        if feat_ring.block != feat_ring.D:
            raise ValueError("the featurizer cache must use the plain [B, R, 3D] layout (block = D)")
        self.Rf, C = feat_ring.R, feat_ring.D
        self.w = _f32(feat_w).reshape(C, self.Rf + 1).t().contiguous()        # tap-major [Rf+1, C]
        self.bias = _f32(feat_bias)
        ci, co, gs, cs = channel_map
        self.proj = ProjStep(None, 0, feat_ring.buf.data_ptr(), self.Rf, 0, self.w.data_ptr(),
                             self.bias.data_ptr() if self.bias is not None else None, ci, co, gs, cs, int(flip_x1x2))
        self._pref = ctypes.byref(self.proj)
        self.is_fir = isinstance(inner, FirStepper)
        self._fn = _lib.lib().hyena_fir_layer_step if self.is_fir else _lib.lib().hyena_iir_layer_step
        self._fn_dpos = _lib.lib().hyena_fir_layer_step_dpos
        self._fn_far = _lib.lib().hyena_fir_layer_step_far
        self._fn_win = _lib.lib().hyena_iir_layer_step_win
        if not self.is_fir and inner.win is not None:
            # the windowed modal step needs a featurizer map with 16-byte pieces (unit-stride or interleaved)
            D = inner.D
            vec = (cs == 1 and ci % 8 == 0 and co % 8 == 0 and gs % 8 == 0) or (cs == 3 and gs == 1 and ci >= D)
            if not vec or D % 8 or feat_ring.buf.data_ptr() % 16 or self.w.data_ptr() % 16:
                inner.unwindow()

    def __call__(self, u, out):
        """u: [B, 3D] bf16 with contiguous channels; out: [B, D] bf16 (float32 allowed for the IIR step)."""
        B = u.shape[0]
        p, n = self.proj, self.inner
        dpos = self.ring.pos_dev is not None
        if (self.is_fir and (n.ring.pos_dev is not None) != dpos) or \
                (not self.is_fir and n.win is not None and (n.pos_dev is not None) != dpos):
            raise RuntimeError("the featurizer cache and the inner cache / windowed state must both be on a RingClock, "
                               "or neither")
        p.u, p.u_batch_stride = u.data_ptr(), u.stride(0)
        p.pos, p.pos_dev = (0, self.ring.pos_dev.data_ptr()) if dpos else (self.ring.pos, None)
        stream = torch.cuda.current_stream().cuda_stream
        if self.is_fir and n.far is not None:
            rc = self._fn_far(self._pref, n.ring.buf.data_ptr(), n.R, n.ring.block, 0 if dpos else n.ring.pos,
                              n.ring.pos_dev.data_ptr() if dpos else None, n.far.data_ptr(), n.far_rebuild(),
                              n.w.data_ptr(), n.bias.data_ptr() if n.bias is not None else None, n.mode,
                              out.data_ptr(), out.stride(0), B, n.D, n.G, stream)
        elif self.is_fir and dpos:
            n.ring.far_owner = None
            rc = self._fn_dpos(self._pref, n.ring.buf.data_ptr(), n.R, n.ring.block, n.ring.pos_dev.data_ptr(), n.w.data_ptr(),
                               n.bias.data_ptr() if n.bias is not None else None, n.mode, out.data_ptr(),
                               out.stride(0), B, n.D, n.G, stream)
        elif self.is_fir:
            n.ring.far_owner = None
            rc = self._fn(self._pref, n.ring.buf.data_ptr(), n.R, n.ring.block, n.ring.pos % n.R, n.w.data_ptr(),
                          n.bias.data_ptr() if n.bias is not None else None, n.mode, out.data_ptr(), out.stride(0),
                          B, n.D, n.G, stream)
        elif n.win is not None:
            rc = self._fn_win(self._pref, n.st.data_ptr(), n.p.data_ptr(), n.r.data_ptr(), int(n.cplx), n.dco.data_ptr(),
                              n.d_is_bf16, out.data_ptr(), int(out.dtype == torch.float32), out.stride(0), B, n.D, n.G,
                              n.S, n._window(), stream)
        else:
            rc = self._fn(self._pref, n.st.data_ptr(), n.p.data_ptr(), n.r.data_ptr(), int(n.cplx), n.dco.data_ptr(),
                          n.d_is_bf16, out.data_ptr(), int(out.dtype == torch.float32), out.stride(0), B, n.D, n.G,
                          n.S, stream)
        if rc:
            _lib.check(rc, "hyena_fir_layer_step" if self.is_fir else "hyena_iir_layer_step")
        if not dpos:
            self.ring.pos = (self.ring.pos + 1) % self.Rf
            if self.is_fir:
                n.ring.pos = (n.ring.pos + 1) % n.ring.period
        return out


class RingClock:
    """Keeps the positions of a set of FirRing caches in device memory and moves them all on with one launch per
    token (hyena_ring_advance), so that a recorded token step (a HIP graph) can be replayed: the step kernels then
    read their ring positions from the device instead of taking them as scalar arguments.

    While a ring is on the clock its host-side `pos` is stale; release() writes the positions back."""

    def __init__(self, rings):
        self.rings = list(rings)
        if not self.rings:
            raise ValueError("no rings")
        dev = self.rings[0].buf.device if hasattr(self.rings[0], "buf") else self.rings[0].state.device
        if any(r.pos_dev is not None for r in self.rings):
            raise RuntimeError("a ring is already on a clock")
        self.pos = torch.tensor([r.pos for r in self.rings], dtype=torch.int32, device=dev)
        self.depth = torch.tensor([r.period for r in self.rings], dtype=torch.int32, device=dev)
        for i, r in enumerate(self.rings):
            r.pos_dev = self.pos[i:i + 1]

    def advance(self):
        rc = _lib.lib().hyena_ring_advance(self.pos.data_ptr(), self.depth.data_ptr(), len(self.rings), _stream())
        _lib.check(rc, "hyena_ring_advance")

    def release(self):
        for r, p in zip(self.rings, self.pos.tolist()):
            r.pos, r.pos_dev = p, None
            if hasattr(r, "_recorded"):
                r._recorded = False     # recordings made on this clock must not be replayed any more


class DecodeLayerSet:
    """Cached decode step of one [Hyena-SE, Hyena-MR, Hyena-LI] layer set: three fused launches.

    window_state: the Hyena-LI step keeps its modal state in windows of several tokens where the library has that form
    (IirStepper windowed=True): state_li then lags the tokens until flush().  far_sums: as in FirStepper, for the
    Hyena-MR cache (None: the default for its depth; False: the whole cache on every token).  With both False every
    kernel runs the reference's own algorithm."""

    def __init__(self, ring_se, w_se, ring_mr, w_mr, D_mr, state_li, poles, residues, D_li, window_state=True,
                 far_sums=None):
        self.se = FirStepper(ring_se, w_se)
        self.mr = FirStepper(ring_mr, w_mr, bias=D_mr, gated_bias=True, far_sums=far_sums)
        self.li = IirStepper(state_li, poles, residues, D_li, windowed=window_state)
        B, D = state_li.shape[0], state_li.shape[1]
        self.out = [torch.empty(B, D, dtype=torch.bfloat16, device=state_li.device) for _ in range(3)]

    def __call__(self, g_se, g_mr, g_li):
        """Each argument is (x2, x1, v), bf16 [B, D]; returns the three outputs."""
        self.se(g_se[1], g_se[0], g_se[2], self.out[0])
        self.mr(g_mr[1], g_mr[0], g_mr[2], self.out[1])
        self.li(g_li[1], g_li[0], g_li[2], self.out[2])
        return self.out

    def flush(self):
        """Brings state_li up to the last token (no-op without windows)."""
        self.li.flush()
