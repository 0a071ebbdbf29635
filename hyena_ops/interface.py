"""Functional signatures of vortex/ops/hyena_se/interface.py on the gfx950 kernels.

The gate-conv-gate operator y = q * conv(h, k * x) with a grouped depthwise causal
filter, in the three layouts the reference accepts.  Arithmetic is the engine's:
k*x rounded to bf16, fp32 accumulation, the convolution rounded to bf16, then the
output gate (vortex/model/engine.py:159, :197-208, :232).  Forward only.
"""
import warnings
from dataclasses import dataclass

import torch

from vortex_amd import ops
from vortex_amd._lib import (HYENA_BIAS_ADD, HYENA_BIAS_ADD_FP32, HYENA_BIAS_GATED_BF16, HYENA_BIAS_GATED_FP32,
                             HYENA_BIAS_NONE)

from .kernel_utils import BwdKernelConfig, FwdKernelConfig  # noqa: F401
from .utils import correction_toeplitz, toeplitz


@dataclass(eq=False)
class DefaultTwoPassChunkedGateConvGateFwdConfig(FwdKernelConfig):
    """vortex/ops/hyena_se/interface.py:27-34: the forward record `two_pass_chunked_gate_conv_gate` falls back to."""
    schedule: str = "default"
    autotune: bool = True
    CHUNK_SIZE: int = 128
    BLOCK_D: int = 32
    THREADBLOCK_SWIZZLE: str = "row"


@dataclass(eq=False)
class DefaultTwoPassChunkedGateConvGateBwdConfig(BwdKernelConfig):
    """vortex/ops/hyena_se/interface.py:36-44 (carried for callers that name it; this build is forward only)."""
    schedule: str = "default"
    autotune: bool = True
    CHUNK_SIZE: int = 128
    BLOCK_D: int = 32
    THREADBLOCK_SWIZZLE: str = "row"
    LOAD_TOEPLITZ: bool = False
    LOAD_BX_LAG: bool = False


def reshape_inputs(x, k, q, num_groups, input_layout, inner_layout):
    """The three feature groups from `input_layout` to `inner_layout` (vortex/ops/hyena_se/interface.py:272-319).

    Layouts: "bdl" [B, D, L], "blgdg" [B, L, G, dg], "bgdgl" [B, G, dg, L], channel d = g*dg + j.  The pairs the
    reference takes: bdl -> bdl | blgdg, blgdg -> bdl | bgdgl, bgdgl -> bdl | bgdgl (its bgdgl -> bdl branch names
    undefined variables, interface.py:309-311; the rearrangement it spells is done here).  Views where torch allows."""
    def one(t):
        if input_layout == "bdl":
            b, d, l = t.shape
            if inner_layout == "bdl":
                return t
            if inner_layout == "blgdg":
                return t.transpose(1, 2).reshape(b, l, num_groups, d // num_groups)
            raise NotImplementedError("inner_layout must be bdl or blgdg")
        if input_layout == "blgdg":
            b, l, g, dg = t.shape
            assert g == num_groups, "number of groups in feature groups and filter must match"
            if inner_layout == "bdl":
                return t.permute(0, 2, 3, 1).reshape(b, g * dg, l)
            if inner_layout == "bgdgl":
                return t.permute(0, 2, 3, 1)
            raise NotImplementedError("inner_layout must be bdl or bgdgl")
        if input_layout == "bgdgl":
            b, g, dg, l = t.shape
            assert g == num_groups, "number of groups in feature groups and filter must match"
            if inner_layout == "bdl":
                return t.reshape(b, g * dg, l)
            if inner_layout == "bgdgl":
                return t
            raise NotImplementedError("inner_layout must be bdl or bgdgl")
        raise NotImplementedError("input_layout must be bdl, blgdg or bgdgl")
    return one(x), one(k), one(q)


def reshape_outputs(y, num_groups, output_layout, inner_layout):
    """The operator output from `inner_layout` ("bdl" or "blgdg") to `output_layout` ("bld", "bdl", "blgdg")
    (vortex/ops/hyena_se/interface.py:322-339)."""
    if inner_layout == "bdl":
        b, d, l = y.shape
        if output_layout == "bld":
            return y.transpose(1, 2)
        if output_layout == "blgdg":
            return y.reshape(b, num_groups, d // num_groups, l).permute(0, 3, 1, 2)
        if output_layout == "bdl":
            return y
        raise NotImplementedError("output_layout must be bld, bdl or blgdg")
    if inner_layout == "blgdg":
        b, l, g, dg = y.shape
        if output_layout == "bld":
            return y.reshape(b, l, g * dg)
        if output_layout == "blgdg":
            return y
        raise NotImplementedError("output_layout must be bld or blgdg")
    raise NotImplementedError("inner_layout must be bdl or blgdg")


def gate_gate(x, k, q):
    """vortex/ops/hyena_se/interface.py:771-773: the operator with the convolution left out."""
    return x * k * q


def _to_bdl(t, layout):
    if layout == "bdl":
        return t
    if layout == "blgdg":
        b, l, g, dg = t.shape
        return t.reshape(b, l, g * dg).transpose(1, 2).contiguous()
    if layout == "bgdgl":
        b, g, dg, l = t.shape
        return t.reshape(b, g * dg, l)
    raise NotImplementedError("input_layout must be bdl, blgdg or bgdgl")


def _from_bdl(y, layout, num_groups):
    b, d, l = y.shape
    if layout == "bdl":
        return y
    if layout == "bld":
        return y.transpose(1, 2)
    if layout == "blgdg":
        return y.transpose(1, 2).reshape(b, l, num_groups, d // num_groups)
    raise NotImplementedError("output_layout must be bld, bdl or blgdg")


def _gcg(x, k, q, h, bias, apply_gated_bias):
    """q * conv(k*x) on [B, D, L] bf16 tensors; h [G, 1, K] in the F.conv1d orientation."""
    B, D, L = x.shape
    taps = ops._f32(h).reshape(h.shape[0], -1)
    K = taps.shape[1]
    mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_FP32 if apply_gated_bias else HYENA_BIAS_ADD)
    (x, pad), (k, _), (q, _) = ops.front_pad8(x), ops.front_pad8(k), ops.front_pad8(q)     # any length, any strides
    y = ops.fir_fwd_rows(ops.rows_of(x), ops.rows_of(q), ops.rows_of(k), taps, B, D, L + pad, K, device=x.device,
                         bias=ops._f32(bias), bias_mode=mode, taps_reversed=True,
                         force_mfma=(K > 8 or mode == HYENA_BIAS_GATED_FP32))
    return y[..., pad:] if pad else y


_WIDE = (torch.float16, torch.float32)      # element types that always run channel-last (hyena_fir_cl_fwd_dtype)


def _cl_ok(x, h):
    """Whether a channel-last kernel covers (b, l, g, dg) inputs with this filter: the MFMA kernel needs filter
    groups of a multiple of 16 channels; float16 / float32 tensors also have a direct-form kernel for any group."""
    return x.dim() == 4 and h.shape[-1] <= 128 and (x.shape[3] % 16 == 0 or x.dtype in _WIDE)


def _to_bld(t, layout):
    """[B, L, D] with contiguous channels from any input layout (a view for blgdg, a transposing copy otherwise)."""
    if layout == "blgdg":
        b, l, g, dg = t.shape
        return t.reshape(b, l, g * dg)
    return _to_bdl(t, layout).transpose(1, 2).contiguous()


def _from_bld(y, layout, num_groups):
    b, l, d = y.shape
    if layout == "bld":
        return y
    if layout == "blgdg":
        return y.reshape(b, l, num_groups, d // num_groups)
    if layout == "bdl":
        return y.transpose(1, 2)
    raise NotImplementedError("output_layout must be bld, bdl or blgdg")


def _gcg_wide(x, k, q, taps, bias, mode, input_layout, output_layout, num_groups):
    """q * fir(k * x) for float16 / float32 tensors in any layout, through the channel-last kernels.  taps [G', K]
    float32 in the F.conv1d orientation; q, k None for the ungated FIR."""
    if taps.shape[1] > 128:
        raise NotImplementedError("filters longer than 128 taps have no FIR kernel")
    xs = _to_bld(x, input_layout)
    ks = _to_bld(k, input_layout) if k is not None else None
    qs = _to_bld(q, input_layout) if q is not None else None
    y = ops.fir_cl_fwd(ks if ks is not None else xs, qs, xs if ks is not None else None, taps, bias=bias,
                       bias_mode=mode, taps_reversed=True)
    return _from_bld(y, output_layout, num_groups)


def _gcg_cl(x, k, q, h, bias, apply_gated_bias, want_y2=False, want_bx=False):
    """q * conv(k*x) on (b, l, g, dg) bf16 tensors without leaving the channel-last layout."""
    b, l, g, dg = x.shape
    taps = ops._f32(h).reshape(h.shape[0], -1)
    mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_FP32 if apply_gated_bias else HYENA_BIAS_ADD)
    flat = lambda t: t.reshape(b, l, g * dg)
    return ops.fir_cl_fwd(flat(k), flat(q), flat(x), taps, bias=ops._f32(bias), bias_mode=mode, taps_reversed=True,
                          want_y2=want_y2, want_bx=want_bx)


def inner_hyena_se(x, k, q, h, bias=None, input_layout="bdl", output_layout="bdl", inner_layout="bdl",
                   apply_gated_bias=False, schedule="default", autotune=False, fwd_kernel_cfg=None,
                   bwd_kernel_cfg=None, use_fast_causal_conv1d=False, kernel_path=None):
    """y = q * causal_depthwise_conv(h, k * x)  (vortex/ops/hyena_se/interface.py:342-397).

    h: [G, 1, K]; group g filters channels g*dg .. (g+1)*dg-1.  Layouts: "bdl" [B, D, L],
    "blgdg" [B, L, G, dg], "bgdgl" [B, G, dg, L] in; "bdl", "bld", "blgdg" out.  (b, l, g, dg) inputs
    with dg a multiple of 16 stay channel-last through the kernel; other cases go through [B, D, L].
    """
    G = h.shape[0]
    if x.dtype in _WIDE:
        assert k.shape == q.shape == x.shape, "feature groups must have the same shape"
        mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_FP32 if apply_gated_bias else HYENA_BIAS_ADD)
        return _gcg_wide(x, k, q, ops._f32(h).reshape(G, -1), ops._f32(bias), mode, input_layout, output_layout, G)
    if input_layout == "blgdg" and _cl_ok(x, h):
        assert k.shape == q.shape == x.shape, "feature groups must have the same shape"
        b, l, g, dg = x.shape
        y = _gcg_cl(x, k, q, h, bias, apply_gated_bias)
        if output_layout == "bld":
            return y
        if output_layout == "blgdg":
            return y.reshape(b, l, g, dg)
        if output_layout == "bdl":
            return y.transpose(1, 2)
        raise NotImplementedError("output_layout must be bld, bdl or blgdg")
    xb, kb, qb = (_to_bdl(t, input_layout) for t in (x, k, q))
    assert kb.shape == qb.shape == xb.shape, "feature groups must have the same shape"
    y = _gcg(xb, kb, qb, h, bias, apply_gated_bias)
    return _from_bdl(y, output_layout, G)


def _fir_per_channel(x, taps, q, k, bias, mode):
    """out = [q *] bias_rule(corr(taps, [k *] x)) on [B, D, L] bf16 with a tap table [G', K], G' in {1, D} or any
    divisor of D in the blocked map; the short kernel up to 8 taps, the MFMA kernel above."""
    B, D, L = x.shape
    K = taps.shape[1]
    if K > 128:
        raise NotImplementedError("filters longer than 128 taps have no FIR kernel")
    (x, pad), (k, _), (q, _) = ops.front_pad8(x), (ops.front_pad8(k) if k is not None else (None, 0)), \
        (ops.front_pad8(q) if q is not None else (None, 0))
    y = ops.fir_fwd_rows(ops.rows_of(x), ops.rows_of(q), ops.rows_of(k), taps, B, D, L + pad, K, device=x.device,
                         bias=bias, bias_mode=mode, taps_reversed=True, force_mfma=K > 8)
    return y[..., pad:] if pad else y


def _bias_rule(weight_dtype, bias, apply_gated_bias, D):
    """(bias [D] float32 or None, bias mode) for causal_conv1d_ref semantics (interface.py:228-243): the arithmetic
    runs in weight.dtype.  float32 weights: conv + bias, or conv + x*bias, formed in float32 and rounded once;
    bf16 weights: F.conv1d adds its bias before its single rounding, the gated bias is bf16 tensor arithmetic."""
    if bias is None:
        return None, HYENA_BIAS_NONE
    b = ops._f32(bias.reshape(-1))
    if b.numel() != D:
        raise ValueError(f"bias must have {D} elements ([D], or [D, 1] for a gated bias)")
    if not apply_gated_bias:
        return b, HYENA_BIAS_ADD_FP32
    # 16-bit weights: the gated bias is tensor arithmetic in that type (three roundings); float32: one float32 sum
    return b, (HYENA_BIAS_GATED_BF16 if weight_dtype in (torch.bfloat16, torch.float16) else HYENA_BIAS_GATED_FP32)


def causal_conv1d_ref(x, weight, bias=None, apply_gated_bias=False, return_final_states=False, final_states_out=None,
                      activation=None, *args, **kwargs):
    """Depthwise causal FIR without gates (vortex/ops/hyena_se/interface.py:207-244), any 1 <= K <= 128.

    x [B, D, L] bf16, weight [D, K] float32 or bf16 (weight[:, K-1] on the current sample); the result is rounded
    to bf16 once, after the bias: out = bf16(conv + bias[d]), or with apply_gated_bias bf16(conv + x*bias[d])
    (bf16 weights: bf16(bf16(conv) + bf16(x*bias[d])), the reference's bf16 tensor arithmetic).  A gated bias is
    [D, 1] in the reference (it multiplies x by plain broadcasting, interface.py:240); [D] is taken as the same
    per-channel coefficient here.  Other input dtypes and the silu activation have no kernel.
    """
    if activation is not None:
        raise NotImplementedError("activation is not supported")
    ops._need_cuda(x, weight)
    B, D, L = x.shape
    if weight.dim() != 2 or weight.shape[0] != D:
        raise ValueError("weight must be [D, K]")
    b, mode = _bias_rule(weight.dtype, bias, apply_gated_bias, D)
    if x.dtype in _WIDE:
        # the arithmetic runs in weight.dtype and the result returns to x.dtype (interface.py:228-243)
        if weight.dtype not in _WIDE:
            raise NotImplementedError("float16 / float32 activations need float16 or float32 weights")
        out = _gcg_wide(x.to(weight.dtype), None, None, ops._f32(weight), b, mode, "bdl", "bdl", D).to(x.dtype)
    else:
        out = _fir_per_channel(x, ops._f32(weight), None, None, b, mode)
    return out if not return_final_states else (out, final_states_out)


def inner_hyena_se_ref(x, k, q, h, bias=None, input_layout="bdl", output_layout="bdl", inner_layout="bdl",
                       apply_gated_bias=False, schedule="default", autotune=False, fwd_kernel_cfg=None,
                       bwd_kernel_cfg=None, use_fast_causal_conv1d=False, kernel_path="unfused_gcg_fast"):
    """y = q * causal_conv1d_ref(k * x) with the reference function's own filter-to-channel map
    (vortex/ops/hyena_se/interface.py:342-397).

    h: [G, 1, K].  Unlike inner_hyena_se (and the model path), this function assigns filters with
    `h.squeeze(1).repeat(d // G, 1)` (interface.py:375-376): channel c is filtered by h[c % G] -- striped, not
    blocked.  The kernels run it with one tap row per channel (a single shared row when G == 1).  Rounding
    follows causal_conv1d_ref (in h.dtype); up to 4 taps on the default kernel_path the reference calls the
    causal_conv1d extension, which accumulates conv + bias in float32 and takes no gated bias.
    """
    if inner_layout != "bdl":
        raise AssertionError("unfused_gcg only supports bdl inner layout")
    if kernel_path not in ("unfused_gcg", "unfused_gcg_fast"):
        raise NotImplementedError("Reference cgcg kernel path not integrated in hyena_se_ref")
    ops._need_cuda(x, k, q, h)
    G = h.shape[0]
    xb, kb, qb = (_to_bdl(t, input_layout) for t in (x, k, q))
    assert kb.shape == qb.shape == xb.shape, "feature groups must have the same shape"
    B, D, L = xb.shape
    if apply_gated_bias and kernel_path == "unfused_gcg_fast":
        warnings.warn("Gated bias not supported for unfused_gcg_fast kernel")
    taps = ops._f32(h).reshape(G, -1)
    K = taps.shape[1]
    if G not in (1, D):
        taps = taps.repeat(D // G, 1)                    # row c = h[c % G]
    if kernel_path == "unfused_gcg_fast" and K <= 4:
        b, mode = _bias_rule(torch.float32, bias, False, D)
    else:
        b, mode = _bias_rule(h.dtype, bias, apply_gated_bias, D)
    if xb.dtype in _WIDE:
        # k*x, the convolution (in h.dtype) and the q gate each rounded to the activations' type, as the reference's
        # tensor arithmetic rounds them; one tap row per channel, so this is the direct-form kernel
        if h.dtype == torch.bfloat16:
            raise NotImplementedError("float16 / float32 activations need float16 or float32 weights")
        return _gcg_wide(xb, kb, qb, taps, b, mode, "bdl", output_layout, G)
    y = _fir_per_channel(xb, taps, qb, kb, b, mode)
    return _from_bdl(y, output_layout, G)


def two_pass_chunked_gate_conv_gate(x, B, C, h, return_toeplitz=True, schedule="default", autotune=False,
                                    fwd_kernel_cfg=None, bwd_kernel_cfg=None):
    """y = C * conv(h, B * x) on (b, l, g, dg) tensors, h (g, 1, K)
    (vortex/ops/hyena_se/interface.py:170-204).  Forward only: no autograd graph is recorded."""
    return inner_hyena_se(x, B, C, h, input_layout="blgdg", output_layout="blgdg")


def _toeplitz_pair(h, chunk, dtype):
    """(T, T_hat) of the operator weights h (g, 1, K): the Toeplitz factors of hyena_ops.utils on hf = h.flip(-1),
    as vortex/ops/hyena_se/ref_fwd.py:216-266 builds them."""
    hf = h.reshape(h.shape[0], h.shape[-1]).flip(-1)
    return toeplitz(hf, chunk, dtype=dtype), correction_toeplitz(hf, chunk, dtype=dtype)


def two_pass_fwd_grouped(x, B, C, h, y=None, return_y2=False, return_toeplitz=False, return_bx_lag=False,
                         verbose=False, schedule="default", autotune=False, version="refactor", CHUNK_SIZE=None,
                         *args, **kwargs):
    """(y, T, T_hat, y2, bx_lag) of vortex/ops/hyena_se/fwd.py:17-43, :290 on (b, l, g, dg) tensors.

    y2 is the convolution before the C gate; bx_lag holds B*x for every chunk but the last (zeros there), as
    fwd_kernels.py:400-409 stores it; T, T_hat are the chunk Toeplitz factors (CHUNK_SIZE required, as in
    fwd.py:199-203).  The kernel itself is not chunk-parametrised; CHUNK_SIZE only shapes these by-products.
    """
    T = T_hat = y2 = bx_lag = None
    b, l, g, dg = x.shape
    if _cl_ok(x, h):
        res = _gcg_cl(x, B, C, h, None, False, want_y2=return_y2, want_bx=return_bx_lag)
        out, y2f, bxf = res if (return_y2 or return_bx_lag) else (res, None, None)
        out = out.reshape(b, l, g, dg)
        if return_y2:
            y2 = y2f.reshape(b, l, g, dg)
        if return_bx_lag:
            assert CHUNK_SIZE is not None, "CHUNK_SIZE must be specified for return_bx_lag"
            bxf[:, max(l - CHUNK_SIZE, 0):] = 0
            bx_lag = bxf.reshape(b, l, g, dg)
    else:
        if return_y2 or return_bx_lag:
            raise NotImplementedError("intermediates need group_dim % 16 == 0 and K <= 128")
        out = two_pass_chunked_gate_conv_gate(x, B, C, h)
    if return_toeplitz:
        assert CHUNK_SIZE is not None, "CHUNK_SIZE must be specified for return_toeplitz"
        T, T_hat = _toeplitz_pair(h, CHUNK_SIZE, x.dtype)
    if y is not None:
        y.copy_(out)
        out = y
    return out, T, T_hat, y2, bx_lag


def hyena_se(x, B, C, h, bias=None, apply_gated_bias=False, schedule="default", autotune=False, fwd_kernel_cfg=None,
             bwd_kernel_cfg=None):
    """vortex/ops/hyena_se/interface.py:247-269 (whose own body passes mismatched arguments);
    computes C * conv(h, B * x) + bias rule on (b, l, g, dg) tensors."""
    if _cl_ok(x, h):
        return _gcg_cl(x, B, C, h, bias, apply_gated_bias).reshape(x.shape)
    xb, kb, qb = (_to_bdl(t, "blgdg") for t in (x, B, C))
    return _from_bdl(_gcg(xb, kb, qb, h, bias, apply_gated_bias), "blgdg", h.shape[0])
