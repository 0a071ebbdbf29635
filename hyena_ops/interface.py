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
from vortex_amd._lib import HYENA_BIAS_ADD, HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE


@dataclass(eq=False)
class FwdKernelConfig:
    """Accepted for signature compatibility (vortex/ops/hyena_se/kernel_utils.py:326-335); the HIP
    kernels have fixed tiles, so every field is ignored."""
    schedule: str = "default"
    autotune: bool = False
    CHUNK_SIZE: int = 128
    BLOCK_D: int = 32
    THREADBLOCK_SWIZZLE: str = "row"
    RETURN_TOEPLITZ: bool = False


@dataclass(eq=False)
class BwdKernelConfig:
    """vortex/ops/hyena_se/kernel_utils.py:337-343; unused (forward only)."""
    schedule: str = "default"
    autotune: bool = False
    CHUNK_SIZE: int = 128
    BLOCK_D: int = 32
    LOAD_TOEPLITZ: bool = False


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
    return ops.fir_fwd_rows(ops.rows_of(x), ops.rows_of(q), ops.rows_of(k), taps, B, D, L, K, device=x.device,
                            bias=ops._f32(bias), bias_mode=mode, taps_reversed=True,
                            force_mfma=(K > 8 or mode == HYENA_BIAS_GATED_FP32))


def inner_hyena_se(x, k, q, h, bias=None, input_layout="bdl", output_layout="bdl", inner_layout="bdl",
                   apply_gated_bias=False, schedule="default", autotune=False, fwd_kernel_cfg=None,
                   bwd_kernel_cfg=None, use_fast_causal_conv1d=False, kernel_path=None):
    """y = q * causal_depthwise_conv(h, k * x)  (vortex/ops/hyena_se/interface.py:342-397).

    h: [G, 1, K]; group g filters channels g*dg .. (g+1)*dg-1.  Layouts: "bdl" [B, D, L],
    "blgdg" [B, L, G, dg], "bgdgl" [B, G, dg, L] in; "bdl", "bld", "blgdg" out.
    """
    G = h.shape[0]
    xb, kb, qb = (_to_bdl(t, input_layout) for t in (x, k, q))
    assert kb.shape == qb.shape == xb.shape, "feature groups must have the same shape"
    y = _gcg(xb, kb, qb, h, bias, apply_gated_bias)
    return _from_bdl(y, output_layout, G)


inner_hyena_se_ref = inner_hyena_se


def causal_conv1d_ref(x, weight, bias=None, apply_gated_bias=False, return_final_states=False, final_states_out=None,
                      activation=None, *args, **kwargs):
    """Depthwise causal FIR without gates (vortex/ops/hyena_se/interface.py:207-244).

    x [B, D, L] bf16, weight [D, K]; bias added after the bf16 rounding, or `+ x*bias` in fp32
    when apply_gated_bias.
    """
    if activation is not None:
        raise NotImplementedError("activation is not supported")
    B, D, L = x.shape
    K = weight.shape[-1]
    mode = HYENA_BIAS_NONE if bias is None else (HYENA_BIAS_GATED_FP32 if apply_gated_bias else HYENA_BIAS_ADD)
    if mode == HYENA_BIAS_GATED_FP32 or K > 8:
        raise NotImplementedError("ungated FIR with per-channel taps is limited to K <= 8 without gated bias")
    out = ops.fir_fwd_rows(ops.rows_of(x), None, None, ops._f32(weight).reshape(D, K), B, D, L, K, device=x.device,
                           bias=ops._f32(bias), bias_mode=mode, taps_reversed=True)
    return out if not return_final_states else (out, final_states_out)


def two_pass_chunked_gate_conv_gate(x, B, C, h, return_toeplitz=True, schedule="default", autotune=False,
                                    fwd_kernel_cfg=None, bwd_kernel_cfg=None):
    """y = C * conv(h, B * x) on (b, l, g, dg) tensors, h (g, 1, K)
    (vortex/ops/hyena_se/interface.py:170-204).  Forward only: no autograd graph is recorded."""
    return inner_hyena_se(x, B, C, h, input_layout="blgdg", output_layout="blgdg")


def two_pass_fwd_grouped(x, B, C, h, *args, **kwargs):
    """(y, T, T_hat, y2, bx_lag) of vortex/ops/hyena_se/fwd.py:17-43, :290 with the
    intermediates, which exist only for the backward pass, returned as None."""
    return two_pass_chunked_gate_conv_gate(x, B, C, h), None, None, None, None


def hyena_se(x, B, C, h, bias=None, apply_gated_bias=False, schedule="default", autotune=False, fwd_kernel_cfg=None,
             bwd_kernel_cfg=None):
    """vortex/ops/hyena_se/interface.py:247-269 (whose own body passes mismatched arguments);
    computes C * conv(h, B * x) + bias rule on (b, l, g, dg) tensors."""
    xb, kb, qb = (_to_bdl(t, "blgdg") for t in (x, B, C))
    return _from_bdl(_gcg(xb, kb, qb, h, bias, apply_gated_bias), "blgdg", h.shape[0])
