"""float16 and float32 tensors at the hyena_ops.interface seam.

The only parity grid the reference holds for two_pass_fwd_grouped runs in these two element types
(vortex/ops/hyena_se/tests/test_fwd.py:25-54: batch 2, seqlen 1024 and 8192, d = 4096, filters of 4, 32 and 128 taps,
inputs and filters drawn from N(0, 1) as in tests/utils.py:11-17, chunk size per tests/utils.py:128-134;
tests/test_two_pass_ref.py:17-51 adds 2 and 4 filter groups), each case compared with gcg_fwd_ref_corrected
(ref_fwd.py:80-127) at atol = rtol = 1e-2 (test_fwd.py:98-102).  The same shapes, distributions, outputs
(y, y2, T, T_hat, bx_lag) and tolerance here, against the oracle's restatement of that reference on the CPU.
float16 runs the MFMA kernel on float16 operands, float32 the direct-form kernel."""
import math

import pytest
import torch

from oracle import hyena_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
ATOL = RTOL = 1e-2          # vortex/ops/hyena_se/tests/test_fwd.py:98-102


def close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    err = (got - ref).abs()
    bad = err > ATOL + RTOL * ref.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} outside atol=rtol=1e-2, worst {err.max().item():.4f}"


def chunk_size(L, K):       # vortex/ops/hyena_se/tests/utils.py:128-134
    return 128 if L > 1024 else max(K, 32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("K", [4, 32, 128])
@pytest.mark.parametrize("g", [1, 2, 4])
@pytest.mark.parametrize("L", [1024, 8192])
def test_two_pass_fwd_grouped_reference_grid(L, g, K, dtype):
    from hyena_ops import interface as I
    bs, d = 2, 4096
    dg = d // g
    gen = torch.Generator().manual_seed(L + 7 * g + K)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    h = torch.randn(g * K, generator=gen).to(dtype).reshape(g, 1, K)
    CH = chunk_size(L, K)
    y_ref = O.gcg_fwd_ref(x, B, C, h)
    y2_ref = O.gcg_fwd_ref(x, B, torch.ones_like(C), h)             # the convolution before the C gate
    y, T, T_hat, y2, bx_lag = I.two_pass_fwd_grouped(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), return_y2=True,
                                                     return_toeplitz=True, return_bx_lag=True, CHUNK_SIZE=CH)
    for t in (y, y2, bx_lag, T, T_hat):
        assert t.dtype == dtype
    assert y.shape == x.shape and y2.shape == x.shape
    close(y, y_ref, "y")
    close(y2, y2_ref, "y2")
    hf = h.flip(-1)[:, 0]
    close(T, O.toeplitz(hf, CH), "T")
    close(T_hat, O.correction_toeplitz(hf, CH), "T_hat")
    bx_ref = (B * x).clone()
    bx_ref[:, L - CH:] = 0                                          # fwd_kernels.py:400-409: every chunk but the last
    assert torch.equal(bx_lag.cpu(), bx_ref)
    # the same call without intermediates, and the gate-conv-gate entry point
    close(I.two_pass_fwd_grouped(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV))[0], y_ref, "y (no intermediates)")
    if L == 1024:
        close(I.two_pass_chunked_gate_conv_gate(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV)), y_ref, "gate_conv_gate")
        if dtype == torch.float32:      # (in float16 the two references round B*x and the convolution differently)
            close(O.gcg_two_pass_chunked(x, B, C, h, CH), y_ref, "two-pass spec vs conv1d")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("bs,L,g,dg,K", [(1, 32, 1, 32, 4), (2, 32, 2, 32, 4),        # the reference's debug configs
                                         (2, 333, 3, 24, 7),                          # groups of 24 channels: direct form
                                         (1, 130, 5, 17, 128), (3, 257, 1, 1, 33)])   # odd widths, one channel
def test_small_and_ragged_shapes(bs, L, g, dg, K, dtype):
    from hyena_ops import interface as I
    gen = torch.Generator().manual_seed(L + K)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    h = (torch.randn(g, 1, K, generator=gen) / math.sqrt(K)).to(dtype)
    y_ref = O.gcg_fwd_ref(x, B, C, h)
    y, _, _, y2, _ = I.two_pass_fwd_grouped(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), return_y2=True)
    close(y, y_ref, "y")
    close(y2, O.gcg_fwd_ref(x, B, torch.ones_like(C), h), "y2")
    # float16 to the last digit: the rounding points of float16 tensor arithmetic (B*x, the convolution, the C gate)
    # around a float32 accumulation, evaluated here in float32 with explicit roundings (the CPU's own float16 conv1d
    # may accumulate in another precision)
    if dtype == torch.float16:
        z32 = O.gcg_fwd_ref((B * x).float(), torch.ones_like(x).float(), torch.ones_like(x).float(), h.float())
        z16 = z32.half()
        ref16 = (C * z16).float()
        ulp16 = lambda t: torch.pow(2.0, torch.floor(torch.log2(t.abs().clamp_min(2.0 ** -14))) - 10)
        assert bool(((y2.float().cpu() - z16.float()).abs() <= ulp16(z16.float())).all())
        assert bool(((y.float().cpu() - ref16).abs() <= ulp16(ref16) + C.float().abs() * ulp16(z16.float())).all())
    else:
        assert (y.cpu() - y_ref).abs().max() <= 1e-5 * y_ref.abs().max()


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("layout_in,layout_out", [("bdl", "bdl"), ("bdl", "bld"), ("blgdg", "bdl"), ("bgdgl", "blgdg")])
def test_inner_hyena_se_layouts(layout_in, layout_out, dtype):
    from hyena_ops import interface as I
    bs, L, g, dg, K = 2, 200, 4, 16, 7
    gen = torch.Generator().manual_seed(5)
    x, k, q = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    h = (torch.randn(g, 1, K, generator=gen) / math.sqrt(K)).to(dtype)
    bias = torch.randn(g * dg, generator=gen)
    ref = O.gcg_fwd_ref(x, k, q, h)                                                   # (b, l, g, dg)
    conv = {"bdl": lambda t: t.permute(0, 2, 3, 1).reshape(bs, g * dg, L), "blgdg": lambda t: t,
            "bgdgl": lambda t: t.permute(0, 2, 3, 1)}[layout_in]
    got = I.inner_hyena_se(conv(x).contiguous().to(DEV), conv(k).contiguous().to(DEV), conv(q).contiguous().to(DEV),
                           h.to(DEV), input_layout=layout_in, output_layout=layout_out)
    back = {"bdl": lambda t: t.reshape(bs, g, dg, L).permute(0, 3, 1, 2), "bld": lambda t: t.reshape(bs, L, g, dg),
            "blgdg": lambda t: t}[layout_out]
    assert got.dtype == dtype
    close(back(got), ref, f"{layout_in}->{layout_out}")
    # the reference function of the same file (striped filter map, arithmetic in h.dtype) and the ungated FIR
    xb, kb, qb = (t.permute(0, 2, 3, 1).reshape(bs, g * dg, L).contiguous() for t in (x, k, q))
    for gated in (False, True):
        b_arg = bias[:, None] if gated else bias
        ref_s = O.inner_hyena_se_ref(xb, kb, qb, h, bias=b_arg.to(dtype), apply_gated_bias=gated, kernel_path="unfused_gcg")
        got_s = I.inner_hyena_se_ref(xb.to(DEV), kb.to(DEV), qb.to(DEV), h.to(DEV), bias=b_arg.to(dtype).to(DEV),
                                     apply_gated_bias=gated, kernel_path="unfused_gcg")
        close(got_s, ref_s, f"inner_hyena_se_ref gated={gated}")
        w = h.squeeze(1).repeat(dg, 1)
        ref_c = O.causal_conv1d_ref(xb, w, b_arg.to(dtype), apply_gated_bias=gated)
        got_c = I.causal_conv1d_ref(xb.to(DEV), w.to(DEV), b_arg.to(dtype).to(DEV), apply_gated_bias=gated)
        assert got_c.dtype == dtype
        close(got_c, ref_c, f"causal_conv1d_ref gated={gated}")
