"""Pins the CPU oracle against what fixes it independently of its own formulas:
brute-force float64 loops, impulse responses, closed forms, the reference's
own known-answer tests, and cross-identities between its code paths."""
import math

import numpy as np
import pytest
import torch

from oracle import hyena_oracle as O


def brute_corr(u, w):
    """z[d,t] = sum_k w[d,k] u[d,t-(K-1)+k], float64 python loops."""
    D, L = u.shape
    K = w.shape[1]
    z = np.zeros((D, L))
    for d in range(D):
        for t in range(L):
            acc = 0.0
            for k in range(K):
                j = t - (K - 1) + k
                if j >= 0:
                    acc += w[d, k] * u[d, j]
            z[d, t] = acc
    return z


def brute_conv(u, h):
    """y[d,t] = sum_k h[d,k] u[d,t-k]"""
    D, L = u.shape
    K = h.shape[1]
    y = np.zeros((D, L))
    for d in range(D):
        for t in range(L):
            acc = 0.0
            for k in range(min(K, t + 1)):
                acc += h[d, k] * u[d, t - k]
            y[d, t] = acc
    return y


def test_orientation_known_answer():
    # cell 26 of the reference's test_log_analysis.ipynb: conv1d([0,1,2],[2,1,0]) = 1
    # (cross-correlation: no flip of the kernel)
    x = torch.tensor([[[0.0, 1.0, 2.0]]])
    w = torch.tensor([[[2.0, 1.0, 0.0]]])
    assert torch.nn.functional.conv1d(x, w).item() == 1.0
    # and the short FIR of the oracle puts w[K-1] on the current sample
    z = O.short_fir_fp32(torch.tensor([[[1.0, 0.0, 0.0, 0.0]]]), torch.tensor([[[5.0, 6.0, 7.0]]]), 3)
    assert z.flatten().tolist() == [7.0, 6.0, 5.0, 0.0]


@pytest.mark.parametrize("K", [3, 7, 16])
def test_short_fir_vs_bruteforce(K):
    g = torch.Generator().manual_seed(K)
    D, L = 6, 37
    u = torch.randn(1, D, L, generator=g)
    w = torch.randn(D, 1, K, generator=g)
    z = O.short_fir_fp32(u, w, K)[0].double().numpy()
    ref = brute_corr(u[0].double().numpy(), w[:, 0].double().numpy())
    np.testing.assert_allclose(z, ref, atol=1e-5)


def test_se_rounding_points():
    # u is rounded to bf16 before the FIR, z is rounded to bf16 before the gate
    x2, x1, v = O.make_gates(2, 32, 64, seed=1)
    h = O.make_se_filter(2, 7)
    out, st = O.se_fir(x2, x1, v, h)
    u = (x1.float() * v.float()).bfloat16()
    w = h.repeat_interleave(16, 0)[:, 0].double().numpy()
    z = np.stack([brute_corr(u[b].double().numpy(), w) for b in range(2)])
    zb = torch.from_numpy(z).float().bfloat16()
    exp = (x2.float() * zb.float()).bfloat16()
    # F.conv1d sums in another order than the loop: allow 1 bf16 ulp on z
    assert (out.float() - exp.float()).abs().max() <= 2 ** -7 * exp.float().abs().max()
    assert torch.equal(st, u[..., -6:])
    assert out.dtype == torch.bfloat16


def test_parallel_fir_matches_se_fir_and_splits():
    B, D, L, G = 2, 32, 48, 2
    g = torch.Generator().manual_seed(3)
    u = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    h = O.make_se_filter(G, 7).repeat_interleave(D // G, 0)
    dims = (D, 4, D // 4, 16, G)
    z, st = O.parallel_fir(u, h, None, L, dims, groups=G, dim_last=False, fir_length=7, gate=True, want_state=True)
    x2, x1, v = u.split(D, 1)
    out, st2 = O.se_fir(x2, x1, v, O.make_se_filter(G, 7))
    assert torch.equal(z, out) and torch.equal(st, st2)
    # column split: head h holds [x2 | x1 | v] of head_dim each
    zc, _ = O.parallel_fir(u, h, None, L, dims, groups=G, dim_last=False, fir_length=7, gate=True,
                           column_split_hyena=True)
    ur = u.reshape(B, 4, 3, D // 4, L)
    outc, _ = O.se_fir(ur[:, :, 0].reshape(B, D, L), ur[:, :, 1].reshape(B, D, L), ur[:, :, 2].reshape(B, D, L),
                       O.make_se_filter(G, 7))
    assert torch.equal(zc, outc)


def test_interleave_index_map():
    z = torch.arange(12.0).reshape(1, 12, 1)
    assert O.interleave(z).flatten().tolist() == [0, 3, 6, 9, 1, 4, 7, 10, 2, 5, 8, 11]
    assert O.interleave(z[..., 0]).flatten().tolist() == [0, 3, 6, 9, 1, 4, 7, 10, 2, 5, 8, 11]


def test_featurizer_fir_dim_last_and_bias():
    B, L, D3, K = 2, 20, 12, 3
    g = torch.Generator().manual_seed(5)
    u = torch.randn(B, L, D3, generator=g).bfloat16()
    w = torch.randn(D3, 1, K, generator=g)
    bias = torch.randn(D3, generator=g)
    z, st = O.parallel_fir(u, w, bias, L, None, fir_length=K, dim_last=True, gate=False, want_state=True)
    ut = u.permute(0, 2, 1)
    ref = np.stack([brute_corr(ut[b].double().numpy(), w[:, 0].double().numpy()) for b in range(B)])
    refb = torch.from_numpy(ref).float().bfloat16()
    exp = refb + bias[None, :, None]          # bf16 + fp32 -> fp32 (torch promotion)
    assert z.dtype == exp.dtype
    assert (z - exp).abs().max() <= 2 ** -7 * exp.abs().max()
    assert torch.equal(st, ut[..., -2:])


def ref_fftconv(x, h):
    # formula held by the reference's test/test_forward.py:13-23
    n = 2 * x.shape[-1]
    y = torch.fft.irfft(torch.fft.rfft(x.float(), n=n) * torch.fft.rfft(h.float(), n=n) / n, n=n, norm="forward")
    return y[..., : x.shape[-1]]


def test_fft_conv_vs_bruteforce_and_ref_fftconv():
    g = torch.Generator().manual_seed(7)
    D, L, K = 4, 50, 20
    u = torch.randn(1, D, L, generator=g)
    h = torch.randn(D, 1, K, generator=g)
    y = O.fft_causal_conv_fp32(u, h)
    ref = brute_conv(u[0].double().numpy(), h[:, 0].double().numpy())
    np.testing.assert_allclose(y[0].double().numpy(), ref, atol=2e-5)
    np.testing.assert_allclose(y.numpy(), ref_fftconv(u, h[:, 0][None]).numpy(), atol=1e-5)
    # impulse response: y = h
    e = torch.zeros(1, D, L)
    e[..., 0] = 1
    np.testing.assert_allclose(O.fft_causal_conv_fp32(e, h)[0, :, :K].numpy(), h[:, 0].numpy(), atol=1e-6)


def test_mr_is_true_convolution_with_fp32_bias():
    B, D, L, G, K = 1, 32, 256, 2, 128
    x2, x1, v = O.make_gates(B, D, L, seed=11)
    h = O.make_mr_filter(G, K)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(12))
    out, st = O.mr_fir(x2, x1, v, h, Db)
    u = (x1.float() * v.float()).bfloat16()
    w = h.repeat_interleave(D // G, 0)[:, 0].double().numpy()
    y = brute_conv(u[0].double().numpy(), w) + u[0].double().numpy() * Db.double().numpy()[:, None]
    zb = torch.from_numpy(y).float().bfloat16()
    exp = (x2[0].float() * zb.float()).bfloat16()
    assert (out[0].float() - exp.float()).abs().max() <= 2 ** -7 * exp.float().abs().max()
    assert torch.equal(st, u[..., -127:])
    # same thing as the short-FIR form on the flipped filter (orientation cross-check)
    z_corr = O.short_fir_fp32(u, h.flip(-1).repeat_interleave(D // G, 0), K)
    z_conv = O.fft_causal_conv_fp32(u.float(), h.repeat_interleave(D // G, 0))
    np.testing.assert_allclose(z_corr.numpy(), z_conv.numpy(), atol=2e-4)


def test_parallel_fir_k128_branch_equals_mr_fir():
    B, D, L, G, K = 2, 32, 160, 2, 128
    g = torch.Generator().manual_seed(13)
    u = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    h = O.make_mr_filter(G, K)
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, 4, D // 4, 16, G)
    z, st = O.parallel_fir(u, h.repeat_interleave(D // G, 0), Db, L, dims, groups=G, gated_bias=True,
                           dim_last=False, fir_length=K, gate=True, want_state=True)
    x2, x1, v = u.split(D, 1)
    out, st2 = O.mr_fir(x2, x1, v, h, Db)
    assert torch.equal(z, out) and torch.equal(st, st2)


def test_toeplitz_known_answer_arange():
    # vortex/ops/hyena_se/tests/test_toeplitz.py:33-66: h = arange, T built from the flipped filter
    for g, K, C in [(1, 4, 16), (2, 4, 32), (2, 128, 128)]:
        h = torch.arange(g * K).reshape(g, 1, K)
        hf = h[:, 0].flip(-1)
        T = O.toeplitz(hf, C)
        Th = O.correction_toeplitz(hf, C)
        for gi in range(g):
            for i in range(C):
                for j in range(C):
                    lag = i - j
                    exp = int(h[gi, 0, K - 1 - lag]) if 0 <= lag < K else 0
                    assert int(T[gi, i, j]) == exp
                    lag2 = i + C - j
                    exp2 = int(h[gi, 0, K - 1 - lag2]) if (j >= i and lag2 < K) else 0
                    assert int(Th[gi, i, j]) == exp2
            if g * K * C > 4096:
                break


@pytest.mark.parametrize("g,K", [(1, 4), (2, 128), (4, 128)])
def test_two_pass_equals_conv1d(g, K):
    # the identity asserted by the reference's test_two_pass_ref.py::test_ref_chunked_fwd (atol 1e-4)
    gen = torch.Generator().manual_seed(17)
    bs, L, dg = 2, 512, 16
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen) for _ in range(3))
    h = torch.randn(g, 1, K, generator=gen)
    y1 = O.gcg_fwd_ref(x, B, C, h)
    y2 = O.gcg_two_pass_chunked(x, B, C, h, L // 2)
    assert torch.allclose(y1, y2, atol=1e-4)
    y3 = O.gcg_two_pass_chunked(x, B, C, h, 128)
    assert torch.allclose(y1, y3, atol=1e-4)


def test_modal_filter_closed_forms():
    lp, r = O.make_modal_complex(3, 16, seed=5, pmax=0.99)
    L = 4096
    h = O.modal_filter(lp, r, L)[0]
    assert torch.allclose(h[:, 0], r.sum(1).real, atol=1e-5)
    p = lp[..., 0].to(torch.complex128).exp()
    geo = (r.to(torch.complex128) * (1 - p ** L) / (1 - p)).sum(1).real
    assert torch.allclose(h.double().sum(1), geo, atol=1e-3)
    lpr, rr = O.make_modal_real(3, 16, seed=6, pmax=0.99)
    hr = O.modal_filter(lpr, rr, L)[0]
    pr = lpr[..., 0].double().exp()
    assert torch.allclose(hr[:, 0], rr.sum(1), atol=1e-5)
    assert torch.allclose(hr.double().sum(1), (rr.double() * (1 - pr ** L) / (1 - pr)).sum(1), atol=1e-3)
    # t=1 term pins the sign/index of the exponent
    assert torch.allclose(hr[:, 1].double(), (rr.double() * pr).sum(1), atol=1e-5)


@pytest.mark.parametrize("cplx", [False, True])
def test_li_fft_equals_recurrence(cplx):
    # FFT long conv + FFT state == explicit modal recurrence (reference test/test_prefill.py:85-229)
    B, D, L, G = 2, 8, 192, 4
    x2, x1, v = O.make_gates(B, D, L, seed=21)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, 16, seed=22, pmax=0.99)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(23)).bfloat16()
    out, y32, state = O.li_prefill(x2, x1, v, lp, r, Db)
    x1v = x1 * v
    y_rec, s_rec = O.prefill_direct_recurrence(x1v, lp, r)
    assert (y32.double() - y_rec).abs().max() <= 1e-4 * y_rec.abs().max()
    assert (state.to(s_rec.dtype) - s_rec).abs().max() <= 1e-5 * s_rec.abs().max()
    # the reference's own FFT state path agrees with the closed form (imag dropped for real poles)
    h = O.modal_filter(lp, r, L)[0].repeat_interleave(D // G, 0)[None]
    _, X_s = O.long_conv_fp32(x1v, h)
    st_fft = O.modal_state_fft(X_s, lp, L, D, G, keep_complex=cplx)
    assert (st_fft.to(s_rec.dtype) - s_rec).abs().max() <= 1e-3 * s_rec.abs().max()
    # gate/cast order
    yb = y32.bfloat16()
    exp = (yb + x1v * Db[:, None]) * x2
    assert torch.equal(out, exp)


def test_parallel_iir_matches_li_prefill_when_G_equals_D():
    B, D, L = 1, 8, 64
    g = torch.Generator().manual_seed(31)
    z_pre = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    lp, r = O.make_modal_real(D, 16, seed=32, pmax=0.99)
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, 2, D // 2, 16, D)
    h = O.modal_filter(lp, r, L)
    y, st = O.parallel_iir(z_pre, h, Db, L, lp, r, dims, want_state=True)
    x2, x1, v = z_pre.split(D, 1)
    out, _, st2 = O.li_prefill(x2, x1, v, lp, r, Db)
    assert torch.equal(y, out.permute(0, 2, 1))
    assert torch.allclose(st, st2, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("K,flip,gated", [(7, False, False), (128, True, True), (3, False, False)])
def test_step_fir_consistent_with_prefill(K, flip, gated):
    # feeding tokens one at a time from the prefill tail reproduces prefill outputs
    B, D, L, n_dec = 2, 16, 160, 5
    g = torch.Generator().manual_seed(41 + K)
    u_all = torch.randn(B, D, L + n_dec, generator=g).bfloat16()
    w = torch.randn(D, 1, K, generator=g) / math.sqrt(K)
    bias = torch.randn(D, generator=g) if gated else None
    if K >= 128:
        full = O.fftconv_with_bias(u_all.float(), w.float(), bias.float()).to(u_all.dtype)
    else:
        full = O.short_fir_fp32(u_all, w, K).to(u_all.dtype)
    state = u_all[..., L - (K - 1): L]
    for i in range(n_dec):
        y, state = O.step_fir(u_all[..., L + i], state, w, bias=bias, gated_bias=gated, flip_filter=flip)
        assert y.dtype == torch.bfloat16 and state.dtype == torch.float32
        assert (y.float() - full[..., L + i].float()).abs().max() <= 2 ** -7 * full.float().abs().max()
        assert torch.equal(state, u_all[..., L + i + 1 - (K - 1): L + i + 1].float())


def test_step_fir_partial_cache_growth():
    # cache shorter than K-1: state is appended, taps are the first cache+1 (non-flip)
    B, D, K = 1, 4, 7
    g = torch.Generator().manual_seed(51)
    w = torch.randn(D, 1, K, generator=g)
    st = torch.randn(B, D, 2, generator=g).bfloat16()
    u = torch.randn(B, D, generator=g).bfloat16()
    y, st2 = O.step_fir(u, st, w)
    exp = w[:, 0, 2] * u.float() + st[..., 0].float() * w[:, 0, 0] + st[..., 1].float() * w[:, 0, 1]
    assert torch.allclose(y.float(), exp.bfloat16().float())
    assert st2.shape[-1] == 3 and torch.equal(st2[..., -1], u.float())


@pytest.mark.parametrize("cplx", [False, True])
def test_step_iir_consistent_with_prefill(cplx):
    B, D, L, n_dec = 2, 8, 96, 4
    x2, x1, v = O.make_gates(B, D, L + n_dec, seed=61)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(D, 16, seed=62, pmax=0.99)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(63)).bfloat16()
    _, _, state = O.li_prefill(x2[..., :L], x1[..., :L], v[..., :L], lp, r, Db)
    out_full, y32_full, _ = O.li_prefill(x2, x1, v, lp, r, Db)
    for i in range(n_dec):
        y, state = O.step_iir(x2[..., L + i], x1[..., L + i], v[..., L + i], Db, r, lp, state)
        yr = y.real if y.is_complex() else y
        x1v = (x1[..., L + i] * v[..., L + i])
        exp = x2[..., L + i].float() * (y32_full[..., L + i] + Db.float() * x1v.float())
        assert (yr.float() - exp).abs().max() <= 2e-2 * exp.abs().max()
    s_ref = O.modal_state_closed_form(x1 * v, lp)
    assert (state.to(s_ref.dtype) - s_ref).abs().max() <= 1e-4 * s_ref.abs().max()


@pytest.mark.parametrize("T", [1, 5, 32])
def test_truncated_fir_branch_of_parallel_iir(T):
    # long_fir_threshold (vortex/model/engine.py:339-349): F.conv1d correlates, so the truncated filter is applied
    # with h[T-1] on the current sample.  Impulse response and a float64 brute force pin the orientation; the
    # whole branch follows with the usual gating.
    B, D, L = 1, 4, 48
    g = torch.Generator().manual_seed(50 + T)
    h = torch.randn(1, D, L, generator=g)
    hb = h[0, :, :T].bfloat16().double()
    x = torch.zeros(B, D, L).bfloat16()
    x[:, :, 7] = 1.0
    y = O.truncated_fir(x, h, T)
    for j in range(T):
        assert torch.equal(y[0, :, 7 + j].double(), hb[:, T - 1 - j])           # y[t0 + j] = h[T-1-j]
    assert y[0, :, :7].abs().max() == 0 and y[0, :, 7 + T:].abs().max() == 0
    x = torch.randn(B, D, L, generator=g).bfloat16()
    y = O.truncated_fir(x, h, T).double()
    want = torch.zeros(B, D, L, dtype=torch.float64)
    for t in range(L):
        for j in range(min(T, t + 1)):
            want[0, :, t] += hb[:, T - 1 - j] * x[0, :, t - j].double()
    assert (y - want).abs().max() <= 2 ** -8 * want.abs().max()                 # one bf16 rounding of the sum
    z_pre = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, 2, D // 2, 16, D)
    out, st = O.parallel_iir(z_pre, h, Db, L, None, None, dims, long_fir_threshold=T)
    x2, x1, v = z_pre.split(D, 1)
    x1v = x1 * v
    assert st is None
    assert torch.equal(out, ((O.truncated_fir(x1v, h, T) + x1v * Db[:, None]) * x2).permute(0, 2, 1))


# ---------------------------------------------------------------- hyena_ops.interface references (a12)

def _bf16_ulp(x):
    """Spacing of bfloat16 at |x| (float64 tensor in, float64 out)."""
    e = torch.floor(torch.log2(x.abs().clamp_min(2.0 ** -126)))
    return torch.pow(2.0, e - 7)


@pytest.mark.parametrize("K,bias_kind", [(3, "none"), (7, "add"), (7, "gated"), (33, "add"), (128, "gated")])
def test_causal_conv1d_ref_vs_bruteforce_fp32_weights(K, bias_kind):
    # interface.py:207-244 with float32 weights: x is upcast, conv + bias (or conv + x*gated_bias) is formed in
    # float32 and rounded ONCE to the input dtype
    g = torch.Generator().manual_seed(K)
    B, D, L = 2, 5, 150
    x = torch.randn(B, D, L, generator=g).bfloat16()
    w = torch.randn(D, K, generator=g) / math.sqrt(K)
    bias = torch.randn(D, generator=g) if bias_kind != "none" else None
    # the gated bias multiplies x [B, D, L] by plain broadcasting (interface.py:240), so a per-channel one is [D, 1]
    out = O.causal_conv1d_ref(x, w, bias[:, None] if bias_kind == "gated" else bias, apply_gated_bias=bias_kind == "gated")
    assert out.dtype == torch.bfloat16 and out.shape == (B, D, L)
    xn, wn = x.double().numpy(), w.double().numpy()
    for b in range(B):
        z = torch.from_numpy(brute_corr(xn[b], wn))
        if bias_kind == "add":
            z = z + bias.double()[:, None]
        if bias_kind == "gated":
            z = z + x[b].double() * bias.double()[:, None]
        # one rounding of the exact value, up to float32 accumulation error: never off by more than half an ulp + eps
        err = (out[b].double() - z).abs()
        assert (err <= 0.5 * _bf16_ulp(z) * 1.02 + 1e-6).all(), (K, bias_kind, err.max())


def test_causal_conv1d_ref_single_rounding_known_answer():
    # conv = 1 + 2^-8 (a bf16 tie that rounds down to 1), bias = 2^-8: one rounding of the sum gives 1 + 2^-7,
    # rounding the convolution first would give bf16(1 + 2^-8) = 1
    x = torch.tensor([[[1.0, 1.0]]]).bfloat16()
    w = torch.tensor([[2.0 ** -8, 1.0]])                     # w[K-1] on the current sample
    b = torch.tensor([2.0 ** -8])
    out = O.causal_conv1d_ref(x, w, b)
    assert out.flatten().tolist() == [1.0, 1.0 + 2.0 ** -7]
    gated = O.causal_conv1d_ref(x, w, b[:, None], apply_gated_bias=True)  # + x * 2^-8 in float32, same sums
    assert gated.flatten().tolist() == [1.0, 1.0 + 2.0 ** -7]
    # float32 in: nothing is rounded to bf16 at all
    out32 = O.causal_conv1d_ref(x.float(), w, b)
    assert out32.dtype == torch.float32 and out32.flatten().tolist() == [1.0 + 2.0 ** -8, 1.0 + 2.0 ** -7]


def test_causal_conv1d_ref_bf16_weights_compute_in_bf16():
    # weight.dtype decides the arithmetic (interface.py:228): with bf16 weights F.conv1d runs in bf16 and the gated
    # bias is bf16 tensor arithmetic, out + x*bias with both roundings.  Pinned to the exact value within 2 ulps.
    g = torch.Generator().manual_seed(5)
    B, D, L, K = 1, 4, 64, 7
    x = torch.randn(B, D, L, generator=g).bfloat16()
    w = (torch.randn(D, K, generator=g) / math.sqrt(K)).bfloat16()
    bias = torch.randn(D, generator=g).bfloat16()
    out = O.causal_conv1d_ref(x, w, bias[:, None], apply_gated_bias=True)
    assert out.dtype == torch.bfloat16
    z = torch.from_numpy(brute_corr(x[0].double().numpy(), w.double().numpy()))
    exact = z + x[0].double() * bias.double()[:, None]
    scale = torch.maximum(z.abs(), (x[0].double() * bias.double()[:, None]).abs())
    assert ((out[0].double() - exact).abs() <= 2.0 * _bf16_ulp(torch.maximum(scale, exact.abs()))).all()


@pytest.mark.parametrize("G", [1, 2, 4, 8])
def test_inner_hyena_se_ref_stripes_filters_over_channels(G):
    # interface.py:375-376: h.squeeze(1).repeat(d // g, 1) -> channel c is filtered by h[c % g].  Impulse input,
    # unit gates: the output rows are the filters themselves, read back in cross-correlation order.
    D, L, K = 8, 16, 5
    h = torch.arange(G * K, dtype=torch.float32).reshape(G, 1, K) + 1
    x = torch.zeros(1, D, L, dtype=torch.bfloat16)
    x[..., 0] = 1
    one = torch.ones_like(x)
    y = O.inner_hyena_se_ref(x, one, one, h, kernel_path="unfused_gcg")
    for c in range(D):
        assert y[0, c, :K].tolist() == h[c % G, 0].flip(-1).tolist(), c
        assert y[0, c, K:].abs().max() == 0
    if 1 < G < D:      # and it is NOT the blocked map of the model path
        blocked = O.gcg_fwd_ref(x.permute(0, 2, 1).reshape(1, L, G, D // G), one.permute(0, 2, 1).reshape(1, L, G, D // G),
                                one.permute(0, 2, 1).reshape(1, L, G, D // G), h.bfloat16())
        assert not torch.equal(blocked.reshape(1, L, D).permute(0, 2, 1).float(), y.float())


@pytest.mark.parametrize("K,path", [(4, "unfused_gcg_fast"), (4, "unfused_gcg"), (7, "unfused_gcg_fast")])
def test_inner_hyena_se_ref_vs_bruteforce_and_layouts(K, path):
    g = torch.Generator().manual_seed(K)
    B, G, dg, L = 2, 3, 4, 40
    D = G * dg
    x, k, q = (torch.randn(B, D, L, generator=g).bfloat16() for _ in range(3))
    h = torch.randn(G, 1, K, generator=g) / math.sqrt(K)
    bias = torch.randn(D, generator=g)
    y = O.inner_hyena_se_ref(x, k, q, h, bias=bias, kernel_path=path)
    kx = (k * x)
    w = h[:, 0].repeat(D // G, 1).double().numpy()
    for b in range(B):
        z = torch.from_numpy(brute_corr(kx[b].double().numpy(), w)) + bias.double()[:, None]
        zb = z.float().bfloat16()                 # one rounding of conv + bias (float32 accumulation: allow one ulp)
        ref = (q[b] * zb).double()
        err = (y[b].double() - ref).abs()
        assert (err <= 1.01 * _bf16_ulp(z) * q[b].double().abs() + _bf16_ulp(ref)).all()
    # layouts: (b, l, g, dg) and (b, g, dg, l) in, "bld" / "blgdg" out are pure re-indexings of the same numbers
    to_blgdg = lambda t: t.permute(0, 2, 1).reshape(B, L, G, dg)
    y2 = O.inner_hyena_se_ref(to_blgdg(x), to_blgdg(k), to_blgdg(q), h, bias=bias, input_layout="blgdg",
                              output_layout="blgdg", kernel_path=path)
    assert torch.equal(y2, to_blgdg(y))
    y3 = O.inner_hyena_se_ref(x.reshape(B, G, dg, L), k.reshape(B, G, dg, L), q.reshape(B, G, dg, L), h, bias=bias,
                              input_layout="bgdgl", output_layout="bld", kernel_path=path)
    assert torch.equal(y3, y.permute(0, 2, 1))


# --------------------------------------------------------------------------
# OracleCascade: the operator module's call sequence (vortex/model/model.py:214-375)
# --------------------------------------------------------------------------

def _cascade_params(kind, D, seed, Ks=3, identity_featurizer=False):
    g = torch.Generator().manual_seed(seed)
    wf = torch.randn(3 * D, 1, Ks, generator=g) / Ks ** 0.5
    if identity_featurizer:
        wf = torch.zeros(3 * D, 1, Ks)
        wf[..., Ks - 1] = 1.0
    p = {"short_filter_weight": wf, "short_filter_bias": None}
    if kind == "se":
        p["h"], p["D"] = O.make_se_filter(D // 2, 7, seed=seed), None
    elif kind == "mr":
        p["h"], p["D"] = O.make_mr_filter(D // 2, 128, seed=seed), torch.randn(D, generator=g).bfloat16()
    else:
        p["log_poles"], p["residues"] = O.make_modal_real(D, 4, seed=seed, pmax=0.99)
        p["D"] = torch.randn(D, generator=g).bfloat16()
    return p


def _make_cascade(kind, p, D, H, cs, il, flip):
    K = {"se": 7, "mr": 128}.get(kind)
    G = D // 2 if K else D
    return O.OracleCascade(O.OracleEngine(hyena_flip_x1x2=flip), p, D, H, G, fir_inner_filter_length=K,
                           column_split_hyena=cs, interleave=il, state_size=4, hyena_flip_x1x2=flip)


@pytest.mark.parametrize("flip", [False, True])
@pytest.mark.parametrize("il", [False, True])
@pytest.mark.parametrize("cs", [False, True])
@pytest.mark.parametrize("kind,L", [("se", 40), ("mr", 150), ("mr", 20), ("li", 64)])
def test_oracle_cascade_prefill_equals_prefill_plus_steps(kind, L, cs, il, flip):
    # what the mathematics fixes for the whole call sequence: a causal operator evaluated on L+n tokens at once
    # equals its evaluation on L tokens followed by n one-token calls, outputs and caches alike.  A wrong split,
    # a missing flip on either branch, a wrong tap orientation or state hand-off breaks it.
    B, D, H, n = 2, 8, 2, 5
    p = _cascade_params(kind, D, seed=70 + L)
    u = torch.randn(B, L + n, 3 * D, generator=torch.Generator().manual_seed(L)).bfloat16()
    full = _make_cascade(kind, p, D, H, cs, il, flip)
    ip_full = O.OracleCache()
    y_full, _ = full.forward(u, ip_full)
    inc = _make_cascade(kind, p, D, H, cs, il, flip)
    ip = O.OracleCache()
    y0, _ = inc.forward(u[:, :L], ip)
    scale = y_full.float().abs().max()
    assert (y0.float() - y_full[:, :L].float()).abs().max() <= 1e-2 * scale
    for i in range(n):
        yi, _ = inc.forward(u[:, L + i:L + i + 1], ip)
        assert yi.shape == (B, 1, D) and yi.dtype == u.dtype
        assert (yi[:, 0].float() - y_full[:, L + i].float()).abs().max() <= 2e-2 * scale, i
    # featurizer cache: the last Ks-1 projection rows, exactly
    assert torch.equal(ip.fir_state_dict[0].float(), ip_full.fir_state_dict[0].float())
    if kind == "li":
        a, b = ip.state_dict[0].double(), ip_full.state_dict[0].double()
        assert (a - b).abs().max() <= 1e-3 * b.abs().max()
    else:
        a, b = ip.fir_inner_state_dict[0].float(), ip_full.fir_inner_state_dict[0].float()
        assert a.shape == b.shape
        assert (a - b).abs().max() <= 2 ** -7 * b.abs().max()          # x1*v of featurizer outputs: one bf16 ulp


def _expected_role(j, D, H, cs, il, flip):
    """(role, channel) a projection channel j ends up as, written from the definitions: interleave sends channel
    3c+i to block i (vortex/model/utils.py:26-38); the plain split cuts [x2 | x1 | v] blocks of D; the column split
    cuts each head's 3*hd channels into [x2 | x1 | v] (utils.py:41-85); the flip swaps the x1 and x2 roles."""
    hd = D // H
    if il:
        j = (j % 3) * D + j // 3
    if cs:
        head, within = divmod(j, 3 * hd)
        role, c = within // hd, head * hd + within % hd
    else:
        role, c = divmod(j, D)
    if flip and role in (0, 1):
        role = 1 - role
    return role, c


@pytest.mark.parametrize("flip", [False, True])
@pytest.mark.parametrize("il", [False, True])
@pytest.mark.parametrize("cs", [False, True])
def test_oracle_cascade_index_known_answer(cs, il, flip):
    # identity featurizer, inner filter = one-sample delay: y[c, t] = x2[c, t] * x1[c, t-1] * v[c, t-1].  All inputs 1
    # except projection channel j, which is 2 at one time step: the 2 shows up in y at that step if j is an x2
    # channel and one step later if it is an x1 or v channel -- on the prefill branch and on the decode branch.
    D, H, Ks, L = 8, 2, 3, 6
    C = 3 * D
    p = _cascade_params("se", D, seed=1, Ks=Ks, identity_featurizer=True)
    h = torch.zeros(D // 2, 1, 7)
    h[..., 5] = 1.0                                     # tap K-2 multiplies the previous sample
    p["h"] = h
    t0 = 3
    u = torch.ones(C, L + 3, C).bfloat16()              # batch element j carries the mark on channel j
    for j in range(C):
        u[j, t0, j] = 2.0
        u[j, L + 1, j] = 2.0                            # and again on the second decode step
    mod = _make_cascade("se", p, D, H, cs, il, flip)
    ip = O.OracleCache()
    y, _ = mod.forward(u[:, :L], ip)
    steps = [mod.forward(u[:, L + i:L + i + 1], ip)[0][:, 0] for i in range(3)]
    for j in range(C):
        role, c = _expected_role(j, D, H, cs, il, flip)
        want = torch.ones(L, D)
        want[0] = 0                                     # no history at t = 0
        want[t0 if role == 0 else t0 + 1, c] = 2.0
        assert torch.equal(y[j].float(), want), (j, role, c)
        for i in range(3):
            w = torch.ones(D)
            if (role == 0 and i == 1) or (role != 0 and i == 2):
                w[c] = 2.0
            assert torch.equal(steps[i][j].float(), w), (j, role, c, i)


def test_prefill_direct_recurrence_ref_hand_computed():
    # three steps by hand.  (1) bf16 state: p = 1 + 2^-8, r = 1, u = 1, 1, 1 in bf16: s = 1; then 2.00390625 which a
    # bf16 state rounds to 2; then p*2 + 1 = 3.0078125, a tie that rounds to even, 3 (a float32 state would give
    # 2.0039 and 3.0117, i.e. an output of 3.015625 after the cast).
    p = torch.tensor([1.0 + 2.0 ** -8, 0.0]).reshape(1, 1, 1, 2)
    r = torch.tensor([1.0, 0.0]).reshape(1, 1, 1, 2)
    u = torch.ones(1, 1, 3).bfloat16()
    y, s = O.prefill_direct_recurrence_ref(u, p, r)
    assert y.dtype == torch.bfloat16 and s.dtype == torch.float32 and s.shape == (1, 1, 1, 2)
    assert y.flatten().tolist() == [1.0, 2.0, 3.0]
    assert s.flatten().tolist() == [3.0, 0.0]
    # (2) the in-place lane update and the lane-0 output with p = i, r = 1 + 5i, u = 1, 0, 0 in float32: the new real
    # lane feeds the imaginary one, so (s_re, s_im) = (1, 1), (-1, -1), (1, 1) where the complex product gives
    # (1, 0), (0, 1), (-1, 0); y = r_re * s_re = 1, -1, 1 where Re(r s) = 1, -5, -1.
    p = torch.tensor([0.0, 1.0]).reshape(1, 1, 1, 2)
    r = torch.tensor([1.0, 5.0]).reshape(1, 1, 1, 2)
    u = torch.tensor([1.0, 0.0, 0.0]).reshape(1, 1, 3)
    y, s = O.prefill_direct_recurrence_ref(u, p, r)
    assert y.flatten().tolist() == [1.0, -1.0, 1.0]
    assert s.flatten().tolist() == [1.0, 1.0]
    # (3) two modes and two channels, real poles, float32: y = sum_s r_s * s_s by hand
    p = torch.tensor([[0.5, 0.25], [0.0, 1.0]])[..., None, None].repeat(1, 1, 1, 2)
    p[..., 1] = 0
    r = torch.tensor([[2.0, 4.0], [1.0, -1.0]])[..., None, None].repeat(1, 1, 1, 2)
    u = torch.tensor([[1.0, 1.0, 0.0], [1.0, 2.0, 3.0]])[None]
    y, s = O.prefill_direct_recurrence_ref(u, p, r)
    # channel 0: s = (1, 1), (1.5, 1.25), (0.75, 0.3125) -> y = 6, 8, 2.75;  channel 1: s = (1, 1), (2, 3), (3, 6)
    assert y[0].tolist() == [[6.0, 8.0, 2.75], [0.0, -1.0, -3.0]]
    assert s[0, :, :, 0].tolist() == [[0.75, 0.3125], [3.0, 6.0]]


def test_prefill_direct_recurrence_ref_is_the_recurrence_for_real_poles_in_float32():
    # with real poles and float32 activations none of the loop's three quirks acts: it is the plain recurrence
    B, D, S, L = 2, 3, 4, 40
    g = torch.Generator().manual_seed(81)
    lp, res = O.make_modal_real(D, S, seed=82, pmax=0.99)
    u = torch.randn(B, D, L, generator=g)
    p4 = torch.stack([lp[..., 0].exp(), torch.zeros(D, S)], -1)[:, :, None]
    r4 = torch.stack([res, torch.zeros(D, S)], -1)[:, :, None]
    y, s = O.prefill_direct_recurrence_ref(u, p4, r4)
    y64, s64 = O.prefill_direct_recurrence(u, lp, res)
    assert (y.double() - y64).abs().max() <= 1e-5 * y64.abs().max()
    assert (s[..., 0].double() - s64).abs().max() <= 1e-5 * s64.abs().max()
    assert s[..., 1].abs().max() == 0
