"""Per-element error statements for the prefill operators (tests/parity.py), next to the normalised maxima of the
other parity tests: every output sample of Hyena-SE, Hyena-MR (single and forced multi-segment launches, taps that
do not decay so that the oldest tap weighs as much as the newest), the channel-last kernel and Hyena-LI must lie
within the forward-error bound of its own accumulation, which a sample that picked up a wrong tap, halo or chunk
state misses by two orders of magnitude wherever it sits.  The observed worst error/bound ratio is part of every
assertion message."""
import pytest
import torch

import vortex_amd as va
from oracle import hyena_oracle as O
from parity import abs_scale, assert_gated_close, bf16_ulp, rel_err
from vortex_amd import ops

pytestmark = pytest.mark.gpu


def flat_taps(G, K, seed):
    """N(0, 1/K) taps without decay: every lag carries the same weight."""
    return torch.randn(G, 1, K, generator=torch.Generator().manual_seed(seed)) / K ** 0.5


@pytest.mark.parametrize("B,D,L,G,K", [(2, 64, 2048, 4, 7), (1, 48, 200, 3, 3), (1, 32, 1000, 2, 8), (2, 16, 4104, 1, 2)])
def test_se_per_element(B, D, L, G, K):
    x2, x1, v = O.make_gates(B, D, L, seed=L + K)
    h = flat_taps(G, K, K)
    ref, _ = O.se_fir(x2, x1, v, h)
    u = x1 * v
    w = h.repeat_interleave(D // G, 0)
    z_ref = O.short_fir_fp32(u, w, K).bfloat16()
    out = va.hyena_se_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda())
    S = abs_scale(u, w[:, 0].flip(-1))
    r = assert_gated_close(out, ref, z_ref, x2, S, 2.0 ** -20, what=f"hyena_se_fwd {B, D, L, G, K}")
    assert r <= 1.0


@pytest.mark.parametrize("nseg", [0, 1, 3, 5])
@pytest.mark.parametrize("B,D,L,G,K,bias", [(1, 32, 4096 + 512, 2, 128, True), (2, 32, 1544, 1, 128, False),
                                           (1, 16, 3000 // 8 * 8, 1, 100, True), (1, 48, 2048, 3, 17, True)])
def test_mr_per_element_across_segments(B, D, L, G, K, bias, nseg, override):
    # nseg = 0: the launcher's own choice; otherwise forced, so that segment starts fall inside short rows
    if nseg:
        override(mr_nseg=nseg)
    x2, x1, v = O.make_gates(B, D, L, seed=L + K + nseg)
    h = flat_taps(G, K, K + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(3)) if bias else torch.zeros(D)
    ref, _ = O.mr_fir(x2, x1, v, h, Db)
    u = x1 * v
    w = h.repeat_interleave(D // G, 0)
    z_ref = (O.fft_causal_conv_fp32(u.float(), w) + u.float() * Db[:, None]).bfloat16()
    out = va.hyena_mr_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda(), Db.cuda() if bias else None)
    assert rel_err(out, ref) <= 2e-2
    S = abs_scale(u, w[:, 0], (u.float() * Db[:, None]).double())
    # taps reach the matrix cores as one bf16 term: 2^-9 relative each, 2^-8 with the accumulation
    assert_gated_close(out, ref, z_ref, x2, S, 2.0 ** -8, fft_floor=4e-6, what=f"hyena_mr_fwd {B, D, L, G, K} nseg={nseg}")
    # with bf16-exact taps the products are exact: the bound tightens to the float32 accumulation
    hb = h.bfloat16().float()
    ref, _ = O.mr_fir(x2, x1, v, hb, Db)
    wb = hb.repeat_interleave(D // G, 0)
    z_ref = (O.fft_causal_conv_fp32(u.float(), wb) + u.float() * Db[:, None]).bfloat16()
    out = va.hyena_mr_fwd(x1.cuda(), x2.cuda(), v.cuda(), hb.cuda(), Db.cuda() if bias else None)
    assert_gated_close(out, ref, z_ref, x2, abs_scale(u, wb[:, 0], (u.float() * Db[:, None]).double()), 2.0 ** -18,
                       fft_floor=4e-6, what=f"hyena_mr_fwd bf16-exact taps {B, D, L, G, K} nseg={nseg}")


@pytest.mark.parametrize("nseg", [1, 4])
@pytest.mark.parametrize("K", [7, 128])
def test_channel_last_per_element(K, nseg, override):
    override(cl_nseg=nseg)
    B, D, L, G = 2, 64, 1160, 4
    x2, x1, v = O.make_gates(B, D, L, seed=K + nseg)
    h = flat_taps(G, K, K + 2).bfloat16().float()
    w = h.repeat_interleave(D // G, 0)
    u = x1 * v
    z_ref = O.fft_causal_conv_fp32(u.float(), w).bfloat16()
    ref = x2 * z_ref
    cl = lambda t: t.permute(0, 2, 1).contiguous().cuda()
    out = ops.fir_cl_fwd(cl(x1), cl(x2), cl(v), h.reshape(G, K).cuda()).permute(0, 2, 1)
    assert_gated_close(out, ref, z_ref, x2, abs_scale(u, w[:, 0]), 2.0 ** -18, fft_floor=4e-6, what=f"hyena_fir_cl_fwd K={K} nseg={nseg}")


@pytest.mark.parametrize("form", ["lone", "coop", "cpw1"])
@pytest.mark.parametrize("L,cplx", [(4096 + 520, True), (2048 + 8, False), (1000, True)])
def test_li_per_element(L, cplx, form, override):
    # float32 long convolution: |y32 - ref| <= 2^-13 * S[t] + (float32 FFT noise of the reference, 4e-6 of max S);
    # gated bf16 output: the bound of parity.py with the three roundings of z = bf16(bf16(y) + bf16(D*x1v))
    override(**{"lone": dict(li_coop=0), "coop": dict(li_coop=1), "cpw1": dict(li_cpw=1)}[form])
    B, G = 2, 2
    D = 16 if form != "cpw1" else 8
    x2, x1, v = O.make_gates(B, D, L, seed=L)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, 16, seed=L + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(1)).bfloat16()
    ref, y32_ref, _ = O.li_prefill(x2, x1, v, lp, r, Db)
    out, y32, _ = va.hyena_li_fwd(x1.cuda(), x2.cuda(), v.cuda(), lp.cuda(), r.cuda(), Db.cuda(), want_fp32=True)
    u = x1 * v
    h = O.modal_filter(lp, r, L, dtype=torch.float64)[0].repeat_interleave(D // G, 0)         # [D, L]
    S = abs_scale(u, h, None)
    err = (y32.double().cpu() - y32_ref.double()).abs()
    bound = 2.0 ** -13 * S + 4e-6 * S.max()
    assert (err <= bound).all(), (form, L, cplx, (err / bound).max().item())
    z_ref = (y32_ref.bfloat16() + u * Db[:, None])
    S2 = S + (u.double() * Db.double()[:, None]).abs()
    assert_gated_close(out, ref, z_ref, x2, S2, 2.0 ** -13, ulps_z=2.0, fft_floor=4e-6, what=f"hyena_li_fwd {form} L={L}")
    assert rel_err(y32, y32_ref) <= 1e-4 and rel_err(out, ref) <= 2e-2


def test_full_size_rows_per_element():
    # configs 1 and 2 at full size (non-temporal accesses, the launchers' own segmenting), sampled rows
    B, D, L, G, K = 1, 4096, 8192, 256, 7
    x2, x1, v = O.make_gates(B, D, L, seed=7)
    h = flat_taps(G, K, 5)
    out = va.hyena_se_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda()).cpu()
    rows = torch.arange(1, D, 97)
    u = x1[:, rows] * v[:, rows]
    w = h.repeat_interleave(D // G, 0)[rows]
    z_ref = O.short_fir_fp32(u, w, K).bfloat16()
    assert_gated_close(out[:, rows], x2[:, rows] * z_ref, z_ref, x2[:, rows], abs_scale(u, w[:, 0].flip(-1)), 2.0 ** -20,
                       what="config 1 rows")
    B, D, L, G, K = 2, 4096, 32768, 256, 128
    g = torch.Generator().manual_seed(9)
    x2, x1, v = (torch.randn(B, D, L, generator=g).bfloat16() for _ in range(3))
    h = flat_taps(G, K, 6)
    Db = torch.randn(D, generator=g)
    out = va.hyena_mr_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda(), Db.cuda()).cpu()
    rows = torch.arange(3, D, 257)
    u = x1[:, rows] * v[:, rows]
    w = h.repeat_interleave(D // G, 0)[rows]
    z_ref = (O.fft_causal_conv_fp32(u.float(), w) + u.float() * Db[rows][:, None]).bfloat16()
    S = abs_scale(u, w[:, 0], (u.float() * Db[rows][:, None]).double())
    assert_gated_close(out[:, rows], x2[:, rows] * z_ref, z_ref, x2[:, rows], S, 2.0 ** -8, fft_floor=4e-6, what="config 2 rows")
