"""Cached decode step at its full configured shape: batch 64, D = 4096 and 8192, FIR caches of 6 (Hyena-SE) and
127 (Hyena-MR) samples, 16 complex modal states, for 131 tokens (the 127-slot ring wraps), outputs and updated
caches against the oracle's step_fir / step_iir (vortex/model/engine.py:406-467).

The step is independent per channel, so the full-width problem is laid out as D / 512 copies of a 512-channel
base problem (filters, caches, inputs tiled along the channel axis): the oracle steps the base problem on the
CPU, the kernels step all D channels, and the test checks the first tile against the oracle and every other
tile -- other blocks, other grid positions, the same arithmetic -- for bit-equality with the first."""
import pytest
import torch

import vortex_amd as va
from oracle import hyena_oracle as O
from parity import assert_gated_close, rel_err
from vortex_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
B, BASE, TOKENS = 64, 512, 131


def tile(t, D, dim=1):
    reps = [1] * t.dim()
    reps[dim] = D // t.shape[dim]
    return t.repeat(*reps)


def tiles_equal(t, D, base=BASE, period=1):
    """Every tile bit-equal to the first -- or, with period p, to the one of the first p tiles it is congruent to
    (the far-sum FIR step staggers its windows over the blocks: blocks p apart do the same arithmetic)."""
    v = t.reshape(t.shape[0], D // base, base, *t.shape[2:])
    idx = torch.arange(D // base, device=t.device) % period
    return bool((v == v[:, idx]).all())


@pytest.mark.parametrize("D", [4096, 8192])
@pytest.mark.parametrize("K,flip,gated", [(7, False, False), (128, True, True)])
def test_fir_step_full_shape(D, K, flip, gated):
    g = torch.Generator().manual_seed(K + D)
    R, Gb = K - 1, BASE // 16
    w = torch.randn(Gb, 1, K, generator=g) / K ** 0.5
    wD = w.repeat_interleave(16, 0)                                  # [BASE, 1, K]
    bias = torch.randn(BASE, generator=g) if gated else None
    st = torch.randn(B, BASE, R, generator=g).bfloat16()
    ring = va.FirRing.from_reference(tile(st, D).to(DEV))
    w2 = w.reshape(Gb, K)
    taps = tile((w2.flip(-1) if flip else w2).contiguous(), D // 16, dim=0).to(DEV)      # [D/16, K], oldest tap first
    bias_d = None if bias is None else tile(bias, D, dim=0).to(DEV)
    ref_state = st
    worst = 0.0
    for step in range(TOKENS):
        x1, x2, v = (torch.randn(B, BASE, generator=g).bfloat16() for _ in range(3))
        u = x1 * v
        y_ref, new_state = O.step_fir(u, ref_state, wD, bias=bias, gated_bias=gated, flip_filter=flip)
        out_ref = y_ref * x2
        y = va.fir_step(tile(x1, D).to(DEV), ring, taps, x2=tile(x2, D).to(DEV), v=tile(v, D).to(DEV), bias=bias_d,
                        gated_bias=gated)
        assert tiles_equal(y, D), step
        assert rel_err(y[:, :BASE], out_ref) <= 2e-2, step
        weff = (wD[:, 0].flip(-1) if flip else wD[:, 0])                              # [BASE, K], oldest first
        S = (ref_state.double().abs() * weff[None, :, :R].double().abs()).sum(-1) + (weff[None, :, R] * u.float()).abs()
        if gated:
            S = S + (bias[None] * u.float()).abs()
        worst = max(worst, assert_gated_close(y[:, :BASE], out_ref, y_ref, x2, S, 2.0 ** -16, what=f"fir_step token {step}"))
        ref_state = new_state
        if step in (0, R - 1, R, TOKENS - 1):
            order = ring.reference_order()
            assert tiles_equal(order, D)
            assert torch.equal(order[:, :BASE].cpu(), ref_state.float()), step
    assert worst <= 1.0


@pytest.mark.parametrize("D", [4096, 8192])
@pytest.mark.parametrize("cplx", [True, False])
def test_iir_step_full_shape(D, cplx):
    S = 16
    g = torch.Generator().manual_seed(D + cplx)
    Gb = BASE // 16
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(Gb, S, seed=D)
    Dp = torch.randn(BASE, generator=g).bfloat16()
    lpD, rD = lp.repeat_interleave(16, 0), r.repeat_interleave(16, 0)
    st_ref = torch.randn(B, BASE, S, generator=g)
    if cplx:
        st_ref = torch.complex(st_ref, torch.randn(B, BASE, S, generator=g))
    state = tile(st_ref, D).contiguous().to(DEV)
    poles = tile(torch.exp(lp[..., 0]), D // 16, dim=0).to(DEV)
    res = tile(r, D // 16, dim=0).to(DEV)
    Dd = tile(Dp, D, dim=0).to(DEV)
    for step in range(TOKENS):
        x1, x2, v = (torch.randn(B, BASE, generator=g).bfloat16() for _ in range(3))
        y_ref, st_ref = O.step_iir(x2, x1, v, Dp, rD, lpD, st_ref)
        y_ref = (y_ref.real if cplx else y_ref).to(torch.bfloat16)
        y = va.iir_step(tile(x1, D).to(DEV), tile(x2, D).to(DEV), tile(v, D).to(DEV), state, poles, res, Dd)
        assert tiles_equal(y, D), step
        assert rel_err(y[:, :BASE], y_ref) <= 2e-2, step
        # per element: |x2| * (2^-16 * sum|r*s| + ulp of the bf16 roundings of res and D*x1v) + ulp(out)
        if step % 10 == 0 or step == TOKENS - 1:
            sabs = (rD[None].abs() * st_ref.abs()).sum(-1).double()
            err = (y[:, :BASE].double().cpu() - y_ref.double()).abs()
            x1v = (x1 * v).double()
            bound = x2.double().abs() * (2.0 ** -16 * sabs + 2.0 ** -7 * (sabs + (Dp.double()[None] * x1v).abs())) \
                + 2.0 ** -7 * y_ref.double().abs() + 1e-30
            assert (err <= bound).all(), (step, (err / bound).max())
    sv = torch.view_as_real(state) if cplx else state
    assert tiles_equal(sv, D)
    sr = torch.view_as_real(st_ref) if cplx else st_ref
    assert rel_err(sv[:, :BASE], sr) <= 1e-4


@pytest.mark.parametrize("D", [4096, 8192])
@pytest.mark.parametrize("kind", ["se", "mr", "li"])
def test_layer_step_full_shape(D, kind):
    # the one-launch layer step from the projection row u [B, 3D] (Evo 2 layout: interleaved gates, 3-tap featurizer)
    g = torch.Generator().manual_seed(D + len(kind))
    Ks, S = 3, 16
    CB, C = 3 * BASE, 3 * D
    Gb = BASE // 16
    wf = torch.randn(CB, 1, Ks, generator=g) / Ks ** 0.5
    fst = torch.randn(B, CB, Ks - 1, generator=g).bfloat16()
    fring = va.FirRing.from_reference(tile(fst, C).to(DEV))
    cmap = ops.gate_channel_map(D, interleave=True)
    if kind == "li":
        lp, r = O.make_modal_complex(Gb, S, seed=D)
        Dp = torch.randn(BASE, generator=g).bfloat16()
        lpD, rD = lp.repeat_interleave(16, 0), r.repeat_interleave(16, 0)
        st_ref = torch.complex(torch.randn(B, BASE, S, generator=g), torch.randn(B, BASE, S, generator=g))
        state = tile(st_ref, D).contiguous().to(DEV)
        inner = ops.IirStepper(state, tile(torch.exp(lp[..., 0]), D // 16, dim=0).to(DEV), tile(r, D // 16, dim=0).to(DEV),
                               tile(Dp, D, dim=0).to(DEV))
    else:
        K = 7 if kind == "se" else 128
        mr = kind == "mr"
        R = K - 1
        w = torch.randn(Gb, 1, K, generator=g) / K ** 0.5
        wD = w.repeat_interleave(16, 0)
        bias = torch.randn(BASE, generator=g) if mr else None
        st_ref = torch.randn(B, BASE, R, generator=g).bfloat16()
        ring = va.FirRing.from_reference(tile(st_ref, D).to(DEV))
        w2 = w.reshape(Gb, K)
        inner = ops.FirStepper(ring, tile((w2.flip(-1) if mr else w2).contiguous(), D // 16, dim=0).to(DEV),
                               bias=None if bias is None else tile(bias, D, dim=0).to(DEV), gated_bias=mr)
    step = ops.LayerStepper(fring, tile(wf.reshape(CB, Ks), C, dim=0).to(DEV), None, cmap, inner)
    # the Hyena-MR stepper keeps far sums: its blocks run in windows staggered with this period
    period = _lib.lib().hyena_fir_far_period(1) if kind == "mr" else 1
    assert (getattr(inner, "far", None) is not None) == (kind == "mr")
    ref_f = fst
    y = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
    for i in range(TOKENS):
        u = torch.randn(B, CB, generator=g).bfloat16()
        z, ref_f = O.step_fir(u, ref_f, wf)
        x2, x1, v = O.interleave(z).split([BASE] * 3, dim=1)
        if kind == "li":
            y_ref, st_ref = O.step_iir(x2, x1, v, Dp, rD, lpD, st_ref)
            y_ref = y_ref.real.to(torch.bfloat16)
        else:
            y_ref, st_ref = O.step_fir(x1 * v, st_ref, wD, bias=bias, gated_bias=mr, flip_filter=mr)
            y_ref = y_ref * x2
        step(tile(u, C).to(DEV), y)
        assert tiles_equal(y, D, period=period), i
        assert rel_err(y[:, :period * BASE], tile(y_ref, period * BASE)) <= 2e-2, i
    assert torch.equal(fring.reference_order()[:, :CB].cpu(), ref_f.float()) and tiles_equal(fring.reference_order(), C, CB)
    if kind == "li":
        sv = torch.view_as_real(state)
        # gates one bf16 ulp from the oracle's (fp32 summation order in the featurizer) feed the state: observed 1.4e-4
        assert tiles_equal(sv, D) and rel_err(sv[:, :BASE], torch.view_as_real(st_ref)) <= 2e-3
    else:
        order = ring.reference_order()
        # x1*v of featurizer outputs: the kernel's fp32 sums can land one bf16 ulp from the oracle's, so not bit-exact
        assert tiles_equal(order, D) and rel_err(order[:, :BASE], st_ref) <= 1e-2


@pytest.mark.parametrize("D", [4096, 8192])
def test_decode_layer_set_full_shape(D):
    """The layer set as it is benchmarked (ops.DecodeLayerSet): the Hyena-SE step, the Hyena-MR step with far sums
    (its cache read whole every third token) and the Hyena-LI step with the complex modal state in windows of four
    tokens, 16 channels per filter, for 135 tokens: every output per element against O.step_fir / O.step_iir, the
    caches bit for bit, the modal state after a flush in the middle of the run and at its end."""
    g = torch.Generator().manual_seed(D + 4)
    Gb, S, n_tok = BASE // 16, 16, 135
    # Hyena-SE (7 taps, plain slicing) and Hyena-MR (128 taps, flipped, gated bias)
    w_se = torch.randn(Gb, 1, 7, generator=g) / 7 ** 0.5
    w_mr = O.make_mr_filter(Gb, 128, seed=D)
    b_mr = torch.randn(BASE, generator=g)
    st_se = torch.randn(B, BASE, 6, generator=g).bfloat16()
    st_mr = torch.randn(B, BASE, 127, generator=g).bfloat16()
    ring_se = va.FirRing.from_reference(tile(st_se, D).to(DEV))
    ring_mr = va.FirRing.from_reference(tile(st_mr, D).to(DEV))
    lp, r = O.make_modal_complex(Gb, S, seed=D + 1)
    Dp = torch.randn(BASE, generator=g).bfloat16()
    lpD, rD = lp.repeat_interleave(16, 0), r.repeat_interleave(16, 0)
    st_li = torch.complex(torch.randn(B, BASE, S, generator=g), torch.randn(B, BASE, S, generator=g))
    state = tile(st_li, D).contiguous().to(DEV)
    step = ops.DecodeLayerSet(
        ring_se, tile(w_se.reshape(Gb, 7), D // 16, dim=0).to(DEV),
        ring_mr, tile(w_mr.reshape(Gb, 128).flip(-1).contiguous(), D // 16, dim=0).to(DEV), tile(b_mr, D, dim=0).to(DEV),
        state, tile(torch.exp(lp[..., 0]), D // 16, dim=0).to(DEV), tile(r, D // 16, dim=0).to(DEV),
        tile(Dp, D, dim=0).to(DEV), window_state=True)
    assert step.mr.far is not None and step.se.far is None and step.li.win is not None
    far_period = _lib.lib().hyena_fir_far_period(1)
    wD_se, wD_mr = w_se.repeat_interleave(16, 0), w_mr.repeat_interleave(16, 0)
    weff_mr = wD_mr[:, 0].flip(-1)
    worst = 0.0

    def state_ok(tok):
        step.flush()
        sv = torch.view_as_real(state)
        assert tiles_equal(sv, D), tok
        assert rel_err(sv[:, :BASE], torch.view_as_real(st_li)) <= 1e-4, tok

    for tok in range(n_tok):
        gates = [tuple(torch.randn(B, BASE, generator=g).bfloat16() for _ in range(3)) for _ in range(3)]    # (x2, x1, v)
        outs = step(*[tuple(tile(t, D).to(DEV) for t in gt) for gt in gates])
        # Hyena-SE
        x2, x1, v = gates[0]
        z_ref, new_se = O.step_fir(x1 * v, st_se, wD_se)
        Sabs = (st_se.double().abs() * wD_se[None, :, 0, :6].double().abs()).sum(-1) + (wD_se[None, :, 0, 6] * (x1 * v).float()).abs()
        assert tiles_equal(outs[0], D), tok
        worst = max(worst, assert_gated_close(outs[0][:, :BASE], z_ref * x2, z_ref, x2, Sabs, 2.0 ** -16, what=f"se token {tok}"))
        st_se = new_se
        # Hyena-MR, far sums: windows staggered over the blocks with period 3
        x2, x1, v = gates[1]
        u = x1 * v
        z_ref, new_mr = O.step_fir(u, st_mr, wD_mr, bias=b_mr, gated_bias=True, flip_filter=True)
        Sabs = (st_mr.double().abs() * weff_mr[None, :, :127].double().abs()).sum(-1) + (weff_mr[None, :, 127] * u.float()).abs() \
            + (b_mr[None] * u.float()).abs()
        assert tiles_equal(outs[1], D, period=far_period), tok
        for t in range(far_period):
            worst = max(worst, assert_gated_close(outs[1][:, t * BASE:(t + 1) * BASE], z_ref * x2, z_ref, x2, Sabs,
                                                  2.0 ** -16, what=f"mr token {tok} tile {t}"))
        st_mr = new_mr
        # Hyena-LI, windowed complex state
        x2, x1, v = gates[2]
        y_ref, st_li = O.step_iir(x2, x1, v, Dp, rD, lpD, st_li)
        y_ref = y_ref.real.to(torch.bfloat16)
        assert tiles_equal(outs[2], D), tok
        assert rel_err(outs[2][:, :BASE], y_ref) <= 2e-2, tok
        sabs = (rD[None].abs() * st_li.abs()).sum(-1).double()
        err = (outs[2][:, :BASE].double().cpu() - y_ref.double()).abs()
        x1v = (x1 * v).double()
        bound = x2.double().abs() * (2.0 ** -16 * sabs + 2.0 ** -7 * (sabs + (Dp.double()[None] * x1v).abs())) \
            + 2.0 ** -7 * y_ref.double().abs() + 1e-30
        assert (err <= bound).all(), (tok, (err / bound).max())
        if tok == 66:
            state_ok(tok)
    assert worst <= 1.0
    state_ok(n_tok)
    for ring, ref in ((ring_se, st_se), (ring_mr, st_mr)):
        order = ring.reference_order()
        assert tiles_equal(order, D) and torch.equal(order[:, :BASE].cpu(), ref.float())
