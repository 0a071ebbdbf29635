"""GPU parity of the one-launch decode layer steps (featurizer step + split + gated FIR / IIR step)
against the oracle's step_fir / step_iir chain, through the C ABI."""
import pytest
import torch

import vortex_amd as va
from vortex_amd import ops
from oracle import hyena_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_err(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def oracle_gates(z, D, H, cs, il, flip):
    """Interleave / split of vortex/model/model.py:332-343 on a [B, 3D] featurizer output."""
    if il:
        z = O.interleave(z)
    if cs:
        x2, x1, v = O.column_split(z, H, D // H)
    else:
        x2, x1, v = z.split([D, D, D], dim=1)
    return (x1, x2, v) if flip else (x2, x1, v)


@pytest.mark.parametrize("B,D,H,G,K,Ks,cs,il,flip,sbias", [
    (3, 512, 8, 32, 7, 3, False, True, False, False),      # Evo 2 layout: interleave, grouped SE taps
    (2, 1024, 16, 64, 128, 3, False, True, False, True),   # MR, gated fp32 bias, featurizer bias
    (2, 256, 4, 256, 7, 4, True, False, False, False),     # head-blocked column split, per-channel taps
    (2, 520, 5, 65, 128, 3, False, False, True, False),    # plain split, x1/x2 flipped, D % 512 != 0
    (1, 64, 4, 4, 7, 2, True, False, True, True),
])
def test_fir_layer_step_sequence_vs_oracle(B, D, H, G, K, Ks, cs, il, flip, sbias):
    g = torch.Generator().manual_seed(K * 100 + D + Ks)
    C, R, Rf = 3 * D, K - 1, Ks - 1
    mr = K >= 128
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g) if sbias else None
    w = torch.randn(G, 1, K, generator=g) / K ** 0.5
    wD = w.repeat_interleave(D // G, 0)
    bias = torch.randn(D, generator=g) if mr else None
    fst = torch.randn(B, C, Rf, generator=g).bfloat16()
    st = torch.randn(B, D, R, generator=g).bfloat16()
    fring, ring = va.FirRing.from_reference(fst.to(DEV)), va.FirRing.from_reference(st.to(DEV))
    taps = (w.reshape(G, K).flip(-1) if mr else w.reshape(G, K)).contiguous().to(DEV)
    inner = ops.FirStepper(ring, taps, bias=None if bias is None else bias.to(DEV), gated_bias=mr)
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    step = ops.LayerStepper(fring, wf.reshape(C, Ks).to(DEV), None if bf is None else bf.to(DEV), cmap, inner,
                            flip_x1x2=flip)
    ref_f, ref_s = fst, st
    for i in range(max(R, Rf) + 3):
        u = torch.randn(B, C, generator=g).bfloat16()
        z, ref_f = O.step_fir(u, ref_f, wf, bias=bf)
        x2, x1, v = oracle_gates(z, D, H, cs, il, flip)
        y_ref, ref_s = O.step_fir(x1 * v, ref_s, wD, bias=bias, gated_bias=mr, flip_filter=mr)
        y_ref = y_ref * x2
        y = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
        step(u.to(DEV), y)
        assert rel_err(y, y_ref) <= 2e-2, i
        if i in (0, Rf, R - 1, R + 2):
            assert torch.equal(fring.reference_order().cpu(), ref_f.float())          # copies of u: exact
            assert rel_err(ring.reference_order(), ref_s) <= 1e-2


@pytest.mark.parametrize("B,D,H,G,S,cplx,cs,il,flip,d_bf16", [
    (3, 512, 8, 512, 16, False, False, True, False, True),    # Evo 2 layout: real poles, one filter per channel
    (2, 256, 4, 16, 16, True, False, True, False, False),     # complex poles, grouped
    (2, 96, 4, 96, 16, True, True, False, True, False),       # column split (head_dim 24), flipped
    (2, 200, 5, 200, 32, False, False, False, False, True),   # plain split, 32 states
    (3, 48, 4, 48, 16, False, True, False, False, True),      # head_dim 12: no 16-byte pieces, scalar featurizer form
    (5, 72, 6, 72, 16, True, True, False, True, False),
    (1, 64, 4, 64, 8, True, True, True, False, False),        # interleave + column split has no fused map
])
def test_iir_layer_step_sequence_vs_oracle(B, D, H, G, S, cplx, cs, il, flip, d_bf16):
    g = torch.Generator().manual_seed(D + S)
    C, Ks = 3 * D, 3
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    if cplx:
        lp, r = O.make_modal_complex(G, S, seed=D)
    else:
        lp, r = O.make_modal_real(G, S, seed=D)
    Dc = torch.randn(D, generator=g)
    Dc = Dc.bfloat16() if d_bf16 else Dc
    fst = torch.randn(B, C, Ks - 1, generator=g).bfloat16()
    st0 = torch.randn(B, D, S, generator=g)
    if cplx:
        st0 = torch.complex(st0, torch.randn(B, D, S, generator=g))
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    if cmap is None:
        return
    state = st0.clone().to(DEV)
    fring = va.FirRing.from_reference(fst.to(DEV))
    poles = torch.exp(lp)[..., 0].contiguous()
    inner = ops.IirStepper(state, poles.to(DEV), r.to(DEV), Dc.to(DEV))
    step = ops.LayerStepper(fring, wf.reshape(C, Ks).to(DEV), None, cmap, inner, flip_x1x2=flip)
    dg = D // G
    lpD, rD = lp.repeat_interleave(dg, 0), r.repeat_interleave(dg, 0)
    ref_f, ref_s = fst, st0
    for i in range(5):
        u = torch.randn(B, C, generator=g).bfloat16()
        z, ref_f = O.step_fir(u, ref_f, wf)
        x2, x1, v = oracle_gates(z, D, H, cs, il, flip)
        y_ref, ref_s = O.step_iir(x2, x1, v, Dc, rD, lpD, ref_s)
        y_ref = y_ref.real if y_ref.is_complex() else y_ref
        y = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
        step(u.to(DEV), y)
        assert rel_err(y, y_ref) <= 2e-2, i
        assert torch.equal(fring.reference_order().cpu(), ref_f.float())
        sr = torch.view_as_real(ref_s) if cplx else ref_s
        sh = torch.view_as_real(state) if cplx else state
        assert rel_err(sh, sr) <= 1e-2, i


def test_windowed_modal_stepper_goes_back_to_the_plain_step_for_scalar_maps():
    # a head-blocked split with heads of 12 channels has no 16-byte pieces, so the fused layer step has no windowed
    # form: LayerStepper flushes the open windows (the state is exact again) and steps the state on every token
    B, D, H, S = 64, 1032, 86, 16
    g = torch.Generator().manual_seed(5)
    C, Ks = 3 * D, 3
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    lp, r = O.make_modal_real(D, S, seed=3)
    Dc = torch.randn(D, generator=g).bfloat16()
    fst = torch.randn(B, C, Ks - 1, generator=g).bfloat16()
    ref_s = torch.randn(B, D, S, generator=g)
    state = ref_s.clone().to(DEV)
    inner = ops.IirStepper(state, torch.exp(lp)[..., 0].contiguous().to(DEV), r.to(DEV), Dc.to(DEV), windowed=True)
    assert inner.win is not None
    y = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
    for i in range(2):                                      # two tokens inside open windows
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        y_ref, ref_s = O.step_iir(x2, x1, v, Dc, r, lp, ref_s)
        inner(x1.to(DEV), x2.to(DEV), v.to(DEV), y)
        assert rel_err(y, y_ref) <= 2e-2, i
    assert rel_err(state, ref_s) > 1e-3                     # lagging
    fring = va.FirRing.from_reference(fst.to(DEV))
    cmap = ops.gate_channel_map(D, head_dim=D // H)
    step = ops.LayerStepper(fring, wf.reshape(C, Ks).to(DEV), None, cmap, inner)
    assert inner.win is None and rel_err(state, ref_s) <= 1e-4
    ref_f = fst
    for i in range(3):
        u = torch.randn(B, C, generator=g).bfloat16()
        z, ref_f = O.step_fir(u, ref_f, wf)
        x2, x1, v = oracle_gates(z, D, H, True, False, False)
        y_ref, ref_s = O.step_iir(x2, x1, v, Dc, r, lp, ref_s)
        step(u.to(DEV), y)
        assert rel_err(y, y_ref) <= 2e-2, i
        assert rel_err(state, ref_s) <= 1e-3, i


def test_layer_step_rejects_bad_maps():
    D = 64
    fring = va.FirRing(torch.zeros(1, 2, 3 * D, dtype=torch.bfloat16, device=DEV))
    ring = va.FirRing(torch.zeros(1, 6, D, dtype=torch.bfloat16, device=DEV))
    inner = ops.FirStepper(ring, torch.zeros(D, 7, device=DEV))
    wf = torch.zeros(3 * D, 3, device=DEV)
    u, y = torch.zeros(1, 3 * D, dtype=torch.bfloat16, device=DEV), torch.empty(1, D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):          # map runs past the 3D channels
        ops.LayerStepper(fring, wf, None, (D, 0, D + 8, 1), inner)(u, y)
    with pytest.raises(NotImplementedError):  # head_dim not a multiple of 8 has no vector kernel
        ops.LayerStepper(fring, wf, None, (4, 12, 4, 1), inner)(u, y)


def _random_cases(seed, n, taps=(2, 3, 4)):
    import random
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        H = rng.choice([1, 2, 4])
        hd = 8 * rng.randint(1, 6)
        D = H * hd
        out.append((rng.randint(1, 5), D, H, rng.choice(taps), rng.choice(["plain", "split", "interleave"]),
                    rng.random() < 0.5, rng.random() < 0.5, rng.randint(0, 10 ** 6)))
    return out


# featurizers of 2-4 taps take the step that requests all its operands at once, longer ones (up to the 8 taps the
# library accepts) the slot-by-slot form
@pytest.mark.parametrize("B,D,H,Ks,layout,flip,sbias,seed", _random_cases(11, 16) + _random_cases(12, 8, (5, 6, 7, 8)))
def test_layer_steps_random(B, D, H, Ks, layout, flip, sbias, seed):
    # both fused layer steps on random channel maps, cache depths and group sizes, several tokens in a row
    import random
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    C = 3 * D
    cs, il = layout == "split", layout == "interleave"
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g) if sbias else None
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    # FIR layer: per-channel taps or 8-channel groups, short or long cache
    K = rng.choice([3, 7, 40, 128])
    G = D if rng.random() < 0.5 else D // 8
    mr = K == 128
    w = torch.randn(G, 1, K, generator=g) / K ** 0.5
    bias = torch.randn(D, generator=g) if mr else None
    fst, st = torch.randn(B, C, Ks - 1, generator=g).bfloat16(), torch.randn(B, D, K - 1, generator=g).bfloat16()
    fring, ring = va.FirRing.from_reference(fst.to(DEV)), va.FirRing.from_reference(st.to(DEV))
    taps = (w.reshape(G, K).flip(-1) if mr else w.reshape(G, K)).contiguous().to(DEV)
    fir = ops.LayerStepper(fring, wf.reshape(C, Ks).to(DEV), None if bf is None else bf.to(DEV), cmap,
                           ops.FirStepper(ring, taps, bias=None if bias is None else bias.to(DEV), gated_bias=mr),
                           flip_x1x2=flip)
    # IIR layer on the same projections
    S = rng.choice([16, 32])
    cplx = rng.random() < 0.5
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(D, S, seed=seed % 1000)
    Dc = torch.randn(D, generator=g).bfloat16()
    s0 = torch.randn(B, D, S, generator=g)
    s0 = torch.complex(s0, torch.randn(B, D, S, generator=g)) if cplx else s0
    state, fring2 = s0.clone().to(DEV), va.FirRing.from_reference(fst.to(DEV))
    iir = ops.LayerStepper(fring2, wf.reshape(C, Ks).to(DEV), None if bf is None else bf.to(DEV), cmap,
                           ops.IirStepper(state, torch.exp(lp)[..., 0].contiguous().to(DEV), r.to(DEV), Dc.to(DEV)),
                           flip_x1x2=flip)
    wD = w.repeat_interleave(D // G, 0)
    ref_f, ref_s, ref_m = fst, st, s0
    for i in range(max(4, Ks + 1)):              # past one turn of the featurizer's ring
        u = torch.randn(B, C, generator=g).bfloat16()
        z, ref_f = O.step_fir(u, ref_f, wf, bias=bf)
        x2, x1, v = oracle_gates(z, D, H, cs, il, flip)
        y_ref, ref_s = O.step_fir(x1 * v, ref_s, wD, bias=bias, gated_bias=mr, flip_filter=mr)
        y = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
        fir(u.to(DEV), y)
        assert rel_err(y, y_ref * x2) <= 2e-2, ("fir", i, K, G)
        y2_ref, ref_m = O.step_iir(x2, x1, v, Dc, r, lp, ref_m)
        y2 = torch.empty(B, D, dtype=torch.bfloat16, device=DEV)
        iir(u.to(DEV), y2)
        assert rel_err(y2, y2_ref.real if cplx else y2_ref) <= 2e-2, ("iir", i, S, cplx)
    assert rel_err(ring.reference_order(), ref_s) <= 1e-2
    assert rel_err(torch.view_as_real(state) if cplx else state, torch.view_as_real(ref_m) if cplx else ref_m) <= 1e-2


def test_ring_positions_on_the_device():
    # hyena_fir_step_dpos / hyena_fir_layer_step_dpos / hyena_ring_advance: the same steps with the ring positions
    # kept in device memory give bit-identical outputs and caches
    B, D, G, K, Ks = 3, 512, 32, 7, 3
    g = torch.Generator().manual_seed(5)
    w = torch.randn(G, K, generator=g).cuda()
    fw = torch.randn(3 * D, Ks, generator=g).cuda()
    cmap = ops.gate_channel_map(D, interleave=True)

    def fresh():
        gg = torch.Generator().manual_seed(6)
        fr = ops.FirRing(torch.randn(B, Ks - 1, 3 * D, generator=gg).bfloat16().cuda(), 1)
        ir = ops.FirRing(torch.randn(B, K - 1, D, generator=gg).bfloat16().cuda(), 4)
        return fr, ir, ops.LayerStepper(fr, fw, None, cmap, ops.FirStepper(ir, w))

    fr_h, ir_h, step_h = fresh()
    fr_d, ir_d, step_d = fresh()
    clock = ops.RingClock([fr_d, ir_d])
    for t in range(15):
        u = torch.randn(B, 3 * D, generator=g).bfloat16().cuda()
        y_h = step_h(u, torch.empty(B, D, dtype=torch.bfloat16, device="cuda"))
        y_d = step_d(u, torch.empty(B, D, dtype=torch.bfloat16, device="cuda"))
        clock.advance()
        assert torch.equal(y_h, y_d), t
    assert clock.pos.tolist() == [fr_h.pos, ir_h.pos]
    assert torch.equal(fr_h.reference_order(), fr_d.reference_order())
    assert torch.equal(ir_h.reference_order(), ir_d.reference_order())
    # the plain (unfused) step through the same clock
    x1, x2, v = (torch.randn(B, D, generator=g).bfloat16().cuda() for _ in range(3))
    y_d = va.fir_step(x1, ir_d, w, x2=x2, v=v)
    y_h = va.fir_step(x1, ir_h, w, x2=x2, v=v)
    clock.advance()
    assert torch.equal(y_h, y_d)
    clock.release()
    assert ir_d.pos == ir_h.pos and ir_d.pos_dev is None
    assert fr_d.pos == (fr_h.pos + 1) % (Ks - 1)          # the clock moved this ring too; no step used it
