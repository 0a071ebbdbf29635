"""GPU parity of the decode-step kernels against the CPU oracle and the committed
reference vectors (tests/golden/decode_steps.npz), through the C ABI."""
import os

import numpy as np
import pytest
import torch

import vortex_amd as va
from oracle import hyena_oracle as O

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_steps.npz"))


def eff_taps(weight, cache, flip):
    """Slicing of vortex/model/engine.py:417-425, as [G, cache+1] oldest tap first."""
    w = weight.reshape(weight.shape[0], -1)
    return (w.flip(-1)[..., -cache - 1:] if flip else w[..., : cache + 1]).contiguous()


@pytest.mark.parametrize("name", ["se", "mr", "feat", "partial", "partial_flip"])
def test_fir_step_golden(name):
    K, cache, flip, gated, _, _ = GOLD[f"fir_{name}_meta"].tolist()
    u = torch.from_numpy(GOLD[f"fir_{name}_u"]).bfloat16()
    st = torch.from_numpy(GOLD[f"fir_{name}_state"]).bfloat16()
    w = torch.from_numpy(GOLD[f"fir_{name}_w"])
    bias = torch.from_numpy(GOLD[f"fir_{name}_bias"]) if f"fir_{name}_bias" in GOLD else None
    ring = va.FirRing.from_reference(st.cuda())
    y = va.fir_step(u.cuda(), ring, eff_taps(w, cache, flip).cuda(), bias=None if bias is None else bias.cuda(),
                    gated_bias=bool(gated))
    ye = torch.from_numpy(GOLD[f"fir_{name}_y"])
    assert (y.float().cpu() - ye).abs().max() <= 2e-2 * ye.abs().max()
    # cache after the step: reference appends while the cache is short, ring keeps its depth
    exp_state = torch.from_numpy(GOLD[f"fir_{name}_state_out"])[..., -cache:]
    assert torch.equal(ring.reference_order().cpu(), exp_state)


@pytest.mark.parametrize("B,D,G,K,flip,gated", [
    (4, 512, 32, 7, False, False),       # SE: dg = 16
    (3, 1024, 64, 128, True, True),      # MR
    (2, 1536, 1536, 3, False, False),    # featurizer: per-channel taps over 3D channels
    (2, 520, 65, 128, True, True),       # D not a multiple of the 512-channel block
])
def test_fir_step_sequence_vs_oracle(B, D, G, K, flip, gated):
    g = torch.Generator().manual_seed(K + D)
    R = K - 1
    w = torch.randn(G, 1, K, generator=g) / K ** 0.5
    wD = w.repeat_interleave(D // G, 0)
    bias = torch.randn(D, generator=g) if gated else None
    st = torch.randn(B, D, R, generator=g).bfloat16()
    ring = va.FirRing.from_reference(st.cuda())
    taps = eff_taps(w, R, flip).cuda()
    ref_state = st
    for step in range(R + 3):            # wraps the ring at least once
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        y_ref, ref_state = O.step_fir(x1 * v, ref_state, wD, bias=bias, gated_bias=gated, flip_filter=flip)
        y_ref = y_ref * x2
        y = va.fir_step(x1.cuda(), ring, taps, x2=x2.cuda(), v=v.cuda(), bias=None if bias is None else bias.cuda(),
                        gated_bias=gated)
        err = (y.float().cpu() - y_ref.float()).abs().max() / y_ref.float().abs().max()
        assert err <= 2e-2, (step, err)
        if step in (0, R - 1, R + 2):
            assert torch.equal(ring.reference_order().cpu(), ref_state)


@pytest.mark.parametrize("D,blocks", [(1536, (1536, 512)), (2048, (2048, 512, 1024)), (4096, (4096, None))])
def test_fir_step_channel_blocked_cache(D, blocks):
    """The cache layouts [B, D/block, R, block] hold the same ring: outputs and contents are bit-equal to the plain
    [B, R, D] cache (block = D) over more steps than the ring has slots, and the plain one matches the oracle."""
    B, G, K = 3, D // 16, 128
    R = K - 1
    g = torch.Generator().manual_seed(D)
    w = torch.randn(G, 1, K, generator=g) / K ** 0.5
    bias = torch.randn(D, generator=g)
    st = torch.randn(B, D, R, generator=g).bfloat16()
    rings = [va.FirRing.from_reference(st.cuda(), block=b) for b in blocks]
    assert rings[0].block == D and all(r.block == 512 for r in rings[1:2])
    assert all(torch.equal(r.reference_order().cpu(), st.float()) for r in rings)
    taps = eff_taps(w, R, True).cuda()
    ref_state = st
    for step in range(R + 4):
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        ys = [va.fir_step(x1.cuda(), r, taps, x2=x2.cuda(), v=v.cuda(), bias=bias.cuda(), gated_bias=True) for r in rings]
        assert all(torch.equal(ys[0], y) for y in ys[1:]), step
        if step in (0, 5, R - 1, R + 3):
            y_ref, ref_state = O.step_fir(x1 * v, ref_state, w.repeat_interleave(16, 0), bias=bias, gated_bias=True,
                                          flip_filter=True)
            y_ref = (y_ref * x2).float()
            assert (ys[0].float().cpu() - y_ref).abs().max() <= 2e-2 * y_ref.abs().max()
            assert all(torch.equal(r.reference_order().cpu(), ref_state) for r in rings), step
        else:
            _, ref_state = O.step_fir(x1 * v, ref_state, w.repeat_interleave(16, 0), bias=bias, gated_bias=True,
                                      flip_filter=True)


@pytest.mark.parametrize("B,D,G,R,gated,on_clock", [
    (3, 1024, 64, 127, True, False),      # Hyena-MR cache, grouped taps
    (2, 1536, 1536, 127, True, False),    # one tap row per channel
    (5, 520, 65, 127, False, False),      # D not a multiple of the 512-channel block
    (1, 512, 32, 40, True, False),        # a shorter deep cache (counter period lcm(3, 40))
    (4, 2048, 128, 127, True, True),      # counter in device memory (what a recorded token step uses)
])
def test_fir_step_far_sums(B, D, G, R, gated, on_clock):
    """The stepper that keeps far sums (it reads its whole cache only every third token, staggered over the blocks)
    against the oracle and against the plain step on a copy of the cache, for more tokens than two ring periods, with
    a plain step on the same cache in between (the stepper then rebuilds its far sums)."""
    from vortex_amd import _lib, ops
    g = torch.Generator().manual_seed(D + R)
    K = R + 1
    w = torch.randn(G, 1, K, generator=g) / K ** 0.5
    wD = w.repeat_interleave(D // G, 0)
    bias = torch.randn(D, generator=g) if gated else None
    st = torch.randn(B, D, R, generator=g).bfloat16()
    taps = eff_taps(w, R, True).cuda()
    rings = [va.FirRing.from_reference(st.cuda()) for _ in range(2)]
    bias_d = None if bias is None else bias.cuda()
    far = ops.FirStepper(rings[0], taps, bias=bias_d, gated_bias=gated)
    plain = ops.FirStepper(rings[1], taps, bias=bias_d, gated_bias=gated, far_sums=False)
    assert far.far is not None and plain.far is None and rings[0].period == _lib.lib().hyena_fir_far_period(R)
    clock = ops.RingClock([rings[0]]) if on_clock else None
    ref_state = st
    ya, yb = (torch.empty(B, D, dtype=torch.bfloat16, device="cuda") for _ in range(2))
    worst = 0.0
    for step in range(2 * R + 7):
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        y_ref, ref_state = O.step_fir(x1 * v, ref_state, wD, bias=bias, gated_bias=gated, flip_filter=True)
        y_ref = (y_ref * x2).float()
        if step in (5, R + 1) and not on_clock:      # something else steps the cache: the far sums are rebuilt afterwards
            ya = va.fir_step(x1.cuda(), rings[0], taps, x2=x2.cuda(), v=v.cuda(), bias=bias_d, gated_bias=gated)
            assert rings[0].far_owner is None
        else:
            far(x1.cuda(), x2.cuda(), v.cuda(), ya)
            if clock is not None:
                clock.advance()
        plain(x1.cuda(), x2.cuda(), v.cuda(), yb)
        assert (ya.float().cpu() - y_ref).abs().max() <= 2e-2 * y_ref.abs().max(), step
        # against the plain step: the same products summed in another order, so at most the last bf16 digit moves
        d = (ya.float() - yb.float()).abs()
        tol = yb.float().abs() * 2.0 ** -7 + 2e-3 * x2.cuda().float().abs()
        assert (d <= tol).all(), (step, (d / tol).max().item())
        worst = max(worst, (d > 0).float().mean().item())
        if step in (0, 6, R, 2 * R + 6):
            if clock is not None:
                torch.cuda.synchronize()
            assert torch.equal(rings[0].reference_order().cpu(), ref_state), step
    assert worst < 0.2, worst          # nearly every output is bit-identical
    if clock is not None:
        clock.release()
        assert rings[0].pos == (2 * R + 7) % rings[0].period


@pytest.mark.parametrize("name", ["real_bf16D", "real_f32D", "cplx_f32D"])
def test_iir_step_golden(name):
    x2, x1, v = (torch.from_numpy(GOLD[f"iir_{name}_{k}"]).bfloat16().cuda() for k in ("x2", "x1", "v"))
    Dp = torch.from_numpy(GOLD[f"iir_{name}_D"])
    if "bf16D" in name:
        Dp = Dp.bfloat16()
    lp, r, st = (torch.from_numpy(GOLD[f"iir_{name}_{k}"]) for k in ("lp", "r", "state"))
    state = st.clone().cuda()
    y = va.iir_step(x1, x2, v, state, torch.exp(lp[..., 0]).cuda(), r.cuda(), Dp.cuda(), out_dtype=torch.float32)
    ye = torch.from_numpy(GOLD[f"iir_{name}_y"])
    ye = ye.real if ye.is_complex() else ye
    se = torch.from_numpy(GOLD[f"iir_{name}_state_out"])
    assert (y.cpu() - ye).abs().max() <= 1e-5 * ye.abs().max()
    assert (state.cpu() - se).abs().max() <= 1e-5 * se.abs().max()


@pytest.mark.parametrize("cplx,G,S", [(False, 256, 16), (True, 256, 16), (True, 16, 16), (False, 1, 16),
                                      (False, 256, 8), (True, 16, 8), (False, 1, 2), (True, 256, 2), (False, 16, 1),
                                      (True, 1, 1), (False, 256, 4), (True, 16, 4), (False, 16, 32), (True, 256, 32)])
def test_iir_step_sequence_vs_oracle(cplx, G, S):
    B, D = 5, 256
    g = torch.Generator().manual_seed(3)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, S, seed=4)
    Dp = torch.randn(D, generator=g).bfloat16()
    lpD, rD = lp.repeat_interleave(D // G, 0), r.repeat_interleave(D // G, 0)
    st_ref = torch.zeros(B, D, S, dtype=torch.complex64 if cplx else torch.float32)
    state = st_ref.clone().cuda()
    poles = torch.exp(lp[..., 0]).cuda()
    for step in range(20):
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        y_ref, st_ref = O.step_iir(x2, x1, v, Dp, rD, lpD, st_ref)
        y_ref = (y_ref.real if cplx else y_ref).to(torch.bfloat16)
        y = va.iir_step(x1.cuda(), x2.cuda(), v.cuda(), state, poles, r.cuda(), Dp.cuda())
        assert (y.float().cpu() - y_ref.float()).abs().max() <= 2e-2 * y_ref.float().abs().max()
    assert (state.cpu() - st_ref).abs().max() <= 1e-4 * st_ref.abs().max()


@pytest.mark.parametrize("cplx,B,D,G,fused,on_clock", [
    (True, 64, 2048, 128, False, False),     # complex poles, grouped
    (False, 64, 4096, 4096, False, False),   # vortex's own: real poles, one filter per channel
    (True, 50, 2048, 2048, True, False),     # layer step from the projection (interleaved gates)
    (False, 37, 2056, 257, True, True),      # counter in device memory; D not a multiple of 256
    (True, 70, 1000, 125, False, False),     # D a multiple of 8 only
    (True, 68, 4104, 513, False, False),     # large enough for two batch elements per block at a window's head (17 of them)
    (False, 130, 4096, 4096, True, True),    # the same from the projection, counters in device memory
])
def test_iir_step_windowed_state(cplx, B, D, G, fused, on_clock):
    """The stepper that reads and writes the modal state once per window of four tokens (windows staggered over the
    batch elements): outputs against the oracle on every token, the state after flush() against the oracle's, a flush
    in the middle of the run (windows restart), and the plain stepper on a copy of the state for comparison."""
    from vortex_amd import _lib, ops
    S, W = 16, _lib.lib().hyena_iir_window_tokens()
    assert _lib.lib().hyena_iir_window_supported(B, D, S, int(cplx))
    g = torch.Generator().manual_seed(D + cplx)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, S, seed=9)
    Dp = torch.randn(D, generator=g).bfloat16()
    lpD, rD = lp.repeat_interleave(D // G, 0), r.repeat_interleave(D // G, 0)
    dt = torch.complex64 if cplx else torch.float32
    st_ref = (torch.randn(B, D, S, generator=g) * 0.5).to(dt)
    states = [st_ref.clone().cuda() for _ in range(2)]
    poles = torch.exp(lp[..., 0]).cuda()
    win = ops.IirStepper(states[0], poles, r.cuda(), Dp.cuda(), windowed=True)
    plain = ops.IirStepper(states[1], poles, r.cuda(), Dp.cuda())
    assert win.win is not None and plain.win is None
    C = 3 * D
    if fused:
        wf = torch.randn(C, 1, 3, generator=g) / 3 ** 0.5
        fst = torch.randn(B, C, 2, generator=g).bfloat16()
        frings = [va.FirRing.from_reference(fst.cuda()) for _ in range(2)]
        cmap = ops.gate_channel_map(D, interleave=True)
        steps = [ops.LayerStepper(fr, wf.reshape(C, 3).cuda(), None, cmap, n) for fr, n in zip(frings, (win, plain))]
        assert win.win is not None
        ref_f = fst
    clock = None
    ya, yb = (torch.empty(B, D, dtype=torch.bfloat16, device="cuda") for _ in range(2))
    as_real = lambda t: torch.view_as_real(t) if cplx else t
    for step in range(4 * W + 2):
        if on_clock and step == W + 1:              # from here on the counters live in device memory
            clock = ops.RingClock([win] + ([frings[0]] if fused else []))
        if fused:
            u = torch.randn(B, C, generator=g).bfloat16()
            z, ref_f = O.step_fir(u, ref_f, wf)
            x2, x1, v = O.interleave(z).split([D] * 3, dim=1)
            steps[0](u.cuda(), ya)
            steps[1](u.cuda(), yb)
        else:
            x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
            win(x1.cuda(), x2.cuda(), v.cuda(), ya)
            plain(x1.cuda(), x2.cuda(), v.cuda(), yb)
        if clock is not None:
            clock.advance()
        y_ref, st_ref = O.step_iir(x2, x1, v, Dp, rD, lpD, st_ref)
        y_ref = (y_ref.real if cplx else y_ref).float()
        assert (ya.float().cpu() - y_ref).abs().max() <= 2e-2 * y_ref.abs().max(), step
        d = (ya.float() - yb.float()).abs().max().item()
        assert d <= 2e-2 * y_ref.abs().max().item(), (step, d)
        if step in (W - 1, 2 * W):                  # the state as anyone else may read it
            win.flush()
            sr = as_real(st_ref)
            assert (as_real(states[0]).cpu() - sr).abs().max() <= (2e-3 if fused else 1e-4) * sr.abs().max(), step
            assert win.warm == 0
    assert not torch.equal(as_real(states[0]).cpu(), as_real(states[1]).cpu())      # the state lags until the flush
    win.flush()
    sr = as_real(st_ref)
    assert (as_real(states[0]).cpu() - sr).abs().max() <= (2e-3 if fused else 1e-4) * sr.abs().max()
    assert (as_real(states[0]) - as_real(states[1])).abs().max() <= 1e-4 * sr.abs().max()
    if clock is not None:
        clock.release()


def test_windowed_stepper_flush_around_a_recorded_step():
    """A recorded token step (a HIP graph) replays the windowed modal step with "every window open" in its arguments.
    A flush while that recording can still be replayed is refused; after release() the flush leaves the exact state,
    eager steps continue the sequence, and a new recording after `period` eager steps replays correctly."""
    from vortex_amd import _lib, ops
    cplx, B, D, G, S = True, 64, 1024, 64, 16
    W = _lib.lib().hyena_iir_window_tokens()
    g = torch.Generator().manual_seed(77)
    lp, r = O.make_modal_complex(G, S, seed=78)
    Dp = torch.randn(D, generator=g).bfloat16()
    lpD, rD = lp.repeat_interleave(D // G, 0), r.repeat_interleave(D // G, 0)
    st_ref = (torch.randn(B, D, S, generator=g) * 0.5).to(torch.complex64)
    state = st_ref.clone().cuda()
    win = ops.IirStepper(state, torch.exp(lp[..., 0]).cuda(), r.cuda(), Dp.cuda(), windowed=True)
    assert win.win is not None
    gx = [torch.empty(B, D, dtype=torch.bfloat16, device="cuda") for _ in range(3)]     # x1, x2, v of the recording
    y = torch.empty(B, D, dtype=torch.bfloat16, device="cuda")

    def token(run):
        nonlocal st_ref
        x1, x2, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
        for dst, src in zip(gx, (x1, x2, v)):
            dst.copy_(src)
        run()
        y_ref, st_ref = O.step_iir(x2, x1, v, Dp, rD, lpD, st_ref)
        assert (y.float().cpu() - y_ref.real.float()).abs().max() <= 2e-2 * y_ref.real.abs().max()

    def record():
        clock = ops.RingClock([win])
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            win(gx[0], gx[1], gx[2], y)
            clock.advance()
        return clock, graph

    eager = lambda: win(gx[0], gx[1], gx[2], y)
    for _ in range(W + 1):
        token(eager)
    clock, graph = record()              # the capture runs no kernel and moves no counter
    for _ in range(7):
        token(graph.replay)
    with pytest.raises(RuntimeError, match="recorded"):
        win.flush()
    clock.release()
    win.flush()
    sr = torch.view_as_real(st_ref)
    assert (torch.view_as_real(state).cpu() - sr).abs().max() <= 1e-4 * sr.abs().max()
    for _ in range(W + 2):
        token(eager)
    clock, graph = record()
    for _ in range(6):
        token(graph.replay)
    clock.release()
    win.flush()
    sr = torch.view_as_real(st_ref)
    assert (torch.view_as_real(state).cpu() - sr).abs().max() <= 1e-4 * sr.abs().max()
