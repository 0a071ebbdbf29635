#!/usr/bin/env python3
"""Benchmark of the Hyena operator hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mr|se|li|decode|mr_cl|mr_layer|se_layer] [--no-extras]

A "step" is one pass of the operator over one batch of synthetic input that is
already resident in HBM.  The headline workload is the Hyena-MR prefill
configuration (B=2, L=32768, D=4096, 256 filter groups, K=128); the other
configurations (Hyena-SE, Hyena-LI prefill, the cached decode step) are
measured the same way and reported under "extra" unless --no-extras is given.
Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X published HBM3E bandwidth

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what the same
# counter reads for the plain copy launch of known size.  These are constants of the committed profile, not
# measurements of this run: `roofline.traffic_source` names the file they were read from.
MEASURED_TRAFFIC = {"mr": 2148.09e6, "se": 271.75e6, "li": 8592.12e6}
TRAFFIC_SOURCE = "profiles/bench_default_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; copy-probe calibrated)"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="mr", choices=["mr", "se", "se_b8", "li", "li_g4096", "decode", "mr_cl", "mr_layer", "li_layer",
                                                         "se_layer", "mr_cl_f16", "cl_f32", "li_layer_seq", "li_layer_seq_g4096", "mr_layer_seq"])
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed run of each workload before its warm-up steps, until clocks have settled")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-model", action="store_true", help="skip the end-to-end model prefill legs")
    ap.add_argument("--no-copy-probe", action="store_true",
                    help="skip the plain 1 GiB device copy whose rate is reported as roofline.copy_probe_gbs")
    ap.add_argument("--launch-override", action="append", default=[], metavar="NAME=VALUE",
                    help="pin one launch-shape choice of the library for the whole run (hyena_set_launch_override), "
                         "e.g. cl_ns=1 for one channel strip per block; recorded in config.launch_overrides")
    return ap.parse_args()


def gates(B, D, L, seed, device):
    g = torch.Generator(device=device).manual_seed(seed)
    return tuple(torch.randn(B, D, L, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
                 for _ in range(3))


class _Synthetic:
    """Seeded synthetic filters and poles of the benchmark configurations (generated on the CPU, as the parity
    tests generate theirs, so every run sees the same values)."""

    @staticmethod
    def make_se_filter(G, K=7, seed=100):
        g = torch.Generator(device="cpu").manual_seed(seed)
        return torch.randn(G, 1, K, generator=g) / math.sqrt(K)

    @staticmethod
    def make_mr_filter(G, K=128, seed=200):
        g = torch.Generator(device="cpu").manual_seed(seed)
        w = torch.randn(G, 1, K, generator=g) / math.sqrt(K)
        a = 0.01 + 0.09 * torch.rand(G, 1, 1, generator=g)
        return w * torch.exp(-a * torch.arange(K)[None, None])

    @staticmethod
    def make_modal_complex(G, S=16, seed=300, pmin=0.9, pmax=0.9999):
        g = torch.Generator(device="cpu").manual_seed(seed)
        mag = pmin + (pmax - pmin) * torch.rand(G, S, generator=g, dtype=torch.float64)
        ang = math.pi * torch.rand(G, S, generator=g, dtype=torch.float64)
        log_poles = torch.complex(mag.log(), ang).to(torch.complex64)[..., None]
        res = torch.complex(torch.randn(G, S, generator=g), torch.randn(G, S, generator=g)) / math.sqrt(2.0)
        return log_poles, res.to(torch.complex64)


SETTLE_S = 0.15     # set from --settle-ms


def time_steps(fn, steps, warmup, settle=None):
    """(wall seconds for `steps` calls, average kernel-side ms per call from HIP events on the launch stream).

    Before the `warmup` untimed steps the workload runs for SETTLE_S seconds, also untimed: after lighter work the
    first tens of launches of a bandwidth-heavy kernel run up to 15 % slower (clock and power management settling),
    and a short run would measure that transient instead of the sustained rate."""
    settle = SETTLE_S if settle is None else settle
    t_end = time.perf_counter() + settle
    while settle > 0 and time.perf_counter() < t_end:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        fn()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return t1 - t0, ev0.elapsed_time(ev1) / steps


def build_workload(name, device):
    """Returns (callable, description dict) for one configuration."""
    import vortex_amd as va
    O = _Synthetic
    from vortex_amd import ops

    if name in ("se", "se_b8"):
        # config 1 (268 MB working set: close to the 256 MB last-level cache) and the same rows at batch 8 (2.1 GB)
        B, D, L, G, K = (1 if name == "se" else 8), 4096, 8192, 256, 7
        x2, x1, v = gates(B, D, L, 1, device)
        h = O.make_se_filter(G, K).reshape(G, K).to(device)
        r1, r2, rv = ops.rows_of(x1), ops.rows_of(x2), ops.rows_of(v)
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)
        fn = lambda: ops.fir_fwd_rows(r1, r2, rv, h, B, D, L, K, device=device, taps_reversed=True, out=out)
        return fn, dict(workload=f"hyena_se_prefill B={B} L={L} D={D} groups={G} K={K}", tokens=B * L,
                        bytes=8 * B * D * L, kernel="se_fir_kernel", keep=(x1, x2, v, h, out))
    if name == "mr":
        B, D, L, G, K = 2, 4096, 32768, 256, 128
        x2, x1, v = gates(B, D, L, 2, device)
        h = O.make_mr_filter(G, K).reshape(G, K).to(device)
        Db = torch.randn(D, generator=torch.Generator().manual_seed(3)).to(device)
        r1, r2, rv = ops.rows_of(x1), ops.rows_of(x2), ops.rows_of(v)
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)
        fn = lambda: ops.fir_fwd_rows(r1, r2, rv, h, B, D, L, K, device=device, bias=Db,
                                      bias_mode=ops.HYENA_BIAS_GATED_FP32, force_mfma=True, out=out)
        return fn, dict(workload=f"hyena_mr_prefill B={B} L={L} D={D} groups={G} K={K}", tokens=B * L,
                        bytes=8 * B * D * L, kernel="mr_fir_kernel", keep=(x1, x2, v, h, Db, out))
    if name in ("li", "li_g4096"):
        # config 3, and the same rows with one filter per channel (vortex's own hcl_filter_groups == hidden_size)
        B, D, L, G, S = 1, 4096, 262144, (256 if name == "li" else 4096), 16
        x2, x1, v = gates(B, D, L, 4, device)
        lp, r = O.make_modal_complex(G, S)
        Db = torch.randn(D, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(device)
        plan = va.ModalPlan(lp.to(device), r.to(device))
        r1, r2, rv = ops.rows_of(x1), ops.rows_of(x2), ops.rows_of(v)
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)
        fn = lambda: ops.li_fwd_rows(r1, r2, rv, plan, Db, B, D, L, device=device, out=out)
        return fn, dict(workload=f"hyena_li_prefill B={B} L={L} D={D} groups={G} poles={S} complex", tokens=B * L,
                        bytes=8 * B * D * L, kernel="li_kernel", keep=(x1, x2, v, plan, Db, out))
    if name in ("mr_cl", "mr_layer", "se_layer"):
        # channel-last variants: gates as three [B, L, D] tensors, or the whole layer from the projection
        # u [B, L, 3D] (Evo 2 layout: interleaved gates, 3-tap featurizer); 8 bytes per output element either way
        mr = name != "se_layer"
        B, D, L, G, K = (2, 4096, 32768, 256, 128) if mr else (1, 4096, 8192, 256, 7)
        g = torch.Generator(device=device).manual_seed(9)
        rnd = lambda *s: torch.randn(*s, generator=g, device=device, dtype=torch.float32)
        h = (O.make_mr_filter(G, K) if mr else O.make_se_filter(G, K)).reshape(G, K).to(device)
        Db = rnd(D) if mr else None
        mode = ops.HYENA_BIAS_GATED_FP32 if mr else ops.HYENA_BIAS_NONE
        out = torch.empty(B, L, D, dtype=torch.bfloat16, device=device)
        if name == "mr_cl":
            x = [rnd(B, L, D).to(torch.bfloat16) for _ in range(3)]
            fn = lambda: ops.fir_cl_fwd(x[1], x[0], x[2], h, bias=Db, bias_mode=mode, out=out)
            what, keep = "hyena_mr_prefill channel-last gates", (x, h, Db, out)
        else:
            u = rnd(B, L, 3 * D).to(torch.bfloat16)
            wf = rnd(3, 3 * D) * 3 ** -0.5
            cmap = ops.gate_channel_map(D, interleave=True)
            fn = lambda: ops.fir_layer_fwd(u, wf, None, cmap, h, bias=Db, bias_mode=mode, taps_reversed=not mr, out=out)
            what, keep = ("hyena_mr" if mr else "hyena_se") + "_layer featurizer+operator from the projection", (u, wf, h, Db, out)
        return fn, dict(workload=f"{what} B={B} L={L} D={D} groups={G} K={K}", tokens=B * L, bytes=8 * B * D * L,
                        kernel="fir_cl_kernel", keep=keep)
    if name in ("mr_cl_f16", "cl_f32"):
        # the element types of the reference's own grid for this operator (vortex/ops/hyena_se/tests/test_fwd.py:25-54):
        # float16 on the MFMA kernel at the config-2 shape, float32 on the direct-form kernel at the grid's largest
        # case (batch 2, seqlen 8192, d 4096, one filter group, 128 taps from N(0, 1))
        f16 = name == "mr_cl_f16"
        B, D, L, G, K = (2, 4096, 32768, 256, 128) if f16 else (2, 4096, 8192, 1, 128)
        dt = torch.float16 if f16 else torch.float32
        g = torch.Generator(device=device).manual_seed(11)
        x = [torch.randn(B, L, D, generator=g, device=device, dtype=torch.float32).to(dt) for _ in range(3)]
        h = (O.make_mr_filter(G, K) if f16 else torch.randn(G, 1, K, generator=torch.Generator().manual_seed(12))).reshape(G, K).to(device)
        out = torch.empty(B, L, D, dtype=dt, device=device)
        fn = lambda: ops.fir_cl_fwd(x[1], x[0], x[2], h, taps_reversed=True, out=out)
        es = 2 if f16 else 4
        return fn, dict(workload=f"gated FIR on (b, l, g, dg) tensors, {'float16 (MFMA)' if f16 else 'float32 (float32 MFMA)'} "
                                 f"B={B} L={L} D={D} groups={G} K={K}", tokens=B * L, bytes=4 * es * B * D * L,
                        kernel="fir_cl_kernel" if f16 else "fir_cl_f32_ring_kernel", keep=(x, h, out),
                        **({} if f16 else {"flops": 2.0 * K * B * D * L}))
    if name == "li_layer":
        # a whole Hyena-LI layer from the projection at the config-3 shape: featurizer + split + x1*v in one launch
        # (rows xv, x2), then the modal scan on them; 8 bytes per output element would be a one-pass layer, the two
        # launches move 16 (10 + 6)
        B, D, L, G, S = 1, 4096, 262144, 256, 16
        g = torch.Generator(device=device).manual_seed(10)
        u = torch.randn(B, L, 3 * D, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
        wf = torch.randn(3, 3 * D, generator=g, device=device, dtype=torch.float32) * 3 ** -0.5
        cmap = ops.gate_channel_map(D, interleave=True)
        lp, r = O.make_modal_complex(G, S)
        Db = torch.randn(D, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(device)
        plan = va.ModalPlan(lp.to(device), r.to(device))
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)

        def fn():
            xv, x2 = ops.featurizer_gates_fwd(u, wf, None, cmap)
            ops.li_fwd_rows(ops.rows_of(xv), ops.rows_of(x2), None, plan, Db, B, D, L, device=device, out=out)

        return fn, dict(workload=f"hyena_li_layer featurizer+gates then modal scan, from the projection B={B} L={L} D={D} "
                                 f"groups={G} poles={S} complex", tokens=B * L, bytes=8 * B * D * L,
                        kernel="proj_gates_kernel + li_kernel", keep=(u, wf, plan, Db, out))
    if name == "mr_layer_seq":
        # the Hyena-MR layer of config 2 from a projection stored sequence-major: featurizer, split, gates and the
        # inner FIR in one launch of the sequence-major MFMA kernel; 6 bytes read + 2 written per (channel, sample)
        B, D, L, G, K = 2, 4096, 32768, 256, 128
        g = torch.Generator(device=device).manual_seed(9)
        p = torch.randn(B, 3 * D, L, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
        w = torch.randn(3 * D, 3, generator=g, device=device, dtype=torch.float32) * 3 ** -0.5
        (q2, q1, qv), chan = ops.projection_rows(p, D, interleave=True)
        taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
        h = O.make_mr_filter(G, K).reshape(G, K).to(device)
        Db = torch.randn(D, generator=g, device=device, dtype=torch.float32)
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)
        fn = lambda: ops.fir_layer_fwd_rows(q1, q2, qv, taps, h, B, D, L, K, device=device, bias=Db,
                                            bias_mode=ops.HYENA_BIAS_GATED_FP32, out=out)
        return fn, dict(workload=f"hyena_mr_layer in one launch from a sequence-major projection B={B} L={L} D={D} "
                                 f"groups={G} K={K}", tokens=B * L, bytes=8 * B * D * L, kernel="mr_fir_kernel",
                        keep=(p, taps, h, Db, out))
    if name in ("li_layer_seq", "li_layer_seq_g4096"):
        # the same layer from the same projection values stored sequence-major ([B, 3D, L], what the projection GEMM
        # writes when asked for the transposed product): featurizer, split, gates and the modal scan in ONE launch,
        # 6 bytes read + 2 written per (channel, sample) -- the algorithmic 8
        B, D, L, S = 1, 4096, 262144, 16
        G = 4096 if name.endswith("g4096") else 256
        g = torch.Generator(device=device).manual_seed(10)
        p = torch.randn(B, 3 * D, L, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
        w = torch.randn(3 * D, 3, generator=g, device=device, dtype=torch.float32) * 3 ** -0.5
        (q2, q1, qv), chan = ops.projection_rows(p, D, interleave=True)
        taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
        lp, r = O.make_modal_complex(G, S)
        Db = torch.randn(D, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(device)
        plan = va.ModalPlan(lp.to(device), r.to(device))
        out = torch.empty(B, D, L, dtype=torch.bfloat16, device=device)
        fn = lambda: ops.li_layer_fwd_rows(q1, q2, qv, taps, plan, Db, B, D, L, device=device, out=out)
        return fn, dict(workload=f"hyena_li_layer in one launch from a sequence-major projection B={B} L={L} D={D} "
                                 f"groups={G} poles={S} complex", tokens=B * L, bytes=8 * B * D * L, kernel="li_kernel",
                        keep=(p, taps, plan, Db, out))
    raise ValueError(name)


def _decode_figures(us, algorithmic_bytes, moved_bytes=None):
    """Figures of one decode kernel or layer set.  A roofline fraction is only formed from bytes the timed launches
    really move: `frac` where they run the reference's algorithm (whole cache, state on every token), otherwise
    `frac_of_bytes_moved` from the average bytes per token of the windowed forms."""
    d = dict(us=us, launch_bound=us < 10.0)
    if moved_bytes is None:
        gbs = algorithmic_bytes / (us * 1e-6) / 1e9
        d.update(bytes=algorithmic_bytes, hbm_gbs=gbs, frac=gbs / HBM_PEAK_GBS)
    else:
        gbs = moved_bytes / (us * 1e-6) / 1e9
        d.update(bytes_moved_per_token=moved_bytes, moved_gbs=gbs, frac_of_bytes_moved=gbs / HBM_PEAK_GBS,
                 reference_algorithm_bytes=algorithmic_bytes)
    return d


def decode_layer_set(D, device, steps, warmup):
    """One [SE, MR, LI] layer set of cached decode at batch 64: three fused launches per token.

    Timed twice: with the kernels that run the reference's algorithm (the whole FIR cache read and the modal state
    read and written on every token; the algorithmic bytes of that algorithm are exactly what these move, so their rate is a
    bandwidth and `frac_reference_algorithm` is the roofline figure), and with the steps the steppers bind by default
    (far sums for the deep cache, the modal state in windows of four tokens), which move fewer bytes per token: for
    those the headline is `us_per_step`, and the fraction is taken of the bytes they move."""
    import vortex_amd as va
    from vortex_amd import ops
    O = _Synthetic
    B, S = 64, 16
    g = torch.Generator(device=device).manual_seed(6)
    rnd = lambda *s: torch.randn(*s, generator=g, device=device, dtype=torch.float32)
    x = [tuple(rnd(B, D).to(torch.bfloat16) for _ in range(3)) for _ in range(3)]
    G = D // 16
    ring_se = va.FirRing(rnd(B, 6, D).to(torch.bfloat16))
    ring_mr = va.FirRing(rnd(B, 127, D).to(torch.bfloat16))
    w_se, w_mr = rnd(G, 7) * 7 ** -0.5, rnd(G, 128) * 128 ** -0.5
    Dmr = rnd(D)
    lp, r = O.make_modal_complex(G, S)
    poles, res = torch.exp(lp[..., 0]).to(device), r.to(device)
    state = torch.zeros(B, D, S, dtype=torch.complex64, device=device)
    Dli = rnd(D).to(torch.bfloat16)
    step = va.DecodeLayerSet(ring_se, w_se, ring_mr, w_mr, Dmr, state, poles, res, Dli)
    # the same set on caches of its own with the reference's algorithm in every kernel
    ref = va.DecodeLayerSet(va.FirRing(rnd(B, 6, D).to(torch.bfloat16)), w_se, va.FirRing(rnd(B, 127, D).to(torch.bfloat16)),
                            w_mr, Dmr, torch.zeros_like(state), poles, res, Dli, window_state=False, far_sums=False)

    wall, ms = time_steps(lambda: step(x[0], x[1], x[2]), steps, warmup)
    _, ms_ref = time_steps(lambda: ref(x[0], x[1], x[2]), steps, warmup)
    # algorithmic bytes: caches read once, one ring slot written per FIR, modal state read+written,
    # 3 gate vectors in and 1 output vector out per operator
    gates_io = 4 * B * D * 2
    b_se, b_mr, b_li = B * D * 2 * 6 + B * D * 2 + gates_io, B * D * 2 * 127 + B * D * 2 + gates_io, \
        2 * state.numel() * 8 + gates_io
    byts = b_se + b_mr + b_li
    # bytes the windowed forms move per token on average
    m_mr, m_li, n_mr, n_li = b_mr, b_li, None, None
    if step.mr.far is not None:
        # far sums: the whole cache every n-th token: per token about (127 / n + (n - 1) / 2) slots, the far buffer
        # (n - 1 float32 rows written per window, one read on n - 1 of n tokens) and the gates
        n_mr = step.mr.far.numel() // (B * D)
        m_mr = B * D * 2 * (127 / n_mr + (n_mr - 1) / 2) + B * D * 4 * 2 * (n_mr - 1) / n_mr + B * D * 2 + gates_io
    if step.li.win is not None:
        # windows of n tokens: 1/n of the state traffic per token, a far row (float32) written on n - 1 tokens of n by
        # the window's first token and read once each, the window's inputs (bf16: one row written per token,
        # (n + n (n - 1) / 2) / n rows read)
        n_li = step.li.period
        m_li = 2 * state.numel() * 8 / n_li + B * D * 4 * 2 * (n_li - 1) / n_li \
            + B * D * 2 * (1 + (n_li + n_li * (n_li - 1) / 2) / n_li) + gates_io
    moved = b_se + m_mr + m_li
    # each step alone, launched back to back: kernels shorter than a launch (about 6 us from Python) read as the
    # launch rate, so `launch_bound` marks figures that are an upper bound of the kernel's own duration
    per = {}
    o = step.out[0]
    for nm, st, xx, alg, mv in (("se_step", step.se, x[0], b_se, None),
                                ("mr_step_whole_cache", ref.mr, x[1], b_mr, None),
                                ("iir_step_state_every_token", ref.li, x[2], b_li, None),
                                ("mr_step_far_sums", step.mr, x[1], b_mr, m_mr if n_mr else None),
                                ("iir_step_windowed_state", step.li, x[2], b_li, m_li if n_li else None)):
        _, kms = time_steps(lambda: st(xx[1], xx[0], xx[2], o), max(steps, 100), warmup)
        per[nm] = _decode_figures(kms * 1e3, alg, mv)
    if n_mr:
        per["mr_step_far_sums"]["window_tokens"] = n_mr
    if n_li:
        per["iir_step_windowed_state"]["window_tokens"] = n_li
    # The same token step (three launches and the counter update) recorded once as a HIP graph and replayed: the ring
    # positions and the window counter then live in device memory (ops.RingClock).  Every cache is full and more
    # than a window of tokens has been stepped by now, which is what a recording needs.
    clock = ops.RingClock([ring_se, ring_mr] + ([step.li] if step.li.win is not None else []))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(x[0], x[1], x[2])
        clock.advance()
    _, gms = time_steps(graph.replay, steps, warmup)
    clock.release()
    ref_gbs = byts / (ms_ref * 1e-3) / 1e9
    return dict(us_per_step=ms * 1e3, wall_us_per_step=wall / steps * 1e6, us_per_step_graph_replay=gms * 1e3,
                what="us_per_step: far-sum Hyena-MR step + modal state in windows (fewer bytes per token than the "
                     "reference's algorithm; not a bandwidth).  reference_algorithm: whole cache and state on every "
                     "token; its bytes are the algorithmic ones, so its frac is the roofline figure",
                bytes_moved_per_token=moved, moved_gbs=moved / (ms * 1e-3) / 1e9,
                frac_of_bytes_moved=moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                reference_algorithm=dict(us_per_step=ms_ref * 1e3, bytes=byts, hbm_gbs=ref_gbs,
                                         frac=ref_gbs / HBM_PEAK_GBS),
                frac_reference_algorithm=ref_gbs / HBM_PEAK_GBS,
                kernels=per)


def decode_layers_from_projection(D, device, steps, warmup):
    """The same layer set stepped from each layer's projection output u [B, 3D] (Evo 2 layout: interleaved
    gates, K=3 featurizer): featurizer step, split, gates and inner step in one launch per layer.  As in
    decode_layer_set, once with the reference's algorithm in the inner steps (the roofline figure) and once with the
    far-sum / windowed steps the steppers bind by default (the time per token)."""
    import vortex_amd as va
    from vortex_amd import ops
    O = _Synthetic
    B, S, C = 64, 16, 3 * D
    g = torch.Generator(device=device).manual_seed(7)
    rnd = lambda *s: torch.randn(*s, generator=g, device=device, dtype=torch.float32)
    G = D // 16
    cmap = ops.gate_channel_map(D, interleave=True)
    lp, r = O.make_modal_complex(G, S)
    w_se, w_mr, b_mr, d_li = rnd(G, 7) * 7 ** -0.5, rnd(G, 128) * 128 ** -0.5, rnd(D), rnd(D).to(torch.bfloat16)
    wf = [rnd(C, 3) * 3 ** -0.5 for _ in range(3)]
    u = [rnd(B, C).to(torch.bfloat16) for _ in range(3)]
    out = [torch.empty(B, D, dtype=torch.bfloat16, device=device) for _ in range(3)]

    def make(shipped):
        state = torch.zeros(B, D, S, dtype=torch.complex64, device=device)
        inner = [ops.FirStepper(va.FirRing(rnd(B, 6, D).to(torch.bfloat16)), w_se),
                 ops.FirStepper(va.FirRing(rnd(B, 127, D).to(torch.bfloat16)), w_mr, bias=b_mr, gated_bias=True,
                                far_sums=None if shipped else False),
                 ops.IirStepper(state, torch.exp(lp[..., 0]).to(device), r.to(device), d_li, windowed=shipped)]
        frings = [va.FirRing(rnd(B, 2, C).to(torch.bfloat16)) for _ in inner]
        layers = [ops.LayerStepper(fr, w, None, cmap, n) for fr, w, n in zip(frings, wf, inner)]

        def fn():
            for l, xx, o in zip(layers, u, out):
                l(xx, o)
        return fn, inner, frings, state

    fn, inner, frings, state = make(True)
    fn_ref, _, _, _ = make(False)
    wall, ms = time_steps(fn, steps, warmup)
    _, ms_ref = time_steps(fn_ref, steps, warmup)
    # inner caches / state as in decode_layer_set; per layer the projection row, two featurizer slots read and
    # one written (3D channels each) and one output row
    byts = B * D * 2 * (6 + 127) + 2 * B * D * 2 + 2 * state.numel() * 8 + 3 * (4 * B * C * 2 + B * D * 2)
    # and replayed as a HIP graph, every ring position and the window counter in device memory
    clock = ops.RingClock(frings + [inner[0].ring, inner[1].ring] + ([inner[2]] if inner[2].win is not None else []))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
        clock.advance()
    _, gms = time_steps(graph.replay, steps, warmup)
    clock.release()
    ref_gbs = byts / (ms_ref * 1e-3) / 1e9
    return dict(us_per_step=ms * 1e3, wall_us_per_step=wall / steps * 1e6, us_per_step_graph_replay=gms * 1e3,
                reference_algorithm=dict(us_per_step=ms_ref * 1e3, bytes=byts, hbm_gbs=ref_gbs, frac=ref_gbs / HBM_PEAK_GBS),
                frac_reference_algorithm=ref_gbs / HBM_PEAK_GBS)


def model_prefill(device, L, iters=2):
    """Evo 2 7B-shaped random-init StripedHyena 2 prefill (32 blocks [SE, MR, LI, attention], hidden 4096,
    MLP 11008, vocab 512): Hyena operators on the HIP kernels, projections / MLP / attention through torch."""
    from vortex_amd.model import StripedHyena2
    m = StripedHyena2(device=device).to_inference(device)
    ids = torch.randint(0, 512, (1, L), device=device, generator=torch.Generator(device=device).manual_seed(8))
    m(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        m(ids)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / iters
    del m
    torch.cuda.empty_cache()
    return {"workload": f"striped_hyena2_7b_shaped_prefill B=1 L={L}", "tokens_per_s": L / dt, "ms": dt * 1e3}


def model_decode(device, L=8192, n=32):
    """Cached generation with the same Evo 2 7B-shaped stack: one prefill over L tokens (untimed), then n single-token
    forwards at batch 1 (Hyena layers: one fused layer-step launch each; attention from its key / value cache)."""
    from vortex_amd.model import StripedHyena2
    m = StripedHyena2(device=device).to_inference(device)
    ids = torch.randint(0, 512, (1, L), device=device, generator=torch.Generator(device=device).manual_seed(8))
    ipd = m.initialize_inference_params(max_seqlen=L + 2 * n + 16)
    x = m(ids, ipd)[:, -1].argmax(-1)[:, None]

    def step(x):
        for p in ipd.values():
            p.seqlen_offset = L if p.seqlen_offset == 0 else p.seqlen_offset + 1
        return m(x, ipd)[:, -1].argmax(-1)[:, None]

    for _ in range(3):
        x = step(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        x = step(x)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / n

    # the same token step recorded once as a HIP graph and replayed (ring and attention positions on the device)
    from vortex_amd.model import RecordedDecodeStep
    with torch.no_grad():
        for p in ipd.values():
            p.seqlen_offset += 1
        rec = RecordedDecodeStep(m, ipd, 1)
        for _ in range(3):
            x = rec(x)[:, -1].argmax(-1)[:, None]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            x = rec(x)[:, -1].argmax(-1)[:, None]
        torch.cuda.synchronize()
        dt_rec = (time.perf_counter() - t0) / n
        rec.release()
    del m, ipd, rec
    torch.cuda.empty_cache()
    return {"workload": f"striped_hyena2_7b_shaped_decode B=1 prompt={L}", "ms_per_token": dt * 1e3,
            "tokens_per_s": 1.0 / dt, "recorded_step_ms_per_token": dt_rec * 1e3,
            "recorded_step_tokens_per_s": 1.0 / dt_rec}


def cpu_baseline(name, budget_s=12.0):
    """The oracle (a PyTorch port of the reference path) timed on the host cores, on a channel slice."""
    from oracle import hyena_oracle as O
    threads = torch.get_num_threads()
    if name == "mr":
        B, D, L, G, K, Ds = 2, 4096, 32768, 256, 128, 1024
        x2, x1, v = O.make_gates(B, Ds, L, seed=2)
        h = O.make_mr_filter(Ds // 16, K)
        Db = torch.randn(Ds)
        f = lambda: O.mr_fir(x2, x1, v, h, Db)
    elif name == "se":
        B, D, L, G, K, Ds = 1, 4096, 8192, 256, 7, 1024
        x2, x1, v = O.make_gates(B, Ds, L, seed=1)
        h = O.make_se_filter(Ds // 16, K)
        f = lambda: O.se_fir(x2, x1, v, h)
    elif name == "li":
        B, D, L, G, K, Ds = 1, 4096, 262144, 256, 0, 32
        x2, x1, v = O.make_gates(B, Ds, L, seed=4)
        lp, r = O.make_modal_complex(Ds // 16, 16)
        Db = torch.randn(Ds).bfloat16()
        f = lambda: O.li_prefill(x2, x1, v, lp, r, Db, want_state=False)
    elif name == "decode":
        # one [SE, MR, LI] layer set at config 4, D = 4096, full shape: the reference's own step functions
        B, D, S = 64, 4096, 16
        g = torch.Generator().manual_seed(6)
        gates3 = [[torch.randn(B, D, generator=g).bfloat16() for _ in range(3)] for _ in range(3)]
        st_se, st_mr = torch.randn(B, D, 6, generator=g), torch.randn(B, D, 127, generator=g)
        w_se, w_mr = torch.randn(D, 1, 7, generator=g), torch.randn(D, 1, 128, generator=g)
        Dm, Dl = torch.randn(D, generator=g), torch.randn(D, generator=g).bfloat16()
        lp, r = O.make_modal_complex(D, S)
        st_li = torch.zeros(B, D, S, dtype=torch.complex64)

        def f():
            (a2, a1, av), (b2, b1, bv), (c2, c1, cv) = gates3
            y0, _ = O.step_fir(a1 * av, st_se, w_se)
            y1, _ = O.step_fir(b1 * bv, st_mr, w_mr, bias=Dm, gated_bias=True, flip_filter=True)
            y2, _ = O.step_iir(c2, c1, cv, Dl, r, lp, st_li)
            return y0 * a2, y1 * b2, y2
        f()
        ts, t_all = [], time.perf_counter()
        while len(ts) < 3 or (time.perf_counter() - t_all < budget_s and len(ts) < 40):
            t0 = time.perf_counter()
            f()
            ts.append(time.perf_counter() - t0)
        t = sorted(ts)[len(ts) // 2]
        return dict(value=t * 1e6, unit="us per layer-set step", cores=threads, kind="port",
                    sample=f"oracle step_fir / step_iir (vortex/model/engine.py:406-467 restated) at the full shape "
                           f"B={B} D={D}, caches of 6 and 127, {S} complex states; median of {len(ts)} steps")
    else:
        return None
    f()
    ts = []
    t_all = time.perf_counter()
    while len(ts) < 3 or (time.perf_counter() - t_all < budget_s and len(ts) < 40):      # about 10 s of CPU work
        t0 = time.perf_counter()
        f()
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[len(ts) // 2]
    return dict(value=B * L / (t * D / Ds), unit="tokens/s", cores=threads, kind="port",
                sample=f"oracle (PyTorch fp32 conv1d/FFT restatement) on {Ds} of {D} channels at full B, L; "
                       f"median of {len(ts)} runs, scaled linearly to {D} channels")


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; the Hyena operator path shards over channels "
              "without communication, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    global SETTLE_S
    SETTLE_S = max(args.settle_ms, 0.0) / 1e3
    from vortex_amd import _lib
    overrides = {}
    for item in args.launch_override:
        k, _, v = item.partition("=")
        overrides[k] = int(v)
        _lib.check(_lib.lib().hyena_set_launch_override(k.encode(), int(v)), "hyena_set_launch_override")

    def run(name, steps, warmup):
        fn, d = build_workload(name, device)
        # cold: the first `steps` launches after `warmup`, with no settle phase (what a short run of this workload
        # after other work sees); then the settled, sustained figure
        _, cold_ms = time_steps(fn, steps, warmup, settle=0.0)
        wall, ms = time_steps(fn, steps, warmup)
        d.pop("keep")
        d.update(wall_s=wall, kernel_ms=ms, tokens_per_s=d["tokens"] * steps / wall,
                 hbm_gbs=d["bytes"] / (ms * 1e-3) / 1e9, cold_kernel_ms=cold_ms,
                 cold_frac=d["bytes"] / (cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
        torch.cuda.empty_cache()
        return d

    copy_gbs = None
    if not args.no_copy_probe:
        # the practical ceiling beside the nominal 8 TB/s: a plain device copy with the kernels' own access shape
        # (16 bytes per lane), 1 GiB read + 1 GiB written per launch
        a = torch.empty(1 << 29, dtype=torch.bfloat16, device=device).normal_()
        b = torch.empty_like(a)
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = a.numel() * 2
        probe = _lib.copy_probe()
        _, cms = time_steps(lambda: _lib.check(probe(a.data_ptr(), b.data_ptr(), nbytes, stream), "copy"), 10, 3)
        copy_gbs = 2 * nbytes / (cms * 1e-3) / 1e9
        del a, b
        torch.cuda.empty_cache()

    main_name = args.workload if args.workload != "decode" else "mr"
    m = run(main_name, args.steps, args.warmup)
    result = {
        "metric": "Hyena-SE/MR/LI prefill tokens/s/GPU at D=4096 + % roofline; decode step us",
        "value": m["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": m["wall_s"] / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 in/out, fp32 accumulate", "data": "synthetic",
        "config": {"workload": m["workload"], "settle_ms": args.settle_ms,
                   **({"launch_overrides": overrides} if overrides else {})},
        "roofline": {"bound": "hbm", "achieved": m["hbm_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": m["hbm_gbs"] / HBM_PEAK_GBS, "copy_probe_gbs": copy_gbs,
                     "copy_probe": "hyena_copy_probe: 1 GiB read + 1 GiB written per launch, 16 bytes per lane, timed "
                                   "in this run; the rate a plain copy reaches beside the nominal peak",
                     "traffic": MEASURED_TRAFFIC.get(main_name),
                     "traffic_source": TRAFFIC_SOURCE if MEASURED_TRAFFIC.get(main_name) else None,
                     "kernel": m["kernel"],
                     "algorithmic_bytes_per_launch": m["bytes"], "kernel_ms": m["kernel_ms"],
                     "cold": {"kernel_ms": m["cold_kernel_ms"], "frac": m["cold_frac"],
                              "what": f"first {args.steps} launches after {args.warmup} warm-up launches, no settle phase"}},
    }
    if not args.no_extras:
        extra = {}
        extra_warmup = args.warmup
        def entry(e):
            return {"workload": e["workload"], "tokens_per_s": e["tokens_per_s"], "kernel_us": e["kernel_ms"] * 1e3,
                    "hbm_gbs": e["hbm_gbs"], "roofline_frac": e["hbm_gbs"] / HBM_PEAK_GBS,
                    "cold_kernel_us": e["cold_kernel_ms"] * 1e3, "cold_roofline_frac": e["cold_frac"]}

        for name in ("se", "se_b8", "mr", "li", "li_g4096"):
            if name == main_name:
                continue
            steps = max(3, min(args.steps, 20 if name.startswith("li") else args.steps))
            extra[name] = entry(run(name, steps, extra_warmup))
        for name in ("mr_cl", "mr_layer", "mr_layer_seq", "se_layer", "li_layer", "li_layer_seq", "li_layer_seq_g4096", "mr_cl_f16",
                     "cl_f32"):
            e = run(name, max(3, min(args.steps, 10 if name.startswith("li_layer") else 20)), extra_warmup)
            extra[name] = entry(e)
            if "flops" in e:    # the float32 form (v_mfma_f32_16x16x4_f32) against the published float32 matrix peak;
                                # the float16 form is bound by memory like the bfloat16 one
                tf = e["flops"] / (e["kernel_ms"] * 1e-3) / 1e12
                extra[name].update(tflops=tf, frac_of_fp32_mfma_peak=tf / 157.3)
        for D in (4096, 8192):
            extra[f"decode_D{D}"] = decode_layer_set(D, device, max(args.steps, 50), max(args.warmup, 5))
        extra["decode_from_projection_D4096"] = decode_layers_from_projection(4096, device, max(args.steps, 50),
                                                                              max(args.warmup, 5))
        if not args.no_model:
            for L in (8192, 131072):
                extra[f"model_L{L}"] = model_prefill(device, L)
            extra["model_decode"] = model_decode(device)
        result["extra"] = extra
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(main_name)
        if "extra" in result:                      # shorter samples of the other workloads' CPU path beside their GPU figures
            for name, key in (("se", "se"), ("li", "li"), ("decode", "decode_D4096")):
                if name != main_name and key in result["extra"]:
                    result["extra"][key]["cpu_baseline"] = cpu_baseline(name, 3.0)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
