"""Seeded sweep over ragged shapes: every prefill kernel against the oracle on sizes that are not
multiples of its tiles (8-sample octets, 512-sample steps, 2048-sample blocks, 128-sample chunks)."""
import random

import pytest
import torch

import vortex_amd as va
from oracle import hyena_oracle as O
from vortex_amd import ops

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def cases(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        B = rng.choice([1, 2, 3])
        L = 8 * rng.randint(1, 700)
        out.append((B, L, rng.randint(0, 10 ** 6)))
    return out


# nt = 1 pins the streaming variants (non-temporal accesses, blocks renumbered so that each XCD takes a contiguous eighth
# of them when 8 divides the grid), which the launchers otherwise pick for tensors beyond the last-level cache only
@pytest.mark.parametrize("nt", [0, 1])
@pytest.mark.parametrize("B,L,seed", cases(1, 12))
def test_se_random(B, L, seed, nt, override):
    override(se_nt=nt)
    rng = random.Random(seed)
    K = rng.randint(2, 8)
    dg = rng.choice([1, 2, 8, 16, 24])
    G = rng.randint(1, 4)
    D = G * dg
    if D % 8:
        D, G = D * 8, G * 8          # strides must stay multiples of 8 elements
    x2, x1, v = O.make_gates(B, D, L, seed=seed)
    h = O.make_se_filter(G, K, seed=seed + 1)
    ref, _ = O.se_fir(x2, x1, v, h)
    out = va.hyena_se_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda())
    assert rel_err(out, ref) <= 2e-2, (B, D, L, G, K)


@pytest.mark.parametrize("nt", [0, 1])
@pytest.mark.parametrize("B,L,seed", cases(2, 10))
def test_mr_random(B, L, seed, nt, override):
    override(mr_nt=nt)
    rng = random.Random(seed)
    K = rng.choice([9, 16, 33, 64, 100, 127, 128])
    G = rng.randint(1, 3)
    D = G * 16 * rng.randint(1, 2)
    x2, x1, v = O.make_gates(B, D, L, seed=seed)
    h = O.make_mr_filter(G, K, seed=seed + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(seed))
    ref, _ = O.mr_fir(x2, x1, v, h, Db)
    out = va.hyena_mr_fwd(x1.cuda(), x2.cuda(), v.cuda(), h.cuda(), Db.cuda())
    assert rel_err(out, ref) <= 2e-2, (B, D, L, G, K)


@pytest.mark.parametrize("coop", ["0", "1"])
@pytest.mark.parametrize("B,L,seed", cases(3, 10))
def test_li_random(B, L, seed, coop, override):
    # coop = "1" forces the cooperative form (four wavefronts per set of channels) wherever groups have four channels
    override(li_coop=int(coop))
    rng = random.Random(seed)
    cplx = rng.random() < 0.5
    S = rng.choice([16, 16, 8, 3])
    dg = rng.choice([1, 2, 4, 8, 16])
    G = rng.randint(1, 3)
    D = G * dg
    if D % 8:
        k = 8 // (D & -D) if (D & -D) < 8 else 1
        D, G = D * k, G * k
    x2, x1, v = O.make_gates(B, D, L, seed=seed)
    # poles from the whole range a checkpoint can hold: log-uniform |p| in [0.05, 0.9999]
    from parity import log_uniform_modal
    lp, r = log_uniform_modal(G, S, cplx, seed + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(seed)).bfloat16()
    x2n, x1n, vn = (torch.randn(B, D, generator=torch.Generator().manual_seed(seed + 2 + i)).bfloat16() for i in range(3))
    cat = lambda t, n: torch.cat([t, n[..., None]], -1)
    full, _, _ = O.li_prefill(cat(x2, x2n), cat(x1, x1n), cat(v, vn), lp, r, Db, want_state=False)
    ref, y32_ref, st_ref = O.li_prefill(x2, x1, v, lp, r, Db)
    out, y32, st = va.hyena_li_fwd(x1.cuda(), x2.cuda(), v.cuda(), lp.cuda(), r.cuda(), Db.cuda(),
                                   want_state=True, want_fp32=True)
    assert rel_err(y32, y32_ref) <= 1e-4, (B, D, L, G, cplx, S)
    assert rel_err(out, ref) <= 2e-2
    sr = torch.view_as_real(st) if cplx else st
    assert torch.isfinite(sr).all()
    assert rel_err(sr, torch.view_as_real(st_ref) if cplx else st_ref) <= 1e-4
    if S & (S - 1) == 0:          # one decode token from the emitted state = position L of a longer prefill
        y = va.iir_step(x1n.cuda(), x2n.cuda(), vn.cuda(), st, torch.exp(lp[..., 0]).cuda(), r.cuda(), Db.cuda())
        assert rel_err(y, full[..., L]) <= 2e-2


@pytest.mark.parametrize("B,L,seed", cases(4, 8))
def test_featurizer_random(B, L, seed):
    rng = random.Random(seed)
    K = rng.randint(2, 5)
    C = 24 * rng.randint(1, 12)
    il = rng.random() < 0.5
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, L, C, generator=g).bfloat16()
    w = torch.randn(C, 1, K, generator=g)
    z = ops.featurizer_fwd(u.cuda(), w.reshape(C, K).cuda(), None, interleave=il)
    ref, _ = O.parallel_fir(u, w, None, fir_length=K, dim_last=True, gate=False)
    if il:
        ref = O.interleave(ref)
    assert rel_err(z, ref) <= 2e-2, (B, L, C, K, il)


def cl_cases(seed, n):
    rng = random.Random(seed)
    return [(rng.choice([1, 2, 3]), rng.randint(1, 3000), rng.randint(0, 10 ** 6)) for _ in range(n)]


@pytest.mark.parametrize("B,L,seed", cl_cases(7, 14) + [(3, 1, 960982)])      # the last: one time row, permuted view
def test_channel_last_fir_random(B, L, seed, override):
    # channel-last kernel: any L (rows are independent), channel counts that leave partial 64-channel blocks,
    # every filter length class, forced segment counts
    rng = random.Random(seed)
    K = rng.choice([1, 2, 7, 16, 17, 18, 33, 64, 97, 98, 99, 127, 128])
    G = rng.randint(1, 5)
    D = G * 16 * rng.randint(1, 3)
    override(cl_nseg=rng.randint(1, 5))
    x2, x1, v = O.make_gates(B, D, L, seed=seed)
    h = O.make_mr_filter(G, K, seed=seed + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(seed))
    gated = rng.random() < 0.5
    u = x1 * v
    w = h.repeat_interleave(D // G, 0)
    conv = O.short_fir_fp32(u, w.flip(-1), K)                       # convolution = correlation with flipped taps
    z = (conv + (u.float() * Db[None, :, None] if gated else 0)).bfloat16()
    ref = x2 * z
    cl = lambda t: t.permute(0, 2, 1).contiguous().cuda()
    out = ops.fir_cl_fwd(cl(x1), cl(x2), cl(v), h.reshape(G, K).cuda(), bias=Db.cuda() if gated else None,
                         bias_mode=ops.HYENA_BIAS_GATED_FP32 if gated else ops.HYENA_BIAS_NONE)
    assert rel_err(out.permute(0, 2, 1), ref) <= 2e-2, (B, D, L, G, K, gated)


@pytest.mark.parametrize("B,L,seed", cl_cases(8, 12))
def test_fused_layer_random(B, L, seed, override):
    rng = random.Random(seed)
    K = rng.choice([2, 4, 7, 17, 18, 64, 128])
    Ks = rng.choice([3, 4])
    G = rng.randint(1, 4)
    H = rng.choice([1, 2])
    D = G * 16 * H
    cs, il = rng.choice([(False, False), (True, False), (False, True)])
    flip, sbias = rng.random() < 0.5, rng.random() < 0.5
    L = max(L, K)
    override(cl_nseg=rng.randint(1, 4))
    g = torch.Generator().manual_seed(seed)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g).bfloat16() if sbias else None
    h = O.make_se_filter(G, K, seed=seed)
    z, _ = O.parallel_fir(u, wf, bf, fir_length=Ks, dim_last=True, gate=False)
    if il:
        z = O.interleave(z)
    x2, x1, v = O.split_gates(z, (D, H, D // H), cs, flip)
    ref = O.se_fir(x2, x1, v, h)[0]
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    y, bx = ops.fir_layer_fwd(u.cuda(), wf.reshape(C, Ks).t().contiguous().cuda(), None if bf is None else bf.cuda(),
                              cmap, h.reshape(G, K).cuda(), taps_reversed=True, flip_x1x2=flip, bx_from=L - (K - 1))
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2, (B, D, L, G, K, Ks, cs, il, flip, sbias)
    if K > 1:
        assert rel_err(bx.permute(0, 2, 1), (x1 * v)[..., L - (K - 1):]) <= 1e-2


@pytest.mark.parametrize("B,L,seed", cl_cases(9, 14))
def test_featurizer_gates_random(B, L, seed, override):
    # the gate-fused featurizer (rows xv = x1*v and x2 for Hyena-LI): any L behind its front padding, channel counts
    # that leave partial 64-channel blocks, both featurizer lengths, every layout with 16-byte pieces, forced numbers
    # of tiles per block; then the modal scan on those rows against the oracle's Hyena-LI on the oracle's gates
    rng = random.Random(seed)
    Ks = rng.choice([3, 4])
    H = rng.choice([1, 2, 3])
    hd = 8 * rng.randint(1, 5)
    D = H * hd
    cs, il = rng.choice([(False, False), (True, False), (False, True)])
    flip, sbias = rng.random() < 0.5, rng.random() < 0.5
    override(cl_nseg=rng.randint(1, 4))
    g = torch.Generator().manual_seed(seed)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g).bfloat16() if sbias else None
    z, _ = O.parallel_fir(u, wf, bf, fir_length=Ks, dim_last=True, gate=False)
    if il:
        z = O.interleave(z)
    x2, x1, v = O.split_gates(z, (D, H, hd), cs, flip)
    pad = (-L) % 8
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=hd if cs else None)
    row_pad = rng.choice([0, 0, 8, 2048])                 # rows of the results further apart than their length
    xv, g2 = ops.featurizer_gates_fwd(u.cuda(), wf.reshape(C, Ks).t().contiguous().cuda(),
                                      None if bf is None else bf.cuda(), cmap, flip_x1x2=flip, front_pad=pad,
                                      row_pad=row_pad)
    assert xv.stride(1) == L + pad + row_pad
    what = (B, D, L, Ks, cs, il, flip, sbias, row_pad)
    assert not xv[..., :pad].any() and not g2[..., :pad].any(), what
    assert rel_err(xv[..., pad:], x1 * v) <= 1e-2 and rel_err(g2[..., pad:], x2) <= 1e-2, what
    lp, r = O.make_modal_real(D, 16, seed=seed)
    Dc = torch.randn(D, generator=g).bfloat16()
    ref, _, _ = O.li_prefill(x2, x1, v, lp, r, Dc, want_state=False)
    plan = ops.ModalPlan(lp.cuda(), r.cuda())
    y, _, _ = ops.li_fwd_rows(ops.rows_of(xv), ops.rows_of(g2), None, plan, Dc.cuda(), B, D, L + pad, device="cuda")
    assert rel_err(y[..., pad:], ref) <= 2e-2, what


@pytest.mark.parametrize("L", [1, 5, 63, 1001, 2049])
def test_lengths_that_are_not_multiples_of_8(L):
    # the tensor-level operators accept any length: they run behind -L % 8 zero samples (ops.front_pad8)
    B, D, G = 2, 32, 2
    x2, x1, v = O.make_gates(B, D, L, seed=L)
    d = lambda t: t.cuda()
    h = O.make_se_filter(G, 7, seed=L)
    assert rel_err(va.hyena_se_fwd(d(x1), d(x2), d(v), d(h)), O.se_fir(x2, x1, v, h)[0]) <= 2e-2
    hm = O.make_mr_filter(G, 128, seed=L)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(L))
    assert rel_err(va.hyena_mr_fwd(d(x1), d(x2), d(v), d(hm), d(Db)), O.mr_fir(x2, x1, v, hm, Db)[0]) <= 2e-2
    lp, r = O.make_modal_complex(G, 16, seed=L, pmax=0.999)
    Dl = torch.randn(D, generator=torch.Generator().manual_seed(L + 1)).bfloat16()
    ref, y32_ref, st_ref = O.li_prefill(x2, x1, v, lp, r, Dl)
    out, y32, st = va.hyena_li_fwd(d(x1), d(x2), d(v), d(lp), d(r), d(Dl), want_state=True, want_fp32=True)
    assert out.shape == (B, D, L) and y32.shape == (B, D, L)
    assert rel_err(out, ref) <= 2e-2 and rel_err(y32, y32_ref) <= 1e-4
    assert rel_err(torch.view_as_real(st), torch.view_as_real(st_ref)) <= 1e-4


@pytest.mark.parametrize("L,bias", [(13, False), (250, True), (1021, False)])
def test_featurizer_front_pad(L, bias):
    B, C, K = 2, 96, 3
    g = torch.Generator().manual_seed(L)
    u = torch.randn(B, L, C, generator=g).bfloat16()
    w = torch.randn(C, 1, K, generator=g) / K ** 0.5
    b = torch.randn(C, generator=g).bfloat16() if bias else None
    pad = (-L) % 8
    z = ops.featurizer_fwd(u.cuda(), w.reshape(C, K).cuda(), None if b is None else b.cuda(), interleave=True,
                           front_pad=pad)
    ref, _ = O.parallel_fir(u, w, b, fir_length=K, dim_last=True, gate=False)
    assert z.shape == (B, C, L + pad) and not z[..., :pad].any()
    assert rel_err(z[..., pad:], O.interleave(ref)) <= 2e-2


def test_kernels_follow_the_current_stream():
    # every entry point enqueues on the stream it is given (the wrappers pass torch's current stream): work issued
    # on a side stream is ordered after that stream's earlier work and gives the default-stream result bit for bit
    import vortex_amd as va
    B, D, L, G = 2, 64, 4096, 4
    g = torch.Generator().manual_seed(12)
    x1, x2, v = (torch.randn(B, D, L, generator=g).bfloat16().cuda() for _ in range(3))
    h7, h128 = torch.randn(G, 1, 7, generator=g).cuda(), (torch.randn(G, 1, 128, generator=g) / 11).cuda()
    Db = torch.randn(D, generator=g).bfloat16().cuda()
    lp = (-(0.01 + torch.rand(G, 16, 1, generator=g))).cuda()
    r = torch.randn(G, 16, generator=g).cuda()

    def run():
        se = va.hyena_se_fwd(x1, x2, v, h7)
        mr = va.hyena_mr_fwd(x1, x2, v, h128, Db)
        li, _, st = va.hyena_li_fwd(x1, x2, v, lp, r, Db, want_state=True)
        cl = va.ops.fir_cl_fwd(x1.transpose(1, 2).contiguous(), x2.transpose(1, 2).contiguous(),
                               v.transpose(1, 2).contiguous(), h128.reshape(G, 128), bias=Db,
                               bias_mode=va.ops.HYENA_BIAS_GATED_FP32)
        y = va.iir_step(x1[..., 0].contiguous(), x2[..., 0].contiguous(), v[..., 0].contiguous(), st,
                        torch.exp(lp[..., 0]), r, Db)
        return se, mr, li, cl, y, st

    want = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        big = torch.randn(64, 1 << 20, device="cuda")
        for _ in range(20):                      # keep the side stream busy ahead of the kernels under test
            big = big * 1.0001
        got = run()
    side.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_offsets_beyond_32_bits():
    # tensors of more than 2^32 elements (B=2, D=4096, L=2^19+4096: 8.1 GiB each): the rows at the far end are only
    # right if every element offset is computed in 64 bits.  Sampled rows against the oracle.
    import vortex_amd as va
    from oracle import hyena_oracle as O
    B, D, L, G = 2, 4096, (1 << 19) + 4096, 256
    assert B * D * L > 1 << 32
    gen = torch.Generator(device="cuda").manual_seed(21)
    x1, x2, v = (torch.randn(B, D, L, generator=gen, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    h7, h128 = O.make_se_filter(G, 7, seed=1), O.make_mr_filter(G, 128, seed=2)
    lp, r = O.make_modal_real(G, 16, seed=3)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(4)).bfloat16()
    groups = (0, 131, 255)

    def check(out, ref_fn, b=1):
        for g in groups:
            rows = slice(16 * g, 16 * g + 16)
            a1, a2, av = x1[b:b + 1, rows].cpu(), x2[b:b + 1, rows].cpu(), v[b:b + 1, rows].cpu()
            ref = ref_fn(a2, a1, av, g, rows)
            err = (out[b:b + 1, rows].float().cpu() - ref.float()).abs().max() / ref.float().abs().max()
            assert err <= 2e-2, (g, err.item())

    out = va.hyena_se_fwd(x1, x2, v, h7.cuda())
    check(out, lambda a2, a1, av, g, rows: O.se_fir(a2, a1, av, h7[g:g + 1])[0])
    out = va.hyena_mr_fwd(x1, x2, v, h128.cuda(), Db.cuda())
    check(out, lambda a2, a1, av, g, rows: O.mr_fir(a2, a1, av, h128[g:g + 1], Db[rows])[0])
    out, _, st = va.hyena_li_fwd(x1, x2, v, lp.cuda(), r.cuda(), Db.cuda(), want_state=True)
    check(out, lambda a2, a1, av, g, rows: O.li_prefill(a2, a1, av, lp[g:g + 1], r[g:g + 1], Db[rows])[0])
    del out
    # channel-last: the same samples as [B, L, D]; the last batch element's rows lie past 2^32 elements
    c1, c2, cv = (t.transpose(1, 2).contiguous() for t in (x1, x2, v))
    del x1, x2, v
    out = va.ops.fir_cl_fwd(c1, c2, cv, h128.reshape(G, 128).cuda(), bias=Db.cuda(), bias_mode=va.ops.HYENA_BIAS_GATED_FP32)
    for g in groups:
        rows = slice(16 * g, 16 * g + 16)
        a1, a2, av = (t[1:2, :, rows].transpose(1, 2).contiguous().cpu() for t in (c1, c2, cv))
        ref = O.mr_fir(a2, a1, av, h128[g:g + 1], Db[rows])[0]
        err = (out[1:2, :, rows].transpose(1, 2).float().cpu() - ref.float()).abs().max() / ref.float().abs().max()
        assert err <= 2e-2, (g, err.item())


@pytest.mark.parametrize("B,L,seed", cases(7, 14))
def test_rows_layers_random(B, L, seed, override):
    """The one-launch layers from a sequence-major projection (hyena_fir_layer_fwd_rows, hyena_li_layer_fwd) on ragged
    shapes, random channel maps, group sizes and segmentations: bit for bit the featurizer kernel followed by the
    operator kernel on its gates, and against the oracle's layer (OracleCascade) within the bf16 tolerance."""
    from vortex_amd._lib import HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE
    rng = random.Random(seed)
    kind = rng.choice(["se", "mr", "mr_short", "li", "li"])
    H = rng.choice([1, 2, 4])
    dg = rng.choice([4, 8, 16, 24, 1]) if kind == "li" else rng.choice([8, 16, 15, 32])
    G = H * rng.randint(1, 2)
    D = G * dg
    if D % 8 or D % H:
        D, G = D * 8, G * 8
    mode = rng.choice(["plain", "interleave", "head"])
    il, hd = mode == "interleave", (D // H if mode == "head" else None)
    override(mr_nseg=rng.randint(1, 3), mr_nt=rng.randint(0, 1), se_nt=rng.randint(0, 1), li_nt=rng.randint(0, 1))
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, L, 3 * D, generator=g).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g) / 3 ** 0.5).to(torch.bfloat16).float()
    ud, wd = u.cuda(), w.cuda()
    z = ops.featurizer_fwd(ud, wd, None, interleave=il)
    r2, r1, rv = (ops.rows_of_projection(z, D, i, hd) for i in range(3))
    p = ud.transpose(1, 2).contiguous()
    (q2, q1, qv), chan = ops.projection_rows(p, D, interleave=il, head_dim=hd)
    ft = torch.stack([wd[chan[1]], wd[chan[0]], wd[chan[2]]]).contiguous()
    params = {"short_filter_weight": w.reshape(3 * D, 1, 3), "short_filter_bias": None}
    if kind == "li":
        lp, rs = O.make_modal_real(G, 16, seed=seed + 1, pmax=0.999)
        Dc = torch.randn(D, generator=g).to(torch.bfloat16)
        plan = ops.ModalPlan(lp.cuda(), rs.cuda())
        # lone wavefronts and the same channels per wavefront on both sides: the scan's additions then come in the same order
        override(li_coop=0, li_cpw=rng.choice([1, 4]) if dg % 4 == 0 else 1)
        y0, _, s0 = ops.li_fwd_rows(r1, r2, rv, plan, Dc.cuda(), B, D, L, device="cuda", want_state=True)
        y1, s1 = ops.li_layer_fwd_rows(q1, q2, qv, ft, plan, Dc.cuda(), B, D, L, device="cuda", want_state=True)
        assert torch.equal(s0, s1), (B, L, D, G, mode)
        params.update(D=Dc, log_poles=lp.repeat_interleave(dg, 0), residues=rs.repeat_interleave(dg, 0))
        ref = O.OracleCascade(O.OracleEngine(), params, D, H, D, column_split_hyena=hd is not None, interleave=il)
    else:
        K = {"se": rng.randint(2, 8), "mr": 128, "mr_short": rng.choice([9, 33, 100])}[kind]
        mr = K >= 128
        h = (torch.randn(G, K, generator=g) / K ** 0.5).to(torch.bfloat16).float()
        Dc = torch.randn(D, generator=g).to(torch.bfloat16) if mr else None
        kw = dict(device="cuda", bias=Dc.float().cuda() if mr else None,
                  bias_mode=HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE, taps_reversed=not mr)
        y0 = ops.fir_fwd_rows(r1, r2, rv, h.cuda(), B, D, L, K, force_mfma=K > 8, **kw)
        y1 = ops.fir_layer_fwd_rows(q1, q2, qv, ft, h.cuda(), B, D, L, K, **kw)
        params.update(D=Dc, h=h.reshape(G, 1, K))
        ref = O.OracleCascade(O.OracleEngine(), params, D, H, G, fir_inner_filter_length=K,
                              column_split_hyena=hd is not None, interleave=il)
    assert torch.equal(y0, y1), (kind, B, L, D, G, mode)
    y_ref, _ = ref.forward(u)
    assert rel_err(y1.permute(0, 2, 1), y_ref) <= 2e-2, (kind, B, L, D, G, mode)
