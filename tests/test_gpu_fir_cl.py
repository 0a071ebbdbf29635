"""GPU parity of the channel-last FIR kernel (hyena_fir_cl_fwd) and the one-launch prefill layer
(hyena_fir_layer_fwd) against the CPU oracle, through the C ABI."""
import os

import pytest
import torch

from vortex_amd import ops
from vortex_amd._lib import HYENA_BIAS_ADD, HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE
from oracle import hyena_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def cl(t):
    """[B, D, L] -> channel-last [B, L, D] contiguous on the GPU."""
    return t.permute(0, 2, 1).contiguous().to(DEV)


@pytest.fixture
def segments(request):
    """Forces a number of segments along L so that short sequences exercise the halo rebuild."""
    from vortex_amd._lib import launch_override
    with launch_override(cl_nseg=request.param):
        yield request.param


@pytest.mark.parametrize("segments", [1, 3], indirect=True)
@pytest.mark.parametrize("B,D,G,L,K", [
    (2, 64, 4, 512, 7), (1, 80, 5, 1000, 7), (2, 128, 8, 131, 4), (1, 64, 2, 8, 7), (1, 192, 12, 777, 2),
])
def test_cl_short_filter_vs_oracle(B, D, G, L, K, segments):
    x2, x1, v = O.make_gates(B, D, L, seed=L + K)
    h = O.make_se_filter(G, K, seed=K)
    ref = O.se_fir(x2, x1, v, h)
    ref = ref[0] if isinstance(ref, tuple) else ref
    y = ops.fir_cl_fwd(cl(x1), cl(x2), cl(v), h.reshape(G, K).to(DEV), taps_reversed=True)
    assert y.shape == (B, L, D)
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2


@pytest.mark.parametrize("segments", [1, 2], indirect=True)
@pytest.mark.parametrize("B,D,G,L,K", [(2, 64, 4, 640, 128), (1, 96, 6, 1333, 128), (1, 64, 1, 300, 100),
                                       (1, 32, 2, 64, 128)])
def test_cl_medium_filter_gated_bias_vs_oracle(B, D, G, L, K, segments):
    x2, x1, v = O.make_gates(B, D, L, seed=L)
    h = O.make_mr_filter(G, K, seed=K)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(5))
    ref, _ = O.mr_fir(x2, x1, v, h, Db)
    y = ops.fir_cl_fwd(cl(x1), cl(x2), cl(v), h.reshape(G, K).to(DEV), bias=Db.to(DEV),
                       bias_mode=HYENA_BIAS_GATED_FP32)
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2


def test_cl_strided_views_and_intermediates():
    # gates as slices of one [B, L, 3D] projection (time stride 3D); y2 and bx as two_pass_fwd_grouped returns them
    B, D, G, L, K = 2, 128, 8, 515, 33
    g = torch.Generator().manual_seed(9)
    u = torch.randn(B, L, 3 * D, generator=g).bfloat16()
    h = torch.randn(G, 1, K, generator=g) / K ** 0.5
    ud = u.to(DEV)
    x2, x1, v = (ud[..., i * D:(i + 1) * D] for i in range(3))
    out, y2, bx = ops.fir_cl_fwd(x1, x2, v, h.reshape(G, K).to(DEV), want_y2=True, want_bx=True, bx_from=L - (K - 1))
    x2c, x1c, vc = (u[..., i * D:(i + 1) * D].permute(0, 2, 1) for i in range(3))
    bx_ref = x1c * vc
    w = h.repeat_interleave(D // G, 0)
    z_ref = O.short_fir_fp32(bx_ref, w.flip(-1), K).bfloat16()          # convolution = correlation with flipped taps
    assert rel_err(y2.permute(0, 2, 1), z_ref) <= 2e-2
    assert rel_err(out.permute(0, 2, 1), x2c * z_ref) <= 2e-2
    assert torch.equal(bx.cpu(), bx_ref[..., L - (K - 1):].permute(0, 2, 1))


@pytest.mark.parametrize("bias_mode", [HYENA_BIAS_NONE, HYENA_BIAS_ADD, HYENA_BIAS_GATED_FP32])
def test_cl_ungated_fir_bias_rules(bias_mode):
    B, D, G, L, K = 1, 64, 64 // 16, 400, 5
    g = torch.Generator().manual_seed(4)
    x = torch.randn(B, D, L, generator=g).bfloat16()
    h = torch.randn(G, 1, K, generator=g) / K ** 0.5
    bias = torch.randn(D, generator=g)
    w = h.repeat_interleave(D // G, 0)
    conv = O.short_fir_fp32(x, w, K)
    if bias_mode == HYENA_BIAS_NONE:
        ref = conv.bfloat16()
    elif bias_mode == HYENA_BIAS_ADD:
        ref = (conv.bfloat16() + bias.bfloat16()[None, :, None])
    else:
        ref = (conv + bias[None, :, None] * x.float()).bfloat16()
    y = ops.fir_cl_fwd(cl(x), None, None, h.reshape(G, K).to(DEV), bias=bias.to(DEV) if bias_mode else None,
                       bias_mode=bias_mode, taps_reversed=True)
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2


def oracle_layer(u, wf, bf, h, Dcoef, D, H, cs, il, flip):
    """Featurizer -> interleave -> split -> inner FIR of vortex/model/model.py:221-291 on u [B, L, 3D]."""
    Ks, K = wf.shape[-1], h.shape[-1]
    z, _ = O.parallel_fir(u, wf, bf, fir_length=Ks, dim_last=True, gate=False)
    if il:
        z = O.interleave(z)
    x2, x1, v = O.split_gates(z, (D, H, D // H, 16, h.shape[0]), cs, flip)
    if K >= 128:
        y, tail = O.mr_fir(x2, x1, v, h, Dcoef)
    else:
        y = O.se_fir(x2, x1, v, h)
        y = y[0] if isinstance(y, tuple) else y
        tail = (x1 * v)[..., -(K - 1):]
    return y, tail


@pytest.mark.parametrize("segments", [1, 2], indirect=True)
@pytest.mark.parametrize("B,L,D,H,G,K,Ks,cs,il,flip,sbias", [
    (2, 512, 64, 4, 4, 7, 3, False, True, False, False),       # Evo 2 layout, Hyena-SE
    (1, 700, 128, 4, 8, 128, 3, False, True, False, False),    # Evo 2 layout, Hyena-MR
    (1, 384, 64, 4, 4, 7, 3, True, False, False, True),        # head-blocked split (head_dim 16), featurizer bias
    (2, 300, 96, 2, 6, 128, 3, False, False, True, False),     # plain split, flipped gates, D % 64 != 0
    (1, 520, 64, 2, 4, 7, 4, False, True, False, True),        # 4-tap featurizer
    (1, 260, 64, 2, 4, 128, 4, True, False, True, False),
])
def test_layer_fwd_vs_oracle(B, L, D, H, G, K, Ks, cs, il, flip, sbias, segments):
    g = torch.Generator().manual_seed(L + K + Ks)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g).bfloat16() if sbias else None
    mr = K >= 128
    h = O.make_mr_filter(G, K, seed=3) if mr else O.make_se_filter(G, K, seed=3)
    Dcoef = torch.randn(D, generator=g) if mr else None
    ref, tail = oracle_layer(u, wf, bf, h, Dcoef, D, H, cs, il, flip)
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    y, bx = ops.fir_layer_fwd(u.to(DEV), wf.reshape(C, Ks).t().contiguous().to(DEV), None if bf is None else bf.to(DEV),
                              cmap, h.reshape(G, K).to(DEV), bias=None if Dcoef is None else Dcoef.to(DEV),
                              bias_mode=HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE, taps_reversed=not mr,
                              flip_x1x2=flip, bx_from=L - (K - 1))
    assert y.shape == (B, L, D)
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2
    assert rel_err(bx.permute(0, 2, 1), tail) <= 1e-2


@pytest.mark.parametrize("nseg", [1, 3])
@pytest.mark.parametrize("B,D,G,L,K", [(2, 384, 24, 640, 128), (1, 448, 28, 1333, 128), (1, 400, 25, 700, 7),
                                       (2, 1024, 64, 300, 17), (1, 384, 6, 2100, 100)])
def test_cl_several_strips_per_block(B, D, G, L, K, nseg, override):
    # blocks of three 64-channel strips that share their barriers (what large tensors run): against the oracle and
    # bit for bit against the one-strip form, with widths that leave the last block one or two empty strips
    # (448 = 7 strips, 400 = 6.25) and segments along L
    from vortex_amd._lib import HYENA_BIAS_NONE as NONE
    x2, x1, v = O.make_gates(B, D, L, seed=L + K)
    mr = K >= 100
    h = O.make_mr_filter(G, K, seed=K) if mr else O.make_se_filter(G, K, seed=K)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(5)) if mr else None
    ref = (O.mr_fir(x2, x1, v, h, Db) if mr else O.se_fir(x2, x1, v, h))[0]
    res = []
    for ns in (3, 1):
        override(cl_ns=ns, cl_nseg=nseg)
        res.append(ops.fir_cl_fwd(cl(x1), cl(x2), cl(v), h.reshape(G, K).to(DEV), bias=None if Db is None else Db.to(DEV),
                                  bias_mode=HYENA_BIAS_GATED_FP32 if mr else NONE, taps_reversed=not mr))
    assert rel_err(res[0].permute(0, 2, 1), ref) <= 2e-2
    assert torch.equal(res[0], res[1])


@pytest.mark.parametrize("nseg", [1, 2])
@pytest.mark.parametrize("B,L,D,H,G,K,Ks,cs,il,flip,sbias", [
    (2, 512, 256, 4, 16, 7, 3, False, True, False, False),
    (1, 700, 320, 4, 20, 128, 3, False, True, False, True),      # five strips: the last block has an empty one
    (1, 384, 256, 4, 16, 128, 4, True, False, True, False),      # head-blocked split (head_dim 64), 4-tap featurizer
])
def test_layer_fwd_several_strips_per_block(B, L, D, H, G, K, Ks, cs, il, flip, sbias, nseg, override):
    g = torch.Generator().manual_seed(L + K + Ks)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g).bfloat16() if sbias else None
    mr = K >= 128
    h = O.make_mr_filter(G, K, seed=3) if mr else O.make_se_filter(G, K, seed=3)
    Dcoef = torch.randn(D, generator=g) if mr else None
    ref, _ = oracle_layer(u, wf, bf, h, Dcoef, D, H, cs, il, flip)
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    res = []
    for ns in (2, 1):
        override(cl_ns=ns, cl_nseg=nseg)
        res.append(ops.fir_layer_fwd(u.to(DEV), wf.reshape(C, Ks).t().contiguous().to(DEV), None if bf is None else bf.to(DEV),
                                     cmap, h.reshape(G, K).to(DEV), bias=None if Dcoef is None else Dcoef.to(DEV),
                                     bias_mode=HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE, taps_reversed=not mr,
                                     flip_x1x2=flip))
    assert rel_err(res[0].permute(0, 2, 1), ref) <= 2e-2
    assert torch.equal(res[0], res[1])


def test_cl_rejects_unsupported():
    x = torch.zeros(1, 16, 24, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):       # 24 channels in 3 groups: group size 8 is not a multiple of 16
        ops.fir_cl_fwd(x, x, x, torch.zeros(3, 4, device=DEV))


def test_cl_filter_longer_than_128_taps_runs_the_direct_form():
    # no MFMA kernel beyond 128 taps: the direct-form kernel in blocks of 128 lags, ungated, against a float32 conv1d
    B, D, L, G, K = 2, 32, 700, 2, 200
    g = torch.Generator().manual_seed(K)
    x = torch.randn(B, D, L, generator=g).bfloat16()
    w = torch.randn(G, K, generator=g) / K ** 0.5                      # w[:, 0] on the current sample
    ref = O.short_fir_fp32(x, w.flip(-1).repeat_interleave(D // G, 0)[:, None], K).bfloat16()
    y = ops.fir_cl_fwd(cl(x), None, None, w.to(DEV))
    assert rel_err(y.permute(0, 2, 1), ref) <= 2e-2


@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("B,L,D,G,K,rev", [(2, 1024, 64, 4, 128, True), (1, 333, 48, 3, 7, True), (3, 130, 128, 1, 32, False),
                                           (1, 2000, 80, 5, 100, True), (2, 520, 96, 2, 60, False), (1, 256, 32, 2, 40, True),
                                           (1, 8, 16, 1, 20, True), (2, 129, 144, 3, 1, True), (1, 700, 4096, 4, 128, True),
                                           (2, 2048 + 40, 64, 2, 128, False)])
def test_cl_float32_matrix_core_form(B, L, D, G, K, rev, gated, override):
    """float32 tensors with 16-channel filter groups run on v_mfma_f32_16x16x4_f32 (hyena_fir_cl_fwd_dtype): against
    a float64 convolution to float32 rounding (1e-5 of the largest output), against the direct form on the vector
    ALUs (the same sums in another order), with the y2 / Bx outputs, for every set of skipped row groups
    (K = 128, 100 | 60 | 40 | 32, 20, 7, 1), ragged lengths and channel counts that leave wavefronts idle."""
    g = torch.Generator().manual_seed(L + K)
    x2, x1, v = (torch.randn(B, L, D, generator=g) for _ in range(3))
    h = torch.randn(G, K, generator=g)
    kw = dict(taps_reversed=rev, want_y2=True, want_bx=True, bx_from=max(L - 9, 0))
    a1, a2, av = (x1.to(DEV), x2.to(DEV), v.to(DEV)) if gated else (x1.to(DEV), None, None)
    res = {}
    for form in (2, 1, 0):          # blocks that walk a ring of tiles, one tile per block, the direct form
        override(cl_f32_mfma=form)
        res[form] = ops.fir_cl_fwd(a1, a2, av, h.to(DEV), **kw)
    u = (x1 * v if gated else x1).double().permute(0, 2, 1)
    taps = (h if rev else h.flip(-1)).double().repeat_interleave(D // G, 0)[:, None]       # [D, 1, K], last tap on the current sample
    z = torch.nn.functional.conv1d(torch.nn.functional.pad(u, (K - 1, 0)), taps, groups=D).permute(0, 2, 1)
    y = z * x2.double() if gated else z
    for i in range(3):
        assert torch.equal(res[2][i], res[1][i])          # the two matrix-core forms: the same sums in the same order
    for form in (1, 0):
        out, y2, bx = (t.cpu().double() for t in res[form])
        scale = y.abs().max()
        assert ((out - y).abs().max() / scale).item() <= 1e-5, form
        assert ((y2 - z).abs().max() / z.abs().max()).item() <= 1e-5, form
        assert torch.equal(bx.float(), u.permute(0, 2, 1)[:, max(L - 9, 0):].float()), form
    assert torch.equal(res[0][2], res[1][2])
    assert ((res[0][0] - res[1][0]).abs().max() / y.abs().max().to(DEV)).item() <= 2e-6


def test_cl_float32_falls_back_to_the_direct_form():
    # groups of 12 channels, an inner bias, or more than 128 taps: no matrix-core form, same entry point, same answers
    from vortex_amd._lib import HYENA_BIAS_GATED_FP32
    g = torch.Generator().manual_seed(2)
    for (D, G, K, bias) in ((48, 4, 16, False), (64, 4, 16, True), (64, 4, 150, False)):
        B, L = 2, 300
        x2, x1, v = (torch.randn(B, L, D, generator=g) for _ in range(3))
        h = torch.randn(G, K, generator=g)
        Db = torch.randn(D, generator=g) if bias else None
        out = ops.fir_cl_fwd(x1.to(DEV), x2.to(DEV), v.to(DEV), h.to(DEV), taps_reversed=True,
                             bias=Db.to(DEV) if bias else None, bias_mode=HYENA_BIAS_GATED_FP32 if bias else 0)
        u = (x1 * v).double().permute(0, 2, 1)
        z = torch.nn.functional.conv1d(torch.nn.functional.pad(u, (K - 1, 0)),
                                       h.double().repeat_interleave(D // G, 0)[:, None], groups=D)
        if bias:
            z = z + Db.double()[None, :, None] * u
        y = z.permute(0, 2, 1) * x2.double()
        assert ((out.cpu().double() - y).abs().max() / y.abs().max()).item() <= 1e-5


def test_cl_impulse_response_across_steps_and_segments():
    # bf16-exact taps, unit gates: the output is the filter itself wherever an impulse sits, bit for bit
    B, D, L, G, K = 1, 64, 4096, 4, 128
    h = O.make_mr_filter(G, K).bfloat16().float()
    x1 = torch.zeros(B, L, D, dtype=torch.bfloat16)
    pos = [0, 127, 300, 1023, 2047, 2050, L - 5]          # step boundaries (128) and segment boundaries (1024)
    for p in pos:
        x1[:, p] = 1
    one = torch.ones(B, L, D, dtype=torch.bfloat16)
    from vortex_amd._lib import launch_override
    with launch_override(cl_nseg=4):
        out = ops.fir_cl_fwd(x1.to(DEV), one.to(DEV), one.to(DEV), h.reshape(G, K).to(DEV)).cpu().float()
    hw = h.repeat_interleave(D // G, 0)[:, 0]            # [D, K]
    exp = torch.zeros(B, L, D)
    for p in pos:
        n = min(K, L - p)
        exp[0, p:p + n] += hw[:, :n].t()
    assert torch.equal(out, exp.bfloat16().float())


def test_layer_full_size_config2():
    # Hyena-MR layer at config 2's shape (B=2, L=32768, D=4096, 256 groups, K=128) from an interleaved projection:
    # the one-launch kernel against the featurizer + sequence-major MR kernels, and sampled channels against the oracle
    B, L, D, G, K, Ks = 2, 32768, 4096, 256, 128, 3
    C = 3 * D
    g = torch.Generator(device=DEV).manual_seed(12)
    u = torch.randn(B, L, C, generator=g, device=DEV, dtype=torch.float32).bfloat16()
    wf = (torch.randn(C, Ks, generator=g, device=DEV) / Ks ** 0.5)
    h = O.make_mr_filter(G, K)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(13))
    cmap = ops.gate_channel_map(D, interleave=True)
    y, bx = ops.fir_layer_fwd(u, wf.t().contiguous(), None, cmap, h.reshape(G, K).to(DEV), bias=Db.to(DEV),
                              bias_mode=HYENA_BIAS_GATED_FP32, bx_from=L - (K - 1))
    z = ops.featurizer_fwd(u, wf, None, interleave=True)
    r2, r1, rv = (ops.rows_of_projection(z, D, i) for i in range(3))
    y2 = ops.fir_fwd_rows(r1, r2, rv, h.reshape(G, K).to(DEV), B, D, L, K, device=u.device, bias=Db.to(DEV),
                          bias_mode=HYENA_BIAS_GATED_FP32, force_mfma=True)
    assert rel_err(y, y2.permute(0, 2, 1)) <= 2e-2
    x1v_tail = (z[:, D:2 * D, L - (K - 1):] * z[:, 2 * D:, L - (K - 1):]).permute(0, 2, 1)
    assert rel_err(bx, x1v_tail) <= 1e-2
    del z, y2
    ds = torch.arange(5, D, 409)                                   # sampled operator channels
    ch = (3 * ds[:, None] + torch.arange(3)[None]).reshape(-1)      # their interleaved projection channels
    us = u[:, :, ch.to(DEV)].cpu()
    n = len(ds)
    ref, _ = oracle_layer(us, wf.cpu()[ch][:, None, :], None, h.repeat_interleave(D // G, 0)[ds], Db[ds], n, 1, False,
                          True, False)
    assert rel_err(y[:, :, ds.to(DEV)].permute(0, 2, 1), ref) <= 2e-2


def test_layer_projection_beyond_32_bit_offsets():
    # a projection of more than 2^32 elements (L = 360448 rows of 3 x 4096 channels, 8.9 GB): the last rows are
    # only right with 64-bit element offsets.  The one-launch layer and the featurizer kernel against the oracle on
    # sampled channels, compared over the last 4096 samples (the filters reach back 130 samples at most).
    B, L, D, G, K, Ks = 1, 360448, 4096, 256, 128, 3
    C = 3 * D
    assert L * C > 1 << 32
    g = torch.Generator(device=DEV).manual_seed(14)
    u = torch.randn(B, L, C, generator=g, device=DEV, dtype=torch.bfloat16)
    wf = (torch.randn(C, Ks, generator=g, device=DEV) / Ks ** 0.5)
    h = O.make_mr_filter(G, K)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(13))
    cmap = ops.gate_channel_map(D, interleave=True)
    y = ops.fir_layer_fwd(u, wf.t().contiguous(), None, cmap, h.reshape(G, K).to(DEV), bias=Db.to(DEV),
                          bias_mode=HYENA_BIAS_GATED_FP32)
    ds = torch.tensor([0, 1777, 4095])
    ch = (3 * ds[:, None] + torch.arange(3)[None]).reshape(-1)
    T = 4096 + 256
    us = u[:, L - T:, ch.to(DEV)].cpu()
    ref, _ = oracle_layer(us, wf.cpu()[ch][:, None, :], None, h.repeat_interleave(D // G, 0)[ds], Db[ds], len(ds), 1,
                          False, True, False)
    assert rel_err(y[:, L - 4096:, ds.to(DEV)].permute(0, 2, 1), ref[..., 256:]) <= 2e-2
    del y
    z = ops.featurizer_fwd(u, wf, None, interleave=True)           # [B, 3D, L]: rows of the three gates
    zs = torch.stack([z[0, i * D + d, L - 4096:] for d in ds.tolist() for i in range(3)]).cpu()
    zr, _ = O.parallel_fir(us, wf.cpu()[ch][:, None, :], None, fir_length=Ks, dim_last=True, gate=False)
    assert rel_err(zs, zr[0][:, 256:]) <= 1e-2
    # and the gate-fused featurizer at the far end of the same projection: bit for bit what the three gate rows give
    xv, g2 = ops.featurizer_gates_fwd(u, wf.t().contiguous(), None, cmap)
    for d in ds.tolist():
        assert torch.equal(xv[0, d, L - 4096:], z[0, D + d, L - 4096:] * z[0, 2 * D + d, L - 4096:])
        assert torch.equal(g2[0, d, L - 4096:], z[0, d, L - 4096:])


@pytest.mark.parametrize("K", [7, 128])
def test_cl_nontemporal_variants_match(K, override):
    # tensors larger than the last-level cache use non-temporal accesses (another instantiation of the kernel):
    # forced on at a small size, it must give the same bits, for the gated form and the fused layer
    B, L, D, G, Ks = 2, 1000, 128, 8, 3
    g = torch.Generator().manual_seed(K)
    x1, x2, v = (torch.randn(B, L, D, generator=g).bfloat16().to(DEV) for _ in range(3))
    u = torch.randn(B, L, 3 * D, generator=g).bfloat16().to(DEV)
    wf = (torch.randn(Ks, 3 * D, generator=g) / Ks ** 0.5).to(DEV)
    h = (O.make_mr_filter(G, K) if K == 128 else O.make_se_filter(G, K)).reshape(G, K).to(DEV)
    cmap = ops.gate_channel_map(D, interleave=True)
    res = {}
    for nt in ("0", "1"):
        override(cl_nt=int(nt))
        res[nt] = (ops.fir_cl_fwd(x1, x2, v, h, taps_reversed=K < 128),
                   ops.fir_layer_fwd(u, wf, None, cmap, h, taps_reversed=K < 128))
    assert torch.equal(res["0"][0], res["1"][0]) and torch.equal(res["0"][1], res["1"][1])


@pytest.mark.parametrize("Ks,nseg", [(3, 3), (4, 2), (3, 1)])
def test_layer_fwd_oldest_tap_across_segments(Ks, nseg, override):
    # Taps that do not decay: the oldest one (lag 127) weighs as much as the newest, so an output at the first
    # sample of a later segment that read a wrong halo sample is off by a whole term.  Checked per element:
    # the first halo samples of a segment are featurizer outputs and need the Ks-1 rows before the halo step.
    from parity import abs_scale, assert_gated_close
    B, L, D, H, G, K = 1, 1024 + 384, 64, 4, 4, 128
    override(cl_nseg=nseg)
    g = torch.Generator().manual_seed(Ks)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    h = (torch.randn(G, 1, K, generator=g) / K ** 0.5).bfloat16().float()           # bf16-exact: the MFMA operand is exact
    ref, _ = oracle_layer(u, wf, None, h, torch.zeros(D), D, H, False, True, False)
    z, _ = O.parallel_fir(u, wf, None, fir_length=Ks, dim_last=True, gate=False)
    x2, x1, v = O.interleave(z).split([D, D, D], dim=1)
    bx = x1 * v
    zr = O.fft_causal_conv_fp32(bx.float(), h.repeat_interleave(D // G, 0)[:, 0]).bfloat16()     # pre-gate value
    y = ops.fir_layer_fwd(u.to(DEV), wf.reshape(C, Ks).t().contiguous().to(DEV), None, ops.gate_channel_map(D, interleave=True),
                          h.reshape(G, K).to(DEV))
    y = y.permute(0, 2, 1)
    assert rel_err(y, ref) <= 2e-2
    S = abs_scale(bx, h.repeat_interleave(D // G, 0)[:, 0])
    # the gates themselves carry the featurizer's own rounding boundary (one bf16 ulp of x1, v or x2 now and then),
    # which moves bx by up to 2^-7 relatively: 2^-6 * S covers it, a wrong halo sample is off by ~S / 11
    assert_gated_close(y, ref, zr, x2, S, 2.0 ** -6, ulps_z=2.0, gate_ulps=1.0, what=f"fused MR layer Ks={Ks} nseg={nseg}")


@pytest.mark.parametrize("segments", [1, 2], indirect=True)      # blocks that walk all tiles of a row / half of them
@pytest.mark.parametrize("B,L,D,H,Ks,cs,il,flip,sbias", [
    (2, 512, 64, 4, 3, False, True, False, False),        # Evo 2 layout: interleaved gates
    (1, 1000, 128, 4, 3, False, True, True, True),        # L % 256 != 0, flipped gates, featurizer bias
    (2, 333, 96, 4, 3, True, False, False, True),         # head-blocked split (head_dim 24), L % 8 != 0, D % 64 != 0
    (1, 700, 200, 5, 4, False, False, False, False),      # plain split, 4-tap featurizer
    (1, 261, 64, 2, 4, False, True, False, True),
    (3, 5, 64, 4, 3, False, True, False, True),           # shorter than one pass
])
def test_featurizer_gates_fwd_vs_oracle_and_unfused_path(B, L, D, H, Ks, cs, il, flip, sbias, segments):
    # the gate-fused featurizer against the oracle's featurizer / interleave / split / x1*v, and bit for bit
    # against the three-tensor featurizer kernel followed by the same split
    g = torch.Generator().manual_seed(L + D + Ks)
    C = 3 * D
    u = torch.randn(B, L, C, generator=g).bfloat16()
    wf = torch.randn(C, 1, Ks, generator=g) / Ks ** 0.5
    bf = torch.randn(C, generator=g).bfloat16() if sbias else None
    z, _ = O.parallel_fir(u, wf, bf, fir_length=Ks, dim_last=True, gate=False)
    if il:
        z = O.interleave(z)
    x2, x1, v = O.split_gates(z, (D, H, D // H, 16, D), cs, flip)
    pad = (-L) % 8
    cmap = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    xv, g2 = ops.featurizer_gates_fwd(u.to(DEV), wf.reshape(C, Ks).t().contiguous().to(DEV),
                                      None if bf is None else bf.to(DEV), cmap, flip_x1x2=flip, front_pad=pad)
    assert xv.shape == g2.shape == (B, D, L + pad)
    assert not xv[..., :pad].any() and not g2[..., :pad].any()
    assert rel_err(xv[..., pad:], (x1 * v)) <= 1e-2 and rel_err(g2[..., pad:], x2) <= 1e-2
    zk = ops.featurizer_fwd(u.to(DEV), wf.reshape(C, Ks).to(DEV), None if bf is None else bf.to(DEV), interleave=il,
                            front_pad=pad)
    hd = D // H if cs else None
    k2, k1, kv = (zk.reshape(B, H, 3, D // H, -1)[:, :, i].reshape(B, D, -1) for i in range(3)) if cs else zk.split(D, 1)
    if flip:
        k1, k2 = k2, k1
    assert torch.equal(xv, k1 * kv) and torch.equal(g2, k2.contiguous())


@pytest.mark.parametrize("cplx,G,D,L", [(True, 8, 128, 4096), (False, 128, 128, 4096),
                                        (True, 32, 32, 65536 + 520),      # one channel per wavefront, whole-piece steps
                                        (False, 2, 32, 2048 * 9 + 8)])    # four channels per wavefront, long enough for them
def test_li_fwd_on_premultiplied_rows(cplx, G, D, L):
    # hyena_li_fwd with v = NULL: x1 holds bf16(x1*v) already; same output and state as the three-gate call
    B, S = 2, 16
    g = torch.Generator().manual_seed(21)
    x1, x2, v = (torch.randn(B, D, L, generator=g).bfloat16().to(DEV) for _ in range(3))
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, S, seed=4)
    Dc = torch.randn(D, generator=g).bfloat16().to(DEV)
    plan = ops.ModalPlan(lp.to(DEV), r.to(DEV))
    want, _, st_want = ops.li_fwd_rows(ops.rows_of(x1), ops.rows_of(x2), ops.rows_of(v), plan, Dc, B, D, L, device=DEV,
                                       want_state=True)
    xv = x1 * v
    got, _, st_got = ops.li_fwd_rows(ops.rows_of(xv), ops.rows_of(x2), None, plan, Dc, B, D, L, device=DEV,
                                     want_state=True)
    assert torch.equal(got, want) and torch.equal(torch.view_as_real(st_got) if cplx else st_got,
                                                  torch.view_as_real(st_want) if cplx else st_want)
    with pytest.raises(NotImplementedError):      # v without x2 has no meaning
        ops.li_fwd_rows(ops.rows_of(x1), None, ops.rows_of(v), plan, Dc, B, D, L, device=DEV)
