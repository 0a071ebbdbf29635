"""hyena_li_layer_fwd: a whole Hyena-LI layer in one pass over a projection stored sequence-major -- the featurizer FIR
of vortex/model/model.py:233-246 (vortex/model/engine.py:188-223), the split of :250-252 under every channel map of
vortex/model/utils.py:26-85, and parallel_iir with its state (engine.py:283-353, :525-559).

Two statements: (1) bit for bit the result of the featurizer kernel followed by hyena_li_fwd on its gates (the same
products in the same order when both run the same work decomposition: lone wavefronts of one or of four channels;
across the two decompositions the scan adds in a different order and the results agree to rounding), on small and
ragged shapes and at the full long-convolution shape; (2) against the oracle's featurizer + gates + FFT convolution
(oracle.hyena_oracle, float32) within the tolerances of hyena_li_fwd: bf16 outputs 2e-2, state 1e-4."""
import pytest
import torch

from oracle import hyena_oracle as O
from vortex_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(B, L, D, G, seed, cplx=False):
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, L, 3 * D, generator=g).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g) / 3 ** 0.5).to(torch.bfloat16).float()
    lp, rs = (O.make_modal_complex if cplx else O.make_modal_real)(G, 16, seed=seed + 1, pmax=0.999)
    Dc = torch.randn(D, generator=g).to(torch.bfloat16)
    return u, w, lp, rs, Dc


def _two_launches(u, w, plan, Dc, D, il, hd):
    B, L, _ = u.shape
    z = ops.featurizer_fwd(u, w, None, interleave=il)
    r2, r1, rv = (ops.rows_of_projection(z, D, i, hd) for i in range(3))
    with _lib.launch_override(li_coop=0):       # lone wavefronts, as the one-pass form runs
        y, _, st = ops.li_fwd_rows(r1, r2, rv, plan, Dc, B, D, L, device=DEV, want_state=True)
    return y, st


def _one_pass(u, w, plan, Dc, D, il, hd, **kw):
    B, L, _ = u.shape
    p = u.transpose(1, 2).contiguous()                                   # what the transposed GEMM would write
    (q2, q1, qv), chan = ops.projection_rows(p, D, interleave=il, head_dim=hd)
    taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
    return ops.li_layer_fwd_rows(q1, q2, qv, taps, plan, Dc, B, D, L, device=DEV, want_state=True, **kw)


@pytest.mark.parametrize("mode", ["plain", "interleave", "head"])
@pytest.mark.parametrize("B,L,D,G", [(2, 1024, 256, 16),        # four channels per wavefront
                                     (1, 4136, 256, 256),       # one filter per channel, a ragged last chunk
                                     (2, 72, 128, 8),           # shorter than a chunk
                                     (1, 8, 64, 64),            # one piece
                                     (3, 2048 + 64, 192, 12),   # three steps of four channels, groups of 16
                                     (1, 65536, 256, 16)])      # long rows: one channel per wavefront
def test_li_layer_equals_featurizer_then_scan(mode, B, L, D, G):
    il, hd = mode == "interleave", (64 if mode == "head" else None)
    u, w, lp, rs, Dc = _case(B, L, D, G, seed=L + D + G)
    u, w, Dc = u.to(DEV), w.to(DEV), Dc.to(DEV)
    plan = ops.ModalPlan(lp.to(DEV), rs.to(DEV))
    for cpw in ((1, 4) if (D // G) % 4 == 0 else (1,)):
        with _lib.launch_override(li_cpw=cpw):
            y0, s0 = _two_launches(u, w, plan, Dc, D, il, hd)
            y1, s1 = _one_pass(u, w, plan, Dc, D, il, hd)
        assert torch.equal(y0, y1), cpw
        assert torch.equal(s0, s1), cpw
        assert bool(torch.isfinite(y1.float()).all())
    # whatever decomposition the library picks by itself for this shape: the same result up to the order of the scan
    y2, s2 = _one_pass(u, w, plan, Dc, D, il, hd)
    assert ((y2.float() - y1.float()).abs().max() / y1.float().abs().max()).item() <= 1e-2
    assert ((s2 - s1).abs().max() / s1.abs().max().clamp_min(1e-30)).item() <= 1e-5


@pytest.mark.parametrize("cpw", [1, 4])
@pytest.mark.parametrize("nt", [0, 1])
def test_li_layer_forms(cpw, nt):
    # both work decompositions and both kinds of memory access on one shape, against each other and the two launches
    B, L, D, G = 2, 4096 + 384, 256, 16
    u, w, lp, rs, Dc = _case(B, L, D, G, seed=5, cplx=True)
    u, w, Dc = u.to(DEV), w.to(DEV), Dc.to(DEV)
    plan = ops.ModalPlan(lp.to(DEV), rs.to(DEV))
    with _lib.launch_override(li_cpw=cpw):
        y0, s0 = _two_launches(u, w, plan, Dc, D, True, None)
    with _lib.launch_override(li_cpw=cpw, li_nt=nt):
        y1, s1 = _one_pass(u, w, plan, Dc, D, True, None)
    assert torch.equal(y0, y1) and torch.equal(torch.view_as_real(s0), torch.view_as_real(s1))
    # the other decomposition adds the scan's terms in another order: the same result to rounding
    with _lib.launch_override(li_cpw=5 - cpw):
        y2, s2 = _one_pass(u, w, plan, Dc, D, True, None)
    assert ((y2.float() - y1.float()).abs().max() / y1.float().abs().max()).item() <= 1e-2
    assert ((s2 - s1).abs().max() / s1.abs().max()).item() <= 1e-5


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("mode", ["plain", "interleave", "head"])
def test_li_layer_vs_oracle(mode, cplx):
    """Against the reference's arithmetic restated on the CPU: featurizer conv1d in float32 rounded to bf16
    (engine.py:196-208), interleave / column split, x1 * v, the FFT long convolution with the modal filter and the
    D term (engine.py:331-353), the gate, and the state of prefill_via_modal_fft (engine.py:525-559)."""
    B, L, D, G, H = 2, 1536, 64, 4, 4
    il, hd = mode == "interleave", (D // H if mode == "head" else None)
    u, w, lp, rs, Dc = _case(B, L, D, G, seed=17, cplx=cplx)
    p = {"short_filter_weight": w.reshape(3 * D, 1, 3), "short_filter_bias": None, "D": Dc,
         "log_poles": lp.repeat_interleave(D // G, 0), "residues": rs.repeat_interleave(D // G, 0)}
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, D, column_split_hyena=hd is not None, interleave=il)
    cache = O.OracleCache()
    y_ref, _ = ref.forward(u, cache)                                     # [B, L, D]
    plan = ops.ModalPlan(lp.to(DEV), rs.to(DEV))
    y, st = _one_pass(u.to(DEV), w.to(DEV), plan, Dc.to(DEV), D, il, hd)
    y = y.permute(0, 2, 1).float().cpu()
    err = ((y - y_ref.float()).abs().max() / y_ref.float().abs().max()).item()
    assert err <= 2e-2, err
    s_ref = cache.state_dict[0]
    s = st.cpu()
    if not cplx:
        s_ref = s_ref.real if s_ref.is_complex() else s_ref
    serr = ((s - s_ref).abs().max() / s_ref.abs().max()).item()
    assert serr <= 1e-4, serr


def test_li_layer_argument_errors():
    B, L, D, G = 1, 64, 64, 4
    u, w, lp, rs, Dc = _case(B, L, D, G, seed=3)
    u, w = u.to(DEV), w.to(DEV)
    plan = ops.ModalPlan(lp.to(DEV), rs.to(DEV))
    p = u.transpose(1, 2).contiguous()
    (q2, q1, qv), chan = ops.projection_rows(p, D)
    taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
    out = torch.empty(B, D, L, dtype=torch.bfloat16, device=DEV)
    call = _lib.lib().hyena_li_layer_fwd
    args = lambda **k: [ops._ref(k.get("x1", q1)), ops._ref(k.get("x2", q2)), ops._ref(k.get("v", qv)),
                        k.get("taps", taps.data_ptr()), k.get("n", 3), plan.workspace.data_ptr(), None, 1, out.data_ptr(),
                        None, B, D, k.get("L", L), G, 16, None]
    EINVAL, EALIGN, ENOSUP = -1, -2, -3
    assert call(*args()) == 0
    assert call(*args(n=4)) == ENOSUP and b"4 taps" in _lib.lib().hyena_last_error_string()
    assert call(*args(taps=None)) == EINVAL
    assert call(*args(v=None)) == EINVAL
    assert call(*args(L=60)) == EALIGN
    with pytest.raises(ValueError):
        ops.projection_rows(p, D, interleave=True, head_dim=16)
    torch.cuda.synchronize()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("G", [256, 4096])
def test_li_layer_full_size(G):
    """The long-convolution configuration (B = 1, L = 262144, D = 4096; 256 shared filters, and one filter per channel
    as vortex configures hcl_filter_groups = hidden_size) from an interleaved projection: bit for bit the featurizer
    kernel followed by the scan, the impulse property (a projection that is zero but for one sample of one operator
    channel's three rows gives that channel's filter scaled by the featurizer's response), and finite everywhere."""
    B, L, D = 1, 262144, 4096
    g = torch.Generator(device=DEV).manual_seed(G)
    u = torch.randn(B, L, 3 * D, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g, device=DEV) / 3 ** 0.5).to(torch.bfloat16).float()
    lp, rs = O.make_modal_complex(G, 16, seed=G, pmax=0.9999)
    Dc = torch.randn(D, generator=g, device=DEV).to(torch.bfloat16)
    plan = ops.ModalPlan(lp.to(DEV), rs.to(DEV))
    with _lib.launch_override(li_cpw=1):       # what the one-pass form picks for rows this long; pinned for the scan alone
        y0, s0 = _two_launches(u, w, plan, Dc, D, True, None)
    y1, s1 = _one_pass(u, w, plan, Dc, D, True, None)
    assert torch.equal(y0, y1)
    assert torch.equal(torch.view_as_real(s0), torch.view_as_real(s1))
    assert bool(torch.isfinite(y1.float()).all())
