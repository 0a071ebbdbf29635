"""The drop-in engine and the operator module, driven through HyenaCascade's call sequence
(vortex/model/model.py:214-375) next to the oracle engine on the same seeded inputs:
prefill, state capture, then token-by-token decode."""
import pytest
import torch

from oracle import hyena_oracle as O
from vortex_amd.cascade import HyenaCascade, HyenaCascadeFIRInferenceParams, HyenaCascadeIIRInferenceParams
from vortex_amd.engine import HyenaInferenceEngine

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def make_params(kind, D, G, seed, Ks=3, bias=False):
    g = torch.Generator().manual_seed(seed)
    p = {"short_filter_weight": torch.randn(3 * D, 1, Ks, generator=g) / Ks ** 0.5,
         "short_filter_bias": torch.randn(3 * D, generator=g).bfloat16() if bias else None}
    if kind == "se":
        p["h"] = O.make_se_filter(G, 7, seed=seed)
        p["D"] = None
    elif kind == "mr":
        p["h"] = O.make_mr_filter(G, 128, seed=seed)
        p["D"] = torch.randn(D, generator=g).bfloat16()
    else:
        p["log_poles"], p["residues"] = (O.make_modal_real if kind == "li_real" else O.make_modal_complex)(
            G, 16, seed=seed, pmax=0.999)
        p["D"] = torch.randn(D, generator=g).bfloat16()
    return p


def to_dev(p):
    return {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in p.items()}


CASES = [
    # kind, B, L, D, heads, G(inner), column_split, interleave, short bias
    ("se", 2, 512, 64, 4, 4, False, True, False),
    ("se", 1, 333, 64, 4, 4, False, True, True),          # lengths that are not multiples of 8
    ("mr", 2, 509, 64, 4, 4, True, False, False),
    ("se", 1, 256, 64, 4, 4, True, False, True),
    ("mr", 2, 640, 64, 4, 4, False, True, False),
    ("mr", 1, 512, 32, 2, 2, True, False, False),
]


@pytest.mark.parametrize("kind,B,L,D,H,G,cs,il,sb", CASES)
def test_engine_dropin_fir_layers(kind, B, L, D, H, G, cs, il, sb):
    K = 7 if kind == "se" else 128
    p = make_params(kind, D, G, seed=L + D, bias=sb)
    g = torch.Generator().manual_seed(1)
    n_dec = 4
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, column_split_hyena=cs,
                          interleave=il)
    hip = O.OracleCascade(HyenaInferenceEngine(), to_dev(p), D, H, G, fir_inner_filter_length=K,
                          column_split_hyena=cs, interleave=il)
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeFIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = hip.forward(u_all[:, :L].to(DEV), ip_hip)
    assert y_hip.shape == y_ref.shape
    assert rel_err(y_hip, y_ref) <= 2e-2
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = hip.forward(tok.to(DEV), ip_hip)
        assert y_hip.shape == y_ref.shape
        assert rel_err(y_hip, y_ref) <= 2e-2, i
    # caches hold the same samples (ring re-ordered oldest first)
    same = torch.equal(ip_hip.fir_state_dict[0].reference_order().cpu(), ip_ref.fir_state_dict[0].float())
    assert same
    # the inner cache holds x1*v of featurizer outputs, which may differ by one bf16 rounding
    assert rel_err(ip_hip.fir_inner_state_dict[0].reference_order(), ip_ref.fir_inner_state_dict[0]) <= 2e-2


@pytest.mark.parametrize("kind,B,L,D,H,cs,il", [
    ("li_real", 2, 512, 32, 2, False, True),
])
def test_engine_dropin_modal_layer_grouped_kernel(kind, B, L, D, H, cs, il):
    # vortex's parallel_iir needs one filter per channel (G == D); the MFMA kernel needs 16 channels per
    # group.  A grouped filter bank expanded to per-channel parameters gives the oracle what it accepts
    # and the kernel what it accepts, on the same numbers.
    G = D // 16
    p = make_params(kind, D, G, seed=7)
    pD = dict(p, log_poles=p["log_poles"].repeat_interleave(16, 0), residues=p["residues"].repeat_interleave(16, 0))
    g = torch.Generator().manual_seed(2)
    n_dec = 3
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    ref = O.OracleCascade(O.OracleEngine(), pD, D, H, D, column_split_hyena=cs, interleave=il)
    hip = O.OracleCascade(HyenaInferenceEngine(), to_dev(p), D, H, G, column_split_hyena=cs, interleave=il)
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = hip.forward(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    assert rel_err(ip_hip.state_dict[0], ip_ref.state_dict[0]) <= 1e-3     # oracle state comes from fp32 FFTs
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = hip.forward(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


@pytest.mark.parametrize("cs,il", [(False, True), (True, False)])
def test_engine_dropin_modal_layer_per_channel_filters(cs, il):
    # vortex's own configuration: hcl_filter_groups == hidden_size, real poles; same parameters on both sides
    B, L, D, H, n_dec = 2, 2048 + 256, 32, 4, 3
    p = make_params("li_real", D, D, seed=5)
    g = torch.Generator().manual_seed(4)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, D, column_split_hyena=cs, interleave=il)
    hip = O.OracleCascade(HyenaInferenceEngine(), to_dev(p), D, H, D, column_split_hyena=cs, interleave=il)
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = hip.forward(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    assert rel_err(ip_hip.state_dict[0], ip_ref.state_dict[0]) <= 1e-3     # oracle state comes from fp32 FFTs
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = hip.forward(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


@pytest.mark.parametrize("L", [517, 200, 40, 3, 1])
@pytest.mark.parametrize("kind", ["se", "mr", "li_real", "li_cplx"])
def test_operator_module_any_prompt_length(kind, L):
    # prompts whose length is not a multiple of 8, or shorter than the filters (the reference then grows its caches
    # step by step, engine.py:443-444), through prefill and decode steps (fused and two-kernel paths)
    B, D, H, G = 2, 64, 4, 4
    K = {"se": 7, "mr": 128}.get(kind)
    p = make_params(kind, D, G, seed=31)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    if K is None:
        pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
        ref = O.OracleCascade(O.OracleEngine(), pr, D, H, D, interleave=True)
    else:
        ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, interleave=True)
    n_dec = 2 if L > 100 else 6
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(L)).bfloat16()
    for fused in (True, False):
        mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K, complex_modal=(kind == "li_cplx"))
        with torch.no_grad():
            mod.short_filter_weight.copy_(p["short_filter_weight"])
            if K:
                mod.h.copy_(p["h"])
            else:
                mod.log_poles.copy_(p["log_poles"])
                mod.residues.copy_(p["residues"])
            if mod.D is not None:
                mod.D.data = p["D"].clone()
        mod = mod.to(DEV)
        mod.fuse_prefill = mod.fuse_decode = fused
        ip_ref = O.OracleCache()
        ip_hip = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
        y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
        y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
        assert y_hip.shape == (B, L, D) and rel_err(y_hip, y_ref) <= 2e-2
        for i in range(n_dec):
            tok = u_all[:, L + i: L + i + 1]
            y_ref, _ = ref.forward(tok, ip_ref)
            y_hip, _ = mod(tok.to(DEV), ip_hip)
            assert rel_err(y_hip, y_ref) <= 2e-2, (fused, i)


@pytest.mark.parametrize("D,H,G", [(640, 10, 64), (768, 12, 64), (1920, 15, 128)])
@pytest.mark.parametrize("kind", ["se", "mr", "li_real"])
def test_operator_module_reference_model_geometries(kind, D, H, G):
    # hidden size / heads / filter groups of shc-evo2-50m-8k-1T.yml, shc-evo2-100m-8k-1T.yml and evo2-1b-8k.yml:
    # groups of 10, 12 and 15 channels; the long-filter layers have one filter per channel
    B, L, n_dec = 1, 264, 3
    K = {"se": 7, "mr": 128}.get(kind)
    Gk = G if K else D
    p = make_params(kind, D, Gk, seed=D)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, Gk, fir_inner_filter_length=K, interleave=True)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(D)).bfloat16()
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=Gk, fir_inner_filter_length=K)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        if K:
            mod.h.copy_(p["h"])
        else:
            mod.log_poles.copy_(p["log_poles"])
            mod.residues.copy_(p["residues"])
        if mod.D is not None:
            mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    ip_ref = O.OracleCache()
    ip_hip = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


@pytest.mark.parametrize("S,bias,L", [(8, False, 512), (2, True, 512), (2, True, 37), (4, False, 200)])
def test_operator_module_small_state_sizes(S, bias, L):
    # the long-filter layers of the older configurations: state_size 8 (shc-evo2-7b-8k-2T-v1.yml) and 2
    # (7b-sh-32k-v1.yml), one filter per channel, head-blocked column split, featurizer bias
    B, D, H, n_dec = 2, 64, 4, 5
    g = torch.Generator().manual_seed(S)
    lp, r = O.make_modal_real(D, S, seed=S, pmax=0.999)
    p = {"short_filter_weight": torch.randn(3 * D, 1, 3, generator=g) / 3 ** 0.5,
         "short_filter_bias": torch.randn(3 * D, generator=g).bfloat16() if bias else None,
         "log_poles": lp, "residues": r, "D": torch.randn(D, generator=g).bfloat16()}
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=True, interleave=False, short_filter_length=3,
               short_filter_bias=bias, state_size=S)
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, D, column_split_hyena=True, interleave=False)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    for fused in (True, False):
        mod = HyenaCascade(cfg, 0)
        with torch.no_grad():
            mod.short_filter_weight.copy_(p["short_filter_weight"])
            if bias:
                mod.short_filter_bias.copy_(p["short_filter_bias"])
            mod.log_poles.copy_(lp)
            mod.residues.copy_(r)
            mod.D.data = p["D"].clone()
        mod = mod.to(DEV)
        mod.fuse_prefill = mod.fuse_decode = fused
        ip_ref, ip_hip = O.OracleCache(), HyenaCascadeIIRInferenceParams()
        y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
        y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2
        assert ip_hip.state_dict[0].shape == (B, D, S)
        for i in range(n_dec):
            tok = u_all[:, L + i: L + i + 1]
            y_ref, _ = ref.forward(tok, ip_ref)
            y_hip, _ = mod(tok.to(DEV), ip_hip)
            assert rel_err(y_hip, y_ref) <= 2e-2, (fused, i)


@pytest.mark.parametrize("flip", [False, True])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("kind,cs,il", [("se", False, True), ("mr", False, True), ("mr", True, False),
                                         ("li_cplx", False, True), ("li_real", True, False), ("se", False, False),
                                         ("li_real", False, False), ("mr", True, True)])
def test_operator_module_prefill_then_decode(kind, cs, il, fused, flip):
    # vortex_amd.cascade.HyenaCascade (fused fast path) against the oracle call sequence, with and without
    # hyena_flip_x1x2 (vortex/model/model.py:342-343, engine.py:157-158, :309-310)
    B, L, D, H, n_dec = 2, 512, 64, 4, 4
    K = {"se": 7, "mr": 128}.get(kind)
    G = 4
    p = make_params(kind, D, G, seed=11)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=cs, interleave=il, short_filter_length=3,
               short_filter_bias=False, state_size=16, hyena_flip_x1x2=flip)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K, complex_modal=(kind == "li_cplx"))
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        if K:
            mod.h.copy_(p["h"])
        else:
            mod.log_poles.copy_(p["log_poles"])
            mod.residues.copy_(p["residues"])
        if mod.D is not None:
            mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    mod.fuse_decode = mod.fuse_prefill = fused
    if K is None:     # oracle needs per-channel modal parameters
        pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0),
                  residues=p["residues"].repeat_interleave(D // G, 0))
        ref = O.OracleCascade(O.OracleEngine(hyena_flip_x1x2=flip), pr, D, H, D, column_split_hyena=cs, interleave=il)
    else:
        ref = O.OracleCascade(O.OracleEngine(hyena_flip_x1x2=flip), p, D, H, G, fir_inner_filter_length=K,
                              column_split_hyena=cs, interleave=il)
    assert ref.hyena_flip_x1x2 == flip
    g = torch.Generator().manual_seed(3)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    ip_ref = O.OracleCache()
    ip_hip = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i
    if fused:   # one launch per step wherever a closed channel map exists (not interleave + column split)
        assert (mod._decode["layer"] is not None) == (not (cs and il))


@pytest.mark.parametrize("kind,cs,il,fused", [("li_cplx", False, True, True), ("li_real", True, False, True),
                                              ("li_cplx", True, True, True), ("li_real", False, False, False)])
def test_operator_module_windowed_modal_state(kind, cs, il, fused):
    # at batch x width of 65536 and more the module's decode step keeps the modal state in windows of four tokens:
    # outputs against the oracle call sequence on every token, the cached state lagging in between and equal to
    # the oracle's after flush_decode_state(), and further tokens after the flush
    from vortex_amd import ops
    B, L, D, H, G = 64, 8, 1024, 8, 64
    p = make_params(kind, D, G, seed=13)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=cs, interleave=il, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, complex_modal=(kind == "li_cplx"))
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.log_poles.copy_(p["log_poles"])
        mod.residues.copy_(p["residues"])
        mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    mod.fuse_decode = mod.fuse_prefill = fused
    assert mod.window_decode_state is False         # the reference keeps the state current: windows are opt-in
    mod.window_decode_state = True
    pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
    ref = O.OracleCascade(O.OracleEngine(), pr, D, H, D, column_split_hyena=cs, interleave=il)
    n_dec = 11
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(4)).bfloat16()
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    as_real = lambda t: torch.view_as_real(t) if t.is_complex() else t
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i
        if i == 6:
            inner = mod._decode["inner"]
            assert isinstance(inner, ops.IirStepper) and inner.win is not None
            assert rel_err(as_real(ip_hip.state_dict[0]), as_real(ip_ref.state_dict[0])) > 1e-2     # lags the tokens
            mod.flush_decode_state()
            assert rel_err(as_real(ip_hip.state_dict[0]), as_real(ip_ref.state_dict[0])) <= 1e-3
    mod.flush_decode_state()
    assert rel_err(as_real(ip_hip.state_dict[0]), as_real(ip_ref.state_dict[0])) <= 1e-3
    mod.flush_decode_state()                               # nothing pending: no launch, same state
    assert rel_err(as_real(ip_hip.state_dict[0]), as_real(ip_ref.state_dict[0])) <= 1e-3


@pytest.mark.parametrize("windowed", [False, True])
def test_operator_module_serves_two_cache_objects_in_turn(windowed):
    # one module, two sequences A and B with their own cache objects, decoded alternately (prefill A, steps on A,
    # prefill B, steps on B, back to A, ...): every output and both final states against the oracle call sequence.
    # With the windowed modal state the pending inputs live in the bound stepper, which has to leave a cache object's
    # state complete whenever the module turns to another one.
    B, D, H, G = 64, 1024, 8, 64
    p = make_params("li_cplx", D, G, seed=21)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, complex_modal=True)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.log_poles.copy_(p["log_poles"])
        mod.residues.copy_(p["residues"])
        mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    mod.window_decode_state = windowed
    pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
    ref = O.OracleCascade(O.OracleEngine(), pr, D, H, D, interleave=True)
    g = torch.Generator().manual_seed(22)
    seqs = {k: torch.randn(B, 8 + 16, 3 * D, generator=g).bfloat16() for k in "AB"}
    caches = {k: (O.OracleCache(), HyenaCascadeIIRInferenceParams()) for k in "AB"}
    used = {k: 0 for k in "AB"}

    def run(k, n):
        ip_ref, ip_hip = caches[k]
        for _ in range(n):
            a = used[k]
            b = 8 if a == 0 else a + 1
            u = seqs[k][:, a:b]
            used[k] = b
            y_ref, _ = ref.forward(u, ip_ref)
            y_hip, _ = mod(u.to(DEV), ip_hip)
            assert rel_err(y_hip, y_ref) <= 2e-2, (k, a)

    for k, n in [("A", 4), ("B", 3), ("A", 3), ("B", 6), ("A", 5), ("B", 1), ("A", 1)]:
        run(k, n)
    if windowed:
        from vortex_amd import ops
        assert isinstance(mod._decode["inner"], ops.IirStepper) and mod._decode["inner"].win is not None
    mod.flush_decode_state()
    for k in "AB":
        a, b = torch.view_as_real(caches[k][1].state_dict[0]), torch.view_as_real(caches[k][0].state_dict[0])
        assert rel_err(a, b) <= 1e-3, k


def test_operator_module_growing_cache_under_a_far_sum_stepper():
    # an inner filter of 64 taps with the plain tap slicing (vortex/model/engine.py:424-425) and a prompt shorter than
    # the filter: the reference grows its cache by one sample per token and shifts the taps with it.  A 63-slot cache
    # is deep enough for the far-sum stepper, whose sums carry a token's taps into the next two outputs; the steps
    # that grow the cache therefore have to read it whole.  Decode through the growth and well past it.
    B, L, D, H, G, K, n_dec = 2, 20, 64, 4, 4, 64, 56
    g = torch.Generator().manual_seed(41)
    p = {"short_filter_weight": torch.randn(3 * D, 1, 3, generator=g) / 3 ** 0.5, "short_filter_bias": None,
         "h": torch.randn(G, 1, K, generator=g) / K ** 0.5, "D": None}
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, interleave=True)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    from vortex_amd import ops
    for fused in (True, False):
        mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K)
        with torch.no_grad():
            mod.short_filter_weight.copy_(p["short_filter_weight"])
            mod.h.copy_(p["h"])
        mod = mod.to(DEV)
        mod.fuse_prefill = mod.fuse_decode = fused
        ip_ref, ip_hip = O.OracleCache(), HyenaCascadeFIRInferenceParams()
        y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
        y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2
        for i in range(n_dec):
            tok = u_all[:, L + i: L + i + 1]
            y_ref, _ = ref.forward(tok, ip_ref)
            y_hip, _ = mod(tok.to(DEV), ip_hip)
            assert rel_err(y_hip, y_ref) <= 2e-2, (fused, i)
        assert mod._decode["inner"].far is not None            # the far-sum stepper was the one bound
        assert rel_err(ip_hip.fir_inner_state_dict[0].reference_order(), ip_ref.fir_inner_state_dict[0]) <= 2e-2


@pytest.mark.parametrize("kind", ["se", "mr", "li_real"])
def test_operator_module_groups_of_15_channels(kind):
    # Evo 2 1B geometry in small: hidden = 16 groups x 15 channels (1920 = 128 x 15 there), 15 heads, interleaved gates
    B, L, H, G, n_dec = 2, 400, 15, 16, 3
    D = 15 * G
    K = {"se": 7, "mr": 128}.get(kind)
    p = make_params(kind, D, G if K else D, seed=41)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G if K else D, fir_inner_filter_length=K)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        if K:
            mod.h.copy_(p["h"])
        else:
            mod.log_poles.copy_(p["log_poles"])
            mod.residues.copy_(p["residues"])
        if mod.D is not None:
            mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, G if K else D, fir_inner_filter_length=K, interleave=True)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(7)).bfloat16()
    ip_ref = O.OracleCache()
    ip_hip = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    y_hip, _ = mod(u_all[:, :L].to(DEV), ip_hip)
    assert rel_err(y_hip, y_ref) <= 2e-2
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


def test_hyena_ops_interface_layouts():
    import hyena_ops
    from hyena_ops import interface as I
    B, L, G, dg, K = 2, 256, 4, 16, 7
    gen = torch.Generator().manual_seed(5)
    x, k, q = (torch.randn(B, L, G, dg, generator=gen).bfloat16() for _ in range(3))
    h = O.make_se_filter(G, K)
    ref = O.gcg_fwd_ref(x.float(), k.float(), q.float(), h)           # fp32 evaluation of the same operator
    y = I.two_pass_chunked_gate_conv_gate(x.to(DEV), k.to(DEV), q.to(DEV), h.to(DEV),
                                          fwd_kernel_cfg=I.FwdKernelConfig(), bwd_kernel_cfg=I.BwdKernelConfig())
    assert y.shape == ref.shape and rel_err(y, ref) <= 2e-2
    xb, kb, qb = (t.reshape(B, L, G * dg).transpose(1, 2).contiguous() for t in (x, k, q))
    y2 = I.inner_hyena_se(xb.to(DEV), kb.to(DEV), qb.to(DEV), h.to(DEV), output_layout="bld")   # blocked groups
    assert rel_err(y2, ref.reshape(B, L, G * dg)) <= 2e-2
    # inner_hyena_se_ref stripes the filters instead (tests/test_gpu_hyena_ops.py)
    # package-level names of vortex/model/layers.py:19
    out = hyena_ops.hyena_se_fwd(kb.to(DEV), qb.to(DEV), xb.to(DEV), h.to(DEV))
    assert rel_err(out.transpose(1, 2), ref.reshape(B, L, G * dg)) <= 2e-2


def test_featurizer_full_width():
    # 3D = 12288 channels as in the 7B configuration, channel-last in, sequence-last out
    B, L, C, K = 1, 1000, 12288, 3
    g = torch.Generator().manual_seed(9)
    u = torch.randn(B, L, C, generator=g).bfloat16()
    w = torch.randn(C, 1, K, generator=g)
    from vortex_amd import ops
    z = ops.featurizer_fwd(u.to(DEV), w.reshape(C, K).to(DEV), None, interleave=True)
    ref, _ = O.parallel_fir(u, w, None, fir_length=K, dim_last=True, gate=False)
    ref = O.interleave(ref)
    assert rel_err(z, ref) <= 2e-2
    assert (z.cpu() == ref).float().mean() > 0.98


def test_hyena_ops_any_length():
    from hyena_ops import interface as I
    B, L, G, dg, K = 2, 203, 2, 16, 5
    gen = torch.Generator().manual_seed(8)
    x, k, q = (torch.randn(B, G * dg, L, generator=gen).bfloat16() for _ in range(3))
    h = O.make_se_filter(G, K)
    ref = O.se_fir(q, k, x, h)[0]
    assert rel_err(I.inner_hyena_se(x.to(DEV), k.to(DEV), q.to(DEV), h.to(DEV)), ref) <= 2e-2
    w = h.repeat_interleave(dg, 0)[:, 0]
    assert rel_err(I.causal_conv1d_ref(x.to(DEV), w.to(DEV)), O.short_fir_fp32(x, w[:, None], K).bfloat16()) <= 2e-2
    xl, kl, ql = (t.permute(0, 2, 1).reshape(B, L, G, dg).contiguous() for t in (x, k, q))
    y = I.two_pass_chunked_gate_conv_gate(xl.to(DEV), kl.to(DEV), ql.to(DEV), h.to(DEV))
    assert rel_err(y.reshape(B, L, G * dg).permute(0, 2, 1), ref) <= 2e-2


def test_two_pass_fwd_grouped_intermediates():
    # (y, T, T_hat, y2, bx_lag) of vortex/ops/hyena_se/fwd.py:290 on (b, l, g, dg) tensors, channel-last kernel
    from hyena_ops import interface as I
    B, L, G, dg, K, CH = 2, 512, 3, 32, 33, 128
    gen = torch.Generator().manual_seed(6)
    x, Bm, Cm = (torch.randn(B, L, G, dg, generator=gen).bfloat16() for _ in range(3))
    h = torch.randn(G, 1, K, generator=gen) / K ** 0.5
    y, T, T_hat, y2, bx_lag = I.two_pass_fwd_grouped(x.to(DEV), Bm.to(DEV), Cm.to(DEV), h.to(DEV), return_y2=True,
                                                     return_toeplitz=True, return_bx_lag=True, CHUNK_SIZE=CH)
    ref = O.gcg_fwd_ref(x.float(), Bm.float(), Cm.float(), h)
    assert y.shape == ref.shape and rel_err(y, ref) <= 2e-2
    assert rel_err(y, O.gcg_two_pass_chunked(x.float(), Bm.float(), Cm.float(), h, CH)) <= 2e-2
    y2_ref = O.gcg_fwd_ref(x.float(), Bm.float(), torch.ones_like(Cm).float(), h)
    assert rel_err(y2, y2_ref) <= 2e-2
    bx = Bm * x
    assert torch.equal(bx_lag[:, :L - CH].cpu(), bx[:, :L - CH]) and not bx_lag[:, L - CH:].any()
    hf = h.flip(-1)[:, 0]
    assert torch.equal(T.cpu(), O.toeplitz(hf, CH).bfloat16())
    assert torch.equal(T_hat.cpu(), O.correction_toeplitz(hf, CH).bfloat16())


@pytest.mark.parametrize("kind", ["se", "mr", "li_real"])
def test_operator_module_padding_mask(kind):
    # left-padded batch: the 0/1 mask of vortex/model/engine.py:226-227 on both FIR outputs
    B, L, D, H, G = 2, 384, 64, 4, 4
    K = {"se": 7, "mr": 128}.get(kind)
    p = make_params(kind, D, G, seed=21)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        if K:
            mod.h.copy_(p["h"])
        else:
            mod.log_poles.copy_(p["log_poles"])
            mod.residues.copy_(p["residues"])
        if mod.D is not None:
            mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    if K is None:
        pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
        ref = O.OracleCascade(O.OracleEngine(), pr, D, H, D, interleave=True)
    else:
        ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, interleave=True)
    u = torch.randn(B, L, 3 * D, generator=torch.Generator().manual_seed(4)).bfloat16()
    mask = torch.ones(B, L)
    mask[0, :37] = 0
    mask[1, :5] = 0
    y_ref, _ = ref.forward(u, None, padding_mask=mask)
    y_hip, _ = mod(u.to(DEV), None, padding_mask=mask.to(DEV))
    assert rel_err(y_hip, y_ref) <= 2e-2


@pytest.mark.parametrize("T,L,cs", [(128, 1024, False), (32, 520, True), (7, 333, False)])
def test_engine_parallel_iir_truncated_fir_branch(T, L, cs):
    # long_fir_threshold (vortex/model/engine.py:339-349): the first T samples of the materialised modal filter as a
    # bf16 depthwise FIR, in the orientation F.conv1d gives them.  Engine against the oracle's restatement.
    B, D, H = 1, 32, 4
    g = torch.Generator().manual_seed(T)
    lp, r = O.make_modal_real(D, 16, seed=T, pmax=0.99)
    h = O.modal_filter(lp, r, L)                                   # [1, D, L]
    z_pre = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, H, D // H, 16, D)
    y_ref, _ = O.parallel_iir(z_pre, h, Db, L, lp, r, dims, column_split_hyena=cs, long_fir_threshold=T)
    eng = HyenaInferenceEngine()
    y = eng.parallel_iir(z_pre.to(DEV), h.to(DEV), Db.to(DEV), L, lp.to(DEV), r.to(DEV), None, dims, 0,
                         column_split_hyena=cs, long_fir_threshold=T)
    assert y.shape == (B, L, D) and rel_err(y, y_ref) <= 2e-2
    with pytest.raises(NotImplementedError):                        # the reference cannot prefill a cache on this branch
        eng.parallel_iir(z_pre.to(DEV), h.to(DEV), Db.to(DEV), L, lp.to(DEV), r.to(DEV), None, dims, 0,
                         inference_params=HyenaCascadeIIRInferenceParams(), long_fir_threshold=T)


@pytest.mark.parametrize("T,L,cs", [(200, 1024, False), (129, 515, True), (700, 1500, False)])
def test_engine_parallel_iir_truncated_fir_longer_than_128(T, L, cs):
    # a long_fir_threshold beyond the MFMA kernel's 128 taps (vortex/model/engine.py:339-349 takes any): the
    # direct-form kernel in blocks of 128 lags, same arithmetic, against the oracle's restatement
    B, D, H = 2, 48, 4
    g = torch.Generator().manual_seed(T)
    lp, r = O.make_modal_real(D, 16, seed=T, pmax=0.99)
    h = O.modal_filter(lp, r, L)
    z_pre = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, H, D // H, 16, D)
    y_ref, _ = O.parallel_iir(z_pre, h, Db, L, lp, r, dims, column_split_hyena=cs, long_fir_threshold=T)
    y = HyenaInferenceEngine().parallel_iir(z_pre.to(DEV), h.to(DEV), Db.to(DEV), L, lp.to(DEV), r.to(DEV), None, dims, 0,
                                            column_split_hyena=cs, long_fir_threshold=T)
    assert y.shape == (B, L, D) and rel_err(y, y_ref) <= 2e-2


@pytest.mark.parametrize("K,L", [(200, 700), (384, 1030), (129, 130)])
def test_inner_fir_longer_than_128(K, L):
    # FIR layers longer than 128 taps (vortex/model/engine.py:174-187 takes any length through its FFT): the operator
    # module and the engine seam against the oracle call sequence, prefill, cache hand-off and decode steps
    B, D, H, G, n_dec = 2, 64, 4, 4, 3
    g = torch.Generator().manual_seed(K)
    p = {"short_filter_weight": torch.randn(3 * D, 1, 3, generator=g) / 3 ** 0.5, "short_filter_bias": None,
         "h": O.make_mr_filter(G, K, seed=K), "D": torch.randn(D, generator=g).bfloat16()}
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=g).bfloat16()
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, interleave=True)
    ip_ref = O.OracleCache()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    # the engine seam under the reference's own call sequence
    hip = O.OracleCascade(HyenaInferenceEngine(), to_dev(p), D, H, G, fir_inner_filter_length=K, interleave=True)
    ip_e = HyenaCascadeFIRInferenceParams()
    y_e, _ = hip.forward(u_all[:, :L].to(DEV), ip_e)
    assert rel_err(y_e, y_ref) <= 2e-2
    # the operator module
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.h.copy_(p["h"])
        mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    ip_m = HyenaCascadeFIRInferenceParams()
    y_m, _ = mod(u_all[:, :L].to(DEV), ip_m)
    assert rel_err(y_m, y_ref) <= 2e-2
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_e, _ = hip.forward(tok.to(DEV), ip_e)
        y_m, _ = mod(tok.to(DEV), ip_m)
        assert rel_err(y_e, y_ref) <= 2e-2 and rel_err(y_m, y_ref) <= 2e-2, i
    # and the functional entry point on explicit gates
    import vortex_amd as va
    x2, x1, v = O.make_gates(B, D, L, seed=K)
    Df = torch.randn(D, generator=g)
    got = va.hyena_mr_fwd(x1.to(DEV), x2.to(DEV), v.to(DEV), p["h"].to(DEV), Df.to(DEV))
    assert rel_err(got, O.mr_fir(x2, x1, v, p["h"], Df)[0]) <= 2e-2


@pytest.mark.parametrize("T,G", [(128, 4), (16, 64)])
def test_operator_module_truncated_fir_config(T, G):
    # `long_fir_threshold` in the model configuration (vortex/model/model.py:185, :310): the operator module builds
    # the T filter samples itself and runs them as a grouped FIR; against the oracle call sequence
    B, L, D, H = 2, 700, 64, 4
    p = make_params("li_real", D, G, seed=T)
    pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
    ref = O.OracleCascade(O.OracleEngine(), pr, D, H, D, interleave=True, long_fir_threshold=T)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16, long_fir_threshold=T)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.log_poles.copy_(p["log_poles"])
        mod.residues.copy_(p["residues"])
        mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    u = torch.randn(B, L, 3 * D, generator=torch.Generator().manual_seed(3)).bfloat16()
    y_ref, _ = ref.forward(u)
    y, _ = mod(u.to(DEV))
    assert rel_err(y, y_ref) <= 2e-2
    with pytest.raises(NotImplementedError):
        mod(u.to(DEV), HyenaCascadeIIRInferenceParams())


@pytest.mark.parametrize("cplx,L", [(False, 1032), (True, 520)])
def test_engine_parallel_iir_recurrence_prefill_seam(cplx, L):
    # prefill_style="recurrence" (vortex/model/engine.py:314-321, :473-504): poles themselves and residues arrive as
    # [D, S, 1, 2] (re, im) lanes, one filter per channel; the state comes back as [B, D, S, 2] float32.  Checked
    # against the explicit recurrence in float64 (what that branch evaluates, without its bf16 state rounding) and,
    # for real poles, against the literal restatement of the reference's loop.
    B, D, H, S = 2, 16, 2, 16
    g = torch.Generator().manual_seed(L)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(D, S, seed=L, pmax=0.99)
    p = torch.exp(lp[..., 0].to(torch.complex64))
    poles = torch.view_as_real(p)[:, :, None, :].contiguous()                            # [D, S, 1, 2]
    res_re = (r.real if cplx else r).float()
    residues = torch.stack([res_re, torch.zeros_like(res_re)], -1)[:, :, None, :].contiguous()
    z_pre = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    Db = torch.randn(D, generator=g).bfloat16()
    dims = (D, H, D // H, S, D)
    x2, x1, v = z_pre.split([D, D, D], dim=1)
    x1v = x1 * v
    # y = sum_s r_re * s_re is what engine.py:500 forms: residues with a zero imaginary lane in the exact recurrence
    y64, s64 = O.prefill_direct_recurrence(x1v, lp.to(torch.complex64) if cplx else lp, res_re.to(torch.complex64) if cplx else res_re)
    y_ref = ((y64.float().bfloat16() + x1v * Db[:, None]) * x2).permute(0, 2, 1)
    ip = HyenaCascadeIIRInferenceParams()
    eng = HyenaInferenceEngine()
    y = eng.parallel_iir(z_pre.to(DEV), None, Db.to(DEV), L, poles.to(DEV), residues.to(DEV), None, dims, 3,
                         inference_params=ip, prefill_style="recurrence")
    assert y.shape == (B, L, D) and rel_err(y, y_ref) <= 2e-2
    st = ip.state_dict[3]
    assert st.shape == (B, D, S, 2) and st.dtype == torch.float32
    s_ref = torch.view_as_real(s64.to(torch.complex128)) if cplx else torch.stack([s64, torch.zeros_like(s64)], -1)
    assert rel_err(st, s_ref) <= 1e-4
    if not cplx:
        # distance to the reference's loop as it is written (bf16 state, rounded every step): with real poles its
        # other two quirks vanish.  The loop itself is 9e-3 (output) and 1.4e-2 (state) away from the exact
        # recurrence on these inputs; the kernel, which carries the state in float32, stays within 2e-2 / 3e-2 of it.
        y_lit, s_lit = O.prefill_direct_recurrence_ref(x1v, poles, residues)
        y_lit = ((y_lit + x1v * Db[:, None]) * x2).permute(0, 2, 1)
        assert rel_err(y, y_lit) <= 2e-2
        assert rel_err(st, s_lit) <= 3e-2
    with pytest.raises(ValueError):
        eng.parallel_iir(z_pre.to(DEV), None, Db.to(DEV), L, lp.to(DEV), r.to(DEV), None, dims, 3,
                         inference_params=HyenaCascadeIIRInferenceParams(), prefill_style="recurrence")
    with pytest.raises(NotImplementedError):
        eng.parallel_iir(z_pre.to(DEV), None, Db.to(DEV), L, lp.to(DEV), r.to(DEV), None, dims, 3,
                         inference_params=HyenaCascadeIIRInferenceParams(), prefill_style="modal-scan")


def test_engine_per_channel_weight_with_groups_argument():
    # vortex's conv1d filters per channel whatever `groups` says (engine.py:203).  A weight whose rows differ inside a
    # group must therefore run per channel; one that was expanded with repeat_interleave may be folded back.
    B, D, H, G, K, L = 1, 32, 2, 4, 7, 256
    g = torch.Generator().manual_seed(0)
    u = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    dims = (D, H, D // H, 16, G)
    eng = HyenaInferenceEngine()
    w_distinct = torch.randn(D, 1, K, generator=g) / K ** 0.5
    w_grouped = (torch.randn(G, 1, K, generator=g) / K ** 0.5).repeat_interleave(D // G, 0)
    for w in (w_distinct, w_grouped):
        ref, _ = O.parallel_fir(u, w, None, L, dims, groups=G, dim_last=False, fir_length=K, gate=True)
        wd = w.to(DEV)
        for _ in range(2):                                          # second call: the cached verdict
            z, _ = eng.parallel_fir(torch.nn.functional.conv1d, u.to(DEV), wd, None, L, dims, groups=G, dim_last=False,
                                    fir_length=K, gate=True)
            assert rel_err(z, ref) <= 2e-2
    # an in-place update of the same tensor object is seen (version counter)
    wd = w_grouped.clone().to(DEV)
    eng.parallel_fir(torch.nn.functional.conv1d, u.to(DEV), wd, None, L, dims, groups=G, dim_last=False, fir_length=K, gate=True)
    wd.copy_(w_distinct)
    ref, _ = O.parallel_fir(u, w_distinct, None, L, dims, groups=G, dim_last=False, fir_length=K, gate=True)
    z, _ = eng.parallel_fir(torch.nn.functional.conv1d, u.to(DEV), wd, None, L, dims, groups=G, dim_last=False,
                            fir_length=K, gate=True)
    assert rel_err(z, ref) <= 2e-2


def test_engine_short_fir_gated_bias_in_bf16():
    # K < 128 with gated_bias (engine.py:218-221): z = bf16(conv), then z + bias*u in bf16 tensor arithmetic
    B, D, H, G, K, L = 2, 32, 2, 2, 7, 264
    g = torch.Generator().manual_seed(1)
    u = torch.randn(B, 3 * D, L, generator=g).bfloat16()
    w = (torch.randn(G, 1, K, generator=g) / K ** 0.5).repeat_interleave(D // G, 0)
    bias = torch.randn(D, generator=g).bfloat16()
    dims = (D, H, D // H, 16, G)
    ref, _ = O.parallel_fir(u, w, bias, L, dims, groups=G, gated_bias=True, dim_last=False, fir_length=K, gate=True)
    z, _ = HyenaInferenceEngine().parallel_fir(torch.nn.functional.conv1d, u.to(DEV), w.to(DEV), bias.to(DEV), L, dims,
                                               groups=G, gated_bias=True, dim_last=False, fir_length=K, gate=True)
    assert rel_err(z, ref) <= 2e-2
    assert (z.cpu() == ref).float().mean() > 0.97


@pytest.mark.parametrize("flip", [False, True])
@pytest.mark.parametrize("kind,cs,il", [("li_cplx", False, True), ("li_real", True, False), ("li_real", False, False)])
def test_operator_module_sequence_major_projection(kind, cs, il, flip):
    """A Hyena-LI layer handed its projection as the [B, L, 3D] view of a [B, 3D, L] tensor (what the projection GEMM
    writes when asked for the transposed product) runs featurizer, gates and scan in one launch
    (hyena_li_layer_fwd).  Against the oracle's call sequence (vortex/model/model.py:214-375): prefill outputs, the
    modal state and the featurizer cache it leaves, and the decode steps that follow from them."""
    B, L, D, H, G, n_dec = 2, 512, 64, 4, 4, 4
    p = make_params(kind, D, G, seed=23)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=cs, interleave=il, short_filter_length=3,
               short_filter_bias=False, state_size=16, hyena_flip_x1x2=flip)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, complex_modal=(kind == "li_cplx"))
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.log_poles.copy_(p["log_poles"])
        mod.residues.copy_(p["residues"])
        mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    pr = dict(p, log_poles=p["log_poles"].repeat_interleave(D // G, 0), residues=p["residues"].repeat_interleave(D // G, 0))
    ref = O.OracleCascade(O.OracleEngine(hyena_flip_x1x2=flip), pr, D, H, D, column_split_hyena=cs, interleave=il)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(5)).bfloat16()
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeIIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    u_seq = u_all[:, :L].to(DEV).transpose(1, 2).contiguous().transpose(1, 2)       # same values, samples contiguous
    assert u_seq.stride(1) == 1 and mod._can_scan_projection_rows(u_seq)
    y_hip, _ = mod(u_seq, ip_hip)
    assert "wf_rows" in mod._f32_cache                       # the one-launch path ran
    assert y_hip.shape == (B, L, D) and rel_err(y_hip, y_ref) <= 2e-2
    s_ref = ip_ref.state_dict[0]
    s_hip = ip_hip.state_dict[0].cpu()
    if not s_hip.is_complex() and s_ref.is_complex():
        s_ref = s_ref.real
    assert rel_err(torch.view_as_real(s_hip) if s_hip.is_complex() else s_hip,
                   torch.view_as_real(s_ref) if s_ref.is_complex() else s_ref) <= 1e-4
    assert torch.equal(ip_hip.fir_state_dict[0].reference_order().cpu().float(), ip_ref.fir_state_dict[0].float())
    # the same module on the same values stored channel-last (two launches): one bf16 digit at most
    y_cl, _ = mod(u_all[:, :L].to(DEV), HyenaCascadeIIRInferenceParams())
    assert rel_err(y_hip, y_cl) <= 2.0 ** -7
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


@pytest.mark.parametrize("flip", [False, True])
@pytest.mark.parametrize("kind,cs,il", [("mr", False, True), ("se", False, True), ("mr", True, False), ("se", False, False)])
def test_operator_module_sequence_major_projection_fir(kind, cs, il, flip):
    """A Hyena-SE / MR layer handed its projection as the [B, L, 3D] view of a [B, 3D, L] tensor runs featurizer, gates
    and the inner FIR in one launch (hyena_fir_layer_fwd_rows).  Against the oracle's call sequence
    (vortex/model/model.py:214-375): prefill outputs, both FIR caches it leaves, and the decode steps after them."""
    B, L, D, H, G, n_dec = 2, 512, 64, 4, 4, 4
    K = {"se": 7, "mr": 128}[kind]
    p = make_params(kind, D, G, seed=29)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=cs, interleave=il, short_filter_length=3,
               short_filter_bias=False, state_size=16, hyena_flip_x1x2=flip)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G, fir_inner_filter_length=K)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.h.copy_(p["h"])
        if mod.D is not None:
            mod.D.data = p["D"].clone()
    mod = mod.to(DEV)
    ref = O.OracleCascade(O.OracleEngine(hyena_flip_x1x2=flip), p, D, H, G, fir_inner_filter_length=K,
                          column_split_hyena=cs, interleave=il)
    u_all = torch.randn(B, L + n_dec, 3 * D, generator=torch.Generator().manual_seed(6)).bfloat16()
    ip_ref, ip_hip = O.OracleCache(), HyenaCascadeFIRInferenceParams()
    y_ref, _ = ref.forward(u_all[:, :L], ip_ref)
    u_seq = u_all[:, :L].to(DEV).transpose(1, 2).contiguous().transpose(1, 2)
    assert mod._can_filter_projection_rows(u_seq)
    y_hip, _ = mod(u_seq, ip_hip)
    assert "wf_rows" in mod._f32_cache                       # the one-launch path ran
    assert y_hip.shape == (B, L, D) and rel_err(y_hip, y_ref) <= 2e-2
    assert torch.equal(ip_hip.fir_state_dict[0].reference_order().cpu().float(), ip_ref.fir_state_dict[0].float())
    inner = ip_hip.fir_inner_state_dict[0].reference_order().cpu().float()
    assert rel_err(inner, ip_ref.fir_inner_state_dict[0].float()) <= 2.0 ** -7
    y_cl, _ = mod(u_all[:, :L].to(DEV), HyenaCascadeFIRInferenceParams())          # channel-last: the fused kernel
    assert rel_err(y_hip, y_cl) <= 2.0 ** -7
    for i in range(n_dec):
        tok = u_all[:, L + i: L + i + 1]
        y_ref, _ = ref.forward(tok, ip_ref)
        y_hip, _ = mod(tok.to(DEV), ip_hip)
        assert rel_err(y_hip, y_ref) <= 2e-2, i


def test_sequence_major_projection_wrapper_feeds_the_one_launch_layer():
    """use_hip_filters(model, sequence_major_projections=True): the wrapped projection of a Hyena-LI block hands the
    cascade the projection's values stored sequence-major, the cascade runs one launch, and the result agrees with
    the same block on the plain linear layer (channel-last projection, two launches) to the last bf16 digit."""
    import types
    from vortex_amd.cascade import SequenceMajorProjection, use_hip_filters
    B, L, D, H, G = 2, 256, 64, 4, 4
    p = make_params("li_real", D, G, seed=31)
    cfg = dict(hidden_size=D, num_attention_heads=H, column_split_hyena=False, interleave=True, short_filter_length=3,
               short_filter_bias=False, state_size=16)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=G)
    with torch.no_grad():
        mod.short_filter_weight.copy_(p["short_filter_weight"])
        mod.log_poles.copy_(p["log_poles"])
        mod.residues.copy_(p["residues"])
        mod.D.data = p["D"].clone()
    lin = torch.nn.Linear(D, 3 * D, bias=False)
    block = types.SimpleNamespace(filter=mod.to(DEV), projections=lin.to(DEV).to(torch.bfloat16))
    use_hip_filters(types.SimpleNamespace(blocks=[block]), sequence_major_projections=True)
    assert isinstance(block.projections, SequenceMajorProjection)
    x = torch.randn(B, L, D, generator=torch.Generator().manual_seed(7)).bfloat16().to(DEV)
    z_seq, z_cl = block.projections(x), block.projections.linear(x)
    assert z_seq.shape == z_cl.shape and z_seq.stride(1) == 1
    assert rel_err(z_seq, z_cl) <= 2.0 ** -7                     # two GEMM kernels, one bf16 digit
    assert block.projections(x[:, :1]).is_contiguous()           # a decode token goes through the layer itself
    y_seq, _ = block.filter(z_seq)
    assert "wf_rows" in block.filter._f32_cache
    y_cl, _ = block.filter(z_seq.contiguous())                   # the same values channel-last: two launches
    assert rel_err(y_seq, y_cl) <= 2.0 ** -7
