"""hyena_fir_layer_fwd_rows: a whole Hyena-SE / MR layer in one pass over a projection stored sequence-major -- the
featurizer FIR of vortex/model/model.py:233-246 (vortex/model/engine.py:188-223), the split under every channel map of
vortex/model/utils.py:26-85 and the gated inner FIR of engine.py:131-260 on the matrix cores.

(1) bit for bit the featurizer kernel followed by hyena_mr_fwd (hyena_se_fwd for filters of at most 8 taps) on its gates, across channel maps, filter lengths,
segmentations along L, group sizes that do not fill an MFMA tile and ragged lengths; (2) against the oracle's
featurizer + gated convolution within the bf16 tolerance 2e-2 and the per-element forward-error bound."""
import pytest
import torch

from oracle import hyena_oracle as O
from vortex_amd import _lib, ops
from vortex_amd._lib import HYENA_BIAS_GATED_FP32, HYENA_BIAS_NONE

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(B, L, D, G, K, seed):
    g = torch.Generator().manual_seed(seed)
    u = torch.randn(B, L, 3 * D, generator=g).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g) / 3 ** 0.5).to(torch.bfloat16).float()
    h = (torch.randn(G, K, generator=g) / K ** 0.5).to(torch.bfloat16).float()
    Dc = torch.randn(D, generator=g).to(torch.bfloat16).float() if K >= 128 else None
    return u, w, h, Dc


def _both(u, w, h, Dc, D, K, il, hd, mfma=None, **ov):
    B, L, _ = u.shape
    mr = K >= 128
    bm = HYENA_BIAS_GATED_FP32 if mr else HYENA_BIAS_NONE
    with _lib.launch_override(**ov):
        z = ops.featurizer_fwd(u, w, None, interleave=il)
        r2, r1, rv = (ops.rows_of_projection(z, D, i, hd) for i in range(3))
        y0 = ops.fir_fwd_rows(r1, r2, rv, h, B, D, L, K, device=DEV, bias=Dc, bias_mode=bm, taps_reversed=not mr,
                              force_mfma=K > 8 if mfma is None else mfma)      # short filters: the direct-form kernel on both sides
        p = u.transpose(1, 2).contiguous()
        (q2, q1, qv), chan = ops.projection_rows(p, D, interleave=il, head_dim=hd)
        taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
        y1 = ops.fir_layer_fwd_rows(q1, q2, qv, taps, h, B, D, L, K, device=DEV, bias=Dc, bias_mode=bm,
                                    taps_reversed=not mr)
    return y0, y1


@pytest.mark.parametrize("mode", ["plain", "interleave", "head"])
@pytest.mark.parametrize("B,L,D,G,K,ov", [(2, 1024, 256, 16, 128, {}),
                                          (1, 4136, 256, 16, 7, {}),                       # a ragged last step
                                          (1, 8192, 256, 16, 128, {"mr_nseg": 4}),         # segments along L: carried history at each start
                                          (1, 4096, 256, 16, 20, {"mr_nseg": 3, "mr_nt": 1}),
                                          (2, 72, 128, 8, 128, {}),                        # shorter than a step
                                          (2, 72, 128, 8, 7, {}),                          # short filter: blocks straddle rows
                                          (3, 8, 128, 8, 4, {}),                           # one octet per row
                                          (1, 2072, 120, 8, 7, {}),
                                          (2, 16, 64, 64, 2, {}),
                                          (1, 16384, 64, 4, 7, {"se_nt": 1}),              # whole blocks per row, streaming accesses
                                          (1, 16384, 64, 4, 7, {"mr_nseg": 2}),
                                          (1, 2048, 120, 8, 128, {}),                      # groups of 15 channels: a part-filled slab
                                          (3, 1536, 64, 64, 128, {"mr_nseg": 3})])         # one filter per channel
def test_fir_layer_rows_equals_featurizer_then_fir(mode, B, L, D, G, K, ov):
    if mode == "head" and D % 64:
        pytest.skip("head-blocked split needs whole heads")
    il, hd = mode == "interleave", (64 if mode == "head" else None)
    u, w, h, Dc = (t.to(DEV) if t is not None else None for t in _case(B, L, D, G, K, seed=L + D + K))
    y0, y1 = _both(u, w, h, Dc, D, K, il, hd, **ov)
    assert torch.equal(y0, y1)
    assert bool(torch.isfinite(y1.float()).all())


@pytest.mark.parametrize("K", [7, 128])
@pytest.mark.parametrize("mode", ["plain", "interleave", "head"])
def test_fir_layer_rows_vs_oracle(mode, K):
    """Against the reference's arithmetic restated on the CPU (OracleCascade: featurizer conv1d rounded to bf16,
    interleave / column split, x1 * v, the inner filter with its D term, the gate)."""
    B, L, D, G, H = 2, 1536, 64, 4, 4
    il, hd = mode == "interleave", (D // H if mode == "head" else None)
    u, w, h, Dc = _case(B, L, D, G, K, seed=K)
    p = {"short_filter_weight": w.reshape(3 * D, 1, 3), "short_filter_bias": None,
         "D": Dc.to(torch.bfloat16) if Dc is not None else None, "h": h.reshape(G, 1, K)}
    ref = O.OracleCascade(O.OracleEngine(), p, D, H, G, fir_inner_filter_length=K, column_split_hyena=hd is not None,
                          interleave=il)
    y_ref, _ = ref.forward(u)
    _, y = _both(u.to(DEV), w.to(DEV), h.to(DEV), Dc.to(DEV) if Dc is not None else None, D, K, il, hd)
    y = y.permute(0, 2, 1).float().cpu()
    err = ((y - y_ref.float()).abs().max() / y_ref.float().abs().max()).item()
    assert err <= 2e-2, err


def test_fir_layer_rows_argument_errors():
    B, L, D, G, K = 1, 64, 64, 4, 128
    u, w, h, Dc = (t.to(DEV) for t in _case(B, L, D, G, K, seed=3))
    p = u.transpose(1, 2).contiguous()
    (q2, q1, qv), chan = ops.projection_rows(p, D)
    taps = torch.stack([w[chan[1]], w[chan[0]], w[chan[2]]]).contiguous()
    out = torch.empty(B, D, L, dtype=torch.bfloat16, device=DEV)
    call = _lib.lib().hyena_fir_layer_fwd_rows
    args = lambda **k: [ops._ref(q1), ops._ref(q2), ops._ref(k.get("v", qv)), k.get("taps", taps.data_ptr()), k.get("n", 3),
                        h.data_ptr(), 0, Dc.data_ptr(), k.get("bm", HYENA_BIAS_GATED_FP32), out.data_ptr(), B, D,
                        k.get("L", L), G, k.get("K", K), None]
    EINVAL, EALIGN, ENOSUP = -1, -2, -3
    assert call(*args()) == 0
    assert call(*args(n=4)) == ENOSUP
    assert call(*args(taps=None)) == EINVAL
    assert call(*args(v=None)) == EINVAL
    assert call(*args(bm=1)) == ENOSUP                 # additive bias: no featurizer kernel
    assert call(*args(K=200)) == ENOSUP
    assert call(*args(L=60)) == EALIGN
    torch.cuda.synchronize()


@pytest.mark.timeout(600)
def test_fir_layer_rows_short_filter_on_streaming_tensors():
    """Hyena-SE rows at batch 8 (2.1 GB: beyond the last-level cache), where the entry point runs short filters on the
    matrix-core kernel: bit for bit the featurizer kernel followed by hyena_mr_fwd with the same filter."""
    B, L, D, G, K = 8, 8192, 4096, 256, 7
    g = torch.Generator(device=DEV).manual_seed(2)
    u = torch.randn(B, L, 3 * D, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g, device=DEV) / 3 ** 0.5).to(torch.bfloat16).float()
    h = O.make_se_filter(G, K).reshape(G, K).to(DEV)
    y0, y1 = _both(u, w, h, None, D, K, True, None, mfma=True)
    assert torch.equal(y0, y1)


@pytest.mark.timeout(600)
def test_fir_layer_rows_full_size():
    """The Hyena-MR configuration (B = 2, L = 32768, D = 4096, 256 groups, K = 128) from an interleaved projection:
    bit for bit the featurizer kernel followed by hyena_mr_fwd."""
    B, L, D, G, K = 2, 32768, 4096, 256, 128
    g = torch.Generator(device=DEV).manual_seed(1)
    u = torch.randn(B, L, 3 * D, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn(3 * D, 3, generator=g, device=DEV) / 3 ** 0.5).to(torch.bfloat16).float()
    h = O.make_mr_filter(G, K).reshape(G, K).to(DEV)
    Dc = torch.randn(D, generator=g, device=DEV)
    y0, y1 = _both(u, w, h, Dc, D, K, True, None)
    assert torch.equal(y0, y1)
    assert bool(torch.isfinite(y1.float()).all())
