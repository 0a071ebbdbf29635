"""The Evo 2 7B-shaped stack at its configured width, depth and prompt length -- hidden 4096, 32 heads, MLP 11008,
vocab 512, L = 8192, all 32 blocks (eight [SE, MR, LI, attention] groups) -- against the float32 CPU restatement of
the reference's layers (oracle/stack_oracle.py: RMSNorm vortex/model/layers.py:191-196, gated MLP :242-246, block
wiring vortex/model/model.py:523-575 and :105-122, tied unembedding layers.py:309-311) with the Hyena oracle inside.

The product runs bf16 GEMMs / SDPA through torch and the Hyena operators on the HIP kernels; the oracle runs the
dense layers in float32 on the same bf16-rounded weights.  Stated bounds, as max|a-b| / max|b| and mean|a-b| / max|b|
of the residual stream: every block on its own (fed the oracle's input) within 2e-2 / 2e-3, one block's worth
of bf16 rounding (observed 6e-3..1.4e-2 / 5e-4..1.5e-3); the chained stack after block i (from 0) within
1e-2 (i+2) / 1.5e-3 (i+2), the rounding of the bf16 residual stream accumulating with depth (observed 1.3e-2 ->
1.3e-1 over the 32 blocks at hidden 4096, 8e-3 -> 3.2e-2 over eight at hidden 256); the logits likewise.  A wiring mistake (a residual taken from the wrong
place, a missing norm, gates in another order) moves these figures to O(1)."""
import time

import pytest
import torch

from oracle.stack_oracle import OracleStack, rms_norm
from vortex_amd.model import EVO2_7B, StripedHyena2

pytestmark = pytest.mark.gpu


def _stat(a, b):
    scale = b.abs().max()
    return round(((a - b).abs().max() / scale).item(), 5), round(((a - b).abs().mean() / scale).item(), 6)


def _compare(cfg, L, seed):
    m = StripedHyena2(cfg, seed=seed, device="cuda").to_inference("cuda")
    ids = torch.randint(0, cfg["vocab_size"], (1, L), device="cuda", generator=torch.Generator(device="cuda").manual_seed(seed + 1))
    with torch.no_grad():
        x = m.embedding(ids)
        hidden = []
        for block in m.blocks:
            x, _ = block(x)
            hidden.append(x.float().cpu())
        logits = (m.norm(x) @ m.embedding.weight.T).float().cpu()
        assert torch.equal(logits, m(ids).float().cpu())                     # the same path forward() takes
    torch.cuda.synchronize()
    t0 = time.time()
    oracle = OracleStack(cfg, m.kinds, m.state_dict())
    ref_hidden = oracle.forward(ids, return_hidden=True)
    ref_logits = rms_norm(ref_hidden[-1], oracle.p["norm.scale"], cfg["eps"]) @ oracle.p["embedding.weight"].T
    print(f"oracle stack: {time.time() - t0:.1f} s on the host", flush=True)
    # (1) every block on its own: fed the oracle's input stream (rounded to bf16), compared with the oracle's output.
    #     One block's worth of bf16 rounding: max <= 2e-2, mean <= 2e-3 of the stream's largest magnitude.
    iso = []
    with torch.no_grad():
        for i, block in enumerate(m.blocks):
            src = oracle.p["embedding.weight"][ids.cpu()] if i == 0 else ref_hidden[i - 1]
            y, _ = block(src.to(torch.bfloat16).cuda())
            iso.append(_stat(y.float().cpu(), ref_hidden[i]))
    # (2) the chained stack: bf16 rounding of the residual stream accumulates about linearly with depth
    chain = [_stat(a, b) for a, b in zip(hidden, ref_hidden)]
    lg = _stat(logits, ref_logits)
    print("isolated blocks (max, mean):", iso, "\nchained:", chain, "\nlogits:", lg, flush=True)
    for i, (mx, mean) in enumerate(iso):
        assert mx <= 2e-2 and mean <= 2e-3, ("isolated block", i, m.kinds[i], iso)
    for i, (mx, mean) in enumerate(chain):
        assert mx <= 1e-2 * (i + 2) and mean <= 1.5e-3 * (i + 2), ("chained, after block", i, chain)
    n = len(m.blocks)
    assert lg[0] <= 1e-2 * (n + 2) and lg[1] <= 1.5e-3 * (n + 2), ("logits", lg)


def test_small_width_stack_vs_oracle():
    # two groups at hidden 256 with grouped filters of every kind, a ragged length, column split off / interleave on
    cfg = dict(EVO2_7B, hidden_size=256, num_layers=8, num_attention_heads=8, inner_mlp_size=704,
               hcs_filter_groups=16, hcm_filter_groups=16, hcl_filter_groups=256)
    _compare(cfg, 1000, 11)


@pytest.mark.timeout(900)
def test_7b_shaped_stack_at_full_depth_vs_oracle():
    """The configuration as it is named: all 32 blocks of the 7B-shaped stack (eight [SE, MR, LI, attention] groups at
    hidden 4096, MLP 11008) on an 8192-token prompt.  Every block on its own against the oracle's block, and the
    chained residual stream and the logits within the depth-dependent bound (the float32 oracle of 32 blocks takes
    about two minutes on the host)."""
    _compare(dict(EVO2_7B), 8192, 41)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("kind", ["hcs", "hcm", "hcl", "hcl_rows", "hcm_rows"])
def test_7b_shaped_hyena_layers_at_L131072(kind):
    """The long leg of the end-to-end configuration (B = 1, L = 131072, hidden 4096): each of the three Hyena operator
    modules of a [SE, MR, LI, attention] group exactly as the stack runs it (projection u [1, L, 3*4096] in the
    interleaved layout, fused prefill paths, cache objects filled), against the oracle's call sequence
    (OracleCascade, vortex/model/model.py:214-375) on sampled filter groups -- the operators are independent per
    channel, so a slice of the projection is a complete small problem -- plus two properties that need no oracle:
    the first 8192 outputs equal a prefill of the first 8192 samples alone, and a prefill of L - 8 samples followed
    by 8 cached one-token steps reproduces the last 8 outputs of the full prefill."""
    from oracle import hyena_oracle as O
    from vortex_amd.cascade import HyenaCascadeFIRInferenceParams, HyenaCascadeIIRInferenceParams
    cfg = dict(EVO2_7B)
    D, L = cfg["hidden_size"], 131072
    # "_rows": the same projection values stored sequence-major ([1, 3D, L], as the stack's Hyena-LI blocks ask their
    # projection GEMM to write them), which the module runs in one launch with the featurizer inside the operator kernel
    rows, kind = kind.endswith("_rows"), kind.split("_")[0]
    m = StripedHyena2(dict(cfg, num_layers=4), seed=31, device="cuda").to_inference("cuda")
    mod = m.blocks[("hcs", "hcm", "hcl").index(kind)].filter
    K = mod.fir_inner_filter_length
    g = torch.Generator(device="cuda").manual_seed(32)
    u = torch.randn(1, L, 3 * D, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    if rows:
        u = u.transpose(1, 2).contiguous().transpose(1, 2)
        assert mod._can_scan_projection_rows(u) or mod._can_filter_projection_rows(u)
    with torch.no_grad():
        if kind == "hcl":       # slow poles too (|p| up to 0.9999): a memory that spans the whole prompt
            mod.log_poles.copy_(-(1e-4 + 0.1 * torch.rand(mod.log_poles.shape, generator=g, device="cuda")))
        if mod.D is not None:   # the skip term is zero-initialised in the stack; give it values
            mod.D.copy_(torch.randn(D, generator=g, device="cuda"))
        ip = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
        y, _ = mod(u, ip)
        torch.cuda.synchronize()
        assert y.shape == (1, L, D) and bool(torch.isfinite(y.float()).all())
        # ---- the oracle's call sequence on sampled operator channels d0 .. d0+15 (one filter group of SE / MR)
        for d0 in (0, 1600, D - 16):
            sl = slice(3 * d0, 3 * (d0 + 16))
            p = {"short_filter_weight": mod.short_filter_weight[sl].float().cpu(), "short_filter_bias": None}
            if K:
                p["h"] = mod.h[d0 // 16: d0 // 16 + 1].float().cpu().repeat(16, 1, 1)     # the group's filter, per channel
                p["D"] = mod.D[d0:d0 + 16].cpu() if mod.D is not None else None
                ref = O.OracleCascade(O.OracleEngine(), p, 16, 1, 16, fir_inner_filter_length=K, interleave=True)
            else:
                p["log_poles"], p["residues"] = mod.log_poles[d0:d0 + 16].float().cpu(), mod.residues[d0:d0 + 16].float().cpu()
                p["D"] = mod.D[d0:d0 + 16].cpu()
                ref = O.OracleCascade(O.OracleEngine(), p, 16, 1, 16, interleave=True)
            ip_ref = O.OracleCache()
            y_ref, _ = ref.forward(u[:, :, sl].cpu(), ip_ref)
            got = y[:, :, d0:d0 + 16].float().cpu()
            s = _stat(got, y_ref.float())
            print(kind, d0, "vs oracle (max, mean):", s, flush=True)
            assert s[0] <= 2e-2 and s[1] <= 2e-3, (kind, d0, s)
            if K:
                a = ip.fir_inner_state_dict[mod.layer_idx].reference_order()[:, d0:d0 + 16].cpu()
                assert _stat(a, ip_ref.fir_inner_state_dict[0].float())[0] <= 2e-2
            else:
                a = ip.state_dict[mod.layer_idx][:, d0:d0 + 16].float().cpu()
                assert _stat(a, ip_ref.state_dict[0].float())[0] <= 1e-3          # the oracle's state comes from fp32 FFTs
            fa = ip.fir_state_dict[mod.layer_idx].reference_order()[:, sl].cpu()
            assert torch.equal(fa, ip_ref.fir_state_dict[0].float())
        # ---- causality: the first 8192 outputs do not depend on what follows (another launch shape, same values)
        y_head, _ = mod(u[:, :8192].contiguous())          # (a channel-last copy: the other path of the module)
        d = (y_head.float() - y[:, :8192].float()).abs().max() / y[:, :8192].float().abs().max()
        assert d <= 2.0 ** -7, d            # at most the last bf16 digit (another segmentation of the same sums)
        # ---- prefill of L - 8 samples, then 8 cached steps, against the last 8 outputs of the full prefill
        ip2 = HyenaCascadeFIRInferenceParams() if K else HyenaCascadeIIRInferenceParams()
        y0, _ = mod(u[:, :L - 8], ip2)
        tail = torch.cat([mod(u[:, L - 8 + i: L - 7 + i], ip2)[0] for i in range(8)], dim=1)
        scale = y.float().abs().max()
        assert (y0.float() - y[:, :L - 8].float()).abs().max() / scale <= 2.0 ** -7
        assert (tail.float() - y[:, L - 8:].float()).abs().max() / scale <= 2e-2
