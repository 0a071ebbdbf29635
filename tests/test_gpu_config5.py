"""The Evo 2 7B-shaped stack at its configured width and prompt length -- hidden 4096, 32 heads, MLP 11008,
vocab 512, L = 8192, one [SE, MR, LI, attention] group (reduced depth) -- against the float32 CPU restatement of
the reference's layers (oracle/stack_oracle.py: RMSNorm vortex/model/layers.py:191-196, gated MLP :242-246, block
wiring vortex/model/model.py:523-575 and :105-122, tied unembedding layers.py:309-311) with the Hyena oracle inside.

The product runs bf16 GEMMs / SDPA through torch and the Hyena operators on the HIP kernels; the oracle runs the
dense layers in float32 on the same bf16-rounded weights.  Stated bounds, as max|a-b| / max|b| and mean|a-b| / max|b|
of the residual stream: every block on its own (fed the oracle's input) within 2e-2 / 2e-3, one block's worth
of bf16 rounding (observed 6e-3..1.4e-2 / 5e-4..1.5e-3); the chained stack after block i (from 0) within
1e-2 (i+2) / 1.5e-3 (i+2), the rounding of the bf16 residual stream accumulating with depth (observed 1.4e-2 ->
2.9e-2 over the four blocks at hidden 4096, 8e-3 -> 3.2e-2 over eight at hidden 256); the logits likewise.  A wiring mistake (a residual taken from the wrong
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
def test_7b_shaped_group_at_L8192_vs_oracle():
    cfg = dict(EVO2_7B, num_layers=4)
    _compare(cfg, 8192, 21)
