"""The end-to-end stack around the operators: runs, is finite, and is batch-invariant
(the property the reference's test/test_forward.py:26-52 asserts for its model)."""
import pytest
import torch

from vortex_amd.model import EVO2_7B, StripedHyena2

pytestmark = pytest.mark.gpu


def test_tiny_stack_runs_and_is_batch_invariant():
    cfg = dict(EVO2_7B, hidden_size=128, num_layers=8, num_attention_heads=4, inner_mlp_size=256,
               hcs_filter_groups=8, hcm_filter_groups=8, hcl_filter_groups=128)
    m = StripedHyena2(cfg, seed=1, device="cuda").to_inference("cuda")
    ids = torch.randint(0, 512, (1, 512), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    y1 = m(ids)
    y4 = m(ids.repeat(4, 1))
    assert y1.shape == (1, 512, 512) and torch.isfinite(y1).all()
    err = (y1[0].float() - y4[2].float()).abs().max() / y1.float().abs().max()
    assert err <= 2e-2      # bf16 GEMMs pick other tilings at batch 4; the Hyena kernels are batch-invariant


def test_hyena_blocks_are_batch_invariant_bitwise():
    cfg = dict(EVO2_7B, hidden_size=64, num_layers=3, num_attention_heads=4, inner_mlp_size=128,
               hcs_filter_groups=4, hcm_filter_groups=4, hcl_filter_groups=16, pattern=("hcs", "hcm", "hcl"))
    m = StripedHyena2(cfg, seed=3, device="cuda").to_inference("cuda")
    g = torch.Generator(device="cuda").manual_seed(4)
    z = torch.randn(1, 1024, 192, device="cuda", generator=g).bfloat16()
    for blk in m.blocks:
        a, _ = blk.filter(z)
        b, _ = blk.filter(z.repeat(3, 1, 1))
        assert torch.equal(a[0], b[1])


@pytest.mark.parametrize("L", [256, 203])
def test_cached_generation_matches_a_longer_prefill(L):
    # generation order of vortex/model/generation.py:164-229: prefill, then one token per forward from the caches
    # (FIR rings, modal states, attention keys / values).  Teacher-forced, so every step's logits can be compared
    # with one prefill over prompt + continuation.
    cfg = dict(EVO2_7B, hidden_size=128, num_layers=8, num_attention_heads=4, inner_mlp_size=256,
               hcs_filter_groups=8, hcm_filter_groups=8, hcl_filter_groups=128)
    m = StripedHyena2(cfg, seed=5, device="cuda").to_inference("cuda")
    n = 6
    ids = torch.randint(0, 512, (2, L + n), device="cuda", generator=torch.Generator(device="cuda").manual_seed(6))
    full = m(ids).float()                                  # logits at every position of the long sequence
    toks, scores = m.generate(ids[:, :L], n, forced=ids[:, L:])
    assert torch.equal(toks, ids[:, L:])
    want = full[:, L - 1:L + n - 1]                        # step i predicts token L + i from position L + i - 1
    err = (scores.float() - want).abs().max() / want.abs().max()
    assert err <= 3e-2, err                                # bf16 GEMM / SDPA paths differ between prefill and decode
