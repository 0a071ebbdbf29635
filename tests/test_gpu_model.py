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


@pytest.mark.parametrize("L,attn", [(256, True), (203, True), (256, False), (203, False)])
def test_recorded_token_step_matches_eager_generation(L, attn):
    # the token step replayed as a HIP graph (ring positions and the attention position in device memory) against
    # the eager loop, teacher-forced over enough tokens for every ring to wrap (the featurizer ring every 2 tokens,
    # the Hyena-SE ring every 6), with the host reading results and synchronising between replays
    cfg = dict(EVO2_7B, hidden_size=128, num_layers=8, num_attention_heads=4, inner_mlp_size=256,
               hcs_filter_groups=8, hcm_filter_groups=8, hcl_filter_groups=128,
               pattern=("hcs", "hcm", "hcl", "attn") if attn else ("hcs", "hcm", "hcl"))
    m = StripedHyena2(cfg, seed=5, device="cuda").to_inference("cuda")
    n = 20
    ids = torch.randint(0, 512, (2, L + n), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    toks_e, scores_e = m.generate(ids[:, :L], n, forced=ids[:, L:])
    toks_g, scores_g = m.generate(ids[:, :L], n, forced=ids[:, L:], graph=True)
    torch.cuda.synchronize()
    assert torch.equal(toks_e, toks_g)
    for i in range(n):
        want, got = scores_e[:, i].float(), scores_g[:, i].float()
        if attn:        # the recorded attention step (masked full-length cache) is another SDPA path: bf16 noise
            err = (got - want).abs().max() / want.abs().max()
            assert err <= 3e-2, (i, err.item())
        else:           # Hyena blocks only: the same kernels on the same data
            assert torch.equal(got, want), i
    # a second generation on the same model records a fresh step and still agrees
    toks_g2, scores_g2 = m.generate(ids[:, :L], n, forced=ids[:, L:], graph=True)
    assert torch.equal(scores_g2, scores_g)


def test_windowed_modal_state_in_generation():
    # at batch x width of 65536 and more the Hyena-LI decode step keeps its modal state in windows of several tokens:
    # the recorded step replays the same kernels as the eager loop bit for bit, both agree with a longer prefill, and
    # the plain per-token state update gives the same logits up to bf16 rounding
    from vortex_amd import ops
    cfg = dict(EVO2_7B, hidden_size=1024, num_layers=3, num_attention_heads=8, inner_mlp_size=1024,
               hcs_filter_groups=8, hcm_filter_groups=8, hcl_filter_groups=1024, pattern=("hcs", "hcm", "hcl"))
    m = StripedHyena2(cfg, seed=11, device="cuda").to_inference("cuda")
    B, L, n = 64, 160, 15
    ids = torch.randint(0, 512, (B, L + n), device="cuda", generator=torch.Generator(device="cuda").manual_seed(12))
    toks_e, scores_e = m.generate(ids[:, :L], n, forced=ids[:, L:])
    inner = m.blocks[2].filter._decode["inner"]
    assert isinstance(inner, ops.IirStepper) and inner.win is not None
    toks_g, scores_g = m.generate(ids[:, :L], n, forced=ids[:, L:], graph=True)
    assert torch.equal(scores_g, scores_e)
    want = m(ids).float()[:, L - 1:L + n - 1]
    err = (scores_e.float() - want).abs().max() / want.abs().max()
    assert err <= 3e-2, err
    _, scores_p = m.generate(ids[:, :L], n, forced=ids[:, L:], window_state=False)
    assert m.blocks[2].filter._decode["inner"].win is None
    err = (scores_e.float() - scores_p.float()).abs().max() / want.abs().max()
    assert err <= 2e-2, err


def test_recorded_step_then_eager_steps():
    # release() hands ring positions back to the host: eager steps after recorded ones continue the same sequence
    from vortex_amd.model import RecordedDecodeStep
    cfg = dict(EVO2_7B, hidden_size=128, num_layers=4, num_attention_heads=4, inner_mlp_size=256,
               hcs_filter_groups=8, hcm_filter_groups=8, hcl_filter_groups=128)
    m = StripedHyena2(cfg, seed=7, device="cuda").to_inference("cuda")
    L, n = 200, 9
    ids = torch.randint(0, 512, (1, L + n), device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    _, want = m.generate(ids[:, :L], n, forced=ids[:, L:])

    with torch.no_grad():
        ipd = m.initialize_inference_params(max_seqlen=L + n)
        got = [m(ids[:, :L], ipd)[:, -1]]
        rec = None
        for i in range(1, n):
            for p in ipd.values():
                p.seqlen_offset = L if p.seqlen_offset == 0 else p.seqlen_offset + 1
            x = ids[:, L + i - 1:L + i]
            if i == 2:
                rec = RecordedDecodeStep(m, ipd, 1)
            if i == 6:
                rec.release()
                rec = None
            got.append((m(x, ipd) if rec is None else rec(x))[:, -1])
    got = torch.stack(got, 1).float()
    err = (got - want.float()).abs().max() / want.float().abs().max()
    assert err <= 3e-2, err
