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


@pytest.mark.parametrize("B,L,seed", cases(1, 12))
def test_se_random(B, L, seed):
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


@pytest.mark.parametrize("B,L,seed", cases(2, 10))
def test_mr_random(B, L, seed):
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


@pytest.mark.parametrize("B,L,seed", cases(3, 10))
def test_li_random(B, L, seed):
    rng = random.Random(seed)
    cplx = rng.random() < 0.5
    dg = rng.choice([1, 2, 4, 8, 16])
    G = rng.randint(1, 3)
    D = G * dg
    if D % 8:
        k = 8 // (D & -D) if (D & -D) < 8 else 1
        D, G = D * k, G * k
    x2, x1, v = O.make_gates(B, D, L, seed=seed)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, 16, seed=seed + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(seed)).bfloat16()
    ref, y32_ref, st_ref = O.li_prefill(x2, x1, v, lp, r, Db)
    out, y32, st = va.hyena_li_fwd(x1.cuda(), x2.cuda(), v.cuda(), lp.cuda(), r.cuda(), Db.cuda(),
                                   want_state=True, want_fp32=True)
    assert rel_err(y32, y32_ref) <= 1e-4, (B, D, L, G, cplx)
    assert rel_err(out, ref) <= 2e-2
    sr = torch.view_as_real(st) if cplx else st
    assert rel_err(sr, torch.view_as_real(st_ref) if cplx else st_ref) <= 1e-4


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
