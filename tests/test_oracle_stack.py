"""Pins the CPU oracle of the layers around the Hyena operators (oracle/stack_oracle.py) with hand-computed
values, explicit loops and structural identities, none of which retypes the oracle's own formulas."""
import math

import pytest
import torch

from oracle import hyena_oracle as O
from oracle import stack_oracle as S


def test_rms_norm_hand_computed():
    # x = (3, 4): ||x|| = 5, hidden^-1/2 = 1/sqrt(2)  ->  y = x / (5/sqrt(2) + eps), then times scale
    x = torch.tensor([[3.0, 4.0], [0.0, 0.0]])
    y = S.rms_norm(x, torch.tensor([2.0, 0.5]), 1e-6)
    d = 5.0 / math.sqrt(2.0) + 1e-6
    assert torch.allclose(y[0], torch.tensor([2.0 * 3.0 / d, 0.5 * 4.0 / d]), atol=1e-7)
    assert y[1].tolist() == [0.0, 0.0]                      # eps keeps the zero row finite
    # a row of ones has ||x|| * hidden^-1/2 = 1: the norm returns the scale itself (up to eps)
    y = S.rms_norm(torch.ones(1, 64), torch.arange(64.0), 0.0)
    assert torch.allclose(y[0], torch.arange(64.0), atol=1e-5)


def test_gated_mlp_hand_computed():
    z = torch.tensor([[1.0, 2.0]])
    w1 = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]])       # l1 z = (1, 2, 3)
    w2 = torch.tensor([[2.0, 0.0], [0.0, -1.0], [1.0, -1.0]])     # l2 z = (2, -2, -1)
    w3 = torch.tensor([[1.0, 1.0, 1.0], [0.0, 1.0, 0.0]])
    assert S.gated_mlp(z, w1, w2, w3, identity_act=True).tolist() == [[-5.0, -4.0]]      # (2, -4, -3) summed / picked
    # exact GELU x * Phi(x): gelu(1) = 0.8413447, gelu(2) = 1.9544997, gelu(3) = 2.9959502
    g = [0.5 * x * (1.0 + math.erf(x / math.sqrt(2.0))) for x in (1.0, 2.0, 3.0)]
    want = [g[0] * 2 - g[1] * 2 - g[2], -2 * g[1]]
    assert torch.allclose(S.gated_mlp(z, w1, w2, w3, identity_act=False), torch.tensor([want]), atol=1e-6)


def test_rotary_is_a_rotation_by_position_times_frequency():
    B, L, H, hd, base = 1, 5, 2, 8, 10000.0
    x = torch.zeros(B, L, H, hd)
    x[..., 1] = 1.0                                   # pair (1, 1 + hd/2) starts at angle 0
    y = S.rotary(x, base, offset=3)
    for l in range(L):
        th = (3 + l) * base ** (-2.0 / hd)            # i = 1 -> exponent -2i/hd
        assert abs(y[0, l, 0, 1].item() - math.cos(th)) < 1e-6 and abs(y[0, l, 0, 1 + hd // 2].item() - math.sin(th)) < 1e-6
        assert y[0, l, 0, [0, 2, 3, 4, 6, 7]].abs().max() == 0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 7, 3, 8, generator=g)
    y = S.rotary(x, base)
    assert torch.equal(y[:, 0], x[:, 0])                                      # position 0: identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)          # rotations preserve the norm
    # relative-position property: <rot(q, m), rot(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, 1, 8, generator=g), torch.randn(1, 1, 1, 8, generator=g)
    d1 = (S.rotary(q, base, 5) * S.rotary(k, base, 2)).sum()
    d2 = (S.rotary(q, base, 13) * S.rotary(k, base, 10)).sum()
    assert abs(d1 - d2) < 1e-4


def test_causal_attention_vs_explicit_softmax_loops():
    g = torch.Generator().manual_seed(1)
    B, L, H, hd = 2, 6, 2, 4
    q, k, v = (torch.randn(B, L, H, hd, generator=g) for _ in range(3))
    o = S.causal_attention(q, k, v)
    for b in range(B):
        for h in range(H):
            for t in range(L):
                s = [sum(q[b, t, h, e].item() * k[b, j, h, e].item() for e in range(hd)) / math.sqrt(hd) for j in range(t + 1)]
                m = max(s)
                w = [math.exp(a - m) for a in s]
                for e in range(hd):
                    want = sum(w[j] * v[b, j, h, e].item() for j in range(t + 1)) / sum(w)
                    assert abs(o[b, t, h, e].item() - want) < 1e-5


def _tiny_params(D, inner, G, K, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    return {"pre_norm.scale": 1 + 0.1 * r(D), "post_norm.scale": 1 + 0.1 * r(D), "projections.weight": r(3 * D, D) / D ** 0.5,
            "out_filter_dense.weight": r(D, D) / D ** 0.5, "out_filter_dense.bias": r(D),
            "mlp.l1.weight": r(inner, D) / D ** 0.5, "mlp.l2.weight": r(inner, D) / D ** 0.5,
            "mlp.l3.weight": r(D, inner) / inner ** 0.5,
            "filter.short_filter_weight": r(3 * D, 1, 3) / 3 ** 0.5, "filter.h": r(G, 1, K) / K ** 0.5}


def test_hyena_block_wiring_by_switching_terms_off():
    # vortex/model/model.py:523-575: two residual branches.  Zeroing a branch's last matrix must leave exactly
    # the other terms; that fixes where each residual is taken from without restating the formula.
    D, inner, G, K, L = 16, 32, 2, 7, 24
    p = _tiny_params(D, inner, G, K, 2)
    u = torch.randn(1, L, D, generator=torch.Generator().manual_seed(3))
    fp = {k[7:]: v for k, v in p.items() if k.startswith("filter.")}
    casc = lambda: O.OracleCascade(O.OracleEngine(), fp, D, 2, G, fir_inner_filter_length=K)
    # (1) MLP off: y = out_filter_dense(filter(projections(pre_norm u))) + u
    p1 = dict(p, **{"mlp.l3.weight": torch.zeros(D, inner)})
    y1 = S.hyena_block(u, p1, casc(), 1e-6, True)
    z = (S.rms_norm(u, p["pre_norm.scale"], 1e-6) @ p["projections.weight"].T).bfloat16()
    f, _ = casc().forward(z)
    want = f.float() @ p["out_filter_dense.weight"].T + p["out_filter_dense.bias"] + u
    assert torch.allclose(y1, want, atol=1e-5)
    # (2) mixer off as well (dense weight and bias zero): the block is the identity
    p2 = dict(p1, **{"out_filter_dense.weight": torch.zeros(D, D), "out_filter_dense.bias": torch.zeros(D)})
    assert torch.equal(S.hyena_block(u, p2, casc(), 1e-6, True), u)
    # (3) mixer off, MLP on: y = mlp(post_norm(u)) + u, the MLP sees the post-mixer stream
    p3 = dict(p, **{"out_filter_dense.weight": torch.zeros(D, D), "out_filter_dense.bias": torch.zeros(D)})
    y3 = S.hyena_block(u, p3, casc(), 1e-6, False)
    want = S.gated_mlp(S.rms_norm(u, p["post_norm.scale"], 1e-6), p["mlp.l1.weight"], p["mlp.l2.weight"],
                       p["mlp.l3.weight"], False) + u
    assert torch.allclose(y3, want, atol=1e-6)


def test_attention_block_wiring_and_first_token():
    # the first token attends to itself only: MHA(x)_0 = out_proj(v_0) whatever q and k are (rotary at position 0
    # is the identity), so block(u)_0 = mlp(post_norm(r)) + r with r = out_proj(v_0) + u_0
    D, H, inner, L = 16, 4, 32, 5
    g = torch.Generator().manual_seed(4)
    r = lambda *s: torch.randn(*s, generator=g)
    p = {"pre_norm.scale": 1 + 0.1 * r(D), "post_norm.scale": 1 + 0.1 * r(D), "Wqkv.weight": r(3 * D, D) / D ** 0.5,
         "out_proj.weight": r(D, D) / D ** 0.5, "out_proj.bias": r(D), "mlp.l1.weight": r(inner, D) / D ** 0.5,
         "mlp.l2.weight": r(inner, D) / D ** 0.5, "mlp.l3.weight": r(D, inner) / inner ** 0.5}
    u = r(1, L, D)
    y = S.attention_block(u, p, H, 10000.0, 1e-6, True)
    x0 = S.rms_norm(u[:, 0], p["pre_norm.scale"], 1e-6)
    v0 = x0 @ p["Wqkv.weight"][2 * D:].T                       # "(three h d)": the last third of the rows is v
    res = v0 @ p["out_proj.weight"].T + p["out_proj.bias"] + u[:, 0]
    want = S.gated_mlp(S.rms_norm(res, p["post_norm.scale"], 1e-6), p["mlp.l1.weight"], p["mlp.l2.weight"],
                       p["mlp.l3.weight"], True) + res
    assert torch.allclose(y[:, 0], want, atol=1e-5)
    # causal: changing the last token changes no earlier output
    u2 = u.clone()
    u2[:, -1] += 1.0
    y2 = S.attention_block(u2, p, H, 10000.0, 1e-6, True)
    assert torch.equal(y2[:, :-1], y[:, :-1]) and not torch.equal(y2[:, -1], y[:, -1])


def test_stack_embedding_and_tied_unembedding():
    # no blocks: logits = rms_norm(E[ids]) @ E^T  (vortex/model/layers.py:309-311: the embedding matrix, transposed)
    E = torch.tensor([[1.0, 0.0], [0.0, 2.0], [3.0, 4.0]])
    st = S.OracleStack(dict(hidden_size=2, eps=0.0), [], {"embedding.weight": E, "norm.scale": torch.ones(2)})
    logits = st.forward(torch.tensor([[2, 0]]))
    n2 = torch.tensor([3.0, 4.0]) / (5.0 / math.sqrt(2.0))
    n0 = torch.tensor([1.0, 0.0]) / (1.0 / math.sqrt(2.0))
    want = torch.stack([torch.stack([n2 @ E[j] for j in range(3)]), torch.stack([n0 @ E[j] for j in range(3)])])[None]
    assert torch.allclose(logits, want, atol=1e-6)
