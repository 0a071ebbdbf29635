"""CPU oracle for the layers around the Hyena operators in a StripedHyena 2 stack.  TEST INFRASTRUCTURE ONLY.

Restates, in plain float32 PyTorch on the CPU, the reference's RMSNorm, gated MLP, block wiring, attention block
and tied unembedding, so that the product's end-to-end stack (bf16, GPU GEMMs) can be compared with something
other than itself.  Only tests/ may import it.  The Hyena operator inside each block is the oracle's own
OracleCascade on OracleEngine (hyena_oracle.py), with the reference's bf16 rounding points; the dense layers
run in float32 on the bf16-rounded weights ("float32 reference of the bf16 stack").

Each function cites the reference lines it follows (paths relative to the reference checkout).  Pins
(tests/test_oracle_stack.py): hand-computed RMSNorm and gated-MLP values, rotary embedding as an explicit 2-D
rotation by position * base^(-2i/d), attention against explicit softmax loops, and the block wiring against
the formulas written out term by term on a one-block stack.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import hyena_oracle as O


def rms_norm(x, scale, eps):
    """vortex/model/layers.py:191-196 (use_flash_rmsnorm False):
    y = x / (||x||_2 * hidden^-1/2 + eps); return scale * y."""
    hidden = x.shape[-1]
    y = x / (x.norm(2, dim=-1, keepdim=True) * hidden ** (-1.0 / 2) + eps)
    return scale * y


def gated_mlp(z, w1, w2, w3, identity_act):
    """vortex/model/layers.py:242-246: l3(act(l1 z) * l2 z); act is GELU (exact, F.gelu's default) on layer 0 and
    the identity on later layers with evo2_style_activations (layers.py:215-218).  Weights [out, in]."""
    z1, z2 = z @ w1.T, z @ w2.T
    a = z1 if identity_act else F.gelu(z1)
    return (a * z2) @ w3.T


def rotary(x, base, offset=0):
    """Non-interleaved rotary embedding over the whole head dimension (vortex/model/rotary.py:19-34 with
    interleaved=False; frequencies base^(-2i/d), vortex/model/rotary.py:422-423).
    x [B, L, H, hd]: pairs (x[i], x[i + hd/2]) rotate by (offset + l) * base^(-2i/hd)."""
    B, L, H, hd = x.shape
    inv = 1.0 / (base ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    t = torch.arange(offset, offset + L, dtype=torch.float32)
    f = torch.outer(t, inv)
    cos = torch.cat([f.cos(), f.cos()], -1)[None, :, None]
    sin = torch.cat([f.sin(), f.sin()], -1)[None, :, None]
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    return x * cos + torch.cat([-x2, x1], -1) * sin


def causal_attention(q, k, v):
    """vortex/model/attention.py:247-283 (the non-flash path): scaled_dot_product_attention, causal, scale
    1/sqrt(hd).  q, k, v [B, L, H, hd] -> [B, L, H, hd]."""
    o = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3),
                                       is_causal=True)
    return o.permute(0, 2, 1, 3)


def attention_block(u, p, num_heads, base, eps, identity_act):
    """vortex/model/model.py:105-122: u = MHA(pre_norm(u)) + u; u = mlp(post_norm(u)) + u, with MHA =
    out_proj(attention(rotary(Wqkv x)))  (vortex/model/attention.py MHA.forward: Wqkv -> "... (three h d)" ->
    rotary on q, k -> inner attention -> out_proj)."""
    B, L, D = u.shape
    hd = D // num_heads
    x = rms_norm(u, p["pre_norm.scale"], eps)
    qkv = (x @ p["Wqkv.weight"].T).view(B, L, 3, num_heads, hd)
    if "Wqkv.bias" in p:
        qkv = qkv + p["Wqkv.bias"].view(3, num_heads, hd)
    q, k, v = rotary(qkv[:, :, 0], base), rotary(qkv[:, :, 1], base), qkv[:, :, 2]
    o = causal_attention(q, k, v).reshape(B, L, D)
    o = o @ p["out_proj.weight"].T
    if "out_proj.bias" in p:
        o = o + p["out_proj.bias"]
    u = o + u
    return gated_mlp(rms_norm(u, p["post_norm.scale"], eps), p["mlp.l1.weight"], p["mlp.l2.weight"],
                     p["mlp.l3.weight"], identity_act) + u


def hyena_block(u, p, cascade, eps, identity_act):
    """vortex/model/model.py:523-575: z = projections(pre_norm(u)); z = filter(z); z_in = out_filter_dense(z) + u;
    y = mlp(post_norm(z_in)) + z_in.  `cascade` is an O.OracleCascade holding the filter's parameters; the
    operator sees and returns bf16 tensors, as every activation of the reference stack is."""
    z = rms_norm(u, p["pre_norm.scale"], eps) @ p["projections.weight"].T
    z, _ = cascade.forward(z.to(torch.bfloat16))
    z = z.float()
    z_in = z @ p["out_filter_dense.weight"].T
    if "out_filter_dense.bias" in p:
        z_in = z_in + p["out_filter_dense.bias"]
    z_in = z_in + u
    return gated_mlp(rms_norm(z_in, p["post_norm.scale"], eps), p["mlp.l1.weight"], p["mlp.l2.weight"],
                     p["mlp.l3.weight"], identity_act) + z_in


class OracleStack:
    """Embedding -> blocks -> RMSNorm -> tied unembedding `x @ E^T` (vortex/model/model.py:693-766,
    vortex/model/layers.py:309-311), float32 on the CPU, from a flat parameter dict named as torch's
    state_dict of the product's stack names them (`blocks.{i}.<sub-name>`).

    cfg keys: hidden_size, num_attention_heads, eps, rotary_emb_base, evo2_style_activations, state_size,
    column_split_hyena, interleave, hcs/hcm filter lengths and hcs/hcm/hcl filter groups; kinds: per block one
    of "hcs", "hcm", "hcl", "attn".
    """

    def __init__(self, cfg, kinds, params):
        self.cfg, self.kinds = cfg, list(kinds)
        f = lambda t: t.detach().cpu().float() if not t.is_complex() else t.detach().cpu()
        self.p = {k: f(v) for k, v in params.items()}

    def block_params(self, i):
        pre = f"blocks.{i}."
        return {k[len(pre):]: v for k, v in self.p.items() if k.startswith(pre)}

    def cascade(self, i, kind):
        cfg, bp = self.cfg, self.block_params(i)
        fp = {k[len("filter."):]: v for k, v in bp.items() if k.startswith("filter.")}
        K = {"hcs": cfg["hcs_filter_length"], "hcm": cfg["hcm_filter_length"], "hcl": None}[kind]
        # the reference's inference model holds every filter parameter except poles and residues in bf16
        # (vortex/model/model.py:1014-1030); the values arrive bf16-rounded and are used as such
        if "D" in fp:
            fp["D"] = fp["D"].to(torch.bfloat16)
        return O.OracleCascade(O.OracleEngine(), fp, cfg["hidden_size"], cfg["num_attention_heads"],
                               cfg[f"{kind}_filter_groups"], layer_idx=i, fir_inner_filter_length=K,
                               column_split_hyena=cfg.get("column_split_hyena", False),
                               interleave=cfg.get("interleave", False), state_size=cfg.get("state_size", 16))

    def forward(self, input_ids, n_blocks=None, return_hidden=False):
        cfg = self.cfg
        x = self.p["embedding.weight"][input_ids.cpu()]
        hidden = []
        for i, kind in enumerate(self.kinds[: n_blocks]):
            ident = bool(cfg.get("evo2_style_activations", False)) and i > 0
            bp = self.block_params(i)
            if kind == "attn":
                x = attention_block(x, bp, cfg["num_attention_heads"], cfg["rotary_emb_base"], cfg["eps"], ident)
            else:
                x = hyena_block(x, bp, self.cascade(i, kind), cfg["eps"], ident)
            hidden.append(x)
        if return_hidden:
            return hidden
        x = rms_norm(x, self.p["norm.scale"], cfg["eps"])
        return x @ self.p["embedding.weight"].T
