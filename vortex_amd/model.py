"""Minimal StripedHyena 2 stack around the gfx950 Hyena operators (random-init, inference only).

Only the Hyena operators (featurizer FIR, Hyena-SE / MR / LI, decode steps) are this package's
kernels; projections, MLP and attention are plain torch matmul / SDPA, as the Evo 2 7B-shaped
end-to-end configuration prescribes.  Formulas follow the reference:
  RMSNorm            vortex/model/layers.py:178-196   y = scale * x / (||x||_2 * D^-1/2 + eps)
  gated MLP          vortex/model/layers.py:199-246   l3(act(l1 z) * l2 z), act = GELU on layer 0,
                                                      identity afterwards (evo2_style_activations)
  Hyena block        vortex/model/model.py:523-575    u + W_o * cascade(W_p * norm(u)), then + MLP
  attention block    vortex/model/model.py:48-122     u + MHA(norm(u)) with rotary embedding, then + MLP
  tied unembedding   vortex/model/layers.py:309-311   logits = x @ E^T
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .cascade import (HyenaCascade, HyenaCascadeFIRInferenceParams, HyenaCascadeIIRInferenceParams,
                      project_sequence_major)

EVO2_7B = dict(
    vocab_size=512, hidden_size=4096, num_layers=32, num_attention_heads=32, inner_mlp_size=11008,
    short_filter_length=3, short_filter_bias=False, state_size=16, eps=1e-6,
    hcs_filter_length=7, hcm_filter_length=128, hcs_filter_groups=256, hcm_filter_groups=256,
    hcl_filter_groups=4096, pattern=("hcs", "hcm", "hcl", "attn"), column_split_hyena=False, interleave=True,
    rotary_emb_base=10000, evo2_style_activations=True,
)


SEQ_MAJOR = "auto"      # "never": every Hyena block hands its operator a channel-last projection


class RMSNorm(nn.Module):
    def __init__(self, hidden, eps):
        super().__init__()
        self.eps, self.hidden = eps, hidden
        self.scale = nn.Parameter(torch.ones(hidden))

    def forward(self, x):
        y = x / (x.norm(2, dim=-1, keepdim=True) * self.hidden ** -0.5 + self.eps)
        return self.scale * y


class GatedMLP(nn.Module):
    def __init__(self, hidden, inner, identity_act, chunk=16384):
        super().__init__()
        self.l1 = nn.Linear(hidden, inner, bias=False)
        self.l2 = nn.Linear(hidden, inner, bias=False)
        self.l3 = nn.Linear(inner, hidden, bias=False)
        self.identity_act, self.chunk = identity_act, chunk

    def _f(self, z):
        a = self.l1(z)
        if not self.identity_act:
            a = F.gelu(a)
        return self.l3(a * self.l2(z))

    def forward(self, z):
        if z.shape[1] <= self.chunk:
            return self._f(z)
        return torch.cat([self._f(z[:, i:i + self.chunk]) for i in range(0, z.shape[1], self.chunk)], dim=1)


def _rotary(x, base, offset=0):
    """x [B, L, H, hd]; non-interleaved rotary embedding over the whole head dimension."""
    B, L, H, hd = x.shape
    inv = 1.0 / (base ** (torch.arange(0, hd, 2, device=x.device, dtype=torch.float32) / hd))
    if isinstance(offset, torch.Tensor):            # position kept on the device (recorded token step)
        t = offset.to(torch.float32) + torch.arange(L, device=x.device, dtype=torch.float32)
    else:
        t = torch.arange(offset, offset + L, device=x.device, dtype=torch.float32)
    f = torch.outer(t, inv)
    cos, sin = f.cos()[None, :, None].to(x.dtype), f.sin()[None, :, None].to(x.dtype)
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1)


class AttentionInferenceParams:
    """Key / value cache of the attention blocks (the role of vortex/model/cache.py:8-28): per layer two
    [B, H, max_seqlen, head_dim] tensors, filled up to seqlen_offset."""

    def __init__(self, max_seqlen):
        self.max_seqlen, self.seqlen_offset = max_seqlen, 0
        self.key_value_memory_dict = {}
        self.offset_dev = None      # int64 [1] device tensor while a recorded token step owns the position


class AttentionBlock(nn.Module):
    def __init__(self, cfg, layer_idx):
        super().__init__()
        D, H = cfg["hidden_size"], cfg["num_attention_heads"]
        self.H, self.base, self.layer_idx = H, cfg["rotary_emb_base"], layer_idx
        self.pre_norm, self.post_norm = RMSNorm(D, cfg["eps"]), RMSNorm(D, cfg["eps"])
        self.Wqkv = nn.Linear(D, 3 * D, bias=False)
        self.out_proj = nn.Linear(D, D, bias=True)
        self.mlp = GatedMLP(D, cfg["inner_mlp_size"], cfg["evo2_style_activations"] and layer_idx > 0)

    def forward(self, u, inference_params=None):
        B, L, D = u.shape
        hd = D // self.H
        qkv = self.Wqkv(self.pre_norm(u)).view(B, L, 3, self.H, hd)
        cached = inference_params is not None and self.layer_idx in inference_params.key_value_memory_dict
        on_device = cached and inference_params.offset_dev is not None
        off = inference_params.offset_dev if on_device else (inference_params.seqlen_offset if cached else 0)
        q, k = _rotary(qkv[:, :, 0], self.base, off).transpose(1, 2), _rotary(qkv[:, :, 1], self.base, off).transpose(1, 2)
        v = qkv[:, :, 2].transpose(1, 2)                                    # [B, H, L, hd]
        if inference_params is not None and not cached:
            # zero-filled: the recorded token step reads every row (masked), and 0 * garbage could be NaN
            kc = k.new_zeros(B, self.H, inference_params.max_seqlen, hd)
            inference_params.key_value_memory_dict[self.layer_idx] = (kc, torch.zeros_like(kc))
        if inference_params is not None:
            kc, vc = inference_params.key_value_memory_dict[self.layer_idx]
            if on_device:
                kc.index_copy_(2, off, k)
                vc.index_copy_(2, off, v)
            else:
                kc[:, :, off:off + L], vc[:, :, off:off + L] = k, v
        if cached and L == 1:
            # one query per head: two batched matrix-vector products over the cache rows seen so far.  A recorded
            # step has fixed shapes, so it reads the whole cache and masks the rows past the position.
            if not on_device:
                kc, vc = kc[:, :, :off + 1], vc[:, :, :off + 1]
            s = torch.matmul(q, kc.transpose(2, 3)).float() * hd ** -0.5         # [B, H, 1, S]
            if on_device:
                s = s.masked_fill(torch.arange(kc.shape[2], device=u.device) > off, float("-inf"))
            o = torch.matmul(torch.softmax(s, dim=-1).to(vc.dtype), vc)
        else:
            if cached:                  # a longer continuation: its queries see the cache and, causally, themselves
                kk, vv = kc[:, :, :off + L], vc[:, :, :off + L]
                mask = torch.ones(L, off + L, dtype=torch.bool, device=u.device).tril(off)
                o = F.scaled_dot_product_attention(q, kk, vv, attn_mask=mask)
            else:
                o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        u = self.out_proj(o.transpose(1, 2).reshape(B, L, D)) + u
        return self.mlp(self.post_norm(u)) + u, None


class HyenaBlock(nn.Module):
    def __init__(self, cfg, layer_idx, kind):
        super().__init__()
        D = cfg["hidden_size"]
        self.pre_norm, self.post_norm = RMSNorm(D, cfg["eps"]), RMSNorm(D, cfg["eps"])
        self.projections = nn.Linear(D, 3 * D, bias=False)
        groups = cfg[f"{kind}_filter_groups"]
        K = {"hcs": cfg["hcs_filter_length"], "hcm": cfg["hcm_filter_length"], "hcl": None}[kind]
        self.filter = HyenaCascade(cfg, layer_idx, hyena_filter_groups=groups, fir_inner_filter_length=K)
        self.kind = kind
        self.out_filter_dense = nn.Linear(D, D, bias=True)
        self.mlp = GatedMLP(D, cfg["inner_mlp_size"], cfg["evo2_style_activations"] and layer_idx > 0)

    def forward(self, u, inference_params=None):
        xn = self.pre_norm(u)
        B, L = xn.shape[0], xn.shape[1]
        # Prefill of a Hyena-LI layer: the projection GEMM writes its product transposed, [B, 3D, L] with the samples
        # contiguous, which the layer then reads once (featurizer, gates and scan in one launch).  The values are
        # those of self.projections(xn), handed over as the [B, L, 3D] view of that memory.  One plain 2-D product per
        # batch element: torch.matmul on the broadcast pair takes twice as long (16.6 against 8.9 ms at L = 131072).
        # Hyena-SE / MR layers keep the channel-last projection: their sequence-major kernels are 7-10 % faster on long
        # prompts, which the slower transposed GEMMs around them (+0.4 ms each at L = 131072) take back.
        if SEQ_MAJOR != "never" and self.kind == "hcl" and L > 1 and L % 8 == 0:
            z = project_sequence_major(self.projections.weight, xn)
        else:
            z = self.projections(xn)
        z, _ = self.filter(z, inference_params=inference_params)
        if B == 1 and L > 1 and z.stride(1) == 1 and z.stride(2) == L:
            # the operator's output is the [B, L, D] view of [B, D, L] memory: the transposed operand goes to the GEMM as it is
            o = torch.addmm(self.out_filter_dense.bias, z[0], self.out_filter_dense.weight.t()).unsqueeze(0)
        else:
            o = self.out_filter_dense(z)
        z_in = o + u
        return self.mlp(self.post_norm(z_in)) + z_in, None


class StripedHyena2(nn.Module):
    """Embedding -> [SE, MR, LI, attention] x N/4 -> RMSNorm -> tied unembedding."""

    def __init__(self, cfg=None, seed=0, device=None):
        super().__init__()
        cfg = dict(EVO2_7B if cfg is None else cfg)
        self.cfg = cfg
        D = cfg["hidden_size"]
        with torch.device(device if device is not None else "cpu"):
            self.embedding = nn.Embedding(cfg["vocab_size"], D)
            pat = cfg["pattern"]
            self.kinds = [pat[i % len(pat)] for i in range(cfg["num_layers"])]
            self.blocks = nn.ModuleList(
                AttentionBlock(cfg, i) if k == "attn" else HyenaBlock(cfg, i, k) for i, k in enumerate(self.kinds))
            self.norm = RMSNorm(D, cfg["eps"])
        self.reset_parameters(seed)

    @torch.no_grad()
    def reset_parameters(self, seed=0):
        dev = self.embedding.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            if name.endswith("scale"):
                p.fill_(1.0)
            elif name.endswith("log_poles"):        # real, stable poles (vortex parametrisation)
                p.copy_(-(0.01 + 0.5 * torch.rand(p.shape, generator=g, device=dev)))
            elif name.endswith(".h"):
                p.copy_(torch.randn(p.shape, generator=g, device=dev) / math.sqrt(p.shape[-1]))
            elif name.endswith("short_filter_weight"):
                p.copy_(torch.randn(p.shape, generator=g, device=dev) / math.sqrt(p.shape[-1]))
            elif name.endswith("residues"):
                p.copy_(torch.randn(p.shape, generator=g, device=dev) / 4.0)
            elif name.endswith(".D") or name.endswith("bias"):
                p.zero_()
            else:
                p.copy_(0.02 * torch.randn(p.shape, generator=g, device=dev))

    def to_inference(self, device):
        """bf16 everywhere except the modal parameters (vortex/model/model.py:1014-1030)."""
        self.to(device)
        for name, p in self.named_parameters():
            if not (name.endswith("log_poles") or name.endswith("residues")):
                p.data = p.data.to(torch.bfloat16)
        return self.eval()

    def initialize_inference_params(self, max_seqlen=8192):
        """vortex/model/model.py:796-830: one cache object per operator family."""
        return {"hcl": HyenaCascadeIIRInferenceParams(), "hcm": HyenaCascadeFIRInferenceParams(),
                "hcs": HyenaCascadeFIRInferenceParams(), "mha": AttentionInferenceParams(max_seqlen)}

    @torch.no_grad()
    def forward(self, input_ids, inference_params_dict=None):
        x = self.embedding(input_ids)
        for kind, block in zip(self.kinds, self.blocks):
            ip = None if inference_params_dict is None else inference_params_dict["mha" if kind == "attn" else kind]
            x, _ = block(x, inference_params=ip)
        x = self.norm(x)
        return x @ self.embedding.weight.T

    @torch.no_grad()
    def generate(self, input_ids, num_tokens, forced=None, graph=False, window_state=True):
        """Greedy cached generation in the order of vortex/model/generation.py:164-229: one prefill over the
        prompt, then one token per forward with the caches' seqlen_offset advanced first.  `forced`
        [B, num_tokens] replaces the sampled tokens (teacher forcing).  graph=True replays the token step as a
        recorded HIP graph from the fifth token on (RecordedDecodeStep).  window_state: the Hyena-LI layers keep their
        modal states in windows of four tokens where that form exists (HyenaCascade.window_decode_state); this loop
        owns its caches and nobody reads them between tokens.  Returns (tokens, logits of every step)."""
        B, L = input_ids.shape
        ipd = self.initialize_inference_params(max_seqlen=L + num_tokens)
        for kind, block in zip(self.kinds, self.blocks):
            if kind != "attn":
                block.filter.window_decode_state = window_state
        x, toks, scores, rec = input_ids, [], [], None
        for i in range(num_tokens):
            if i > 0:
                x = x[:, -1:]
                for p in ipd.values():
                    p.seqlen_offset = L if p.seqlen_offset == 0 else p.seqlen_offset + 1
            if graph and i == 5:                    # four eager token steps have bound the decode kernels and opened
                rec = RecordedDecodeStep(self, ipd, B)   # every window of the windowed modal steps by now
            logits = (self.forward(x, ipd) if rec is None else rec(x))[:, -1]
            new = logits.argmax(-1) if forced is None else forced[:, i]
            toks.append(new)
            scores.append(logits)
            x = new[:, None]
        if rec is not None:
            rec.release()
        return torch.stack(toks, 1), torch.stack(scores, 1)


class RecordedDecodeStep:
    """The cached one-token forward of a StripedHyena2 recorded once as a HIP graph and replayed per token.

    A replay cannot change scalar kernel arguments, so everything that moves from token to token lives in device
    memory while this object is in use: the ring positions of the FIR caches (ops.RingClock, read by the step
    kernels, advanced by one launch at the end of the step) and the attention position (an int64 tensor the
    recorded step increments).  Needs caches that are full (prompt at least as long as the longest FIR filter)
    and one eager token step beforehand, which binds the decode kernels to the caches.  release() hands the
    positions back to the host-side fields so that eager steps can follow."""

    def __init__(self, model, ipd, batch):
        self.model, self.ipd = model, ipd
        dev = model.embedding.weight.device
        rings = []
        for kind, block in zip(model.kinds, model.blocks):
            if kind == "attn":
                continue
            ip, i = ipd[kind], block.filter.layer_idx
            if i not in ip.fir_state_dict:
                raise RuntimeError("run the prefill and one token step before recording")
            rings.append(ip.fir_state_dict[i])
            if block.filter.fir_inner_filter_length:
                rings.append(ip.fir_inner_state_dict[i])
            inner = (block.filter._decode or {}).get("inner")
            if isinstance(inner, ops.IirStepper) and inner.win is not None:     # a windowed modal step counts tokens too
                if inner.warm < inner.period:
                    raise RuntimeError(f"step {inner.period} tokens eagerly before recording (windowed modal state)")
                rings.append(inner)
        if any(getattr(r, "valid", r.R) < r.R for r in rings if isinstance(r, ops.FirRing)):
            raise NotImplementedError("a cache is still filling up (prompt shorter than a filter): step eagerly")
        mha = ipd["mha"]
        self.clock = ops.RingClock(rings)
        mha.offset_dev = torch.tensor([mha.seqlen_offset], dtype=torch.int64, device=dev)
        self.tokens = torch.zeros(batch, 1, dtype=torch.int64, device=dev)
        self.steps = 0
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = model.forward(self.tokens, ipd)
            self.clock.advance()
            mha.offset_dev.add_(1)

    def __call__(self, tokens):
        self.tokens.copy_(tokens)
        self.graph.replay()
        self.steps += 1
        return self.logits.clone()                  # the recorded step writes the same buffer every time

    def release(self):
        self.clock.release()
        self.ipd["mha"].offset_dev = None
