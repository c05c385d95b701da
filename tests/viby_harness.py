"""A Viby-shaped decoder used to drive the Canon path the way the real model does.

It restates the forward pass of the reference model (model/model.py): pre-norm blocks (:1006-1068)
with Canon-A on the normed attention input (C = hidden), Canon-B on cat(q, k, v) (:765-794,
C = q + k + v), Canon-C on the normed MLP input, Canon-D on cat(gate, up) (:961-971,
C = 2 * intermediate), one conv state per (layer, site) on the cache object, rotate-half rotary
embedding from a precomputed table (:118-125, 182-196), attention written out as scores + masks +
softmax with a per-head sink column (:796-925: causal mask, key-padding mask from the attention mask,
sliding window of `sliding_window` keys except in every sixth layer, :1029-1030), SwiGLU (:973-976),
tied embedding / lm_head (:1168), greedy decoding that feeds one token per step with the
whole-history attention mask (:1308-1327).  tests/test_viby_reference.py checks it against logits,
tokens and conv states recorded from the reference model itself at a small configuration.
"""
from __future__ import annotations

import math
import types
from typing import Callable, Optional

import torch
import torch.nn.functional as F
from torch import nn


def viby_config(**over):
    cfg = dict(hidden_size=640, num_hidden_layers=18, num_attention_heads=4, num_key_value_heads=1,
               head_dim=160, intermediate_size=1728, vocab_size=25600, rms_norm_eps=1e-6,
               rope_theta=1e6, sliding_window=512, max_position_embeddings=32768,
               canon_kernel=4, canon_bias=False, canon_activation=False)
    cfg.update(over)
    return types.SimpleNamespace(**cfg)


def rope_tables(dim: int, end: int, theta: float):
    # model/model.py:118-125
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: (dim // 2)].float() / dim))
    t = torch.arange(end, device=freqs.device)
    freqs = torch.outer(t, freqs).float()
    return torch.cat([torch.cos(freqs), torch.cos(freqs)], dim=-1), torch.cat([torch.sin(freqs), torch.sin(freqs)], dim=-1)


def rotate_half(x):
    return torch.cat((-x[..., x.shape[-1] // 2:], x[..., : x.shape[-1] // 2]), dim=-1)


def apply_rope(q, k, cos, sin):
    # q, k [B, T, H, d]; cos, sin [T, d]  (model/model.py:182-196)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def sink_attention(q, key, value, sinks, blocked, scale):
    """softmax(q k^T * scale with `blocked` entries at the dtype's minimum, plus one sink logit per head)
    applied to value, the sink column dropped after the softmax (model/model.py:823-925).
    q [B, H, Tq, d]; key, value [B, H, Tk, d]; blocked: bool, broadcastable to [B, H, Tq, Tk];
    scale: 1 / sqrt(d) as a tensor of q's dtype (the reference builds it per call, :826)."""
    B, H, Tq, d = q.shape
    scores = torch.einsum("bhqd,bhkd->bhqk", q, key) * scale
    scores = scores.masked_fill(blocked, torch.finfo(scores.dtype).min)
    sink = sinks.view(1, H, 1, 1).to(scores.dtype).expand(B, -1, Tq, 1)
    weights = F.softmax(torch.cat([scores, sink], dim=-1), dim=-1)[..., :-1]
    return torch.einsum("bhqk,bhkd->bhqd", weights, value)


class Block(nn.Module):
    def __init__(self, cfg, make_canon: Callable[[int, str], nn.Module], parts: bool = False):
        super().__init__()
        self.parts = parts
        H, hd = cfg.hidden_size, cfg.head_dim
        self.nq, self.nkv, self.hd = cfg.num_attention_heads, cfg.num_key_value_heads, hd
        self.window = cfg.sliding_window
        self.input_layernorm = nn.RMSNorm(H, eps=cfg.rms_norm_eps)
        self.post_attention_layernorm = nn.RMSNorm(H, eps=cfg.rms_norm_eps)
        self.q_proj = nn.Linear(H, self.nq * hd, bias=False)
        self.k_proj = nn.Linear(H, self.nkv * hd, bias=False)
        self.v_proj = nn.Linear(H, self.nkv * hd, bias=False)
        self.o_proj = nn.Linear(self.nq * hd, H, bias=False)
        self.sinks = nn.Parameter(torch.zeros(self.nq))
        # a buffer, so that it follows the model's dtype and no tensor is created inside a captured step
        self.register_buffer("attn_scale", torch.tensor(1.0 / math.sqrt(hd)), persistent=False)
        self.gate_proj = nn.Linear(H, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(H, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, H, bias=False)
        self.canon_a = make_canon(H, "a")
        self.canon_b = make_canon((self.nq + 2 * self.nkv) * hd, "b")
        self.canon_c = make_canon(H, "c")
        self.canon_d = make_canon(2 * cfg.intermediate_size, "d")

    def forward(self, h, layer_idx, cache, mask, pos0, rope):
        B, T, _ = h.shape
        x = self.canon_a(self.input_layernorm(h), attention_mask=mask, cache=cache, layer_idx=layer_idx)
        if self.parts:      # the projections go to the Canon layer where they are (no cat, no split)
            q, k, v = self.canon_b.forward_parts((self.q_proj(x), self.k_proj(x), self.v_proj(x)),
                                                 attention_mask=mask, cache=cache, layer_idx=layer_idx)
        else:               # model/model.py:772-789
            qkv = torch.cat([self.q_proj(x), self.k_proj(x), self.v_proj(x)], dim=-1)
            qkv = self.canon_b(qkv, attention_mask=mask, cache=cache, layer_idx=layer_idx)
            q, k, v = qkv.split([self.nq * self.hd, self.nkv * self.hd, self.nkv * self.hd], dim=-1)
        q = q.reshape(B, T, self.nq, self.hd)
        k = k.reshape(B, T, self.nkv, self.hd)
        v = v.reshape(B, T, self.nkv, self.hd).transpose(1, 2)
        rep = self.nq // self.nkv
        win = 0 if (layer_idx + 1) % 6 == 0 else self.window            # model/model.py:1029-1030
        cos_t, sin_t = rope
        dev = h.device
        if getattr(cache, "static_kv", None) is not None:
            # decode step over preallocated K / V (shapes never change, so the step can be captured as a HIP
            # graph): the position lives in a device tensor, the new row is written in place, and attention
            # runs over the whole buffer with the rows beyond the position blocked
            pos = cache.pos_t + torch.arange(T, device=dev)
            q, k = apply_rope(q, k, cos_t.index_select(0, pos), sin_t.index_select(0, pos))
            q, k = q.transpose(1, 2), k.transpose(1, 2)
            K, V = cache.static_kv[layer_idx]
            K.index_copy_(2, pos, k)
            V.index_copy_(2, pos, v)
            k_abs = torch.arange(K.shape[2], device=dev)[None, :]
            q_abs = pos[:, None]
            blocked = k_abs > q_abs
            if win > 0:
                blocked = blocked | (k_abs < q_abs - win)
            att = sink_attention(q, K.repeat_interleave(rep, dim=1), V.repeat_interleave(rep, dim=1), self.sinks, blocked, self.attn_scale)
        else:
            q, k = apply_rope(q, k, cos_t[pos0: pos0 + T], sin_t[pos0: pos0 + T])
            q, k = q.transpose(1, 2), k.transpose(1, 2)
            if cache.kv[layer_idx] is not None:
                pk, pv = cache.kv[layer_idx]
                k, v = torch.cat([pk, k], dim=2), torch.cat([pv, v], dim=2)
            cache.kv[layer_idx] = (k, v)
            Tk = k.shape[2]
            past = Tk - T
            blocked = torch.triu(torch.ones((T, Tk), device=dev, dtype=torch.bool), diagonal=1 + past)
            if mask is not None:         # key padding, model/model.py:848-884 (the mask covers the whole history)
                am = mask
                if am.size(1) < Tk:
                    am = torch.cat([am, torch.ones((am.size(0), Tk - am.size(1)), dtype=am.dtype, device=dev)], dim=1)
                elif am.size(1) > Tk:
                    am = am[:, -Tk:]
                blocked = blocked | (am == 0)[:, None, None, :]
            if win > 0:
                q_abs = torch.arange(T, device=dev) + past
                k_abs = torch.arange(Tk, device=dev)
                blocked = blocked | ~(k_abs[None, :] >= (q_abs[:, None] - win))
            att = sink_attention(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), self.sinks, blocked, self.attn_scale)
        h = h + self.o_proj(att.transpose(1, 2).contiguous().view(B, T, self.nq * self.hd))
        x = self.canon_c(self.post_attention_layernorm(h), attention_mask=mask, cache=cache, layer_idx=layer_idx)
        gate, up = self.gate_proj(x), self.up_proj(x)
        if self.parts:
            gate, up = self.canon_d.forward_parts((gate, up), attention_mask=mask, cache=cache, layer_idx=layer_idx)
        else:               # model/model.py:962-971
            gu = self.canon_d(torch.cat([gate, up], dim=-1), attention_mask=mask, cache=cache, layer_idx=layer_idx)
            gate, up = gu[..., : gate.shape[-1]], gu[..., gate.shape[-1]:]
        return h + self.down_proj(F.silu(gate) * up)


class DecodeCache:
    """What the layers hang their per-layer state on: kv[i] = (K, V), the Canon layers' canon_cache_<name>
    lists (model/model.py:227-241 does the same on the HF cache object).  A plain class, so that attribute
    reads and writes trace under torch.compile."""

    def __init__(self, n_layers: int):
        self._max_layers = n_layers
        self.kv = [None] * n_layers
        self.seen = 0


class VibyShaped(nn.Module):
    def __init__(self, cfg, make_canon, parts: bool = False):
        super().__init__()
        self.cfg = cfg
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList(Block(cfg, make_canon, parts) for _ in range(cfg.num_hidden_layers))
        self.norm = nn.RMSNorm(cfg.hidden_size, eps=cfg.rms_norm_eps)
        # the rotary table is a buffer of the model: it takes the model's dtype with it (model/model.py:1111-1112)
        cos, sin = rope_tables(cfg.head_dim, cfg.max_position_embeddings, cfg.rope_theta)
        self.register_buffer("freqs_cos", cos, persistent=False)
        self.register_buffer("freqs_sin", sin, persistent=False)

    def new_cache(self):
        return DecodeCache(self.cfg.num_hidden_layers)

    def forward(self, ids, cache, mask, all_positions: bool = False):
        h = self.embed_tokens(ids)
        rope = (self.freqs_cos, self.freqs_sin)
        for i, layer in enumerate(self.layers):
            h = layer(h, i, cache, mask, cache.seen, rope)
        cache.seen += ids.shape[1]
        last = self.norm(h if all_positions else h[:, -1])
        return F.linear(last, self.embed_tokens.weight).float()   # tied head (the last position unless asked)

    @torch.no_grad()
    def generate(self, ids, steps, forced: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        """Prefill + `steps` greedy tokens.  With `forced` [B, steps] those tokens are fed instead of
        the argmax (teacher forcing), so two back ends see identical inputs.  `mask`: the prompt's attention
        mask (all ones by default).  Returns (tokens [B, steps], logits [steps, B, V] of every step incl. the
        prefill's, cache)."""
        cache = self.new_cache()
        B, T = ids.shape
        if mask is None:
            mask = torch.ones(B, T, dtype=torch.int64, device=ids.device)
        logits = [self.forward(ids, cache, mask)]
        toks = []
        for s in range(steps):
            nxt = logits[-1].argmax(dim=-1) if forced is None else forced[:, s]
            toks.append(nxt)
            mask = torch.cat([mask, mask.new_ones(B, 1)], dim=1)
            if s + 1 < steps:
                logits.append(self.forward(nxt[:, None], cache, mask))
        return torch.stack(toks, dim=1), torch.stack(logits), cache


@torch.no_grad()
def generate_graphed(model: VibyShaped, ids: torch.Tensor, steps: int, capture=True, compile_kwargs=None):
    """Prefill eagerly, then ONE captured HIP graph per generated token (all layers: 72 Canon update launches,
    projections, attention over a preallocated KV buffer, head, argmax, feeding the token back), replayed
    steps-1 times without any host work in between.  With capture=False the same step function is called
    eagerly instead (same kernels, launched one by one): the reference the replays must match bit for bit.
    With capture="compile" the step function goes through torch.compile(fullgraph=True, **compile_kwargs)
    instead (what eval_model.py:157 does to the reference model).
    Returns (tokens [B, steps], logits [steps, B, V])."""
    dev = ids.device
    B, T = ids.shape
    n = model.cfg.num_hidden_layers
    cache = model.new_cache()
    mask = torch.ones(B, T, dtype=torch.int64, device=dev)
    logits0 = model.forward(ids, cache, mask)
    # move the prefill's K / V into buffers of the final length
    cache.static_kv = []
    for k, v in cache.kv:
        K = torch.zeros(k.shape[0], k.shape[1], T + steps, k.shape[3], dtype=k.dtype, device=dev)
        V = torch.zeros_like(K)
        K[:, :, :T].copy_(k)
        V[:, :, :T].copy_(v)
        cache.static_kv.append((K, V))
    cache.kv = [None] * n
    cache.pos_t = torch.tensor([T], device=dev)
    tok = logits0.argmax(dim=-1)[:, None].clone()       # static input of the step
    one = torch.ones(B, 1, dtype=torch.int64, device=dev)  # mask column of the new token
    out_logits = torch.empty_like(logits0)

    def step():
        lg = model.forward(tok, cache, one)
        out_logits.copy_(lg)
        tok.copy_(lg.argmax(dim=-1)[:, None])
        cache.pos_t.add_(1)

    tok0 = tok.clone()
    graph = None
    if capture == "compile":
        step = torch.compile(step, fullgraph=True, **(compile_kwargs or {}))
    elif capture:
        # the package's helper: warm-up on a side stream, every carried state put back, capture
        from causal_conv1d.canon import GraphedDecodeStep
        # (the K / V row the warm-up writes at position T is written again, with the same values, by the first replay)
        graph = GraphedDecodeStep(step, cache, state=[tok, cache.pos_t, out_logits])
    toks, logits = [tok0[:, 0].clone()], [logits0]
    for _ in range(steps - 1):
        if graph is not None:
            graph.replay()
        else:
            step()
        logits.append(out_logits.clone())
        toks.append(tok[:, 0].clone())
    torch.cuda.synchronize()
    return torch.stack(toks, dim=1), torch.stack(logits)


def init_weights(model: nn.Module, seed: int, dtype, device) -> nn.Module:
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("canon_a.weight") or ".canon_" in name:
                if name.endswith("weight"):
                    # kaiming-uniform(a=sqrt 5) over fan_in = K, as CanonLayer.reset_parameters
                    bound = 1.0 / (p.shape[-1] ** 0.5)
                    p.copy_((torch.rand(p.shape, generator=g) * 2 - 1) * bound)
                else:
                    p.zero_()
            elif name.endswith("sinks"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.5)
            elif p.dim() == 1:
                p.fill_(1.0)
            else:
                p.copy_(torch.randn(p.shape, generator=g) * 0.02)
    return model.to(device=device, dtype=dtype)
