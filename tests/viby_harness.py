"""A Viby-shaped decoder used only to drive the Canon path the way the real model does.

It reproduces what fixes the shapes and the order of the Canon calls
(reference: model/model.py): pre-norm blocks (:1006-1068) with Canon-A on the
normed attention input (C = hidden), Canon-B on cat(q, k, v) (:765-794,
C = q + k + v), Canon-C on the normed MLP input, Canon-D on cat(gate, up)
(:961-971, C = 2 * intermediate), one conv state per (layer, site) on the cache
object, tied embedding / lm_head, greedy decoding that feeds one token per step
with the whole-history attention mask (:1308-1327).

Everything that is NOT the Canon path is deliberately plain (causal softmax
attention with grouped KV heads and rotary embedding, SwiGLU, RMSNorm): the
harness compares Canon back ends against each other inside an otherwise
identical network, it does not claim parity with the reference's attention.
"""
from __future__ import annotations

import types
from typing import Callable, Optional

import torch
import torch.nn.functional as F
from torch import nn


def viby_config(**over):
    cfg = dict(hidden_size=640, num_hidden_layers=18, num_attention_heads=4, num_key_value_heads=1,
               head_dim=160, intermediate_size=1728, vocab_size=25600, rms_norm_eps=1e-6,
               rope_theta=1e6, canon_kernel=4, canon_bias=False, canon_activation=False)
    cfg.update(over)
    return types.SimpleNamespace(**cfg)


def rotary(x: torch.Tensor, pos: torch.Tensor, theta: float) -> torch.Tensor:
    # x [B, H, T, d], pos [T]
    d = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=x.device, dtype=torch.float32) / d))
    ang = pos.to(torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos()[None, None], ang.sin()[None, None]
    x1, x2 = x[..., 0::2].float(), x[..., 1::2].float()
    out = torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).flatten(-2)
    return out.to(x.dtype)


class Block(nn.Module):
    def __init__(self, cfg, make_canon: Callable[[int, str], nn.Module], parts: bool = False):
        super().__init__()
        self.parts = parts
        H, hd = cfg.hidden_size, cfg.head_dim
        self.nq, self.nkv, self.hd, self.theta = cfg.num_attention_heads, cfg.num_key_value_heads, hd, cfg.rope_theta
        self.input_layernorm = nn.RMSNorm(H, eps=cfg.rms_norm_eps)
        self.post_attention_layernorm = nn.RMSNorm(H, eps=cfg.rms_norm_eps)
        self.q_proj = nn.Linear(H, self.nq * hd, bias=False)
        self.k_proj = nn.Linear(H, self.nkv * hd, bias=False)
        self.v_proj = nn.Linear(H, self.nkv * hd, bias=False)
        self.o_proj = nn.Linear(self.nq * hd, H, bias=False)
        self.gate_proj = nn.Linear(H, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(H, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, H, bias=False)
        self.canon_a = make_canon(H, "a")
        self.canon_b = make_canon((self.nq + 2 * self.nkv) * hd, "b")
        self.canon_c = make_canon(H, "c")
        self.canon_d = make_canon(2 * cfg.intermediate_size, "d")

    def forward(self, h, layer_idx, cache, mask, pos0):
        B, T, _ = h.shape
        x = self.canon_a(self.input_layernorm(h), attention_mask=mask, cache=cache, layer_idx=layer_idx)
        if self.parts:      # the projections go to the Canon layer where they are (no cat, no split)
            q, k, v = self.canon_b.forward_parts((self.q_proj(x), self.k_proj(x), self.v_proj(x)),
                                                 attention_mask=mask, cache=cache, layer_idx=layer_idx)
        else:               # model/model.py:772-789
            qkv = torch.cat([self.q_proj(x), self.k_proj(x), self.v_proj(x)], dim=-1)
            qkv = self.canon_b(qkv, attention_mask=mask, cache=cache, layer_idx=layer_idx)
            q, k, v = qkv.split([self.nq * self.hd, self.nkv * self.hd, self.nkv * self.hd], dim=-1)
        q = q.reshape(B, T, self.nq, self.hd).transpose(1, 2)
        k = k.reshape(B, T, self.nkv, self.hd).transpose(1, 2)
        v = v.reshape(B, T, self.nkv, self.hd).transpose(1, 2)
        rep = self.nq // self.nkv
        if getattr(cache, "static_kv", None) is not None:
            # decode step over preallocated K / V (shapes never change, so the step can be captured as a HIP
            # graph): the position lives in a device tensor, the new row is written in place, and attention
            # runs over the whole buffer with the rows beyond the position masked out
            pos = cache.pos_t + torch.arange(T, device=h.device)
            q, k = rotary(q, pos, self.theta), rotary(k, pos, self.theta)
            K, V = cache.static_kv[layer_idx]
            K.index_copy_(2, pos, k)
            V.index_copy_(2, pos, v)
            seen = torch.arange(K.shape[2], device=h.device)[None, None, None, :] <= cache.pos_t
            att = F.scaled_dot_product_attention(q, K.repeat_interleave(rep, dim=1), V.repeat_interleave(rep, dim=1),
                                                 attn_mask=seen)
        else:
            pos = torch.arange(pos0, pos0 + T, device=h.device)
            q, k = rotary(q, pos, self.theta), rotary(k, pos, self.theta)
            if cache.kv[layer_idx] is not None:
                pk, pv = cache.kv[layer_idx]
                k, v = torch.cat([pk, k], dim=2), torch.cat([pv, v], dim=2)
            cache.kv[layer_idx] = (k, v)
            att = F.scaled_dot_product_attention(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1),
                                                 is_causal=(T > 1))
        h = h + self.o_proj(att.transpose(1, 2).reshape(B, T, self.nq * self.hd))
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

    def new_cache(self):
        return DecodeCache(self.cfg.num_hidden_layers)

    def forward(self, ids, cache, mask):
        h = self.embed_tokens(ids)
        for i, layer in enumerate(self.layers):
            h = layer(h, i, cache, mask, cache.seen)
        cache.seen += ids.shape[1]
        last = self.norm(h[:, -1])
        return F.linear(last, self.embed_tokens.weight).float()   # tied head, last position only

    @torch.no_grad()
    def generate(self, ids, steps, forced: Optional[torch.Tensor] = None):
        """Prefill + `steps` greedy tokens.  With `forced` [B, steps] those tokens are fed instead of
        the argmax (teacher forcing), so two back ends see identical inputs.  Returns
        (tokens [B, steps], logits [steps, B, V] of every step incl. the prefill's, cache)."""
        cache = self.new_cache()
        B, T = ids.shape
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

    # warm-up on a side stream (library handles, allocator), then put every carried state back
    sites = [name for name in ("a", "b", "c", "d") if hasattr(cache, f"canon_cache_{name}")]
    saved = {name: [t.clone() for t in getattr(cache, f"canon_cache_{name}")] for name in sites}
    tok0 = tok.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for name in sites:
        for t, old in zip(getattr(cache, f"canon_cache_{name}"), saved[name]):
            t.copy_(old)
    tok.copy_(tok0)
    cache.pos_t.fill_(T)

    graph = None
    if capture == "compile":
        step = torch.compile(step, fullgraph=True, **(compile_kwargs or {}))
    elif capture:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
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
            elif p.dim() == 1:
                p.fill_(1.0)
            else:
                p.copy_(torch.randn(p.shape, generator=g) * 0.02)
    return model.to(device=device, dtype=dtype)
