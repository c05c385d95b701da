"""``CanonLayer`` on the fused HIP kernels: one launch per call.

Same constructor, parameters and ``forward`` signature as the reference's
``CanonLayer`` (``model/model.py:201-225`` and ``:400-406``), so it can replace
that class inside ``VibyBlock`` / ``Attention`` / ``FeedForward``
(``model/model.py:765-794, 961-971, 1021-1027, 1049-1055``):

* parameters ``weight [C, 1, K]`` and ``bias_param [C] | None`` with the same
  names and initialisation (``model/model.py:212-225``), so checkpoints load;
* per-layer conv states live on the cache object as the list attribute
  ``canon_cache_<name>`` (``model/model.py:227-241``).

What one call does, and which reference branch defines it.  The reference has
three branches whose residual/state conventions differ; this module follows
the plain-PyTorch branch, which is the one that runs wherever no accelerated
package is installed and the one the parity vectors come from:

* block of T tokens (``model/model.py:587-675``): ``xm = x * mask``;
  ``out = xm + act(conv(xm) + bias)``; with a cache, the last
  ``state_len = max(8, K)`` masked inputs are captured right-aligned (history,
  if a state already exists, is taken from it: chunked continuation);
* single token with a cache (``model/model.py:262-289, 367-398``): the token is
  multiplied by the last mask column, the state is shifted left and the token
  appended, ``out = x + act(conv + bias)`` (residual on the unmasked token).

``rounding='eager'`` reproduces that branch's intermediate bf16/fp16 roundings
bit for bit; the default ``'fused'`` rounds once.

``forward_parts`` takes the channel ranges as separate tensors (q, k, v for
Canon-B, gate and up for Canon-D) and returns one output per part, so the
``torch.cat`` / ``split`` around the layer (``model/model.py:772-789, 962-971``)
is not needed; the state on the cache is the same single tensor either way.

Training: a block call without a cache is differentiable (fused backward
kernel), and so are a prefill with state capture and the single-token step
of ``forward`` (its own backward kernel; the cache tensor then carries the
graph from step to step) and the chunked continuation of ``forward``
(``initial_states``; the captured state is differentiable, so the graph
continues across chunk boundaries and into the decode steps).  The cached paths of ``forward_parts`` are
inference paths: run them under ``torch.no_grad()`` /
``torch.inference_mode()``.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn

from . import (_canon_decode_step, causal_conv1d_fn, causal_conv1d_fn_parts, causal_conv1d_update,
               causal_conv1d_update_parts)

STATE_LEN_MIN = 8  # model/model.py:286, :626


class CanonLayer(nn.Module):
    def __init__(self, hidden_size: int, config, name: str, rounding: str = "fused"):
        super().__init__()
        self.name = name
        self.hidden_size = hidden_size
        self.kernel_size = config.canon_kernel
        self.bias = config.canon_bias
        self.activation = config.canon_activation
        self.rounding = rounding
        self.weight = nn.Parameter(torch.randn(hidden_size, 1, self.kernel_size))
        if self.bias:
            self.bias_param = nn.Parameter(torch.zeros(hidden_size))
        else:
            self.register_parameter("bias_param", None)
        self._taps_view = None   # (address of the weight, its (C, K) view): see _taps

    def reset_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias_param is not None:
            fan_in = self.weight.size(1) * self.weight.size(2)
            bound = 1.0 / math.sqrt(fan_in) if fan_in > 0 else 0.0
            nn.init.uniform_(self.bias_param, -bound, bound)

    # -- cache plumbing: a list per site hung on the cache object --------------
    def _slot(self, cache):
        attr = f"canon_cache_{self.name}"
        if not hasattr(cache, attr):
            setattr(cache, attr, [None] * getattr(cache, "_max_layers", 256))
        return getattr(cache, attr)

    def _state_len(self) -> int:
        return max(STATE_LEN_MIN, self.kernel_size)

    @staticmethod
    def _block_mask(attention_mask, B: int, T: int):
        # the mask columns of the T tokens of this call (model/model.py:589-600)
        if attention_mask is not None and attention_mask.dim() == 2:
            if tuple(attention_mask.shape) == (B, T):
                return attention_mask
            if attention_mask.size(0) == B and attention_mask.size(1) >= T:
                return attention_mask[:, -T:]
        return None

    def _taps(self) -> torch.Tensor:
        """``weight`` as (C, K).  Outside autograd the view is kept (it stays valid while the parameter keeps its
        storage; in-place updates show through it), which saves the decode step a tensor operation."""
        w = self.weight
        if torch.is_grad_enabled() and w.requires_grad:
            return w.squeeze(1)
        kept = self._taps_view
        if kept is None or kept[0] != w.data_ptr() or kept[1].device != w.device or kept[1].dtype != w.dtype:
            kept = (w.data_ptr(), w.detach().squeeze(1))
            self._taps_view = kept
        return kept[1]

    def forward(self, x: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                cache=None, layer_idx: Optional[int] = None) -> torch.Tensor:
        B, T, D = x.shape
        use_cache = cache is not None and layer_idx is not None
        act = "silu" if self.activation else None

        if use_cache and T == 1:
            slot = self._slot(cache)
            state = slot[layer_idx]
            token_mask = None          # the whole mask here: its last column scales the token (model/model.py:277-282)
            if attention_mask is not None and attention_mask.dim() == 2 and attention_mask.shape[0] == B:
                token_mask = attention_mask
            if state is None:
                state = torch.zeros(B, D, self._state_len(), dtype=x.dtype, device=x.device)
                slot[layer_idx] = state
            if torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad or state.requires_grad
                                            or (self.bias_param is not None and self.bias_param.requires_grad)):
                y = causal_conv1d_update(x[:, 0], state, self._taps(), self.bias_param, activation=act,
                                         token_mask=token_mask[:, -1] if token_mask is not None else None,
                                         residual="unmasked", rounding=self.rounding)
                return y.unsqueeze(1)
            return _canon_decode_step(x, state, self._taps(), self.bias_param, token_mask, act, self.rounding)

        state = self._slot(cache)[layer_idx] if use_cache else None
        taps = self._taps()

        mask = self._block_mask(attention_mask, B, T)

        new_state = None
        if use_cache:
            new_state = torch.empty(B, D, state.size(-1) if state is not None else self._state_len(),
                                    dtype=x.dtype, device=x.device)
        history = state if (state is not None and self.kernel_size > 1) else None
        out = causal_conv1d_fn(x.transpose(1, 2), taps, self.bias_param, activation=act,
                               initial_states=history, final_states_out=new_state,
                               attention_mask=mask, residual="masked", rounding=self.rounding)
        if use_cache:
            out, new_state = out
            if state is not None:
                state.copy_(new_state)   # the cached tensor object stays the same
            else:
                state = new_state
            self._slot(cache)[layer_idx] = state
        return out.transpose(1, 2)

    def forward_parts(self, xs, attention_mask: Optional[torch.Tensor] = None,
                      cache=None, layer_idx: Optional[int] = None):
        """``forward(torch.cat(xs, dim=-1)).split(...)`` without the cat: ``xs`` are (B, T, D_i) tensors
        whose widths add up to ``hidden_size``; returns a tuple of (B, T, D_i) outputs."""
        xs = tuple(xs)
        B, T = xs[0].shape[:2]
        D = sum(x.shape[2] for x in xs)
        if D != self.hidden_size:
            raise ValueError(f"the parts hold {D} channels, the layer has {self.hidden_size}")
        use_cache = cache is not None and layer_idx is not None
        state = self._slot(cache)[layer_idx] if use_cache else None
        taps = self._taps()
        act = "silu" if self.activation else None

        if use_cache and T == 1:
            token_mask = None
            if attention_mask is not None and attention_mask.dim() == 2 and attention_mask.shape[0] == B:
                token_mask = attention_mask[:, -1]
            if state is None:
                state = torch.zeros(B, D, self._state_len(), dtype=xs[0].dtype, device=xs[0].device)
            ys = causal_conv1d_update_parts([x[:, 0] for x in xs], state, taps, self.bias_param, activation=act,
                                            token_mask=token_mask, residual="unmasked", rounding=self.rounding)
            self._slot(cache)[layer_idx] = state
            return tuple(y.unsqueeze(1) for y in ys)

        mask = self._block_mask(attention_mask, B, T)
        new_state = None
        if use_cache:
            new_state = torch.empty(B, D, state.size(-1) if state is not None else self._state_len(),
                                    dtype=xs[0].dtype, device=xs[0].device)
        history = state if (state is not None and self.kernel_size > 1) else None
        outs = causal_conv1d_fn_parts([x.transpose(1, 2) for x in xs], taps, self.bias_param, activation=act,
                                      initial_states=history, final_states_out=new_state,
                                      attention_mask=mask, residual="masked", rounding=self.rounding)
        if use_cache:
            outs, new_state = outs
            if state is not None:
                state.copy_(new_state)
            else:
                state = new_state
            self._slot(cache)[layer_idx] = state
        return tuple(o.transpose(1, 2) for o in outs)


class GraphedDecodeStep:
    """One decode step of a model built on ``CanonLayer``, captured once as a HIP graph and replayed per token.

    A decode loop is host bound outside a graph: the 72 update launches of an 18-layer model take 2-4 us each on
    the device and 8-12 us each to issue from Python.  The reference removes that cost by compiling the model with
    ``mode="reduce-overhead"`` (``eval_model.py:157``), which is graph capture; this is the same thing done by hand
    around a step function the caller owns.

    ``step``  a callable without arguments that runs ONE decode step: it may read and write only tensors that exist
              before the capture (a token buffer, a position tensor, preallocated K / V buffers, the conv states the
              Canon layers keep on ``cache``) and must not create tensors that outlive it other than through those.
              The K / V history therefore has to live in buffers of the final length (an attention that concatenates
              a growing history cannot be replayed); the Canon states already have that form.
    ``cache`` the cache object the ``CanonLayer``s hang their ``canon_cache_<name>`` lists on; the prefill must have
              run, so that every state tensor exists.
    ``state`` further tensors the step modifies (token, position, K / V buffers, ...).

    The constructor runs the step once on a side stream as a warm-up (loads code objects, fills the allocator's
    pools and the prepared-call table of the decode launches), puts every conv state and every tensor in ``state``
    back to what it was, and captures.  ``replay()`` then advances the model by one token; its results equal the
    step launched kernel by kernel bit for bit.  No ``hipMemsetAsync`` is recorded by the Canon launches (the
    library clears with fill kernels).
    """

    SITES = ("a", "b", "c", "d")

    def __init__(self, step, cache, state=()):
        lists = [getattr(cache, f"canon_cache_{name}") for name in self.SITES if hasattr(cache, f"canon_cache_{name}")]
        carried = [t for states in lists for t in states if t is not None] + list(state)
        with torch.no_grad():
            saved = [t.clone() for t in carried]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            for t, old in zip(carried, saved):
                t.copy_(old)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                step()
            # the capture only records: nothing ran, the states are still the restored ones

    def replay(self) -> None:
        self.graph.replay()
