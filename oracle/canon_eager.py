"""Module-level oracle: the eager (plain torch ops) Canon layer, restated.

TEST INFRASTRUCTURE ONLY.  It follows the fall-back branch of the reference's
``CanonLayer`` (model/model.py:587-675 for a block of tokens, :262-289 and
:367-398 for the single-token step), including its rounding points: every
torch op rounds to the tensor dtype, so in bf16 the conv output, the SiLU
output and the residual sum are each rounded.

The cache is a plain ``dict`` keyed by whatever the caller likes (the
reference hangs per-layer lists on the HF cache object, model/model.py:227-241;
only the stored tensor matters here).
"""
from __future__ import annotations

from typing import Hashable, MutableMapping, Optional

import torch
import torch.nn.functional as F

STATE_LEN_MIN = 8  # model/model.py:286 and :626 -> max(8, kernel_size)


class EagerCanon:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 activation: bool = False):
        # the parameter is [C, 1, W] in the reference (model/model.py:212)
        self.weight = weight if weight.dim() == 3 else weight.unsqueeze(1)
        self.bias = bias
        self.activation = bool(activation)
        self.channels, _, self.width = self.weight.shape

    # -- single token, model/model.py:372-398 --------------------------------
    def _step(self, token: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        W = self.width
        state.copy_(torch.roll(state, shifts=-1, dims=-1))
        state[:, :, -1] = token
        taps = self.weight.squeeze(1)
        y = (state[:, :, -W:] * taps.unsqueeze(0)).sum(dim=-1)
        if self.bias is not None:
            y = self.bias.unsqueeze(0).expand(token.shape[0], -1).clone() + y
        else:
            y = torch.zeros_like(token) + y
        return F.silu(y) if self.activation else y

    def forward(self, x: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                cache: Optional[MutableMapping] = None, key: Hashable = None) -> torch.Tensor:
        B, T, D = x.shape
        W = self.width
        state = cache.get(key) if cache is not None else None

        if cache is not None and T == 1:  # model/model.py:417-422, 274-289, 367-370
            token = x[:, 0]
            if (attention_mask is not None and attention_mask.dim() == 2
                    and attention_mask.shape[0] == B):
                token = token * attention_mask[:, -1].unsqueeze(-1).to(token.dtype)
            if state is None:
                state = torch.zeros(B, D, max(STATE_LEN_MIN, W), dtype=x.dtype, device=x.device)
            y = self._step(token, state).unsqueeze(1)
            cache[key] = state
            return x + y  # the residual is the unmasked token here

        # model/model.py:590-602: only these two mask shapes are honoured
        if attention_mask is not None and attention_mask.dim() == 2:
            if tuple(attention_mask.shape) == (B, T):
                x = x * attention_mask.unsqueeze(-1)
            elif attention_mask.size(0) == B and attention_mask.size(1) >= T:
                x = x * attention_mask[:, -T:].unsqueeze(-1)
        xc = x.transpose(1, 2)  # [B, D, T] view

        have_history = state is not None and W > 1  # model/model.py:607-620
        if have_history:
            conv_in = torch.cat([state[:, :, -(W - 1):], xc], dim=-1)
        else:
            conv_in = F.pad(xc, (W - 1, 0))

        if cache is not None:  # model/model.py:623-661
            if state is None:
                state = torch.zeros(B, D, max(STATE_LEN_MIN, W), dtype=x.dtype, device=x.device)
            S = state.size(-1)
            if not have_history:      # start of a sequence: right aligned, zeros on the left
                if T <= S:
                    state[:, :, -T:] = xc
                else:
                    state[:, :, :] = xc[:, :, -S:]
            elif T >= S:              # continuation that overwrites the whole window
                state[:, :, :] = xc[:, :, -S:]
            else:                     # continuation: slide left by T, append
                state.copy_(torch.roll(state, shifts=-T, dims=-1))
                state[:, :, -T:] = xc
            cache[key] = state

        y = F.conv1d(conv_in, self.weight, bias=self.bias, groups=self.channels)
        if self.activation:
            y = F.silu(y)
        return x + y.transpose(1, 2)  # the residual is the masked input here
