"""Gradient oracle of the prefill: torch autograd (CPU, float64) through the
reference's eager formulation.

TEST INFRASTRUCTURE ONLY.  The formulation is the one of the eager CanonLayer
(model/model.py:590-675): ``xm = x * mask``, ``z = conv1d(pad(xm), w, bias,
groups=C)``, ``y = silu(z)`` if activated, ``out = y (+ xm | + x)``; its
gradients are what ``loss.backward()`` of the reference computes
(trainer/base_trainer.py:274).  Everything is evaluated in float64 from the
quantised inputs, so the result is the exact-arithmetic gradient up to 1e-15.

With ``seq_idx`` (packed sequences: the slot of the call signature that the
reference passes as None, model/model.py:465, and that its MPS back end rejects,
causal_conv1d_mps/autograd.py:64-65) a tap contributes only
when its time step carries the same sequence index as the output step, so the
convolution is written as a sum of shifted, gated copies of ``xm``.  That
form is pinned by the tests in two ways: its output against the C oracle of
the packed forward, and its gradients against this same function run without
``seq_idx`` on every sequence cut out on its own.

With ``initial_states`` the zero padding is replaced by their last W-1
entries (``torch.cat`` instead of ``F.pad``); pinned by the tests through the
split property: a block cut in two, the second half continued from the first
half's last inputs, has the gradients of the block convolved in one go.

``update_grads`` does the same for one decode step in the formulation of
the eager module's step (model/model.py:372-398): the window is the last
W-1 state slots and the token, ``out = act(bias + sum_k w[k] * window[k])``
plus the residual, and the new state is the old one shifted left by one with
the token appended.  The loss whose gradient it returns is
``sum(out * dout) + sum(new_state * dstate_out)``, so it covers the gradient
that reaches a step through the state it hands to the next one.  Pinned by
the tests through the prefill: a chain of such steps has the gradients of
``conv1d_grads`` on the same tokens laid out along time.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def conv1d_grads(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], dout: torch.Tensor,
                 mask: Optional[torch.Tensor] = None, activation=None, residual=0,
                 seq_idx: Optional[torch.Tensor] = None, initial_states: Optional[torch.Tensor] = None,
                 dfinal: Optional[torch.Tensor] = None):
    """x, dout logical [B, C, L]; weight [C, W] and bias [C] are first rounded to x.dtype, as the
    forward does.  Returns (dx, dweight, dbias, out) in float64; with ``initial_states`` [B, C, S >= W-1]
    (the inputs before t = 0 instead of the zero padding, unmasked: the chunked continuation of
    model/model.py:647-659) also their gradient as a fifth entry.  ``dfinal`` [B, C, S_out]: a gradient arriving
    through the captured state (the last S_out entries of initial_states ++ xm, zero filled on the left,
    model/model.py:470-489); the loss differentiated is then sum(out * dout) + sum(final * dfinal)."""
    C, W = weight.shape
    x64 = x.detach().cpu().double().requires_grad_(True)
    w64 = weight.detach().cpu().to(x.dtype).double().requires_grad_(True)
    b64 = bias.detach().cpu().to(x.dtype).double().requires_grad_(True) if bias is not None else None
    xm = x64 if mask is None else x64 * mask.detach().cpu().double().unsqueeze(1)
    h64 = None
    if initial_states is not None:
        assert seq_idx is None
        h64 = initial_states.detach().cpu().double().requires_grad_(True)
        z = F.conv1d(torch.cat([h64[:, :, h64.shape[2] - (W - 1):], xm], dim=2), w64.unsqueeze(1), b64, groups=C)
    elif seq_idx is None:
        z = F.conv1d(F.pad(xm, (W - 1, 0)), w64.unsqueeze(1), b64, groups=C)
    else:
        L = x64.shape[2]
        q = seq_idx.detach().cpu().long()
        z = torch.zeros_like(xm) if b64 is None else b64.view(1, C, 1).expand_as(xm).clone()
        for k in range(W):
            back = W - 1 - k                       # tap k reads time step t - back
            if back >= L:
                continue
            keep = (q[:, back:] == q[:, :L - back]).double().unsqueeze(1)          # [B, 1, L - back]
            z = z + F.pad(w64[:, k].view(1, C, 1) * xm[:, :, :L - back] * keep, (back, 0))
    y = F.silu(z) if activation in ("silu", "swish", True, 1) else z
    if residual in (True, 1, "masked"):
        y = y + xm
    elif residual in (2, "unmasked"):
        y = y + x64
    loss = (y * dout.detach().cpu().double()).sum()
    if dfinal is not None:
        assert seq_idx is None
        S_out = dfinal.shape[2]
        hist = xm if h64 is None else torch.cat([h64, xm], dim=2)
        final = F.pad(hist, (S_out, 0))[:, :, -S_out:]
        loss = loss + (final * dfinal.detach().cpu().double()).sum()
    loss.backward()
    if h64 is not None:
        return x64.grad, w64.grad, (b64.grad if b64 is not None else None), y.detach(), h64.grad
    return x64.grad, w64.grad, (b64.grad if b64 is not None else None), y.detach()


def update_grads(x: torch.Tensor, conv_state: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                 dout: torch.Tensor, dstate_out: Optional[torch.Tensor] = None, token_mask: Optional[torch.Tensor] = None,
                 activation=None, residual=0):
    """x, dout [B, C]; conv_state, dstate_out [B, C, S] (the state BEFORE the step); weight [C, W] and
    bias [C] are first rounded to x.dtype.  Returns (dx, dstate, dweight, dbias, out, new_state) in float64."""
    C, W = weight.shape
    x64 = x.detach().cpu().double().requires_grad_(True)
    s64 = conv_state.detach().cpu().double().requires_grad_(True)
    w64 = weight.detach().cpu().to(x.dtype).double().requires_grad_(True)
    b64 = bias.detach().cpu().to(x.dtype).double().requires_grad_(True) if bias is not None else None
    xt = x64 if token_mask is None else x64 * token_mask.detach().cpu().double().unsqueeze(1)
    window = torch.cat([s64[:, :, s64.shape[2] - (W - 1):], xt.unsqueeze(-1)], dim=-1)      # [B, C, W]
    z = (window * w64.unsqueeze(0)).sum(-1)
    if b64 is not None:
        z = z + b64
    y = F.silu(z) if activation in ("silu", "swish", True, 1) else z
    if residual in (True, 1, "masked"):
        y = y + xt
    elif residual in (2, "unmasked"):
        y = y + x64
    new_state = torch.cat([s64[:, :, 1:], xt.unsqueeze(-1)], dim=-1)
    loss = (y * dout.detach().cpu().double()).sum()
    if dstate_out is not None:
        loss = loss + (new_state * dstate_out.detach().cpu().double()).sum()
    loss.backward()
    return (x64.grad, s64.grad if s64.grad is not None else torch.zeros_like(s64), w64.grad,
            b64.grad if b64 is not None else None, y.detach(), new_state.detach())


def update_grads_ext(x: torch.Tensor, conv_state: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                     dout: torch.Tensor, dstate_out: Optional[torch.Tensor] = None, token_mask: Optional[torch.Tensor] = None,
                     activation=None, residual=0, cache_seqlens: Optional[torch.Tensor] = None,
                     conv_state_indices: Optional[torch.Tensor] = None):
    """Gradients of the decode step in upstream's other two state modes, by torch autograd (float64) through the
    step written with gather / scatter:

    cache_seqlens [B]       ring buffer (the reference's update kernel, causal_conv1d.metal:755-775): the token goes
                            to slot p = cache_seqlens % S, tap k < W-1 reads slot (p - (W-1) + k) mod S, the other
                            slots stay.
    conv_state_indices [B]  state pool: entry b uses row conv_state_indices[b] of conv_state [R, C, S]; an index
                            outside [0, R) skips the entry (its output row is zero, no state row changes).

    x, dout [B, C]; conv_state, dstate_out [R, C, S] (R = B without a pool).  Returns
    (dx, dstate, dweight, dbias, out, new_state) in float64, dstate and new_state with conv_state's shape."""
    C, W = weight.shape
    B = x.shape[0]
    R, _, S = conv_state.shape
    x64 = x.detach().cpu().double().requires_grad_(True)
    s64 = conv_state.detach().cpu().double().requires_grad_(True)
    w64 = weight.detach().cpu().to(x.dtype).double().requires_grad_(True)
    b64 = bias.detach().cpu().to(x.dtype).double().requires_grad_(True) if bias is not None else None
    xt = x64 if token_mask is None else x64 * token_mask.detach().cpu().double().unsqueeze(1)
    if conv_state_indices is not None:
        idx = conv_state_indices.detach().cpu().long()
        live = (idx >= 0) & (idx < R)
    else:
        idx = torch.arange(B)
        live = torch.ones(B, dtype=torch.bool)
    rows = s64[idx.clamp(0, R - 1)]                                    # [B, C, S]
    if cache_seqlens is not None:
        p = torch.remainder(cache_seqlens.detach().cpu().long(), S)    # non-negative
        hist_slots = torch.remainder(p[:, None] - (W - 1) + torch.arange(W - 1)[None, :], S)      # [B, W-1]
        write_slot = p
    else:
        hist_slots = (S - (W - 1) + torch.arange(W - 1))[None, :].expand(B, W - 1)
        write_slot = None
    hist = rows.gather(2, hist_slots[:, None, :].expand(B, C, W - 1))
    window = torch.cat([hist, xt.unsqueeze(-1)], dim=-1)               # [B, C, W]
    z = (window * w64.unsqueeze(0)).sum(-1)
    if b64 is not None:
        z = z + b64
    y = F.silu(z) if activation in ("silu", "swish", True, 1) else z
    if residual in (True, 1, "masked"):
        y = y + xt
    elif residual in (2, "unmasked"):
        y = y + x64
    y = y * live[:, None].double()                                      # a skipped entry's output is a constant zero
    if write_slot is not None:
        new_rows = rows.scatter(2, write_slot[:, None, None].expand(B, C, 1), xt.unsqueeze(-1))
    else:
        new_rows = torch.cat([rows[:, :, 1:], xt.unsqueeze(-1)], dim=-1)
    new_state = s64.clone()
    new_state[idx[live]] = new_rows[live]
    loss = (y * dout.detach().cpu().double()).sum()
    if dstate_out is not None:
        loss = loss + (new_state * dstate_out.detach().cpu().double()).sum()
    loss.backward()
    return (x64.grad, s64.grad if s64.grad is not None else torch.zeros_like(s64), w64.grad,
            b64.grad if b64 is not None else None, y.detach(), new_state.detach())
