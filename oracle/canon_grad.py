"""Gradient oracle of the prefill: torch autograd (CPU, float64) through the
reference's eager formulation.

TEST INFRASTRUCTURE ONLY.  The formulation is the one of the eager CanonLayer
(model/model.py:590-675): ``xm = x * mask``, ``z = conv1d(pad(xm), w, bias,
groups=C)``, ``y = silu(z)`` if activated, ``out = y (+ xm | + x)``; its
gradients are what ``loss.backward()`` of the reference computes
(trainer/base_trainer.py:274).  Everything is evaluated in float64 from the
quantised inputs, so the result is the exact-arithmetic gradient up to 1e-15.

With ``seq_idx`` (packed sequences, the varlen contract of
causal_conv1d_mps/causal_conv1d_interface.py:253-261) a tap contributes only
when its time step carries the same sequence index as the output step, so the
convolution is written as a sum of shifted, gated copies of ``xm``.  That
form is pinned by the tests in two ways: its output against the C oracle of
the packed forward, and its gradients against this same function run without
``seq_idx`` on every sequence cut out on its own.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def conv1d_grads(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], dout: torch.Tensor,
                 mask: Optional[torch.Tensor] = None, activation=None, residual=0,
                 seq_idx: Optional[torch.Tensor] = None
                 ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
    """x, dout logical [B, C, L]; weight [C, W] and bias [C] are first rounded to x.dtype, as the
    forward does.  Returns (dx, dweight, dbias, out) in float64."""
    C, W = weight.shape
    x64 = x.detach().cpu().double().requires_grad_(True)
    w64 = weight.detach().cpu().to(x.dtype).double().requires_grad_(True)
    b64 = bias.detach().cpu().to(x.dtype).double().requires_grad_(True) if bias is not None else None
    xm = x64 if mask is None else x64 * mask.detach().cpu().double().unsqueeze(1)
    if seq_idx is None:
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
    y.backward(dout.detach().cpu().double())
    return x64.grad, w64.grad, (b64.grad if b64 is not None else None), y.detach()
