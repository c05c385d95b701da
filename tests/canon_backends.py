"""Canon back ends the harness model (tests/viby_harness.py) can be built with."""
import torch
from torch import nn

from oracle import canon_oracle as co
from oracle.canon_eager import EagerCanon


class TorchEagerCanon(nn.Module):
    """The eager restatement (plain torch ops).  host=False: on whatever device the input lives on.
    host=True: on the CPU whatever the model's device (the layer's input is copied to the host and its output
    back), i.e. the arithmetic of the reference's own CPU path inside a model that otherwise runs on the GPU."""

    def __init__(self, C, cfg, name, host=False):
        super().__init__()
        self.name, self.host = name, host
        self.weight = nn.Parameter(torch.randn(C, 1, cfg.canon_kernel))
        self.act = cfg.canon_activation

    def forward(self, x, attention_mask=None, cache=None, layer_idx=None):
        store = cache.__dict__.setdefault("eager_states", {})
        if not self.host:
            return EagerCanon(self.weight, None, self.act).forward(x, attention_mask, store, (self.name, layer_idx))
        mask = attention_mask.cpu() if attention_mask is not None else None
        y = EagerCanon(self.weight.detach().cpu(), None, self.act).forward(x.detach().cpu(), mask, store, (self.name, layer_idx))
        return y.to(x.device)


class OracleCanon(nn.Module):
    """The C oracle on the host (eager rounding points), called with the semantics of the eager CanonLayer."""

    def __init__(self, C, cfg, name, round_mode):
        super().__init__()
        self.name, self.K, self.round_mode = name, cfg.canon_kernel, round_mode
        self.weight = nn.Parameter(torch.randn(C, 1, cfg.canon_kernel))

    def forward(self, x, attention_mask=None, cache=None, layer_idx=None):
        store = cache.__dict__.setdefault("oracle_states", {})
        key = (self.name, layer_idx)
        xc, w = x.detach().cpu(), self.weight.detach().cpu().squeeze(1)
        B, T, D = xc.shape
        if T == 1 and key in store:
            tok = xc[:, 0]
            xt = (tok * attention_mask[:, -1].cpu().unsqueeze(-1).to(tok.dtype)) if attention_mask is not None else tok
            y = co.conv1d_update(xt.contiguous(), store[key], w, None, round_mode=1)
            return (tok + y).unsqueeze(1).to(x.device)     # residual on the unmasked token, rounded
        mask = attention_mask.cpu() if attention_mask is not None else None
        out, fs = co.conv1d_fwd(xc.transpose(1, 2), w, None, mask=mask, final_state_len=max(8, self.K),
                                residual=1, round_mode=1)
        store[key] = fs
        return out.transpose(1, 2).contiguous().to(x.device)


class NoCanon(nn.Module):
    """The Canon layer switched off."""

    def forward(self, x, attention_mask=None, cache=None, layer_idx=None):
        return x


def hip_factory(cfg, rounding):
    from causal_conv1d.canon import CanonLayer
    return lambda C, name: CanonLayer(C, cfg, name, rounding=rounding)
