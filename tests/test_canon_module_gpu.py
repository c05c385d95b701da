"""The drop-in CanonLayer (HIP kernels) against vectors of the reference's own
CanonLayer (tests/golden/, produced from model/model.py's eager branch) and
against the eager restatement at larger sizes."""
import json
import os
import types

import numpy as np
import pytest
import torch

from helpers import assert_parity, bits, right_padded_mask
from oracle.canon_eager import EagerCanon

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _cases():
    with open(os.path.join(GOLDEN, "canon_layer_cases.json")) as f:
        return json.load(f)["cases"]


def _tensor(arrays, key, dtype):
    a = torch.from_numpy(arrays[key])
    return a.view(torch.bfloat16) if dtype == torch.bfloat16 else a


def make_layer(D, W, w, b, act, dtype, rounding):
    from causal_conv1d.canon import CanonLayer
    cfg = types.SimpleNamespace(canon_kernel=W, canon_bias=b is not None, canon_activation=act)
    layer = CanonLayer(D, cfg, "a", rounding=rounding).to(device=DEV, dtype=dtype)
    with torch.no_grad():
        layer.weight.copy_(w.view(D, 1, W))
        if b is not None:
            layer.bias_param.copy_(b)
    return layer


@pytest.mark.parametrize("rounding", ["eager", "fused"])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_canon_layer_golden_vectors(case, rounding):
    arrays = np.load(os.path.join(GOLDEN, "canon_layer_cases.npz"))
    name, dtype = case["name"], getattr(torch, case["dtype"])
    w = _tensor(arrays, f"{name}/weight", dtype)
    b = _tensor(arrays, f"{name}/bias", dtype) if case["bias"] else None
    layer = make_layer(case["D"], case["W"], w, b, case["activation"], dtype, rounding)
    cache = types.SimpleNamespace()
    with torch.no_grad():
        for i, call in enumerate(case["calls"]):
            key = f"{name}/call{i}"
            x = _tensor(arrays, f"{key}/x", dtype)
            mask = torch.from_numpy(arrays[f"{key}/mask"]).to(DEV) if call["mask"] else None
            out = layer(x.to(DEV), attention_mask=mask, cache=cache if call["cache"] else None,
                        layer_idx=0 if call["cache"] else None)
            want = _tensor(arrays, f"{key}/out", dtype)
            if call["cache"]:
                want_state = _tensor(arrays, f"{key}/state", dtype)
                assert torch.equal(bits(cache.canon_cache_a[0]), bits(want_state)), (name, i, "state")
            if rounding == "eager" and dtype != torch.float32:
                # same rounding points as the reference: bit exact (1 ulp where SiLU's exp differs)
                assert_parity(out, want, exact=not case["activation"], what=f"{name}/call{i}")
            elif dtype == torch.float32:
                assert_parity(out, want, exact=False, what=f"{name}/call{i}", res=x)
            else:
                # single rounding vs the reference's three: within the reference's own bf16 tolerance
                torch.testing.assert_close(out.cpu().float(), want.float(), rtol=5e-3, atol=2e-2)


@pytest.mark.parametrize("site,C", [("a", 640), ("b", 960), ("d", 3456)])
def test_canon_layer_prefill_then_decode_at_model_shapes(site, C):
    """Benchmark shapes of the four call sites: prefill with a padding mask, then 8 decode steps."""
    torch.manual_seed(5)
    B, T = 4, 256
    dtype = torch.bfloat16
    w = (torch.randn(C, 4) * 0.3).to(dtype)
    x = torch.randn(B, T, C).to(dtype)
    mask = right_padded_mask([256, 200, 131, 17], T)
    ref = EagerCanon(w, None, False)
    ref_cache = {}
    want = ref.forward(x, mask, ref_cache, 0)
    layer = make_layer(C, 4, w, None, False, dtype, "eager")
    cache = types.SimpleNamespace()
    with torch.no_grad():
        got = layer(x.to(DEV), attention_mask=mask.to(DEV), cache=cache, layer_idx=3)
        assert_parity(got, want, exact=True, what=f"site {site} prefill")
        state = cache.canon_cache_a[3]
        assert torch.equal(bits(state), bits(ref_cache[0]))
        full_mask = mask
        for step in range(8):
            tok = torch.randn(B, 1, C).to(dtype)
            full_mask = torch.cat([full_mask, torch.tensor([[1], [1], [0], [1]])], dim=1)
            want = ref.forward(tok, full_mask, ref_cache, 0)
            got = layer(tok.to(DEV), attention_mask=full_mask.to(DEV), cache=cache, layer_idx=3)
            assert cache.canon_cache_a[3] is state            # updated in place, same object
            assert torch.equal(bits(state), bits(ref_cache[0])), step
            assert_parity(got, want, exact=False, what=f"site {site} step {step}")


def test_decode_token_as_one_hip_graph():
    """All 72 Canon update launches of one generated token (18 layers x sites a, b, c, d) captured into
    one HIP graph and replayed with eager work and synchronisations in between: every replay must give
    the bits of the eager launches (states are carried in place from replay to replay)."""
    import causal_conv1d as cc
    torch.manual_seed(12)
    B, S, layers = 16, 4, 18
    sites = [("a", 640), ("b", 960), ("c", 640), ("d", 3456)]
    dtype = torch.bfloat16
    weights = {n: (torch.randn(C, 4) * 0.3).to(dtype).to(DEV) for n, C in sites}
    toks = {n: torch.randn(B, C).to(dtype).to(DEV) for n, C in sites}          # static input buffers
    states_g = {(n, l): torch.randn(B, C, S).to(dtype).to(DEV) for n, C in sites for l in range(layers)}
    states_e = {k: v.clone() for k, v in states_g.items()}
    outs_g = {}

    def one_token(states, outs):
        for l in range(layers):
            for n, _ in sites:
                outs[(n, l)] = cc.causal_conv1d_update(toks[n], states[(n, l)], weights[n], residual=True)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_token({k: v.clone() for k, v in states_g.items()}, {})              # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one_token(states_g, outs_g)
    for k in states_g:                    # capture does not run the kernels; start both from the same state
        assert torch.equal(bits(states_g[k]), bits(states_e[k]))
    for replay in range(4):
        for n, C in sites:
            toks[n].copy_(torch.randn(B, C).to(dtype))                          # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        outs_e = {}
        one_token(states_e, outs_e)
        torch.cuda.synchronize()
        for k in states_g:
            assert torch.equal(bits(states_g[k]), bits(states_e[k])), (replay, k)
            assert torch.equal(bits(outs_g[k]), bits(outs_e[k])), (replay, k)


def test_unmodified_model_call_pattern():
    """What the reference's own CanonLayer does around the two package calls on its accelerated branch
    (model/model.py:454-491 prefill, :299-313 decode), spelled out with the package's functions and the
    reference's keywords: mask multiply, transpose to (B, D, T), conv, state = last K masked inputs,
    `x + output`; then `x_token + update(...)` on that state.  Checked against the CPU oracle."""
    import causal_conv1d as cc
    from oracle import canon_oracle as co
    torch.manual_seed(33)
    B, T, D, K = 4, 50, 640, 4
    dtype = torch.bfloat16
    x = torch.randn(B, T, D).to(dtype)
    weight = (torch.randn(D, 1, K) * 0.3).to(dtype)           # the module's parameter shape
    mask = right_padded_mask([50, 31, 4, 17], T)
    for activation in (None, "silu"):
        xg, wg, mg = x.to(DEV), weight.to(DEV), mask.to(DEV)
        masked_x = xg * mg.unsqueeze(-1)
        x_conv = masked_x.transpose(1, 2)
        y_conv = cc.causal_conv1d_fn(x=x_conv, weight=wg.squeeze(1), bias=None, activation=activation, seq_idx=None)
        assert y_conv.stride() == x_conv.stride()
        out = xg + y_conv.transpose(1, 2)
        conv_state = torch.zeros(B, D, K, device=DEV, dtype=dtype)
        conv_state[:, :, :] = x_conv[:, :, -K:]

        xm = (x.float() * mask[:, :, None].float()).to(dtype)
        want_y, want_state = co.conv1d_fwd(xm.transpose(1, 2).contiguous(), weight.squeeze(1), None,
                                           activation=activation, final_state_len=K)
        if activation is None:
            assert torch.equal(bits(y_conv.contiguous()), bits(want_y))
        else:
            assert (y_conv.float().cpu() - want_y.float()).abs().max() <= 2 ** -7 * want_y.float().abs().max()
        assert torch.equal(bits(conv_state), bits(want_state))
        want_out = (x.float() + want_y.transpose(1, 2).float()).to(dtype)      # the eager add rounds once more
        assert (out.float().cpu() - want_out.float()).abs().max() <= 2 ** -6 * want_out.float().abs().max()

        for step in range(3):
            x_token = torch.randn(B, D).to(dtype)
            held = conv_state
            y = cc.causal_conv1d_update(x=x_token.to(DEV), conv_state=conv_state, weight=wg.squeeze(1), bias=None,
                                        activation=activation)
            want = co.conv1d_update(x_token, want_state, weight.squeeze(1), None, activation=activation)
            assert conv_state is held and torch.equal(bits(conv_state), bits(want_state))
            if activation is None:
                assert torch.equal(bits(y), bits(want))
            else:
                assert (y.float().cpu() - want.float()).abs().max() <= 2 ** -7 * want.float().abs().max()


def test_prepared_decode_call_agrees_with_the_checked_path():
    """The decode fast path (a signature seen once is launched from a prepared argument block): second and later
    calls with a mask that grew, a token that is a non-contiguous view, and a trainable bias under autograd give
    what the fully checked path gives, and the table of signatures never grows beyond its limit."""
    import causal_conv1d as cc
    from oracle import canon_oracle as co
    torch.manual_seed(9)
    B, C, dtype = 5, 96, torch.bfloat16
    w = (torch.randn(C, 4) * 0.3).to(dtype)
    b = (torch.randn(C) * 0.1).to(dtype)
    layer = make_layer(C, 4, w, b, False, dtype, "fused")
    cache = types.SimpleNamespace()
    state_ref = torch.zeros(B, C, 8, dtype=dtype)
    with torch.no_grad():
        for step, width in enumerate([3, 4, 9, 9, 17]):           # the mask's length changes from call to call
            wide = torch.randn(B, 3, 2 * C).to(dtype)
            tok = wide[:, 1:2, ::2] if step % 2 else wide[:, 1:2, :C].contiguous()   # strided view / dense token
            mask = torch.ones(B, width, dtype=torch.int64)
            mask[step % B, -1] = 0
            got = layer(tok.to(DEV) if tok.is_contiguous() else wide.to(DEV)[:, 1:2, ::2], attention_mask=mask.to(DEV),
                        cache=cache, layer_idx=0)
            xt = tok[:, 0] * mask[:, -1:].to(dtype)
            want = tok[:, 0] + co.conv1d_update(xt.contiguous(), state_ref, w, b)   # the residual is the unmasked token
            assert torch.equal(bits(cache.canon_cache_a[0]), bits(state_ref)), step
            assert_parity(got[:, 0], want.to(dtype), exact=False, what=f"step {step}", res=tok[:, 0])
    # a frozen weight with a trainable bias takes the autograd path, not the prepared launch
    layer.weight.requires_grad_(False)
    layer.bias_param.requires_grad_(True)
    tok = torch.randn(B, 1, C).to(dtype).to(DEV)
    y = layer(tok, attention_mask=None, cache=types.SimpleNamespace(), layer_idx=0)
    assert y.requires_grad
    y.float().sum().backward()
    assert layer.bias_param.grad is not None and torch.isfinite(layer.bias_param.grad.float()).all()
    # the table keeps its size: new signatures push the oldest ones out
    known = cc._known_updates()
    with torch.no_grad():
        for n in range(cc._KNOWN_UPDATES_MAX + 8):
            x = torch.zeros(1, 2 + 2 * n, dtype=dtype, device=DEV)
            st = torch.zeros(1, 2 + 2 * n, 3, dtype=dtype, device=DEV)
            wt = torch.zeros(2 + 2 * n, 4, dtype=dtype, device=DEV)
            cc.causal_conv1d_update(x, st, wt)
            cc.causal_conv1d_update(x, st, wt)
    assert len(known) == cc._KNOWN_UPDATES_MAX
    torch.cuda.synchronize()
