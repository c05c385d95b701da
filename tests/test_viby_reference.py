"""The harness model (tests/viby_harness.py) against the reference model itself: a 2-layer hidden-64
``VibyForCausalLM`` with Canon A-D was run in the build container (tests/golden/make_viby_tiny_vectors.py, fp32,
CPU, the reference's plain-PyTorch Canon branch) and its parameters, prompt, logits, greedy tokens and conv states
are stored in tests/golden/viby_tiny_model.npz.  Loaded with those parameters the harness must compute the same:
on the CPU with the eager Canon restatement (nearly bit for bit: the same torch operations in the same order)
and on the GPU with the HIP Canon layers (fp32: to the rounding of the GPU's matrix products)."""
import os
import types

import numpy as np
import pytest
import torch

from canon_backends import TorchEagerCanon, hip_factory
from viby_harness import VibyShaped, viby_config

HERE = os.path.dirname(os.path.abspath(__file__))
STEPS = 8


def load_fixture():
    z = np.load(os.path.join(HERE, "golden", "viby_tiny_model.npz"))
    return {k: torch.from_numpy(z[k]) for k in z.files}


def build(fx, make_canon, device):
    cfg = viby_config(hidden_size=64, intermediate_size=96, num_attention_heads=4, num_key_value_heads=1,
                      head_dim=16, num_hidden_layers=2, vocab_size=128, sliding_window=6, max_position_embeddings=64)
    model = VibyShaped(cfg, make_canon(cfg))
    # the reference's parameter names (model/model.py:692-747, 950-961, 1006-1027, 1108-1112, 1160-1168)
    names = {"embed_tokens.weight": "model.embed_tokens.weight", "norm.weight": "model.norm.weight"}
    for i in range(cfg.num_hidden_layers):
        ref, own = f"model.layers.{i}.", f"layers.{i}."
        for n in ("input_layernorm.weight", "post_attention_layernorm.weight", "canon_a.weight", "canon_c.weight"):
            names[own + n] = ref + n
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            names[own + n + ".weight"] = ref + "self_attn." + n + ".weight"
        names[own + "sinks"] = ref + "self_attn.sinks"
        names[own + "canon_b.weight"] = ref + "self_attn.canon_b.weight"
        for n in ("gate_proj", "up_proj", "down_proj"):
            names[own + n + ".weight"] = ref + "mlp." + n + ".weight"
        names[own + "canon_d.weight"] = ref + "mlp.canon_d.weight"
    own_params = dict(model.named_parameters())
    assert set(own_params) == set(names), set(own_params) ^ set(names)
    with torch.no_grad():
        for own, ref in names.items():
            own_params[own].copy_(fx["param/" + ref])
    assert torch.equal(fx["param/lm_head.weight"], fx["param/model.embed_tokens.weight"])      # tied head
    return model.to(device).eval(), cfg


@torch.no_grad()
def run(model, fx, device):
    ids, mask = fx["input_ids"].to(device), fx["attention_mask"].to(device)
    cache = model.new_cache()
    prefill = model.forward(ids, cache, mask, all_positions=True)
    toks, logits = [], []
    last = prefill[:, -1]
    for _ in range(STEPS):
        nxt = last.argmax(dim=-1)
        toks.append(nxt)
        mask = torch.cat([mask, mask.new_ones(mask.shape[0], 1)], dim=1)
        last = model.forward(nxt[:, None], cache, mask)
        logits.append(last)
    return prefill.cpu(), torch.stack(toks, dim=1).cpu(), torch.stack(logits).cpu(), cache


def check(fx, prefill, toks, logits, states, tol):
    assert torch.equal(toks, fx["tokens"]), (toks, fx["tokens"])
    for got, want, what in ((prefill, fx["prefill_logits"], "prefill logits"), (logits, fx["step_logits"], "step logits")):
        err = (got - want).abs().max().item()
        assert err <= tol * want.abs().max().item(), f"{what}: max |diff| {err:.3e}"
    for site in "abcd":
        for layer in range(2):
            got, want = states(site, layer).cpu(), fx[f"state/{site}/{layer}"]
            assert got.shape == want.shape, (site, layer, got.shape, want.shape)
            err = (got - want).abs().max().item()
            assert err <= tol * max(want.abs().max().item(), 1.0), f"state {site}{layer}: max |diff| {err:.3e}"


def test_harness_with_eager_canon_reproduces_the_reference_model_on_the_cpu():
    fx = load_fixture()
    model, _ = build(fx, lambda cfg: (lambda C, name: TorchEagerCanon(C, cfg, name)), "cpu")
    prefill, toks, logits, cache = run(model, fx, "cpu")
    check(fx, prefill, toks, logits, lambda site, layer: cache.eager_states[(site, layer)], tol=2e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("rounding", ["fused", "eager"])
def test_harness_with_hip_canon_reproduces_the_reference_model(rounding):
    fx = load_fixture()
    model, _ = build(fx, lambda cfg: hip_factory(cfg, rounding), "cuda")
    prefill, toks, logits, cache = run(model, fx, "cuda")
    check(fx, prefill, toks, logits, lambda site, layer: getattr(cache, f"canon_cache_{site}")[layer], tol=2e-4)
