"""Writes ``viby_tiny_model.npz``: a small random ``VibyForCausalLM`` of the reference (2 layers, hidden 64,
Canon A-D) together with what it computes: logits of a right-padded prompt at every position, eight greedy
decode steps through the cache (tokens and logits) and the conv states of all Canon layers at the end.

Run in the build container only (it imports the reference from ``/root/reference``, which does not exist
anywhere else):

    python tests/golden/make_viby_tiny_vectors.py

The reference runs its plain-PyTorch Canon branch here (neither accelerated package is installed) in fp32
on the CPU.  tests/test_viby_reference.py loads the arrays into the test harness (tests/viby_harness.py)
and requires the same numbers, which pins the harness -- block order, the four Canon call sites and their
channel order, cache plumbing, attention with window / sinks / padding, greedy loop -- to the model itself.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

REF = "/root/reference/model/model.py"
HERE = os.path.dirname(os.path.abspath(__file__))

CONFIG = dict(hidden_size=64, intermediate_size=96, num_attention_heads=4, num_key_value_heads=1,
              num_hidden_layers=2, vocab_size=128, sliding_window=6, max_position_embeddings=64,
              canon_set="ABCD", canon_kernel=4, canon_bias=False, canon_activation=False)
STEPS = 8


def load_reference():
    spec = importlib.util.spec_from_file_location("viby_reference_model", REF)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = mod
    spec.loader.exec_module(mod)
    assert not mod.HAS_CAUSAL_CONV1D_CUDA and not mod.HAS_CAUSAL_CONV1D_MPS
    return mod


def main():
    ref = load_reference()
    torch.manual_seed(2024)
    model = ref.VibyForCausalLM(ref.VibyConfig(**CONFIG)).float().eval()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("sinks"):
                p.copy_(torch.randn(p.shape) * 0.5)           # zeros at construction: make them count
            elif name.endswith("layernorm.weight") or name.endswith("norm.weight"):
                p.copy_(1.0 + 0.1 * torch.randn(p.shape))
    B, T = 3, 14
    g = torch.Generator().manual_seed(7)
    ids = torch.randint(0, CONFIG["vocab_size"], (B, T), generator=g)
    mask = torch.ones(B, T, dtype=torch.int64)
    mask[1, 11:] = 0                                           # right padded prompts
    mask[2, 5:] = 0
    arrays = {"input_ids": ids.numpy(), "attention_mask": mask.numpy()}
    for name, p in model.state_dict().items():
        arrays["param/" + name] = p.detach().numpy().copy()

    with torch.no_grad():
        out = model(input_ids=ids, attention_mask=mask, use_cache=True)
        cache = out.past_key_values
        arrays["prefill_logits"] = out.logits.numpy().copy()          # [B, T, V]
        toks, step_logits = [], []
        logits = out.logits[:, -1]
        for _ in range(STEPS):
            nxt = logits.argmax(dim=-1)
            toks.append(nxt)
            mask = torch.cat([mask, mask.new_ones(B, 1)], dim=1)
            out = model(input_ids=nxt[:, None], attention_mask=mask, past_key_values=cache, use_cache=True)
            logits = out.logits[:, -1]
            step_logits.append(logits)
        arrays["tokens"] = torch.stack(toks, dim=1).numpy()            # [B, STEPS]
        arrays["step_logits"] = torch.stack(step_logits).numpy()       # [STEPS, B, V]: after feeding token s
    for site in "abcd":
        states = getattr(cache, f"canon_cache_{site}")
        for layer in range(CONFIG["num_hidden_layers"]):
            arrays[f"state/{site}/{layer}"] = states[layer].numpy().copy()   # [B, C, 8]
    path = os.path.join(HERE, "viby_tiny_model.npz")
    np.savez_compressed(path, **arrays)
    print("wrote", path, os.path.getsize(path), "bytes;", len(arrays), "arrays; torch", torch.__version__)
    print("tokens", arrays["tokens"].tolist())


if __name__ == "__main__":
    main()
