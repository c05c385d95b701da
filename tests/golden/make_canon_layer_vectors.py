"""Writes ``canon_layer_cases.npz`` + ``canon_layer_cases.json``: golden vectors
of the reference's own ``CanonLayer`` (eager CPU branch).

Run in the build container only (it imports the reference from
``/root/reference``, which does not exist anywhere else):

    python tests/golden/make_canon_layer_vectors.py

Each case is a short script of calls on one layer sharing one cache object:
block prefill with / without padding mask, masks longer than the block, state
capture for blocks shorter / equal / longer than the 8-slot state, chunked
continuation (roll path and overwrite path) and single-token steps.  The
committed fixtures pin the control flow that ``oracle/canon_eager.py``
restates; the arithmetic itself is pinned elsewhere against torch's conv1d.
"""
import importlib.util
import json
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/model/model.py"
HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference():
    spec = importlib.util.spec_from_file_location("viby_reference_model", REF)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = mod
    spec.loader.exec_module(mod)
    assert not mod.HAS_CAUSAL_CONV1D_CUDA and not mod.HAS_CAUSAL_CONV1D_MPS
    return mod


def to_np(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().copy()
    return t.contiguous().numpy().copy()


def right_padded_mask(B, T, lens):
    m = torch.zeros(B, T, dtype=torch.int64)
    for b, n in enumerate(lens):
        m[b, :n] = 1
    return m


def main():
    ref = load_reference()
    torch.manual_seed(1234)
    arrays = {}
    manifest = []

    # (name, dtype, D, W, bias, activation, calls); a call is (T, mask spec, use_cache)
    # mask spec: None | ("exact", lens) | ("longer", extra, lens) | ("ones_step",)
    specs = [
        ("fp32_plain", torch.float32, 8, 4, False, False,
         [(12, None, False)]),
        ("fp32_bias_silu_mask", torch.float32, 8, 4, True, True,
         [(16, ("exact", [16, 9]), False)]),
        ("fp32_mask_longer", torch.float32, 8, 4, False, False,
         [(6, ("longer", 5, [11, 7]), False)]),
        ("fp32_cache_long_then_steps", torch.float32, 8, 4, True, False,
         [(13, ("exact", [13, 10]), True), (1, ("step", [14, 10]), True),
          (1, ("step", [15, 10]), True), (1, None, True)]),
        ("fp32_cache_short_then_chunks", torch.float32, 8, 4, False, True,
         [(3, None, True), (2, None, True), (9, None, True), (8, None, True), (1, None, True)]),
        ("fp32_cache_exact8", torch.float32, 8, 4, False, False,
         [(8, None, True), (5, ("exact", [5, 2]), True)]),
        ("fp32_step_from_empty", torch.float32, 8, 4, True, True,
         [(1, None, True), (1, None, True), (1, None, True), (1, None, True), (1, None, True)]),
        ("fp32_width3", torch.float32, 8, 3, True, False,
         [(10, ("exact", [10, 4]), True), (1, None, True), (4, None, True)]),
        ("fp32_width2", torch.float32, 8, 2, False, True,
         [(7, None, True), (1, None, True)]),
        ("bf16_bias_mask", torch.bfloat16, 16, 4, True, False,
         [(20, ("exact", [20, 12]), True), (1, None, True), (1, None, True)]),
        ("bf16_silu", torch.bfloat16, 16, 4, False, True,
         [(17, None, True), (1, None, True), (6, None, True)]),
    ]

    for name, dtype, D, W, has_bias, act, calls in specs:
        cfg = types.SimpleNamespace(canon_kernel=W, canon_bias=has_bias, canon_activation=act)
        layer = ref.CanonLayer(D, cfg, "a")
        with torch.no_grad():
            layer.weight.copy_(torch.randn(D, 1, W) * 0.5)
            if has_bias:
                layer.bias_param.copy_(torch.randn(D) * 0.1)
        layer = layer.to(dtype)
        arrays[f"{name}/weight"] = to_np(layer.weight.detach())
        if has_bias:
            arrays[f"{name}/bias"] = to_np(layer.bias_param.detach())
        cache = types.SimpleNamespace()
        B = 2
        entry = {"name": name, "dtype": str(dtype).replace("torch.", ""), "D": D, "W": W,
                 "bias": has_bias, "activation": act, "calls": []}
        for i, (T, mspec, use_cache) in enumerate(calls):
            x = torch.randn(B, T, D).to(dtype)
            mask = None
            if mspec is not None:
                if mspec[0] == "exact":
                    mask = right_padded_mask(B, T, mspec[1])
                elif mspec[0] == "longer":
                    mask = right_padded_mask(B, T + mspec[1], mspec[2])
                elif mspec[0] == "step":
                    # generation passes the whole-history mask; the last column counts
                    total = max(mspec[1])
                    mask = right_padded_mask(B, total, mspec[1])
            with torch.no_grad():
                out = layer(x, attention_mask=mask,
                            cache=cache if use_cache else None,
                            layer_idx=0 if use_cache else None)
            key = f"{name}/call{i}"
            arrays[f"{key}/x"] = to_np(x)
            if mask is not None:
                arrays[f"{key}/mask"] = mask.numpy().copy()
            arrays[f"{key}/out"] = to_np(out)
            if use_cache:
                arrays[f"{key}/state"] = to_np(cache.canon_cache_a[0])
            entry["calls"].append({"T": T, "mask": mask is not None, "cache": use_cache})
        manifest.append(entry)

    np.savez_compressed(os.path.join(HERE, "canon_layer_cases.npz"), **arrays)
    with open(os.path.join(HERE, "canon_layer_cases.json"), "w") as f:
        json.dump({"source": "CanonLayer eager CPU branch, model/model.py:587-675 and :262-398",
                   "torch": torch.__version__, "cases": manifest}, f, indent=1)
    print("wrote", len(arrays), "arrays,", len(manifest), "cases")


if __name__ == "__main__":
    main()
