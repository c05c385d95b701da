"""Benchmark configuration 5: a Viby-shaped model (tests/viby_harness.py) run with the HIP Canon layers
and with reference Canon back ends inside an otherwise identical network."""
import time

import pytest
import torch
from torch import nn

from canon_backends import NoCanon, OracleCanon, TorchEagerCanon, hip_factory
from helpers import bits
from viby_harness import generate_graphed, VibyShaped, init_weights, viby_config

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_small_model_hip_equals_oracle_bit_for_bit():
    cfg = viby_config(hidden_size=64, num_hidden_layers=3, num_attention_heads=2, num_key_value_heads=1,
                      head_dim=32, intermediate_size=96, vocab_size=512)
    ids = torch.randint(0, cfg.vocab_size, (2, 40), generator=torch.Generator().manual_seed(1)).to(DEV)
    hip = init_weights(VibyShaped(cfg, hip_factory(cfg, "eager")), 7, torch.bfloat16, DEV)
    ref = init_weights(VibyShaped(cfg, lambda C, n: OracleCanon(C, cfg, n, 1)), 7, torch.bfloat16, DEV)
    toks_h, logits_h, cache_h = hip.generate(ids, 6)
    toks_r, logits_r, cache_r = ref.generate(ids, 6)
    assert torch.equal(toks_h, toks_r)
    assert torch.equal(logits_h, logits_r)
    for site in "abcd":
        for layer in range(cfg.num_hidden_layers):
            got = getattr(cache_h, f"canon_cache_{site}")[layer]
            want = cache_r.oracle_states[(site, layer)]
            assert torch.equal(bits(got), bits(want)), (site, layer)


def test_model_with_concat_free_canon_b_d_is_bit_identical(capsys):
    """Canon-B / Canon-D fed q, k, v and gate, up as separate tensors: same logits and states as the cat path,
    at the small size and at the full model's shapes (with the time both take)."""
    cfg = viby_config(hidden_size=64, num_hidden_layers=3, num_attention_heads=2, num_key_value_heads=1,
                      head_dim=32, intermediate_size=96, vocab_size=512)
    ids = torch.randint(0, cfg.vocab_size, (2, 40), generator=torch.Generator().manual_seed(1)).to(DEV)
    for rounding in ("fused", "eager"):
        cat = init_weights(VibyShaped(cfg, hip_factory(cfg, rounding)), 7, torch.bfloat16, DEV)
        par = init_weights(VibyShaped(cfg, hip_factory(cfg, rounding), parts=True), 7, torch.bfloat16, DEV)
        toks_c, logits_c, cache_c = cat.generate(ids, 6)
        toks_p, logits_p, cache_p = par.generate(ids, 6)
        assert torch.equal(toks_c, toks_p) and torch.equal(logits_c, logits_p)
        for site in "abcd":
            for a, b in zip(getattr(cache_c, f"canon_cache_{site}"), getattr(cache_p, f"canon_cache_{site}")):
                assert torch.equal(bits(a), bits(b)), site

    cfg = viby_config()
    B, T, steps = 16, 1024, 16
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(5)).to(DEV)
    times, results = {}, {}
    for name, parts in (("cat", False), ("parts", True)):
        m = init_weights(VibyShaped(cfg, hip_factory(cfg, "fused"), parts=parts), 11, torch.bfloat16, DEV)
        m.generate(ids[:2, :64], 2)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        toks, logits, _ = m.generate(ids, steps, forced=results["cat"][0] if parts else None)
        torch.cuda.synchronize()
        times[name] = time.perf_counter() - t0
        results[name] = (toks, logits)
        del m
        torch.cuda.empty_cache()
    assert torch.equal(results["cat"][1], results["parts"][1])
    with capsys.disabled():
        print(f"\n[concat-free Canon-B/D] B{B} x L{T} prefill + {steps} steps: cat path {times['cat']:.3f} s, "
              f"parts {times['parts']:.3f} s")


def test_config5_full_model_fused_rounding_timing_and_noise_bound(capsys):
    cfg = viby_config()
    B, T, steps = 16, 1024, 128
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(5)).to(DEV)
    hip = init_weights(VibyShaped(cfg, hip_factory(cfg, "fused")), 11, torch.bfloat16, DEV)
    hip.generate(ids[:2, :64], 2)                       # warm-up (library load, allocator)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks, logits, cache = hip.generate(ids, steps)
    torch.cuda.synchronize()
    t_hip = time.perf_counter() - t0
    # shapes of the carried states: one [B, C, 8] tensor per (site, layer)
    for site, C in (("a", 640), ("b", 960), ("c", 640), ("d", 3456)):
        states = getattr(cache, f"canon_cache_{site}")
        assert len(states) == cfg.num_hidden_layers
        assert all(tuple(s.shape) == (B, C, 8) for s in states)
    del hip, cache
    torch.cuda.empty_cache()

    # the same network with the eager torch Canon, fed the tokens the HIP run produced
    ref = init_weights(VibyShaped(cfg, lambda C, n: TorchEagerCanon(C, cfg, n)), 11, torch.bfloat16, DEV)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks_r, logits_r, _ = ref.generate(ids, steps, forced=toks)
    torch.cuda.synchronize()
    t_ref = time.perf_counter() - t0

    # the same network with the Canon layers switched off: what is left is everything else (projections,
    # attention, norms, python), so the difference is the share of the 72 Canon calls per forward
    bare = init_weights(VibyShaped(cfg, lambda C, n: NoCanon()), 11, torch.bfloat16, DEV)
    bare.generate(ids[:2, :64], 2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    bare.generate(ids, steps, forced=toks)
    torch.cuda.synchronize()
    t_bare = time.perf_counter() - t0
    del bare
    torch.cuda.empty_cache()

    # A second, weaker check beside the bit-exact one above: in the default rounding mode the HIP layers round once
    # where the eager module rounds three times, so logits agree to bf16 noise accumulated over 18 layers and the
    # greedy choice agrees wherever it is not a near tie
    diff = (logits - logits_r).abs()
    scale = logits_r.abs().max().item()
    assert diff.max().item() <= 0.05 * scale, (diff.max().item(), scale)
    top2 = logits_r.topk(2, dim=-1).values
    margin = top2[..., 0] - top2[..., 1]
    decided = margin > 4 * diff.max(dim=-1).values
    agree = logits.argmax(-1) == logits_r.argmax(-1)
    assert bool(agree[decided].all())
    with capsys.disabled():
        print(f"\n[config 5] B{B} x L{T} prefill + {steps} greedy steps, 18 layers bf16: "
              f"HIP Canon {t_hip:.2f} s, eager torch Canon {t_ref:.2f} s, Canon layers off {t_bare:.2f} s "
              f"(Canon share {100 * (t_hip - t_bare) / t_hip:.0f} % with HIP, {100 * (t_ref - t_bare) / t_ref:.0f} % eager); "
              f"greedy tokens equal at {agree.float().mean().item() * 100:.1f} % of steps "
              f"({decided.float().mean().item() * 100:.1f} % decided beyond rounding noise), "
              f"max |dlogit| {diff.max().item():.4f} of scale {scale:.2f}")


def test_config5_full_size_eager_rounding_equals_the_cpu_eager_module_bit_for_bit(capsys):
    """Configuration 5 by its own criterion: 18 layers, B16 x L1024 prefill, 128 greedy steps through the conv
    caches, bf16.  The HIP Canon layers with the eager module's rounding points against the eager module itself
    (torch operations on the host, the reference's CPU path) inside the same network: identical greedy tokens,
    identical logits at every step and all 72 conv states equal bit for bit.  Both runs decode freely (no
    teacher forcing): one differing bit anywhere would show."""
    cfg = viby_config()
    B, T, steps = 16, 1024, 128
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(5)).to(DEV)
    hip = init_weights(VibyShaped(cfg, hip_factory(cfg, "eager")), 11, torch.bfloat16, DEV)
    toks, logits, cache = hip.generate(ids, steps)
    states = {(site, layer): getattr(cache, f"canon_cache_{site}")[layer].cpu()
              for site in "abcd" for layer in range(cfg.num_hidden_layers)}
    del hip, cache
    torch.cuda.empty_cache()
    ref = init_weights(VibyShaped(cfg, lambda C, n: TorchEagerCanon(C, cfg, n, host=True)), 11, torch.bfloat16, DEV)
    t0 = time.perf_counter()
    toks_r, logits_r, cache_r = ref.generate(ids, steps)
    torch.cuda.synchronize()
    t_ref = time.perf_counter() - t0
    assert len(states) == 72
    assert torch.equal(toks, toks_r), f"greedy tokens differ first at step {(toks != toks_r).any(0).nonzero()[0].item()}"
    assert torch.equal(bits(logits.bfloat16()), bits(logits_r.bfloat16())) and torch.equal(logits, logits_r)
    for key, got in states.items():
        assert torch.equal(bits(got), bits(cache_r.eager_states[key])), key
    with capsys.disabled():
        print(f"\n[config 5, eager rounding] B{B} x L{T} prefill + {steps} greedy steps: tokens, logits and all 72 conv "
              f"states identical to the host eager module (which took {t_ref:.1f} s)")


def test_config5_decode_as_one_hip_graph_per_token(capsys):
    """The whole decode step of the 18-layer model (72 Canon update launches among everything else) captured
    once and replayed for every generated token: bit-identical to the same step launched eagerly, same tokens
    and logits as the growing-KV loop up to the attention kernel's rounding (it runs over a fixed-length KV
    buffer here), and the time it takes."""
    cfg = viby_config()
    B, T, steps = 16, 1024, 128
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(5)).to(DEV)
    model = init_weights(VibyShaped(cfg, hip_factory(cfg, "fused")), 11, torch.bfloat16, DEV)
    model.generate(ids[:2, :64], 2)
    generate_graphed(model, ids[:2, :64], 3)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks_e, logits_e, _ = model.generate(ids, steps)
    torch.cuda.synchronize()
    t_eager = time.perf_counter() - t0
    t0 = time.perf_counter()
    toks_g, logits_g = generate_graphed(model, ids, steps)
    torch.cuda.synchronize()
    t_graph = time.perf_counter() - t0
    # the same step function launched kernel by kernel: the replays must reproduce it bit for bit
    toks_s, logits_s = generate_graphed(model, ids, steps, capture=False)
    assert torch.equal(toks_s, toks_g) and torch.equal(logits_s, logits_g)
    assert torch.equal(logits_e[0], logits_g[0])                     # the prefill is the same code
    # teacher-forced comparison is not possible inside a graph: compare up to the first diverging token
    same = (toks_e == toks_g).all(dim=0).int().cumprod(0).sum().item()
    assert same >= 4, same
    diff = (logits_e[:same + 1] - logits_g[:same + 1]).abs().max().item()
    scale = logits_e.abs().max().item()
    assert diff <= 0.05 * scale, (diff, scale)
    with capsys.disabled():
        print(f"\n[config 5, graph-captured decode] B{B} x L{T} prefill + {steps} greedy steps: eager loop {t_eager:.2f} s, "
              f"one HIP graph per token {t_graph:.2f} s; first {same} of {steps} steps identical for every sequence, "
              f"max |dlogit| {diff:.4f} of scale {scale:.2f} over them")
