"""Pins the CPU oracle before anything is compared against it.

  * storage conversions            vs torch's own casts
  * prefill arithmetic             vs torch's conv1d (the reference's oracle,
                                   causal-conv1d-mps/test.py:83-107) on the
                                   reference's grid (test.py:110-116, seed 42)
  * indices / history / state      vs a brute-force loop on tiny shapes
  * invariants                     streaming, chunking, state-length
                                   independence, linearity, causality,
                                   permutation equivariance, mask special cases
  * eager module restatement       vs golden vectors produced by the real
                                   CanonLayer (tests/golden/)
"""
import itertools
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import canon_oracle as co
from oracle.canon_eager import EagerCanon

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def bits(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in representable values of the (16-bit) storage type."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(i >= 0x8000, 0x8000 - i, i)
    return (key(a) - key(b)).abs()


# --------------------------------------------------------------------------
# conversions
# --------------------------------------------------------------------------
def test_conversions_match_torch():
    L = co.lib()
    g = torch.Generator().manual_seed(0)
    vals = torch.cat([
        torch.randn(4000, generator=g),
        torch.randn(2000, generator=g) * 1e-6,
        torch.randn(2000, generator=g) * 6e4,
        torch.randn(500, generator=g) * 1e-41,       # fp32 subnormals
        torch.tensor([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9,
                      float("inf"), float("-inf"), 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                      2.0 ** -14, 2.0 ** -14 * 0.9999, 3.3895314e38, 1.0 + 2.0 ** -8,
                      1.0 + 2.0 ** -8 + 2.0 ** -20, 1.0 + 3 * 2.0 ** -8]),
    ])
    want_bf = vals.bfloat16().view(torch.int16).to(torch.int32) & 0xFFFF
    want_h = vals.half().view(torch.int16).to(torch.int32) & 0xFFFF
    for v, wb, wh in zip(vals.tolist(), want_bf.tolist(), want_h.tolist()):
        assert L.canon_oracle_float_to_bf16(v) == wb, v
        assert L.canon_oracle_float_to_f16(v) == wh, v
    assert L.canon_oracle_float_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0
    # every 16-bit pattern back to float
    allbits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    bf = allbits.view(torch.bfloat16).float()
    hf = allbits.view(torch.float16).float()
    for i in range(0, 65536, 7):
        b = int(allbits[i]) & 0xFFFF
        x, y = L.canon_oracle_bf16_to_float(b), float(bf[i])
        assert x == y or (x != x and y != y)
        x, y = L.canon_oracle_f16_to_float(b), float(hf[i])
        assert x == y or (x != x and y != y)


# --------------------------------------------------------------------------
# arithmetic vs torch conv1d on the reference's grid
# --------------------------------------------------------------------------
def torch_reference(x, weight, bias, silu):
    """fp32 restatement of causal-conv1d-mps/test.py:83-107."""
    itype = x.dtype
    xq = x.float()
    wq = weight.to(itype).float()
    bq = bias.to(itype).float() if bias is not None else None
    W = weight.shape[1]
    y = F.conv1d(F.pad(xq, (W - 1, 0)), wq.unsqueeze(1), bias=bq, groups=x.shape[1])
    return F.silu(y) if silu else y


@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_fwd_matches_torch_conv1d_on_reference_grid(dim, has_bias, silu, itype):
    for seqlen in [1, 2, 8, 16, 32, 64, 128, 256]:
        torch.manual_seed(42)
        x = torch.randn(2, dim, seqlen).to(itype)
        w = torch.randn(dim, 4)
        b = torch.randn(dim) if has_bias else None
        got = co.conv1d_fwd(x, w, b, activation="silu" if silu else None)
        want32 = torch_reference(x, w, b, silu)
        if itype == torch.float32:
            if not silu:
                # torch evaluates the depthwise conv as the same fma chain
                scale = want32.abs().clamp_min(1.0)
                assert ((got - want32).abs() / scale).max().item() <= 1e-6
                assert (got != want32).float().mean().item() <= 0.01
            else:
                torch.testing.assert_close(got, want32, rtol=1e-6, atol=1e-6)
        else:
            want = want32.to(itype)
            d = ulp_diff(got, want)
            assert d.max().item() <= 1, (seqlen, d.max().item())
            assert (d > 0).float().mean().item() <= 0.002


# --------------------------------------------------------------------------
# brute force on tiny shapes
# --------------------------------------------------------------------------
def brute_fwd(x, w, bias, mask, init, S_out, silu, res_mode):
    """float64-free, index-by-index restatement (fp32 only, python loops)."""
    B, C, L = x.shape
    W = w.shape[1]
    out = np.zeros((B, C, L), np.float32)
    fs = np.zeros((B, C, S_out), np.float32) if S_out else None
    for b in range(B):
        for c in range(C):
            xm = [np.float32(x[b, c, t] * (mask[b, t] if mask is not None else np.float32(1)))
                  for t in range(L)]
            hist = [np.float32(0)] * (W - 1) if init is None else list(init[b, c, init.shape[2] - (W - 1):]) if W > 1 else []
            seq = hist + xm     # seq[t + W - 1] == xm[t]
            for t in range(L):
                acc = np.float64(bias[c]) if bias is not None else np.float64(0)
                acc = np.float32(acc)
                for k in range(W):
                    # fma: exact product in float64, one rounding of the sum
                    acc = np.float32(np.float64(w[c, k]) * np.float64(seq[t + k]) + np.float64(acc))
                if silu:
                    acc = np.float32(acc / np.float32(np.float32(1) + np.exp(-acc, dtype=np.float32)))
                if res_mode == 1:
                    acc = np.float32(acc + xm[t])
                elif res_mode == 2:
                    acc = np.float32(acc + x[b, c, t])
                out[b, c, t] = acc
            if S_out:
                full = ([np.float32(0)] * S_out + (list(init[b, c]) if init is not None else []) + xm)
                fs[b, c] = full[-S_out:]
    return out, fs


@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("L", [1, 2, 3, 4, 5, 9])
def test_fwd_matches_brute_force(W, L):
    rng = np.random.default_rng(100 * W + L)
    B, C = 2, 3
    for has_bias, has_mask, has_init, silu, res_mode in itertools.product(
            [False, True], [False, True], [False, True], [False, True], [0, 1, 2]):
        x = rng.standard_normal((B, C, L)).astype(np.float32)
        w = rng.standard_normal((C, W)).astype(np.float32)
        bias = rng.standard_normal(C).astype(np.float32) if has_bias else None
        mask = (rng.random((B, L)) > 0.4).astype(np.float32) if has_mask else None
        S_in = int(rng.integers(W - 1, 6)) if W > 1 else 2
        init = rng.standard_normal((B, C, S_in)).astype(np.float32) if has_init else None
        S_out = int(rng.integers(1, 9))
        want, want_fs = brute_fwd(x, w, bias, mask, init, S_out, silu, res_mode)
        t = torch.from_numpy
        got, got_fs = co.conv1d_fwd(
            t(x), t(w), None if bias is None else t(bias),
            mask=None if mask is None else t(mask),
            initial_state=None if init is None else t(init),
            final_state_len=S_out, activation="silu" if silu else None, residual=res_mode)
        if silu:
            np.testing.assert_allclose(got.numpy(), want, rtol=2e-6, atol=1e-6)
        else:
            np.testing.assert_array_equal(got.numpy(), want)
        np.testing.assert_array_equal(got_fs.numpy(), want_fs)


def test_update_matches_brute_force():
    rng = np.random.default_rng(7)
    B, C = 3, 5
    for W, S, has_bias, silu, res in itertools.product([2, 3, 4], [3, 4, 8], [False, True],
                                                       [False, True], [False, True]):
        if S < W - 1:
            continue
        x = rng.standard_normal((B, C)).astype(np.float32)
        st = rng.standard_normal((B, C, S)).astype(np.float32)
        w = rng.standard_normal((C, W)).astype(np.float32)
        bias = rng.standard_normal(C).astype(np.float32) if has_bias else None
        want = np.zeros((B, C), np.float32)
        for b in range(B):
            for c in range(C):
                seq = list(st[b, c, S - (W - 1):]) + [x[b, c]]
                acc = np.float32(bias[c]) if has_bias else np.float32(0)
                for k in range(W):
                    acc = np.float32(np.float64(w[c, k]) * np.float64(seq[k]) + np.float64(acc))
                if silu:
                    acc = np.float32(acc / np.float32(np.float32(1) + np.exp(-acc, dtype=np.float32)))
                if res:
                    acc = np.float32(acc + x[b, c])
                want[b, c] = acc
        want_state = np.concatenate([st[:, :, 1:], x[:, :, None]], axis=2)
        t = torch.from_numpy
        st_t = t(st.copy())
        got = co.conv1d_update(t(x), st_t, t(w), None if bias is None else t(bias),
                               activation="silu" if silu else None, residual=res)
        if silu:
            np.testing.assert_allclose(got.numpy(), want, rtol=2e-6, atol=1e-6)
        else:
            np.testing.assert_array_equal(got.numpy(), want)
        np.testing.assert_array_equal(st_t.numpy(), want_state)


# --------------------------------------------------------------------------
# invariants
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S", [3, 4, 8])
def test_streaming_equals_prefill(dtype, S):
    torch.manual_seed(S)
    B, C, L = 2, 24, 19
    x = torch.randn(B, C, L).to(dtype)
    w = (torch.randn(C, 4) * 0.3).to(dtype)
    b = (torch.randn(C) * 0.1).to(dtype)
    for act in (None, "silu"):
        full, fs = co.conv1d_fwd(x, w, b, final_state_len=S, activation=act)
        state = torch.zeros(B, C, S, dtype=dtype)
        cols = [co.conv1d_update(x[:, :, t].contiguous(), state, w, b, activation=act)
                for t in range(L)]
        assert torch.equal(bits(torch.stack(cols, dim=-1)), bits(full))
        assert torch.equal(bits(state), bits(fs))
        assert torch.equal(bits(fs), bits(x[:, :, -S:]))


def test_chunked_prefill_equals_one_shot():
    torch.manual_seed(3)
    B, C, L = 2, 10, 23
    x = torch.randn(B, C, L)
    w = torch.randn(C, 4)
    mask = (torch.rand(B, L) > 0.3).float()
    full, fs = co.conv1d_fwd(x, w, None, mask=mask, final_state_len=5, residual=1)
    for cut in (1, 2, 3, 7, 20, 22):
        a, sa = co.conv1d_fwd(x[:, :, :cut], w, None, mask=mask[:, :cut], final_state_len=3, residual=1)
        bpart, sb = co.conv1d_fwd(x[:, :, cut:], w, None, mask=mask[:, cut:], initial_state=sa,
                                  final_state_len=5, residual=1)
        assert torch.equal(torch.cat([a, bpart], dim=-1), full)
        if L - cut >= 5 or cut >= 3:
            # enough history travelled through the 3-slot intermediate state
            k = min(5, (L - cut) + 3)
            assert torch.equal(sb[:, :, -k:], fs[:, :, -k:])


def test_linearity_causality_permutation_and_masks():
    torch.manual_seed(5)
    B, C, L = 3, 12, 40
    x1, x2 = torch.randn(B, C, L).double(), torch.randn(B, C, L).double()
    # values on a coarse grid make every fp32 operation exact -> exact linearity
    q = lambda t: (t * 8).round().div(8).float()
    x1, x2 = q(x1), q(x2)
    w = q(torch.randn(C, 4).double())
    y1, y2 = co.conv1d_fwd(x1, w), co.conv1d_fwd(x2, w)
    assert torch.equal(co.conv1d_fwd(x1 + x2, w), y1 + y2)
    assert torch.equal(co.conv1d_fwd(x1, 2 * w), 2 * y1)
    # causality: a change at t0 reaches t0 .. t0+3 only
    xp = x1.clone()
    xp[:, :, 17] += 1.0
    d = (co.conv1d_fwd(xp, w) != y1).any(dim=0).any(dim=0)
    assert d.nonzero().flatten().tolist() == [17, 18, 19, 20]
    # batch / channel permutation equivariance
    pb, pc = torch.randperm(B), torch.randperm(C)
    assert torch.equal(co.conv1d_fwd(x1[pb][:, pc], w[pc]), y1[pb][:, pc])
    # masks: all ones == none; all zeros -> act(bias) (+ masked residual == 0)
    bias = torch.randn(C)
    ones, zeros = torch.ones(B, L), torch.zeros(B, L)
    for act in (None, "silu"):
        assert torch.equal(co.conv1d_fwd(x1, w, bias, mask=ones, activation=act, residual=1),
                           co.conv1d_fwd(x1, w, bias, activation=act, residual=1))
        z = co.conv1d_fwd(x1, w, bias, mask=zeros, activation=act, residual=1)
        want = F.silu(bias) if act else bias
        torch.testing.assert_close(z, want[None, :, None].expand(B, C, L), rtol=1e-6, atol=1e-7)
    # masking multiplies: -x * 0 keeps its sign bit (the captured state must be bit exact)
    neg = -x1.abs() - 1
    _, fs = co.conv1d_fwd(neg, w, mask=zeros, final_state_len=4)
    assert torch.equal(bits(fs), bits(torch.full_like(fs, -0.0)))


# --------------------------------------------------------------------------
# eager module restatement vs the real CanonLayer's vectors
# --------------------------------------------------------------------------
def _load_golden():
    with open(os.path.join(GOLDEN, "canon_layer_cases.json")) as f:
        manifest = json.load(f)
    arrays = np.load(os.path.join(GOLDEN, "canon_layer_cases.npz"))
    return manifest["cases"], arrays


def golden_tensor(arrays, key, dtype):
    a = torch.from_numpy(arrays[key])
    return a.view(torch.bfloat16) if dtype == torch.bfloat16 else a


@pytest.mark.parametrize("case", _load_golden()[0], ids=lambda c: c["name"])
def test_eager_restatement_matches_canon_layer_golden(case):
    _, arrays = _load_golden()
    name = case["name"]
    dtype = getattr(torch, case["dtype"])
    w = golden_tensor(arrays, f"{name}/weight", dtype)
    b = golden_tensor(arrays, f"{name}/bias", dtype) if case["bias"] else None
    layer = EagerCanon(w, b, case["activation"])
    cache = {}
    for i, call in enumerate(case["calls"]):
        key = f"{name}/call{i}"
        x = golden_tensor(arrays, f"{key}/x", dtype)
        mask = torch.from_numpy(arrays[f"{key}/mask"]) if call["mask"] else None
        out = layer.forward(x, mask, cache if call["cache"] else None, "k")
        want = golden_tensor(arrays, f"{key}/out", dtype)
        assert torch.equal(bits(out), bits(want)), (name, i)
        if call["cache"]:
            want_state = golden_tensor(arrays, f"{key}/state", dtype)
            assert torch.equal(bits(cache["k"]), bits(want_state)), (name, i)


# --------------------------------------------------------------------------
# kernel-level oracle vs the eager module (ties the two oracles together)
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", [False, True])
def test_eager_rounding_mode_reproduces_eager_module(dtype, act):
    torch.manual_seed(11)
    B, T, D = 3, 50, 32
    x = torch.randn(B, T, D).to(dtype)
    w = (torch.randn(D, 4) * 0.4).to(dtype)
    bias = (torch.randn(D) * 0.1).to(dtype)
    lens = [50, 31, 7]
    mask = torch.zeros(B, T, dtype=torch.int64)
    for i, n in enumerate(lens):
        mask[i, :n] = 1
    cache = {}
    want = EagerCanon(w, bias, act).forward(x, mask, cache, 0)
    got, fs = co.conv1d_fwd(x.transpose(1, 2), w, bias, mask=mask, final_state_len=8,
                            activation="silu" if act else None, residual=1, round_mode=1)
    got = got.transpose(1, 2)
    assert torch.equal(bits(fs), bits(cache[0]))
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    elif not act:
        assert torch.equal(bits(got), bits(want))
    else:
        d = ulp_diff(got, want)   # expf of libm vs torch's vectorised exp
        assert d.max().item() <= 1 and (d > 0).float().mean().item() < 0.01
    # and the single-rounding result stays within one ulp of exact arithmetic
    if dtype != torch.float32:
        fused = co.conv1d_fwd(x.transpose(1, 2), w, bias, mask=mask,
                              activation="silu" if act else None, residual=1)
        x64 = (x * mask.unsqueeze(-1)).double().transpose(1, 2)
        y64 = F.conv1d(F.pad(x64, (3, 0)), w.double().unsqueeze(1), bias.double(), groups=D)
        if act:
            y64 = F.silu(y64)
        exact = (y64 + x64).to(dtype)
        assert ulp_diff(fused, exact).max().item() <= 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_eager_step_mode_reproduces_eager_module(dtype):
    torch.manual_seed(13)
    B, D, S = 4, 48, 8
    w = (torch.randn(D, 4) * 0.4).to(dtype)
    bias = (torch.randn(D) * 0.1).to(dtype)
    for act in (False, True):
        layer = EagerCanon(w, bias, act)
        cache = {0: torch.randn(B, D, S).to(dtype)}
        state = cache[0].clone()
        for _ in range(6):
            x = torch.randn(B, 1, D).to(dtype)
            want = layer.forward(x, None, cache, 0)[:, 0]
            got = co.conv1d_update(x[:, 0].contiguous(), state, w, bias,
                                   activation="silu" if act else None, residual=True, round_mode=1)
            assert torch.equal(bits(state), bits(cache[0]))
            if dtype == torch.float32:
                torch.testing.assert_close(got, want, rtol=2e-6, atol=2e-6)
            else:
                d = ulp_diff(got, want)
                assert d.max().item() <= 1 and (d > 0).float().mean().item() < 0.02


# ---- packed sequences (seq_idx): pinned by brute force and by the defining property ------------
def test_seq_idx_oracle_brute_force_and_separate_sequences():
    g = torch.Generator().manual_seed(81)
    for W, L in itertools.product([2, 3, 4], [1, 2, 5, 9, 17]):
        B, C = 2, 3
        x = torch.randn(B, C, L, generator=g)
        w = torch.randn(C, W, generator=g)
        b = torch.randn(C, generator=g)
        seq = torch.randint(0, 3, (B, L), generator=g).sort(dim=1).values.to(torch.int32)
        got = co.conv1d_fwd_seq(x, w, b, seq)
        # index by index, every tap spelled out
        for bi, c, t in itertools.product(range(B), range(C), range(L)):
            acc = np.float32(b[c])
            for k in range(W):
                src = t - (W - 1) + k
                v = np.float32(x[bi, c, src]) if src >= 0 and seq[bi, src] == seq[bi, t] else np.float32(0)
                # the product of two floats is exact in float64, so this is the fused multiply-add up to double rounding
                acc = np.float32(np.float64(np.float32(w[c, k])) * np.float64(v) + np.float64(acc))
            assert abs(float(got[bi, c, t]) - float(acc)) <= 1e-6 * max(1.0, abs(float(acc))), (W, L, bi, c, t)
        # a packed row equals its sequences run one by one, bit for bit
        for bi in range(B):
            bounds = [0] + [t for t in range(1, L) if seq[bi, t] != seq[bi, t - 1]] + [L]
            for lo, hi in zip(bounds[:-1], bounds[1:]):
                alone = co.conv1d_fwd(x[bi:bi + 1, :, lo:hi].contiguous(), w, b)
                assert torch.equal(got[bi:bi + 1, :, lo:hi], alone), (W, L, bi, lo, hi)
    # one sequence per row is the plain conv; SiLU, mask and residual ride along unchanged
    x = torch.randn(2, 4, 33, generator=g).bfloat16()
    w = torch.randn(4, 4, generator=g).bfloat16()
    mask = (torch.rand(2, 33, generator=g) > 0.3).to(torch.int64)
    same = torch.zeros(2, 33, dtype=torch.int32)
    for act, res in [(None, 0), ("silu", 1), ("silu", 2)]:
        a = co.conv1d_fwd_seq(x, w, None, same, mask=mask, activation=act, residual=res)
        b_ = co.conv1d_fwd(x, w, None, mask=mask, activation=act, residual=res)
        assert torch.equal(a.view(torch.int16), b_.view(torch.int16))


def test_gradient_oracle_of_packed_sequences_is_pinned():
    """The float64 gradient oracle with seq_idx: its forward equals the C oracle of the packed forward,
    and its gradients equal those of every sequence differentiated on its own with the plain conv1d
    formulation (dx cut out per sequence, dweight / dbias summed)."""
    from oracle.canon_grad import conv1d_grads
    g = torch.Generator().manual_seed(5)
    B, C, L = 2, 5, 23
    x = torch.randn(B, C, L, generator=g)
    dout = torch.randn(B, C, L, generator=g)
    mask = (torch.rand(B, L, generator=g) > 0.2).float()
    seq = torch.tensor([[0] * 7 + [1] * 3 + [2] * 1 + [3] * 12, [0] * 23], dtype=torch.int32)
    for W in (2, 3, 4):
        w = torch.randn(C, W, generator=g)
        b = torch.randn(C, generator=g)
        for act, res in itertools.product((None, "silu"), (0, 1, 2)):
            dx, dw, db, out = conv1d_grads(x, w, b, dout, mask, act, res, seq_idx=seq)
            want = co.conv1d_fwd_seq(x, w, b, seq, mask, act, res)
            torch.testing.assert_close(out.float(), want, rtol=1e-5, atol=1e-5)
            dx2, dw2, db2 = torch.zeros_like(dx), torch.zeros_like(dw), torch.zeros_like(db)
            for bi in range(B):
                cuts = [0] + [t for t in range(1, L) if seq[bi, t] != seq[bi, t - 1]] + [L]
                for s0, s1 in zip(cuts[:-1], cuts[1:]):
                    a, aw, ab, _ = conv1d_grads(x[bi:bi + 1, :, s0:s1], w, b, dout[bi:bi + 1, :, s0:s1],
                                                mask[bi:bi + 1, s0:s1], act, res)
                    dx2[bi, :, s0:s1] = a[0]
                    dw2 += aw
                    db2 += ab
            torch.testing.assert_close(dx, dx2, rtol=1e-12, atol=1e-12)
            torch.testing.assert_close(dw, dw2, rtol=1e-12, atol=1e-12)
            torch.testing.assert_close(db, db2, rtol=1e-12, atol=1e-12)


def test_ring_buffer_and_state_pool_update_equal_the_shift_register():
    g = torch.Generator().manual_seed(83)
    for dtype, W, S in itertools.product([torch.float32, torch.bfloat16], [2, 3, 4], [3, 4, 7, 8]):
        if S < W - 1:
            continue
        B, C, rows = 3, 5, 7
        w = torch.randn(C, W, generator=g).to(dtype)
        b = torch.randn(C, generator=g).to(dtype)
        start = torch.randn(B, C, S, generator=g).to(dtype)
        shift = start.clone()
        ring = start.clone()                      # ring position 0 = oldest entry = shift-register slot 0
        pool = torch.randn(rows, C, S, generator=g).to(dtype)
        rows_of = torch.tensor([5, 0, 3], dtype=torch.int32)
        pool[rows_of.long()] = start
        untouched = pool.clone()
        for step in range(2 * S + 3):
            x = torch.randn(B, C, generator=g).to(dtype)
            want = co.conv1d_update(x, shift, w, b, activation="silu", residual=True)
            got = co.conv1d_update_ext(x, ring, w, b, activation="silu", residual=True,
                                       cache_seqlens=torch.full((B,), step, dtype=torch.int32))
            assert torch.equal(got.view(torch.int16 if dtype != torch.float32 else torch.int32),
                               want.view(torch.int16 if dtype != torch.float32 else torch.int32)), (dtype, W, S, step)
            pos = (step + 1) % S
            assert torch.equal(torch.cat([ring[:, :, pos:], ring[:, :, :pos]], dim=2), shift), (dtype, W, S, step)
            got2 = co.conv1d_update_ext(x, pool, w, b, activation="silu", residual=True, conv_state_indices=rows_of)
            assert torch.equal(got2, want)
            assert torch.equal(pool[rows_of.long()], shift)
        others = [r for r in range(rows) if r not in rows_of.tolist()]
        assert torch.equal(pool[others], untouched[others])
        # entries whose index lies outside the pool are skipped: the rest is the call without them
        before = pool.clone()
        x = torch.randn(B, C, generator=g).to(dtype)
        want = co.conv1d_update_ext(x[1:2], pool, w, b, activation="silu", residual=True, conv_state_indices=rows_of[1:2])
        after = pool.clone()
        pool.copy_(before)
        got = co.conv1d_update_ext(x, pool, w, b, activation="silu", residual=True,
                                   conv_state_indices=torch.tensor([-1, int(rows_of[1]), rows], dtype=torch.int32))
        assert torch.equal(got[1:2], want) and torch.equal(pool, after)
        assert not got[0].any() and not got[2].any()


def test_update_gradient_oracle_chained_equals_the_prefill_gradient_oracle():
    """oracle/canon_grad.update_grads, chained backwards through the state it hands on, must give the
    gradients of conv1d_grads (torch autograd through F.conv1d) on the same tokens laid out along time;
    a wrong slot, a dropped state term or a missing residual fails this."""
    from oracle.canon_grad import conv1d_grads, update_grads
    torch.manual_seed(0)
    for (S, W), act, res, masked in itertools.product([(4, 4), (3, 4), (8, 4), (5, 3), (1, 2)], [None, "silu"],
                                                      [0, 1, 2], [False, True]):
        B, C, T = 2, 5, 6
        x, w, b = torch.randn(B, C, T).double(), torch.randn(C, W).double(), torch.randn(C).double()
        dout = torch.randn(B, C, T).double()
        mask = (torch.rand(B, T) > 0.3).double() if masked else None
        dx_ref, dw_ref, db_ref, out_ref = conv1d_grads(x, w, b, dout, mask=mask, activation=act, residual=res)
        states = [torch.zeros(B, C, S, dtype=torch.float64)]
        for t in range(T):
            r = update_grads(x[:, :, t], states[-1], w, b, dout[:, :, t], None, None if mask is None else mask[:, t],
                             act, res)
            assert torch.allclose(r[4], out_ref[:, :, t], atol=1e-12)
            states.append(r[5])
        ds, dw, db = None, torch.zeros_like(w), torch.zeros_like(b)
        dx = torch.zeros_like(x)
        for t in reversed(range(T)):
            r = update_grads(x[:, :, t], states[t], w, b, dout[:, :, t], ds, None if mask is None else mask[:, t],
                             act, res)
            dx[:, :, t], ds = r[0], r[1]
            dw += r[2]
            db += r[3]
        for got, want in ((dx, dx_ref), (dw, dw_ref), (db, db_ref)):
            assert torch.allclose(got, want, atol=1e-11), (S, W, act, res, masked)


def test_update_gradient_oracle_of_ring_and_pool_modes_equals_the_shift_register_form():
    """oracle/canon_grad.update_grads_ext (the step written with gather / scatter) is pinned by what defines its
    two modes.  Ring: with the state rotated so that slot (p + j) mod S holds entry j of a shift register, and the
    gradient of the updated state rotated by p + 1, its gradients are those of update_grads, rotated back.  Pool:
    entries that name rows of a pool give update_grads of those rows; rows nobody names hand their gradient on;
    an index outside the pool contributes nothing.  Both together; and neither equals update_grads itself."""
    from oracle.canon_grad import update_grads, update_grads_ext
    torch.manual_seed(3)
    for (S, W), act, res, masked, through in itertools.product([(4, 4), (3, 4), (8, 4), (5, 3), (1, 2)], [None, "silu"],
                                                               [0, 1, 2], [False, True], [False, True]):
        B, C = 4, 5
        x, st = torch.randn(B, C).double(), torch.randn(B, C, S).double()
        w, b, dout = torch.randn(C, W).double(), torch.randn(C).double(), torch.randn(B, C).double()
        dso = torch.randn(B, C, S).double() if through else None
        mask = torch.tensor([1.0, 0.0, 1.0, 1.0]).double() if masked else None
        plain = update_grads(x, st, w, b, dout, dso, mask, act, res)
        same = update_grads_ext(x, st, w, b, dout, dso, mask, act, res)
        for u, v in zip(plain, same):
            assert torch.allclose(u, v, atol=1e-13)
        # ring buffer
        seqlens = torch.tensor([0, 1, S + 2, 7 * S + (S - 1)], dtype=torch.int32)
        p = seqlens.long() % S
        j = torch.arange(S)
        to_slot = (p[:, None] + j[None, :]) % S                  # slot of entry j before the step
        to_slot_after = (p[:, None] + 1 + j[None, :]) % S        # slot of entry j after it
        def rotate(t, slots):                                   # ring[slot] = register[entry]
            r = torch.empty_like(t)
            r.scatter_(2, slots[:, None, :].expand_as(t), t)
            return r
        ring = update_grads_ext(x, rotate(st, to_slot), w, b, dout, None if dso is None else rotate(dso, to_slot_after),
                                mask, act, res, cache_seqlens=seqlens)
        assert torch.allclose(ring[0], plain[0], atol=1e-13) and torch.allclose(ring[2], plain[2], atol=1e-13)
        assert torch.allclose(ring[3], plain[3], atol=1e-13) and torch.allclose(ring[4], plain[4], atol=1e-13)
        assert torch.allclose(ring[1], rotate(plain[1], to_slot), atol=1e-13), (S, W)
        assert torch.allclose(ring[5], rotate(plain[5], to_slot_after), atol=1e-13), (S, W)
        # state pool of 7 rows: entries 0, 1, 3 name rows 5, 0, 2; entry 2 is skipped
        idx = torch.tensor([5, 0, -3, 2], dtype=torch.int32)
        live = torch.tensor([0, 1, 3])
        pool = torch.randn(7, C, S).double()
        pool[idx[live].long()] = st[live]
        dpool = torch.randn(7, C, S).double() if through else None
        if through:
            dpool[idx[live].long()] = dso[live]
        got = update_grads_ext(x, pool, w, b, dout, dpool, mask, act, res, conv_state_indices=idx)
        sub = update_grads(x[live], st[live], w, b, dout[live], None if dso is None else dso[live],
                           None if mask is None else mask[live], act, res)
        assert torch.allclose(got[0][live], sub[0], atol=1e-13) and not got[0][2].any() and not got[4][2].any()
        assert torch.allclose(got[2], sub[2], atol=1e-13) and torch.allclose(got[3], sub[3], atol=1e-13)
        assert torch.allclose(got[1][idx[live].long()], sub[1], atol=1e-13)
        for r in (1, 3, 4, 6):
            assert torch.equal(got[1][r], dpool[r] if through else torch.zeros(C, S).double())
            assert torch.equal(got[5][r], pool[r])
        assert torch.allclose(got[5][idx[live].long()], sub[5], atol=1e-13)


def test_gradient_oracle_with_initial_states_equals_the_block_in_one_go():
    """conv1d_grads(initial_states=...) on the second half of a block, continued from the (masked) last inputs
    of the first half, plus conv1d_grads on the first half, must add up to conv1d_grads on the whole block."""
    from oracle.canon_grad import conv1d_grads
    torch.manual_seed(1)
    for W, S, act, res, masked, L1 in itertools.product([2, 3, 4], [3, 5], [None, "silu"], [0, 1, 2], [False, True],
                                                        [1, 2, 7]):
        if S < W - 1:
            continue
        B, C, L2 = 2, 3, 5
        x = torch.randn(B, C, L1 + L2).double()
        w, b, dout = torch.randn(C, W).double(), torch.randn(C).double(), torch.randn(B, C, L1 + L2).double()
        mask = (torch.rand(B, L1 + L2) > 0.3).double() if masked else None
        m1, m2 = (None, None) if mask is None else (mask[:, :L1], mask[:, L1:])
        whole = conv1d_grads(x, w, b, dout, mask=mask, activation=act, residual=res)
        # state after the first half: its last S masked inputs, zero filled on the left
        xm1 = x[:, :, :L1] if m1 is None else x[:, :, :L1] * m1.unsqueeze(1)
        state = F.pad(xm1, (S, 0))[:, :, -S:]
        second = conv1d_grads(x[:, :, L1:], w, b, dout[:, :, L1:], mask=m2, activation=act, residual=res,
                              initial_states=state)
        first = conv1d_grads(x[:, :, :L1], w, b, dout[:, :, :L1], mask=m1, activation=act, residual=res)
        assert torch.allclose(torch.cat([first[3], second[3]], dim=2), whole[3], atol=1e-12)
        # the state's gradient flows back into the inputs it copied (times their mask)
        n = min(S, L1)
        back = torch.zeros_like(first[0])
        back[:, :, L1 - n:] = second[4][:, :, S - n:] * (1.0 if m1 is None else m1[:, L1 - n:].unsqueeze(1))
        assert torch.allclose(torch.cat([first[0] + back, second[0]], dim=2), whole[0], atol=1e-11), (W, S, act, res)
        # ... which is what the oracle does itself when handed the state's gradient as dfinal
        chained = conv1d_grads(x[:, :, :L1], w, b, dout[:, :, :L1], mask=m1, activation=act, residual=res, dfinal=second[4])
        assert torch.allclose(chained[0], first[0] + back, atol=1e-11), (W, S, act, res, "dfinal")
        assert torch.allclose(chained[1], first[1], atol=1e-11) and torch.allclose(chained[3], first[3], atol=1e-12)
        assert torch.allclose(first[1] + second[1], whole[1], atol=1e-11)
        assert torch.allclose(first[2] + second[2], whole[2], atol=1e-11)
        assert float(second[4][:, :, :S - (W - 1)].abs().max()) == 0.0 if S > W - 1 else True
