"""Backward of the prefill (dx, dweight, dbias) against torch autograd of the reference's eager
formulation (oracle/canon_grad.py, float64), by finite differences as the reference's own tests
do (causal-conv1d-mps/test.py:8-80, 259-291), and through the drop-in CanonLayer."""
import itertools
import types

import pytest
import torch

from helpers import bits, right_padded_mask
from oracle.canon_grad import conv1d_grads

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def cc():
    import causal_conv1d
    return causal_conv1d


def gpu_grads(cc, x_cpu, w, b, dout_cpu, layout, mask=None, act=None, residual=False, seq_idx=None):
    xg = x_cpu.to(DEV)
    dg = dout_cpu.to(DEV)
    if layout == "blc":
        xg = xg.transpose(1, 2).contiguous().transpose(1, 2)
        dg = dg.transpose(1, 2).contiguous().transpose(1, 2)
    xg.requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True) if b is not None else None
    out = cc.causal_conv1d_fn(xg, wg, bg, activation=act,
                              attention_mask=None if mask is None else mask.to(DEV), residual=residual,
                              seq_idx=None if seq_idx is None else seq_idx.to(DEV))
    out.backward(dg)
    torch.cuda.synchronize()
    return xg.grad, wg.grad, (bg.grad if bg is not None else None), out.detach()


def check(got, want64, dtype, what, sum_terms=1):
    """dx-like tensors: fp32 to 2e-5 of the tensor's scale; 16-bit to 1 ulp of the rounded float64
    value.  Sums over `sum_terms` products are compared relative to the magnitude of the sum."""
    got = got.detach().cpu()
    if sum_terms > 1:
        # fp32 accumulation in a fixed order vs exact: 1e-4 of the tensor's scale; a 16-bit result is
        # additionally rounded once to its storage type (one ulp of its own value)
        scale = want64.abs().max().item() + 1e-30
        ulp = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
        err = (got.double() - want64).abs()
        bound = 1e-4 * scale + ulp * want64.abs()
        assert bool((err <= bound).all()), f"{what}: worst excess {(err - bound).max().item():.3e} (scale {scale:.3e})"
    elif dtype == torch.float32:
        scale = want64.abs().max().item() + 1e-30
        err = (got.double() - want64).abs().max().item() / scale
        assert err <= 2e-5, f"{what}: {err:.3e}"
    else:
        # one rounding to the storage type of a value computed in fp32 from a handful of terms that
        # may cancel: one ulp of the value plus 1e-5 of the tensor's scale
        scale = want64.abs().max().item() + 1e-30
        ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
        err = (got.double() - want64).abs()
        bound = ulp * want64.abs() + 1e-5 * scale
        assert bool((err <= bound).all()), f"{what}: worst excess {(err - bound).max().item():.3e} (scale {scale:.3e})"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["bcl", "blc"])
def test_backward_matches_autograd_of_the_eager_formulation(cc, dtype, layout):
    g = torch.Generator().manual_seed(17)
    shapes = [(2, 16, 40), (3, 24, 129), (1, 8, 5), (2, 40, 3), (4, 64, 256)]
    for (B, C, L), W in itertools.product(shapes, [2, 3, 4]):
        for has_bias, act, residual, has_mask in [(False, None, False, False), (True, "silu", "masked", True),
                                                  (True, None, "unmasked", True), (False, "silu", True, False)]:
            x = torch.randn(B, C, L, generator=g).to(dtype)
            w = (torch.randn(C, W, generator=g) * 0.5).to(dtype)
            b = (torch.randn(C, generator=g) * 0.2).to(dtype) if has_bias else None
            dout = torch.randn(B, C, L, generator=g).to(dtype)
            mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L) if has_mask else None
            dx, dw, db, out = gpu_grads(cc, x, w, b, dout, layout, mask, act, residual)
            rdx, rdw, rdb, _ = conv1d_grads(x, w, b, dout, mask, act, residual)
            what = f"{dtype} {layout} {B}x{C}x{L} W{W} bias{has_bias} {act} {residual} mask{has_mask}"
            assert dx.stride() == (x.to(DEV).stride() if layout == "bcl" else dx.stride())
            check(dx, rdx, dtype, what + " dx")
            check(dw, rdw, dtype, what + " dweight", sum_terms=B * L)
            if has_bias:
                check(db, rdb, dtype, what + " dbias", sum_terms=B * L)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_backward_blocks_that_walk_several_tiles(cc, dtype):
    """Channel-contiguous tensors large enough that a block walks more than one 32-step tile of its chunk
    (dz handed from tile to tile), with a ragged end (200 = 6 tiles + 8 steps), SiLU, mask and bias."""
    g = torch.Generator().manual_seed(29)
    B, C, L = 16, 2048, 200
    x = torch.randn(B, C, L, generator=g).to(dtype)
    w = (torch.randn(C, 4, generator=g) * 0.5).to(dtype)
    b = (torch.randn(C, generator=g) * 0.2).to(dtype)
    dout = torch.randn(B, C, L, generator=g).to(dtype)
    mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
    for act, residual, m in [("silu", "masked", mask), (None, "unmasked", mask), ("silu", False, None)]:
        dx, dw, db, _ = gpu_grads(cc, x, w, b, dout, "blc", m, act, residual)
        rdx, rdw, rdb, _ = conv1d_grads(x, w, b, dout, m, act, residual)
        what = f"{dtype} multi-tile {act} {residual} mask{m is not None}"
        check(dx, rdx, dtype, what + " dx")
        check(dw, rdw, dtype, what + " dweight", sum_terms=B * L)
        check(db, rdb, dtype, what + " dbias", sum_terms=B * L)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_time_contiguous_rows_with_partly_idle_vector_slots(cc, dtype):
    """Time-contiguous rows whose vector count is not a multiple of 64: the planner gives a lane 2 or 4 vectors
    to keep a row in one segment, so some of a lane's slots lie past the end of the row (65, 144 vectors),
    and rows that need two segments of four (300 vectors).  Forward and backward against the float64 oracle."""
    g = torch.Generator().manual_seed(30)
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    for nvec in (65, 144, 300):
        B, C, L = 2, 1024, nvec * E      # 2048 rows: enough for the planner to give a lane several vectors
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, 4, generator=g) * 0.5).to(dtype)
        b = (torch.randn(C, generator=g) * 0.2).to(dtype)
        dout = torch.randn(B, C, L, generator=g).to(dtype)
        mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
        for act, residual, m in [("silu", "masked", mask), (None, "unmasked", None)]:
            dx, dw, db, out = gpu_grads(cc, x, w, b, dout, "bcl", m, act, residual)
            rdx, rdw, rdb, rout = conv1d_grads(x, w, b, dout, m, act, residual)
            what = f"{dtype} {nvec} vectors {act} {residual} mask{m is not None}"
            check(out, rout, dtype, what + " out")
            check(dx, rdx, dtype, what + " dx")
            check(dw, rdw, dtype, what + " dweight", sum_terms=B * L)
            check(db, rdb, dtype, what + " dbias", sum_terms=B * L)


def test_backward_finite_differences_like_the_reference_tests(cc):
    """causal-conv1d-mps/test.py:259-272 and :275-291: eps 1e-3, atol 1e-3, rtol 1e-2, loss = out.sum()."""
    torch.manual_seed(0)
    for layout, (B, C, L) in itertools.product(["bcl", "blc"], [(2, 8, 16)]):
        x = torch.randn(B, C, L, device=DEV)
        if layout == "blc":
            x = x.transpose(1, 2).contiguous().transpose(1, 2)
        w = torch.randn(C, 4, device=DEV)
        b = torch.randn(C, device=DEV)
        mask = torch.ones(B, L, device=DEV)
        mask[1, 11:] = 0
        params = [x, w, b]

        def f():
            return cc.causal_conv1d_fn(x, w, b, activation="silu", attention_mask=mask, residual="unmasked")

        for p in params:
            p.requires_grad_(True)
            p.grad = None
        f().sum().backward()
        analytic = [p.grad.clone() for p in params]
        eps = 1e-3
        with torch.no_grad():
            for p, a in zip(params, analytic):
                num = torch.zeros_like(p)
                flat, nflat = p.view(-1) if p.is_contiguous() else None, None
                idx = list(itertools.product(*[range(s) for s in p.shape]))
                for i in idx:
                    old = p[i].item()
                    p[i] = old + eps
                    lp = f().double().sum().item()
                    p[i] = old - eps
                    lm = f().double().sum().item()
                    p[i] = old
                    num[i] = (lp - lm) / (2 * eps)
                assert torch.allclose(a, num, atol=1e-3, rtol=1e-2), (layout, (a - num).abs().max().item())


@pytest.mark.parametrize("layout", ["blc", "bcl"])
def test_backward_at_model_shape_is_deterministic_and_correct(cc, layout):
    g = torch.Generator().manual_seed(23)
    B, C, L = 4, 3456, 1024                      # Canon-D channel count, benchmark sequence length
    x = torch.randn(B, C, L, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.3).bfloat16()
    b = (torch.randn(C, generator=g) * 0.1).bfloat16()
    dout = torch.randn(B, C, L, generator=g).bfloat16()
    mask = right_padded_mask([1024, 800, 333, 128], L)
    dx, dw, db, _ = gpu_grads(cc, x, w, b, dout, layout, mask, None, "masked")
    dx2, dw2, db2, _ = gpu_grads(cc, x, w, b, dout, layout, mask, None, "masked")
    assert torch.equal(bits(dx), bits(dx2)) and torch.equal(bits(dw), bits(dw2)) and torch.equal(bits(db), bits(db2))
    rdx, rdw, rdb, _ = conv1d_grads(x, w, b, dout, mask, None, "masked")
    check(dx, rdx, torch.bfloat16, "model shape dx")
    check(dw, rdw, torch.bfloat16, "model shape dweight", sum_terms=B * L)
    check(db, rdb, torch.bfloat16, "model shape dbias", sum_terms=B * L)
    # fp32 master weights with bf16 activations (autocast-style): gradients come back in fp32
    xg = x.to(DEV).requires_grad_(True)
    w32 = w.float().to(DEV).requires_grad_(True)
    cc.causal_conv1d_fn(xg, w32, None, residual=True).backward(dout.to(DEV))
    assert w32.grad.dtype == torch.float32
    rdx, rdw, _, _ = conv1d_grads(x, w.float(), None, dout, None, None, 1)
    check(w32.grad, rdw, torch.float32, "fp32 weight grad", sum_terms=B * L)


def test_canon_layer_trains(cc):
    """One SGD step through the drop-in CanonLayer equals the same step through the eager restatement."""
    from causal_conv1d.canon import CanonLayer
    from oracle.canon_eager import EagerCanon
    torch.manual_seed(3)
    B, T, D = 3, 64, 96
    cfg = types.SimpleNamespace(canon_kernel=4, canon_bias=True, canon_activation=True)
    layer = CanonLayer(D, cfg, "a").to(DEV)
    layer.reset_parameters()
    x = torch.randn(B, T, D)
    mask = right_padded_mask([64, 40, 9], T)
    target = torch.randn(B, T, D)
    xg = x.to(DEV).requires_grad_(True)
    loss = ((layer(xg, attention_mask=mask.to(DEV)) - target.to(DEV)) ** 2).mean()
    loss.backward()
    w_ref = layer.weight.detach().cpu().double().requires_grad_(True)
    b_ref = layer.bias_param.detach().cpu().double().requires_grad_(True)
    x_ref = x.double().requires_grad_(True)
    ref_out = EagerCanon(w_ref, b_ref, True).forward(x_ref, mask.double())
    ((ref_out - target.double()) ** 2).mean().backward()
    torch.testing.assert_close(loss.item(), ((ref_out - target.double()) ** 2).mean().item(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(xg.grad.cpu().double(), x_ref.grad, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(layer.weight.grad.cpu().double(), w_ref.grad, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(layer.bias_param.grad.cpu().double(), b_ref.grad, rtol=1e-4, atol=1e-7)


def test_unsupported_gradients_raise(cc):
    x = torch.randn(2, 8, 16, device=DEV, requires_grad=True)
    w = torch.randn(8, 4, device=DEV)
    out, fs = cc.causal_conv1d_fn(x, w, return_final_states=True)
    assert out.requires_grad and fs.requires_grad          # the captured state is differentiable


def test_backward_more_than_2_31_elements(cc):
    """Index arithmetic past 32 bits in the backward kernels: dx of a batch row inside a 2.26e9-element
    call equals dx of that row differentiated alone (dx has no term across batch rows)."""
    B, C, L = 64, 3456, 10240
    g = torch.Generator(device=DEV).manual_seed(5)
    w = (torch.randn(C, 4, generator=g, device=DEV) * 0.3).bfloat16().requires_grad_(True)
    for layout in ("blc", "bcl"):
        shape = (B, L, C) if layout == "blc" else (B, C, L)
        x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        dout = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        for b in range(B):
            x[b].normal_(generator=g)
            dout[b].normal_(generator=g)
        if layout == "blc":
            x, dout = x.transpose(1, 2), dout.transpose(1, 2)
        x.requires_grad_(True)
        cc.causal_conv1d_fn(x, w, activation="silu", residual=True).backward(dout)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(w.grad).all())
        for b in (0, 40, 63):
            xb = x[b:b + 1].detach().requires_grad_(True)
            cc.causal_conv1d_fn(xb, w, activation="silu", residual=True).backward(dout[b:b + 1])
            assert torch.equal(bits(x.grad[b:b + 1]), bits(xb.grad)), (layout, b)
        w.grad = None
        del x, dout
        torch.cuda.empty_cache()


def test_backward_randomised(cc):
    """60 seeded random backward calls across layouts, sizes around the tile boundaries, dtypes, widths and options
    against float64 autograd of the eager formulation."""
    g = torch.Generator().manual_seed(777)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    def pick(seq):
        return seq[ri(0, len(seq) - 1)]

    for case in range(60):
        dtype = pick([torch.bfloat16, torch.float32, torch.float16])
        W = pick([2, 3, 4])
        B, C = ri(1, 3), pick([1, 4, 8, 12, 64, 100, 260])
        L = pick([1, 2, 3, 5, 31, 32, 33, 64, 65, 127, 128, 129, 200, 257])
        layout = pick(["bcl", "blc"])
        act, res = pick([None, "silu"]), pick([False, "masked", "unmasked"])
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.5).to(dtype)
        b = (torch.randn(C, generator=g) * 0.2).to(dtype) if ri(0, 1) else None
        dout = torch.randn(B, C, L, generator=g).to(dtype)
        mask = right_padded_mask([ri(1, L) for _ in range(B)], L) if ri(0, 1) else None
        dx, dw, db, _ = gpu_grads(cc, x, w, b, dout, layout, mask, act, res)
        rdx, rdw, rdb, _ = conv1d_grads(x, w, b, dout, mask, act, res)
        what = f"case {case}: {dtype} {layout} {B}x{C}x{L} W{W} {act} {res} mask{mask is not None} bias{b is not None}"
        check(dx, rdx, dtype, what + " dx")
        check(dw, rdw, dtype, what + " dweight", sum_terms=B * L)
        if b is not None:
            check(db, rdb, dtype, what + " dbias", sum_terms=B * L)


def packed_seq_idx(B, L, g, max_len):
    """[B, L] int32: each row cut into consecutive sequences of random lengths 1..max_len, numbered from 0."""
    q = torch.empty(B, L, dtype=torch.int32)
    for b in range(B):
        t, n = 0, 0
        while t < L:
            step = int(torch.randint(1, max_len + 1, (1,), generator=g))
            q[b, t:t + step] = n
            t, n = t + step, n + 1
    return q


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layout", ["bcl", "blc"])
def test_backward_of_packed_sequences(cc, dtype, layout):
    """Gradients of a call with seq_idx: no term may cross a sequence boundary, in dx (through the dz of
    later steps), in dweight or in the recomputed pre-activation.  Sequences shorter than the kernel
    width, boundaries next to chunk ends and a padding mask on top are all in the draw."""
    g = torch.Generator().manual_seed(4242)
    for case, (B, C, L, W, max_len) in enumerate([(2, 24, 97, 4, 9), (1, 7, 160, 3, 40), (3, 64, 33, 2, 3),
                                                  (2, 130, 515, 4, 64), (1, 8, 1, 4, 1), (2, 16, 1024, 4, 300)]):
        for act, res in ((None, False), ("silu", "masked"), ("silu", "unmasked")):
            x = torch.randn(B, C, L, generator=g).to(dtype)
            w = (torch.randn(C, W, generator=g) * 0.5).to(dtype)
            b = (torch.randn(C, generator=g) * 0.2).to(dtype) if case % 2 == 0 else None
            dout = torch.randn(B, C, L, generator=g).to(dtype)
            seq = packed_seq_idx(B, L, g, max_len)
            mask = right_padded_mask([max(1, L - 5 * i) for i in range(B)], L) if case % 3 == 0 else None
            dx, dw, db, out = gpu_grads(cc, x, w, b, dout, layout, mask, act, res, seq_idx=seq)
            rdx, rdw, rdb, rout = conv1d_grads(x, w, b, dout, mask, act, res, seq_idx=seq)
            what = f"case {case} {dtype} {layout} {B}x{C}x{L} W{W} {act} {res}"
            check(out, rout, dtype, what + " out")
            check(dx, rdx, dtype, what + " dx")
            check(dw, rdw, dtype, what + " dweight", sum_terms=B * L)
            if b is not None:
                check(db, rdb, dtype, what + " dbias", sum_terms=B * L)


def test_backward_of_packed_sequences_equals_the_sequences_on_their_own(cc):
    """Oracle-free: the gradients of a packed row are those of its sequences run as separate calls
    (dx cut out per sequence, dweight / dbias summed over them)."""
    g = torch.Generator().manual_seed(99)
    C, W = 48, 4
    lengths = [5, 1, 2, 40, 3, 77]
    L = sum(lengths)
    x = torch.randn(1, C, L, generator=g)
    w = torch.randn(C, W, generator=g) * 0.5
    b = torch.randn(C, generator=g) * 0.2
    dout = torch.randn(1, C, L, generator=g)
    seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lengths)]).unsqueeze(0)
    dx, dw, db, out = gpu_grads(cc, x, w, b, dout, "bcl", None, "silu", "unmasked", seq_idx=seq)
    dw_sum, db_sum, t = torch.zeros(C, W, dtype=torch.float64), torch.zeros(C, dtype=torch.float64), 0
    for n in lengths:
        sdx, sdw, sdb, sout = gpu_grads(cc, x[:, :, t:t + n].contiguous(), w, b, dout[:, :, t:t + n].contiguous(),
                                        "bcl", None, "silu", "unmasked")
        torch.testing.assert_close(out[:, :, t:t + n], sout, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(dx[:, :, t:t + n], sdx, rtol=1e-5, atol=1e-6)
        dw_sum += sdw.cpu().double()
        db_sum += sdb.cpu().double()
        t += n
    torch.testing.assert_close(dw.cpu().double(), dw_sum, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(db.cpu().double(), db_sum, rtol=1e-4, atol=1e-5)


def test_forward_and_backward_inside_a_captured_graph(cc):
    """A training step's Canon part (forward, backward with its reduction, scratch from torch's allocator)
    captured once as a device graph and replayed with new data between eager work: every replay must give
    what the eager call gives on the same data."""
    torch.manual_seed(31)
    B, L, C = 4, 256, 264
    x = torch.randn(B, L, C, device=DEV).bfloat16().requires_grad_()
    w = (torch.randn(C, 4, device=DEV) * 0.3).requires_grad_()
    b = (torch.randn(C, device=DEV) * 0.1).requires_grad_()
    mask = right_padded_mask([256, 100, 31, 200], L).to(DEV)
    dout = torch.randn(B, L, C, device=DEV).bfloat16()

    def step():
        y = cc.causal_conv1d_fn(x.transpose(1, 2), w, b, activation="silu", attention_mask=mask, residual=True)
        gx, gw, gb = torch.autograd.grad(y, (x, w, b), dout.transpose(1, 2))
        return y.detach(), gx, gw, gb

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture (library handles, allocator)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for i in range(4):
        with torch.no_grad():                    # new data in the captured tensors, eager work in between
            x.copy_(torch.randn(B, L, C, device=DEV).bfloat16())
            dout.copy_(torch.randn(B, L, C, device=DEV).bfloat16())
            w.mul_(1.01)
        want = [t.clone() for t in step()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, exp in zip(("y", "dx", "dweight", "dbias"), outs, want):
            assert torch.equal(bits(got), bits(exp)), (i, name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["bcl", "blc"])
def test_backward_through_initial_states(cc, dtype, layout):
    """A call continued from an initial state (the chunked continuation of model/model.py:647-659): dx, dweight,
    dbias and the gradient of the state itself against float64 autograd; rows shorter and longer than the
    history, several time chunks per row, all widths."""
    torch.manual_seed(17)
    for (B, C, L, S, W), act, residual, masked in itertools.product(
            [(2, 24, 1, 3, 4), (2, 24, 2, 4, 4), (3, 40, 5, 8, 4), (2, 16, 700, 3, 4), (2, 24, 37, 2, 3), (2, 24, 9, 4, 2),
             (2, 520, 70, 4, 4)],
            [None, "silu"], [False, True, "unmasked"], [False, True]):
        x = torch.randn(B, C, L).to(dtype)
        w, b = (torch.randn(C, W) * 0.5).to(dtype), (torch.randn(C) * 0.1).to(dtype)
        init = torch.randn(B, C, S).to(dtype)
        dout = torch.randn(B, C, L).to(dtype)
        mask = (torch.rand(B, L) > 0.3).to(torch.int64) if masked else None
        xg, dg = x.to(DEV), dout.to(DEV)
        if layout == "blc":
            xg = xg.transpose(1, 2).contiguous().transpose(1, 2)
            dg = dg.transpose(1, 2).contiguous().transpose(1, 2)
        xg.requires_grad_(True)
        wg, bg = w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
        ig = init.to(DEV).requires_grad_(True)
        out = cc.causal_conv1d_fn(xg, wg, bg, activation=act, initial_states=ig, residual=residual,
                                  attention_mask=None if mask is None else mask.to(DEV))
        out.backward(dg)
        torch.cuda.synchronize()
        want = conv1d_grads(x, w, b, dout, mask=mask, activation=act, residual=residual, initial_states=init)
        tag = f"{dtype} {layout} B{B} C{C} L{L} S{S} W{W} act={act} res={residual} mask={masked}"
        check(xg.grad, want[0], dtype, "dx " + tag)
        check(ig.grad, want[4], dtype, "dinit " + tag)
        check(wg.grad, want[1], dtype, "dweight " + tag, sum_terms=B * L)
        check(bg.grad, want[2], dtype, "dbias " + tag, sum_terms=B * L)
    # only the state needs a gradient
    ig = torch.randn(2, 8, 3, device=DEV, requires_grad=True)
    w = torch.randn(8, 4, device=DEV)
    cc.causal_conv1d_fn(torch.randn(2, 8, 6, device=DEV), w, initial_states=ig).sum().backward()
    want = torch.stack([w[:, 0], w[:, 0] + w[:, 1], w[:, 0] + w[:, 1] + w[:, 2]], dim=1).expand(2, 8, 3)
    assert torch.allclose(ig.grad, want, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layout", ["bcl", "blc"])
def test_backward_through_final_states(cc, dtype, layout):
    """A gradient that arrives through the captured final state (model/model.py:470-489 keeps the last
    inputs for the next call) reaches x, and initial_states where the state is longer than the row."""
    torch.manual_seed(23)
    for (B, C, L, S_in, S_out), act, residual, masked in itertools.product(
            [(2, 24, 40, 0, 4), (2, 24, 2, 3, 8), (3, 16, 5, 4, 3), (2, 16, 300, 0, 8), (2, 24, 1, 8, 4), (2, 520, 70, 3, 8)],
            [None, "silu"], [False, True], [False, True]):
        W = 4
        x = torch.randn(B, C, L).to(dtype)
        w, b = (torch.randn(C, W) * 0.5).to(dtype), (torch.randn(C) * 0.1).to(dtype)
        init = torch.randn(B, C, S_in).to(dtype) if S_in else None
        dout, dfin = torch.randn(B, C, L).to(dtype), torch.randn(B, C, S_out).to(dtype)
        mask = (torch.rand(B, L) > 0.3).to(torch.int64) if masked else None
        xg, dg = x.to(DEV), dout.to(DEV)
        if layout == "blc":
            xg = xg.transpose(1, 2).contiguous().transpose(1, 2)
            dg = dg.transpose(1, 2).contiguous().transpose(1, 2)
        xg.requires_grad_(True)
        wg, bg = w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
        ig = init.to(DEV).requires_grad_(True) if S_in else None
        out, fs = cc.causal_conv1d_fn(xg, wg, bg, activation=act, initial_states=ig, residual=residual,
                                      attention_mask=None if mask is None else mask.to(DEV),
                                      final_states_out=torch.empty(B, C, S_out, dtype=dtype, device=DEV))
        ((out.float() * dg.float()).sum() + (fs.float() * dfin.to(DEV).float()).sum()).backward()
        torch.cuda.synchronize()
        want = conv1d_grads(x, w, b, dout, mask=mask, activation=act, residual=residual, initial_states=init,
                            dfinal=dfin)
        tag = f"{dtype} {layout} B{B} C{C} L{L} S_in{S_in} S_out{S_out} act={act} res={residual} mask={masked}"
        check(xg.grad, want[0], dtype, "dx " + tag)
        if S_in:
            check(ig.grad, want[4], dtype, "dinit " + tag)
        check(wg.grad, want[1], dtype, "dweight " + tag, sum_terms=B * L)
        check(bg.grad, want[2], dtype, "dbias " + tag, sum_terms=B * L)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_multi_part_call_differentiates_through_both_states(cc, dtype):
    """causal_conv1d_fn_parts with initial_states and a captured final state that the loss reads: the gradients of
    every part, of weight / bias and of the initial state against float64 autograd on the concatenation, and
    against the single-tensor call on the concatenation (same kernels on the same rows: same bits)."""
    torch.manual_seed(31)
    for dims, L, S_in, S_out, act, residual, masked in [((24, 8, 8), 40, 3, 4, "silu", True, True),
                                                       ((64, 64), 70, 4, 8, None, False, False),
                                                       ((16, 40), 2, 8, 3, "silu", "unmasked", True),
                                                       ((520, 8, 1032, 64), 33, 3, 8, None, True, False)]:
        B, C, W = 2, sum(dims), 4
        x = torch.randn(B, C, L).to(dtype)
        w, b = (torch.randn(C, W) * 0.5).to(dtype), (torch.randn(C) * 0.1).to(dtype)
        init = torch.randn(B, C, S_in).to(dtype)
        dout, dfin = torch.randn(B, C, L).to(dtype), torch.randn(B, C, S_out).to(dtype)
        mask = (torch.rand(B, L) > 0.3).to(torch.int64) if masked else None
        mg = None if mask is None else mask.to(DEV)

        def leaves():
            parts = [t.transpose(1, 2).contiguous().to(DEV).transpose(1, 2).requires_grad_(True) for t in x.split(list(dims), dim=1)]
            return parts, w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True), init.to(DEV).requires_grad_(True)

        parts, wg, bg, ig = leaves()
        outs, fs = cc.causal_conv1d_fn_parts(parts, wg, bg, activation=act, initial_states=ig, residual=residual,
                                             attention_mask=mg, final_states_out=torch.empty(B, C, S_out, dtype=dtype, device=DEV))
        loss = sum((o.float() * d.to(DEV).float()).sum() for o, d in zip(outs, dout.split(list(dims), dim=1)))
        (loss + (fs.float() * dfin.to(DEV).float()).sum()).backward()
        torch.cuda.synchronize()
        want = conv1d_grads(x, w, b, dout, mask=mask, activation=act, residual=residual, initial_states=init, dfinal=dfin)
        tag = f"{dtype} dims{dims} L{L} S_in{S_in} S_out{S_out} act={act} res={residual} mask={masked}"
        dx = torch.cat([p.grad.contiguous() for p in parts], dim=1)
        check(dx, want[0], dtype, "dx " + tag)
        check(ig.grad, want[4], dtype, "dinit " + tag)
        check(wg.grad, want[1], dtype, "dweight " + tag, sum_terms=B * L)
        check(bg.grad, want[2], dtype, "dbias " + tag, sum_terms=B * L)
        # the single-tensor call on the concatenation
        parts1, w1, b1, i1 = leaves()
        xcat = torch.cat([p.detach() for p in parts1], dim=1).transpose(1, 2).contiguous().transpose(1, 2).requires_grad_(True)
        out1, fs1 = cc.causal_conv1d_fn(xcat, w1, b1, activation=act, initial_states=i1, residual=residual, attention_mask=mg,
                                        final_states_out=torch.empty(B, C, S_out, dtype=dtype, device=DEV))
        ((out1.float() * dout.to(DEV).float()).sum() + (fs1.float() * dfin.to(DEV).float()).sum()).backward()
        assert torch.equal(bits(dx), bits(xcat.grad.contiguous())), "dx vs concatenation " + tag
        assert torch.equal(bits(ig.grad), bits(i1.grad)), "dinit vs concatenation " + tag
        assert torch.equal(bits(fs), bits(fs1)), tag


def test_block_in_two_chunks_trains_like_the_block_in_one_go(cc):
    """Prefill of a first chunk with state capture, the second chunk continued from that state: the gradient
    flows through the state, so x, weight and bias get the gradients of the single call over both chunks."""
    torch.manual_seed(29)
    B, C, L1, L2, S = 2, 48, 37, 21, 4
    x = torch.randn(B, C, L1 + L2, device=DEV)
    w, b = torch.randn(C, 4, device=DEV) * 0.5, torch.randn(C, device=DEV) * 0.1
    dout = torch.randn(B, C, L1 + L2, device=DEV)
    mask = (torch.rand(B, L1 + L2, device=DEV) > 0.2).to(torch.int64)

    x1, w1, b1 = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    cc.causal_conv1d_fn(x1, w1, b1, activation="silu", attention_mask=mask, residual=True).backward(dout)

    x2, w2, b2 = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    o1, state = cc.causal_conv1d_fn(x2[:, :, :L1], w2, b2, activation="silu", attention_mask=mask[:, :L1],
                                    residual=True, final_states_out=torch.empty(B, C, S, device=DEV))
    o2 = cc.causal_conv1d_fn(x2[:, :, L1:], w2, b2, activation="silu", attention_mask=mask[:, L1:], residual=True,
                             initial_states=state)
    torch.cat([o1, o2], dim=2).backward(dout)
    torch.cuda.synchronize()
    for got, ref, tol in ((x2.grad, x1.grad, 2e-5), (w2.grad, w1.grad, 1e-4), (b2.grad, b1.grad, 1e-4)):
        assert (got - ref).abs().max().item() <= tol * (ref.abs().max().item() + 1e-30)
