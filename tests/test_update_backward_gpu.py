"""Backward of the decode step (dx, dconv_state, dweight, dbias) against torch autograd of the eager
step formulation (oracle/canon_grad.py, float64), by finite differences as the reference's own test
does (causal-conv1d-mps/test.py:294-321), and as a chain of steps against the backward of the prefill."""
import itertools

import pytest
import torch

from oracle.canon_grad import conv1d_grads, update_grads, update_grads_ext
from test_backward_gpu import check

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def cc():
    import causal_conv1d
    return causal_conv1d


def quantised(shape, dtype, scale=1.0):
    return (torch.randn(*shape) * scale).to(dtype)


def run_step(cc, x, state, w, b, dout, dstate_out, mask, act, residual):
    """One differentiable step on the GPU; the loss also reads the updated state when dstate_out is given."""
    xg = x.to(DEV).requires_grad_(True)
    s0 = state.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True) if b is not None else None
    s = s0.clone()                      # the in-place update needs a non-leaf tensor
    out = cc.causal_conv1d_update(xg, s, wg, bg, activation=act, residual=residual,
                                  token_mask=None if mask is None else mask.to(DEV))
    loss = (out.float() * dout.to(DEV).float()).sum()
    if dstate_out is not None:
        loss = loss + (s.float() * dstate_out.to(DEV).float()).sum()
    loss.backward()
    torch.cuda.synchronize()
    return xg.grad, s0.grad, wg.grad, (bg.grad if bg is not None else None), out.detach(), s.detach()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("S,W", [(3, 4), (4, 4), (8, 4), (2, 3), (5, 2)])
def test_update_backward_matches_autograd_of_the_eager_step(cc, dtype, S, W):
    torch.manual_seed(S * 10 + W)
    B, C = 5, 200
    for act, residual, use_mask, use_bias, through_state in itertools.product(
            [None, "silu"], [False, True, "unmasked"], [False, True], [True, False], [False, True]):
        if use_mask != (residual is not False) and act is None:
            continue                                   # thin the grid: 28 of the 48 combinations per shape
        x, st = quantised((B, C), dtype), quantised((B, C, S), dtype)
        w, b = quantised((C, W), dtype, 0.5), quantised((C,), dtype, 0.1) if use_bias else None
        dout = quantised((B, C), dtype)
        dso = quantised((B, C, S), dtype) if through_state else None
        mask = torch.tensor([1, 0, 1, 1, 0], dtype=torch.int64) if use_mask else None
        got = run_step(cc, x, st, w, b, dout, dso, mask, act, residual)
        want = update_grads(x, st, w, b, dout, dso, mask, act, residual)
        tag = f"{dtype} S{S} W{W} act={act} res={residual} mask={use_mask} bias={use_bias} state={through_state}"
        check(got[0], want[0], dtype, "dx " + tag)
        check(got[1], want[1], dtype, "dstate " + tag)
        check(got[2], want[2], dtype, "dweight " + tag, sum_terms=B)
        if use_bias:
            check(got[3], want[3], dtype, "dbias " + tag, sum_terms=B)
        # the state handed on is bit-exactly the shifted state with the (masked) token appended
        assert torch.equal(got[5].cpu().double(), want[5]), "state " + tag


def run_step_ext(cc, x, state, w, b, dout, dstate_out, mask, act, residual, seqlens, indices):
    """run_step in the ring-buffer / state-pool modes (state: the whole pool when indices are given)."""
    xg = x.to(DEV).requires_grad_(True)
    s0 = state.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True) if b is not None else None
    s = s0.clone()
    out = cc.causal_conv1d_update(xg, s, wg, bg, activation=act, residual=residual,
                                  token_mask=None if mask is None else mask.to(DEV),
                                  cache_seqlens=None if seqlens is None else seqlens.to(DEV),
                                  conv_state_indices=None if indices is None else indices.to(DEV))
    loss = (out.float() * dout.to(DEV).float()).sum()
    if dstate_out is not None:
        loss = loss + (s.float() * dstate_out.to(DEV).float()).sum()
    loss.backward()
    torch.cuda.synchronize()
    return xg.grad, s0.grad, wg.grad, (bg.grad if bg is not None else None), out.detach(), s.detach()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("S,W", [(3, 4), (4, 4), (8, 4), (2, 3), (5, 2)])
def test_update_backward_in_ring_buffer_and_state_pool_modes(cc, dtype, S, W):
    """The decode modes of upstream's signature: cache_seqlens (the mode the reference's own update autograd
    differentiates, causal_conv1d_mps/autograd.py:341-498) and conv_state_indices, alone and together, against
    torch autograd through the step written with gather / scatter."""
    torch.manual_seed(S * 10 + W + 100)
    B, C, R = 6, 72, 9
    seqlens = torch.tensor([0, 1, 5, 7, 2 * S + 1, 123], dtype=torch.int32)
    # a pool of nine rows: entries use rows 4, 0, 8, 2, a negative index and one past the pool skip their entries,
    # rows 1, 3, 5, 6, 7 are nobody's
    indices = torch.tensor([4, 0, -1, 8, 9, 2], dtype=torch.int32)
    for (ring, pool), act, residual, use_mask, through_state in itertools.product(
            [(True, False), (False, True), (True, True)], [None, "silu"], [False, True, "unmasked"], [False, True],
            [False, True]):
        if act is None and use_mask != (residual is not False):
            continue
        rows = R if pool else B
        x, st = quantised((B, C), dtype), quantised((rows, C, S), dtype)
        w, b = quantised((C, W), dtype, 0.5), quantised((C,), dtype, 0.1)
        dout = quantised((B, C), dtype)
        dso = quantised((rows, C, S), dtype) if through_state else None
        mask = torch.tensor([1, 0, 1, 1, 0, 1], dtype=torch.int64) if use_mask else None
        sl, ix = (seqlens if ring else None), (indices if pool else None)
        got = run_step_ext(cc, x, st, w, b, dout, dso, mask, act, residual, sl, ix)
        want = update_grads_ext(x, st, w, b, dout, dso, mask, act, residual, sl, ix)
        tag = f"{dtype} S{S} W{W} ring={ring} pool={pool} act={act} res={residual} mask={use_mask} state={through_state}"
        check(got[0], want[0], dtype, "dx " + tag)
        check(got[1], want[1], dtype, "dstate " + tag)
        live = B - 2 if pool else B
        check(got[2], want[2], dtype, "dweight " + tag, sum_terms=live)
        check(got[3], want[3], dtype, "dbias " + tag, sum_terms=live)
        assert torch.equal(got[5].cpu().double(), want[5]), "state " + tag
        if pool:
            # a skipped entry has a zero output row and a zero dx row; rows of the pool that no entry names hand
            # the gradient of the updated pool through untouched (zero when the loss does not read the pool)
            for e in (2, 4):
                assert not got[4][e].any() and not got[0][e].any(), tag
            for r in (1, 3, 5, 6, 7):
                passed = dso[r].to(DEV) if through_state else torch.zeros(C, S, dtype=dtype, device=DEV)
                assert torch.equal(got[1][r], passed), tag


def test_chain_of_ring_buffer_steps_has_the_gradients_of_the_shift_register_chain(cc):
    """T tokens through an 8-slot ring (cache_seqlens = 0, 1, 2, ...) and through the shift register, same start
    (the ring's slot j is the register's entry j at step 0): equal outputs, and bit-equal gradients of the tokens
    and parameters (the same products in the same order; only the slot arithmetic differs)."""
    torch.manual_seed(7)
    B, C, S, T = 3, 40, 8, 11
    w0, b0 = quantised((C, 4), torch.bfloat16, 0.5), quantised((C,), torch.bfloat16, 0.1)
    xs0 = quantised((T, B, C), torch.bfloat16)
    st0 = quantised((B, C, S), torch.bfloat16)
    results = []
    for ring in (False, True):
        w = w0.to(DEV).requires_grad_(True)
        b = b0.to(DEV).requires_grad_(True)
        xs = xs0.to(DEV).requires_grad_(True)
        s_leaf = st0.to(DEV).requires_grad_(True)
        s = s_leaf.clone()
        outs = []
        for t in range(T):
            sl = torch.full((B,), t, dtype=torch.int32, device=DEV) if ring else None
            outs.append(cc.causal_conv1d_update(xs[t], s, w, b, activation="silu", residual=True, cache_seqlens=sl))
        loss = sum((o.float() * (i + 1)).sum() for i, o in enumerate(outs)) + (s.float() ** 2).sum()
        loss.backward()
        results.append((torch.stack(outs).detach(), xs.grad, w.grad, b.grad, s_leaf.grad))
    (o0, dx0, dw0, db0, ds0), (o1, dx1, dw1, db1, ds1) = results
    assert torch.equal(o0, o1) and torch.equal(dx0, dx1) and torch.equal(dw0, dw1) and torch.equal(db0, db1)
    # the ring starts at slot 0 = the register's oldest entry, so the initial states coincide slot by slot
    assert torch.equal(ds0, ds1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_multi_part_decode_step_has_the_gradients_of_the_single_tensor_step(cc, dtype):
    """causal_conv1d_update_parts under autograd (q / k / v or gate / up tokens as separate tensors, one state):
    outputs, updated state and every gradient, the one through the updated state included, equal those of
    causal_conv1d_update on the concatenation (float64 autograd as the common yardstick)."""
    torch.manual_seed(41)
    for dims, S, act, residual, use_mask in [((24, 8, 8), 4, "silu", True, True), ((64, 64), 3, None, False, False),
                                             ((16, 40), 8, "silu", "unmasked", True)]:
        B, C = 5, sum(dims)
        x, st = quantised((B, C), dtype), quantised((B, C, S), dtype)
        w, b = quantised((C, 4), dtype, 0.5), quantised((C,), dtype, 0.1)
        dout, dso = quantised((B, C), dtype), quantised((B, C, S), dtype)
        mask = torch.tensor([1, 0, 1, 1, 0], dtype=torch.int64) if use_mask else None
        parts = [t.contiguous().to(DEV).requires_grad_(True) for t in x.split(list(dims), dim=1)]
        s0 = st.to(DEV).requires_grad_(True)
        wg, bg = w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
        s = s0.clone()
        outs = cc.causal_conv1d_update_parts(parts, s, wg, bg, activation=act, residual=residual,
                                             token_mask=None if mask is None else mask.to(DEV))
        loss = sum((o.float() * d.to(DEV).float()).sum() for o, d in zip(outs, dout.split(list(dims), dim=1)))
        (loss + (s.float() * dso.to(DEV).float()).sum()).backward()
        want = update_grads(x, st, w, b, dout, dso, mask, act, residual)
        tag = f"{dtype} dims{dims} S{S} act={act} res={residual} mask={use_mask}"
        check(torch.cat([p.grad for p in parts], dim=1), want[0], dtype, "dx " + tag)
        check(s0.grad, want[1], dtype, "dstate " + tag)
        check(wg.grad, want[2], dtype, "dweight " + tag, sum_terms=B)
        check(bg.grad, want[3], dtype, "dbias " + tag, sum_terms=B)
        assert torch.equal(s.detach().cpu().double(), want[5]), "state " + tag


def test_update_backward_finite_differences_like_the_reference_test(cc):
    """causal-conv1d-mps/test.py:294-321: batch 2, dim 8, width 4, state_len 8, SiLU, residual; eps 1e-3,
    atol 1e-3, rtol 1e-2, loss = out.sum() (test.py:8-80).  The state gradient is checked as well."""
    torch.manual_seed(0)
    B, C, W, S = 2, 8, 4, 8
    x = torch.randn(B, C, device=DEV, requires_grad=True)
    state = torch.randn(B, C, S, device=DEV, requires_grad=True)
    w = torch.randn(C, W, device=DEV, requires_grad=True)
    b = torch.randn(C, device=DEV, requires_grad=True)
    params = [x, state, w, b]

    def f():
        return cc.causal_conv1d_update(x, state.clone(), w, b, activation="silu", residual=True)

    f().sum().backward()
    analytic = [p.grad.clone() for p in params]
    eps = 1e-3
    with torch.no_grad():
        for p, a in zip(params, analytic):
            num = torch.zeros_like(p)
            for i in itertools.product(*[range(s) for s in p.shape]):
                old = p[i].item()
                p[i] = old + eps
                lp = f().double().sum().item()
                p[i] = old - eps
                lm = f().double().sum().item()
                p[i] = old
                num[i] = (lp - lm) / (2 * eps)
            assert torch.allclose(a, num, atol=1e-3, rtol=1e-2), (tuple(p.shape), (a - num).abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chain_of_steps_has_the_gradients_of_the_prefill(cc, dtype):
    """T decode steps from a zero state, differentiated end to end through the carried state, against the
    float64 gradient of the prefill over the same tokens, and against this library's own prefill backward."""
    torch.manual_seed(3)
    B, C, T, S, W = 3, 264, 7, 4, 4
    x, w, b = quantised((B, C, T), dtype), quantised((C, W), dtype, 0.5), quantised((C,), dtype, 0.1)
    dout = quantised((B, C, T), dtype)
    xg = x.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True)
    state = torch.zeros(B, C, S, dtype=dtype, device=DEV)
    outs = []
    for t in range(T):
        outs.append(cc.causal_conv1d_update(xg[:, :, t], state, wg, bg, activation="silu", residual=True))
    out = torch.stack(outs, dim=-1)
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    want = conv1d_grads(x, w, b, dout, activation="silu", residual=1)
    if dtype == torch.float32:
        check(xg.grad, want[0], dtype, "dx chain")
    else:
        # every step rounds the gradient it hands back through the state to the storage type (up to three
        # roundings on the way to a token): three ulps of the tensor's scale
        scale = want[0].abs().max().item()
        assert (xg.grad.cpu().double() - want[0]).abs().max().item() <= 3 * 2.0 ** -8 * scale
    if dtype == torch.float32:
        check(wg.grad, want[1], dtype, "dweight chain", sum_terms=B * T)
        check(bg.grad, want[2], dtype, "dbias chain", sum_terms=B * T)
    else:
        # autograd adds the T per-step parameter gradients in the parameters' 16-bit type: T roundings
        for got, ref in ((wg.grad, want[1]), (bg.grad, want[2])):
            assert (got.cpu().double() - ref).abs().max().item() <= T * 2.0 ** -8 * scale_of(ref)
    assert torch.equal(state[:, :, 1:].cpu(), x[:, :, T - 3:])       # and the state is the last tokens, bit for bit
    if dtype == torch.float32:
        x2 = x.to(DEV).requires_grad_(True)
        w2 = w.to(DEV).requires_grad_(True)
        cc.causal_conv1d_fn(x2, w2, b.to(DEV), activation="silu", residual=True).backward(dout.to(DEV))
        assert (x2.grad - xg.grad).abs().max().item() <= 2e-5 * scale_of(x2.grad)
        assert (w2.grad - wg.grad).abs().max().item() <= 1e-4 * scale_of(w2.grad)


def scale_of(t):
    return t.abs().max().item() + 1e-30


def test_update_backward_at_decode_shape_is_deterministic(cc):
    """B 256, C 3456, S 3 bf16 (the decode configuration): same bits on every run (fixed-order reduction,
    no float atomics), gradients within the bar of the float64 oracle; strided token and dout."""
    torch.manual_seed(5)
    B, C, S, W = 256, 3456, 3, 4
    dtype = torch.bfloat16
    x3 = quantised((B, C, 1), dtype)                       # the (batch, dim, 1) form: the token is a view
    st, w, b = quantised((B, C, S), dtype), quantised((C, W), dtype, 0.5), quantised((C,), dtype, 0.1)
    dout = quantised((B, C), dtype)
    runs = []
    for _ in range(2):
        xg = x3.to(DEV).requires_grad_(True)
        s0 = st.to(DEV).requires_grad_(True)
        wg = w.to(DEV).requires_grad_(True)
        bg = b.to(DEV).requires_grad_(True)
        out = cc.causal_conv1d_update(xg, s0.clone(), wg, bg, activation="silu")
        assert out.shape == (B, C, 1)
        out.backward(dout.to(DEV).unsqueeze(-1))
        torch.cuda.synchronize()
        runs.append((xg.grad[:, :, 0], s0.grad, wg.grad, bg.grad))
    for a, b_ in zip(*runs):
        assert torch.equal(a, b_)
    want = update_grads(x3[:, :, 0], st, w, b, dout, None, None, "silu", 0)
    check(runs[0][0], want[0], dtype, "dx")
    check(runs[0][1], want[1], dtype, "dstate")
    check(runs[0][2], want[2], dtype, "dweight", sum_terms=B)
    check(runs[0][3], want[3], dtype, "dbias", sum_terms=B)


def test_update_backward_argument_handling(cc):
    x = torch.randn(2, 8, device=DEV, requires_grad=True)
    w = torch.randn(8, 4, device=DEV)
    # the eager module's rounding points in the forward, the gradient of the unrounded step in the backward
    xe = x.detach().clone().requires_grad_(True)
    se, sf = torch.randn(2, 8, 4, device=DEV), None
    sf = se.clone()
    oe = cc.causal_conv1d_update(xe, se, w, activation="silu", rounding="eager")
    xf = x.detach().clone().requires_grad_(True)
    of = cc.causal_conv1d_update(xf, sf, w, activation="silu")
    oe.sum().backward()
    of.sum().backward()
    assert torch.allclose(oe, of, rtol=1e-5, atol=1e-6) and torch.equal(xe.grad, xf.grad)
    # a state that is a leaf requiring grad cannot be updated in place: torch says so itself
    with pytest.raises(RuntimeError, match="leaf"):
        cc.causal_conv1d_update(x, torch.zeros(2, 8, 4, device=DEV, requires_grad=True), w)
    # only the token needs a gradient: no parameter gradients are formed, the cache tensor is updated in place
    state = torch.randn(2, 8, 4, device=DEV)
    before = state.clone()
    out = cc.causal_conv1d_update(x, state, w)
    out.sum().backward()
    assert torch.equal(state[:, :, :3], before[:, :, 1:]) and torch.equal(state[:, :, 3], x.detach())
    assert torch.allclose(x.grad, w[:, 3].expand(2, 8))
    # under no_grad nothing is recorded and no copy of the state is made
    with torch.no_grad():
        assert not cc.causal_conv1d_update(x, state, w).requires_grad


def test_canon_layer_trains_through_single_token_steps(cc):
    """The drop-in CanonLayer fed token by token through its cache (model/model.py:270-317) has the
    parameter and input gradients of the same layer called once on the whole block (:587-675)."""
    import types
    from causal_conv1d.canon import CanonLayer
    torch.manual_seed(11)
    B, T, D = 3, 6, 192
    cfg = types.SimpleNamespace(canon_kernel=4, canon_bias=True, canon_activation=True)
    layer = CanonLayer(D, cfg, "a").to(DEV)
    layer.reset_parameters()
    x = torch.randn(B, T, D, device=DEV)
    dout = torch.randn(B, T, D, device=DEV)

    xb = x.clone().requires_grad_(True)
    layer(xb).backward(dout)
    want = (xb.grad.clone(), layer.weight.grad.clone(), layer.bias_param.grad.clone())
    layer.zero_grad()

    xs = x.clone().requires_grad_(True)
    cache = types.SimpleNamespace()
    ys = [layer(xs[:, t:t + 1], cache=cache, layer_idx=0) for t in range(T)]
    torch.cat(ys, dim=1).backward(dout)
    torch.cuda.synchronize()
    for got, ref, tol in zip((xs.grad, layer.weight.grad, layer.bias_param.grad), want, (2e-5, 1e-4, 1e-4)):
        assert (got - ref).abs().max().item() <= tol * scale_of(ref)


def test_canon_layer_prefill_then_steps_trains_like_the_block(cc):
    """Prefill with state capture, a continued chunk, then single-token steps, all through the layer's cache
    (model/model.py:470-489, 647-659, 270-317): the graph runs through the cached state, so inputs and
    parameters get the gradients of one call over the whole block."""
    import types
    from causal_conv1d.canon import CanonLayer
    torch.manual_seed(13)
    B, D, T1, T2, T3 = 2, 128, 9, 5, 3
    T = T1 + T2 + T3
    cfg = types.SimpleNamespace(canon_kernel=4, canon_bias=True, canon_activation=True)
    layer = CanonLayer(D, cfg, "a").to(DEV)
    layer.reset_parameters()
    x = torch.randn(B, T, D, device=DEV)
    dout = torch.randn(B, T, D, device=DEV)

    xb = x.clone().requires_grad_(True)
    layer(xb).backward(dout)
    want = (xb.grad.clone(), layer.weight.grad.clone(), layer.bias_param.grad.clone())
    layer.zero_grad()

    xs = x.clone().requires_grad_(True)
    cache = types.SimpleNamespace()
    ys = [layer(xs[:, :T1], cache=cache, layer_idx=0), layer(xs[:, T1:T1 + T2], cache=cache, layer_idx=0)]
    ys += [layer(xs[:, t:t + 1], cache=cache, layer_idx=0) for t in range(T1 + T2, T)]
    torch.cat(ys, dim=1).backward(dout)
    torch.cuda.synchronize()
    for got, ref, tol in zip((xs.grad, layer.weight.grad, layer.bias_param.grad), want, (2e-5, 1e-4, 1e-4)):
        assert (got - ref).abs().max().item() <= tol * scale_of(ref)
