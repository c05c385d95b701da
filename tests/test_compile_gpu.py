"""The package under torch.compile: the reference compiles its whole model (trainer/train_pretrain.py:39,
trainer/train_full_sft.py:54, eval_model.py:157 with fullgraph=True), so the calls must trace without a
graph break and the traced graph must launch the same kernels as the eager call (same bits)."""
import types

import pytest
import torch

from helpers import bits, right_padded_mask

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def cc():
    import causal_conv1d
    return causal_conv1d


@pytest.fixture(autouse=True)
def fresh_dynamo():
    torch._dynamo.reset()
    yield
    torch._dynamo.reset()


def graphs_of(fn, *args):
    """(result, list of traced graphs) of fn compiled with fullgraph=True; the backend runs the graph as it is."""
    seen = []

    def backend(gm, example_inputs):
        seen.append(gm)
        return gm.forward

    out = torch.compile(fn, backend=backend, fullgraph=True)(*args)
    return out, seen


def op_names(gm):
    return [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]


def test_prefill_traces_as_one_operator_and_matches_eager(cc):
    torch.manual_seed(0)
    B, L, C = 4, 300, 264
    x = torch.randn(B, L, C, device=DEV).bfloat16()
    w = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()
    b = (torch.randn(C, device=DEV) * 0.1).bfloat16()
    mask = right_padded_mask([300, 17, 128, 299], L, dtype=torch.int64).to(DEV)

    def f(x, w, b, mask):
        # what CanonLayer does around the call (model/model.py:454-466, 491)
        y = cc.causal_conv1d_fn(x.transpose(1, 2), w, b, activation="silu", attention_mask=mask, residual=True)
        return y.transpose(1, 2) * 2.0

    want = f(x, w, b, mask)
    got, seen = graphs_of(f, x, w, b, mask)
    assert len(seen) == 1 and any("canon_conv1d.fwd" in n for n in op_names(seen[0])), op_names(seen[0])
    assert torch.equal(bits(got), bits(want))

    # final states through the traced graph: the caller's tensor is filled
    def g(x, w, state):
        y, st = cc.causal_conv1d_fn(x.transpose(1, 2), w, final_states_out=state)
        return y, st

    st_e = torch.zeros(B, C, 8, device=DEV, dtype=torch.bfloat16)
    st_c = torch.zeros_like(st_e)
    y_e, _ = g(x, w, st_e)
    (y_c, st_ret), _ = graphs_of(g, x, w, st_c)
    assert torch.equal(bits(y_c), bits(y_e)) and torch.equal(bits(st_c), bits(st_e)) and torch.equal(bits(st_ret), bits(st_e))


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_training_step_has_the_eager_gradients(cc, backend):
    torch.manual_seed(1)
    B, L, C = 2, 256, 128
    x0 = torch.randn(B, L, C, device=DEV).bfloat16()
    w0 = torch.randn(C, 4, device=DEV) * 0.3          # fp32 master weights, bf16 activations
    b0 = torch.randn(C, device=DEV) * 0.1
    mask = right_padded_mask([256, 100], L, dtype=torch.int64).to(DEV)
    dout = torch.randn(B, L, C, device=DEV).bfloat16()

    def step(fn):
        x, w, b = x0.clone().requires_grad_(), w0.clone().requires_grad_(), b0.clone().requires_grad_()
        y = fn(x, w, b)
        y.backward(dout)
        return y.detach(), x.grad, w.grad, b.grad

    def f(x, w, b):
        h = x * 1.5
        y = cc.causal_conv1d_fn(h.transpose(1, 2), w, b, attention_mask=mask, residual=True).transpose(1, 2)
        return y + 1.0

    want = step(f)
    got = step(torch.compile(f, backend=backend, fullgraph=True))
    for name, a, e in zip(("y", "dx", "dweight", "dbias"), got, want):
        if backend == "inductor" and name in ("y", "dx"):
            # the surrounding elementwise ops are fused by the compiler and may round once less
            torch.testing.assert_close(a.float(), e.float(), rtol=2e-2, atol=2e-2, msg=name)
        else:
            assert torch.equal(bits(a), bits(e)), name


def test_compiled_training_step_over_packed_sequences(cc):
    """seq_idx travels through the traced forward into the traced backward."""
    torch.manual_seed(11)
    B, L, C = 2, 96, 64
    x0 = torch.randn(B, L, C, device=DEV)
    w0 = torch.randn(C, 4, device=DEV) * 0.3
    seq = torch.tensor([[0] * 10 + [1] * 2 + [2] * 84, [0] * 50 + [1] * 46], dtype=torch.int32, device=DEV)
    dout = torch.randn(B, L, C, device=DEV)

    def step(fn):
        x, w = x0.clone().requires_grad_(), w0.clone().requires_grad_()
        y = fn(x, w)
        y.backward(dout)
        return y.detach(), x.grad, w.grad

    def f(x, w):
        return cc.causal_conv1d_fn(x.transpose(1, 2), w, None, activation="silu", seq_idx=seq).transpose(1, 2)

    want = step(f)
    got = step(torch.compile(f, backend="aot_eager", fullgraph=True))
    for name, a, e in zip(("y", "dx", "dweight"), got, want):
        assert torch.equal(bits(a), bits(e)), name


def test_decode_step_traces_and_updates_the_state_in_place(cc):
    torch.manual_seed(2)
    B, C, S = 8, 264, 4
    w = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()
    st_e = torch.randn(B, C, S, device=DEV).bfloat16()
    st_c = st_e.clone()
    tm = torch.tensor([1, 0, 1, 1, 1, 0, 1, 1], device=DEV)

    def f(tok, state):
        return cc.causal_conv1d_update(tok, state, w, None, None, token_mask=tm, residual=True) + 0.0

    for step in range(3):
        tok = torch.randn(B, C, device=DEV).bfloat16()
        want = f(tok, st_e)
        got, seen = graphs_of(f, tok, st_c)
        assert len(seen) == 1 and any("canon_conv1d.update" in n for n in op_names(seen[0]))
        assert torch.equal(bits(got), bits(want)) and torch.equal(bits(st_c), bits(st_e)), step


def test_multi_part_calls_trace(cc):
    torch.manual_seed(3)
    B, L, dims = 2, 96, (64, 16, 16)
    C = sum(dims)
    qkv = [torch.randn(B, L, d, device=DEV).bfloat16() for d in dims]
    w = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()
    st_e = torch.zeros(B, C, 8, device=DEV, dtype=torch.bfloat16)
    st_c = torch.zeros_like(st_e)

    def prefill(q, k, v, state):
        outs, _ = cc.causal_conv1d_fn_parts([t.transpose(1, 2) for t in (q, k, v)], w, final_states_out=state,
                                            residual=True)
        return [o.transpose(1, 2) for o in outs]

    want = prefill(*qkv, st_e)
    got, seen = graphs_of(prefill, *qkv, st_c)
    assert len(seen) == 1 and any("canon_conv1d.fwd_parts" in n for n in op_names(seen[0]))
    assert all(torch.equal(bits(a), bits(e)) for a, e in zip(got, want)) and torch.equal(bits(st_c), bits(st_e))

    def decode(q, k, v, state):
        return list(cc.causal_conv1d_update_parts([q, k, v], state, w, residual=True))

    toks = [torch.randn(B, d, device=DEV).bfloat16() for d in dims]
    want = decode(*toks, st_e)
    got, seen = graphs_of(decode, *toks, st_c)
    assert len(seen) == 1 and any("canon_conv1d.update_parts" in n for n in op_names(seen[0]))
    assert all(torch.equal(bits(a), bits(e)) for a, e in zip(got, want)) and torch.equal(bits(st_c), bits(st_e))


def test_canon_layer_module_compiles_without_a_graph_break(cc):
    from causal_conv1d.canon import CanonLayer
    torch.manual_seed(4)
    cfg = types.SimpleNamespace(canon_kernel=4, canon_bias=False, canon_activation=False)
    layer = CanonLayer(128, cfg, "a").to(device=DEV, dtype=torch.bfloat16)
    x = torch.randn(2, 200, 128, device=DEV).bfloat16()
    mask = right_padded_mask([200, 77], 200, dtype=torch.int64).to(DEV)
    with torch.no_grad():
        want = layer(x, mask)
        got, seen = graphs_of(lambda x, mask: layer(x, mask), x, mask)
    assert len(seen) == 1 and any("canon_conv1d.fwd" in n for n in op_names(seen[0]))
    assert torch.equal(bits(got), bits(want))


def test_decode_under_cuda_graph_trees(cc):
    """mode='reduce-overhead' (eval_model.py:157): the compiler may capture the step in a device graph (it
    decides per graph, e.g. not when it sees its inputs mutated).  Either way the kernel is launched on
    torch's current stream and allocates through torch, so repeated calls stay correct."""
    torch.manual_seed(5)
    B, C, S = 16, 640, 4
    w = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()
    st_e = torch.randn(B, C, S, device=DEV).bfloat16()
    st_c = st_e.clone()

    def f(tok, state):
        return cc.causal_conv1d_update(tok * 1.0, state, w, residual=True) * 1.0

    fc = torch.compile(f, mode="reduce-overhead", fullgraph=True)
    for step in range(6):
        tok = torch.randn(B, C, device=DEV).bfloat16()
        want = f(tok, st_e)
        got = fc(tok, st_c).clone()
        torch.cuda.synchronize()
        assert torch.equal(bits(got), bits(want)) and torch.equal(bits(st_c), bits(st_e)), step


def test_the_reference_modules_accelerated_branch_compiles_whole(cc):
    """The statements of the reference CanonLayer's accelerated branches (model/model.py:427-495 prefill,
    :293-317 decode: try / except around the calls, the reference's keywords, state by slicing), traced with
    fullgraph=True as eval_model.py:157 does, against the same statements run eagerly."""
    torch.manual_seed(6)
    B, T, D, K = 4, 50, 640, 4
    weight = (torch.randn(D, 1, K, device=DEV) * 0.3).bfloat16()      # the module's parameter shape
    mask = right_padded_mask([50, 31, 4, 17], T).to(DEV)

    def prefill(x, weight, mask):
        try:
            masked_x = x * mask.unsqueeze(-1).to(x.dtype)
            x_conv = masked_x.transpose(1, 2)
            output = cc.causal_conv1d_fn(x=x_conv, weight=weight.squeeze(1), bias=None, activation=None, seq_idx=None)
            conv_state = torch.zeros(x.shape[0], x.shape[2], K, device=x.device, dtype=x.dtype)
            conv_state[:, :, :] = x_conv[:, :, -K:]
            return x + output.transpose(1, 2), conv_state
        except Exception as e:      # the reference prints and falls back to its eager path here
            raise AssertionError(f"accelerated branch failed: {e}")

    def decode(x_token, conv_state, weight):
        try:
            y = cc.causal_conv1d_update(x=x_token, conv_state=conv_state, weight=weight.squeeze(1), bias=None,
                                        activation=None)
            return x_token + y
        except Exception as e:
            raise AssertionError(f"accelerated branch failed: {e}")

    x = torch.randn(B, T, D, device=DEV).bfloat16()
    want, state_e = prefill(x, weight, mask)
    (got, state_c), seen = graphs_of(prefill, x, weight, mask)
    assert len(seen) == 1 and torch.equal(bits(got), bits(want)) and torch.equal(bits(state_c), bits(state_e))
    for step in range(3):
        tok = torch.randn(B, D, device=DEV).bfloat16()
        want = decode(tok, state_e, weight)
        got, seen = graphs_of(decode, tok, state_c, weight)
        assert len(seen) == 1 and torch.equal(bits(got), bits(want)) and torch.equal(bits(state_c), bits(state_e)), step


def test_whole_model_with_canon_layers_and_caches_traces_as_one_graph(cc):
    """A Viby-shaped model (Canon A-D on the HIP CanonLayer, conv states on the cache object, q/k/v and gate/up
    either concatenated or as parts): prefill and single-token steps each trace without a graph break and
    reproduce the eager logits."""
    import viby_harness as vh
    from causal_conv1d.canon import CanonLayer

    class Cache:   # a plain object, as the HF cache the reference hangs its lists on (model/model.py:227-241)
        def __init__(self, n):
            self._max_layers, self.kv, self.seen = n, [None] * n, 0

    cfg = vh.viby_config(num_hidden_layers=2, hidden_size=128, intermediate_size=256, vocab_size=512)
    for parts in (False, True):
        model = vh.init_weights(vh.VibyShaped(cfg, lambda C, name: CanonLayer(C, cfg, name), parts=parts), 0,
                                torch.bfloat16, DEV).eval()
        ids = torch.randint(0, 512, (2, 40), generator=torch.Generator().manual_seed(7)).to(DEV)
        steps = [ids] + [torch.randint(0, 512, (2, 1), generator=torch.Generator().manual_seed(8 + i)).to(DEV)
                         for i in range(2)]
        with torch.no_grad():
            cache_e, cache_c = Cache(cfg.num_hidden_layers), Cache(cfg.num_hidden_layers)
            seen_tokens = 0
            for i, tok in enumerate(steps):
                seen_tokens += tok.shape[1]
                mask = torch.ones(2, seen_tokens, dtype=torch.int64, device=DEV)
                want = model.forward(tok, cache_e, mask)
                torch._dynamo.reset()
                got, seen = graphs_of(model.forward, tok, cache_c, mask)
                assert len(seen) == 1, (parts, i, len(seen))
                assert torch.equal(got, want), (parts, i)
                for site in "abcd":
                    for a, e in zip(getattr(cache_c, f"canon_cache_{site}"), getattr(cache_e, f"canon_cache_{site}")):
                        assert torch.equal(bits(a), bits(e)), (parts, i, site)


def test_compiled_training_through_the_multi_part_call(cc):
    """Traced training graphs differentiate through the multi-part operator (one fused backward per part on
    its rows of the weights, as the eager path): same bits."""
    torch.manual_seed(9)
    B, L, dims = 2, 128, (64, 32)
    C = sum(dims)
    parts0 = [torch.randn(B, L, d, device=DEV).bfloat16() for d in dims]
    w0 = torch.randn(C, 4, device=DEV) * 0.3
    douts = [torch.randn(B, L, d, device=DEV).bfloat16() for d in dims]

    def step(fn):
        xs = [p.clone().requires_grad_() for p in parts0]
        w = w0.clone().requires_grad_()
        outs = fn(xs[0], xs[1], w)
        torch.autograd.backward(outs, douts)
        return [o.detach() for o in outs], [x.grad for x in xs], w.grad

    def f(a, b, w):
        outs = cc.causal_conv1d_fn_parts([a.transpose(1, 2), b.transpose(1, 2)], w, activation="silu", residual=True)
        return [o.transpose(1, 2) for o in outs]

    outs_e, dx_e, dw_e = step(f)
    outs_c, dx_c, dw_c = step(torch.compile(f, backend="aot_eager", fullgraph=True))
    for a, e in zip(outs_c + dx_c + [dw_c], outs_e + dx_e + [dw_e]):
        assert torch.equal(bits(a), bits(e))


def test_compiled_training_through_the_captured_state(cc):
    """A block processed as two chunks inside one traced function, the second continued from the state the
    first captured: the traced operators pass the state's gradient on, as the eager calls do."""
    torch.manual_seed(7)
    B, C, L1, L2, S = 2, 64, 40, 24, 4
    x0 = torch.randn(B, C, L1 + L2, device=DEV)
    w0, b0 = torch.randn(C, 4, device=DEV) * 0.3, torch.randn(C, device=DEV) * 0.1
    dout = torch.randn(B, C, L1 + L2, device=DEV)

    def whole(x, w, b):
        return cc.causal_conv1d_fn(x, w, b, activation="silu", residual=True)

    def chunked(x, w, b):
        o1, state = cc.causal_conv1d_fn(x[:, :, :L1], w, b, activation="silu", residual=True,
                                        final_states_out=torch.empty(B, C, S, device=DEV))
        o2 = cc.causal_conv1d_fn(x[:, :, L1:], w, b, activation="silu", residual=True, initial_states=state)
        return torch.cat([o1, o2], dim=2)

    def step(fn):
        x, w, b = x0.clone().requires_grad_(), w0.clone().requires_grad_(), b0.clone().requires_grad_()
        y = fn(x, w, b)
        y.backward(dout)
        return y.detach(), x.grad, w.grad, b.grad

    want = step(whole)
    for fn in (chunked, torch.compile(chunked, backend="aot_eager", fullgraph=True)):
        got = step(fn)
        for name, a, e, tol in zip(("y", "dx", "dweight", "dbias"), got, want, (1e-6, 2e-5, 1e-4, 1e-4)):
            assert (a - e).abs().max().item() <= tol * (e.abs().max().item() + 1e-30), name


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("mode", ["shift", "ring"])
def test_compiled_decode_steps_have_the_eager_gradients(cc, backend, mode):
    """A chain of single-token steps traced with gradients (the step as a function with its backward registered,
    the state overwritten by a copy the tracer understands): outputs, final state and every gradient, the one
    that flows from step to step through the state included, equal those of the same chain run eagerly."""
    torch.manual_seed(11)
    B, C, S, T = 4, 128, 4, 3
    xs0 = torch.randn(T, B, C, device=DEV).bfloat16()
    st0 = torch.randn(B, C, S, device=DEV).bfloat16()
    w0 = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()
    b0 = (torch.randn(C, device=DEV) * 0.1).bfloat16()
    tm = torch.tensor([1, 1, 0, 1], device=DEV)
    seqlens = [torch.full((B,), 5 + t, dtype=torch.int32, device=DEV) if mode == "ring" else None for t in range(T)]

    def chain(xs, state0, w, b):
        s = state0.clone()
        outs = []
        for t in range(T):
            outs.append(cc.causal_conv1d_update(xs[t], s, w, b, activation="silu", token_mask=tm, residual=True,
                                                cache_seqlens=seqlens[t]))
        return torch.stack(outs), s

    def run(fn):
        xs, st, w, b = (t.clone().requires_grad_() for t in (xs0, st0, w0, b0))
        outs, s = fn(xs, st, w, b)
        loss = (outs.float() * torch.arange(1, T + 1, device=DEV).view(T, 1, 1)).sum() + (s.float() ** 2).sum()
        loss.backward()
        return outs.detach(), s.detach(), xs.grad, st.grad, w.grad, b.grad

    want = run(chain)
    got = run(torch.compile(chain, backend=backend, fullgraph=True))
    for name, a, e in zip(("out", "state", "dx", "dstate", "dweight", "dbias"), got, want):
        if backend == "inductor" and name in ("dweight", "dbias"):
            # the three steps' bf16 contributions are added up by the compiler in one fused kernel (one rounding)
            # and by eager autograd one after the other (two)
            torch.testing.assert_close(a.float(), e.float(), rtol=2e-2, atol=2e-2, msg=name)
        else:
            assert torch.equal(bits(a), bits(e)), name


def test_compiled_decode_step_with_gradients_on_a_cache_tensor(cc):
    """The state as an argument of the traced function (a cache tensor that lives outside it, as CanonLayer keeps
    it): each compiled call overwrites it, and the gradient flows back through it from call to call."""
    torch.manual_seed(12)
    B, C, S, T = 2, 64, 4, 3
    xs0 = torch.randn(T, B, C, device=DEV).bfloat16()
    w0 = (torch.randn(C, 4, device=DEV) * 0.3).bfloat16()

    def step(x, state, w):
        return cc.causal_conv1d_update(x, state, w, residual=True) * 2.0

    def run(fn):
        xs, w = xs0.clone().requires_grad_(), w0.clone().requires_grad_()
        state = torch.zeros(B, C, S, device=DEV, dtype=torch.bfloat16)
        outs = [fn(xs[t], state, w) for t in range(T)]
        (torch.stack(outs).float().sum() + (state.float() ** 2).sum()).backward()
        return torch.stack(outs).detach(), state.detach(), xs.grad, w.grad

    want = run(step)
    got = run(torch.compile(step, backend="aot_eager", fullgraph=True))
    for name, a, e in zip(("out", "state", "dx", "dweight"), got, want):
        assert torch.equal(bits(a), bits(e)), name
