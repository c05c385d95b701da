"""Channel ranges as separate tensors (q/k/v for Canon-B, gate/up for Canon-D,
model/model.py:772-789 and 962-971) vs the CPU oracle on the concatenated input, and vs the
single-tensor HIP call on the concatenation (those two must agree bit for bit: same arithmetic,
only the addressing differs).
"""
import itertools

import pytest
import torch

from helpers import assert_parity, bits, right_padded_mask
from oracle import canon_oracle as co

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def cc():
    import causal_conv1d
    return causal_conv1d


def blc_parts(x_cat_cpu, dims, how):
    """The channel ranges of a logical [B, C, L] tensor as channel-contiguous [B, C_i, L] views on the GPU:
    'separate' = one (B, L, C_i) allocation per part; 'sliced' = views into one (B, L, C) projection output."""
    if how == "sliced":
        full = x_cat_cpu.transpose(1, 2).contiguous().to(DEV)          # (B, L, C)
        return [t.transpose(1, 2) for t in full.split(dims, dim=2)]
    return [t.transpose(1, 2).contiguous().to(DEV).transpose(1, 2) for t in x_cat_cpu.split(dims, dim=1)]


@pytest.mark.parametrize("dims", [(640, 160, 160), (1728, 1728), (520, 8, 1032, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_prefill_parts_one_launch(cc, dims, dtype):
    g = torch.Generator().manual_seed(sum(dims))
    B, L, C = 3, 200, sum(dims)
    x = torch.randn(B, C, L, generator=g).to(dtype)
    w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype)
    mask = right_padded_mask([200, 131, 7], L)
    init = torch.randn(B, C, 8, generator=g).to(dtype)
    for how, act, use_mask, use_state in itertools.product(["separate", "sliced"], [None, "silu"], [False, True],
                                                           [False, True]):
        m = mask if use_mask else None
        want = co.conv1d_fwd(x, w, b, mask=m, activation=act, residual=1,
                             initial_state=init if use_state else None, final_state_len=8 if use_state else None)
        want_out, want_state = want if use_state else (want, None)
        xs = blc_parts(x, list(dims), how)
        # two dense tensors of one shape take the pair launch, everything else the launch over a table of parts
        pair = len(dims) == 2 and dims[0] == dims[1] and how == "separate"
        assert cc.kernel_plan_fwd_parts(xs, w.to(DEV)) == ("blc_vec_pair" if pair else "blc_vec_parts")
        fs = torch.full((B, C, 8), float("nan"), dtype=dtype, device=DEV) if use_state else None
        r = cc.causal_conv1d_fn_parts(xs, w.to(DEV), b.to(DEV), activation=act, residual="masked",
                                      attention_mask=None if m is None else m.to(DEV),
                                      initial_states=init.to(DEV) if use_state else None, final_states_out=fs)
        outs = r[0] if use_state else r
        what = f"parts/{dims}/{dtype}/{how}/{act}/mask{use_mask}/state{use_state}"
        assert all(o.stride(1) == 1 and o.shape == xi.shape for o, xi in zip(outs, xs)), what   # channel contiguous, dense
        got = torch.cat([o.contiguous() for o in outs], dim=1)
        xm = x if m is None else (x.float() * m[:, None, :].float()).to(dtype)
        assert_parity(got, want_out, exact=act is None, what=what, res=xm)
        # the single-tensor call on the concatenation: identical bits
        x_cat = torch.cat(xs, dim=1).transpose(1, 2).contiguous().transpose(1, 2)
        fs1 = torch.empty_like(fs) if use_state else None
        r1 = cc.causal_conv1d_fn(x_cat, w.to(DEV), b.to(DEV), activation=act, residual="masked",
                                 attention_mask=None if m is None else m.to(DEV),
                                 initial_states=init.to(DEV) if use_state else None, final_states_out=fs1)
        one = r1[0] if use_state else r1
        assert torch.equal(bits(got), bits(one.contiguous())), what
        if use_state:
            assert torch.equal(bits(fs), bits(want_state)), what
            assert torch.equal(bits(fs), bits(fs1)), what


def test_prefill_parts_metric_shape(cc):
    """Canon-D at the benchmark shape: gate and up as two (8, 1024, 1728) tensors."""
    g = torch.Generator().manual_seed(5)
    B, L, dims = 8, 1024, [1728, 1728]
    C = sum(dims)
    x = torch.randn(B, C, L, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.02).bfloat16()
    want = co.conv1d_fwd(x, w, None, residual=1)
    xs = blc_parts(x, dims, "separate")
    assert cc.kernel_plan_fwd_parts(xs, w.to(DEV)) == "blc_vec_pair"
    outs = cc.causal_conv1d_fn_parts(xs, w.to(DEV), residual=True)
    assert_parity(torch.cat([o.contiguous() for o in outs], dim=1), want, exact=True, what="parts/metric")
    # the same launch size with everything on: bias, padding mask, fp32 taps, final states (a large launch fetches its
    # taps ahead of everything else, through the addresses among its leading arguments)
    b = (torch.randn(C, generator=g) * 0.1).bfloat16()
    mask = right_padded_mask([1024, 1000, 517, 3, 1024, 64, 999, 1], L)
    for wt in (w, w.float()):
        want, want_state = co.conv1d_fwd(x, wt, b.to(wt.dtype), mask=mask, residual=1, final_state_len=3)
        outs, fs = cc.causal_conv1d_fn_parts(xs, wt.to(DEV), b.to(wt.dtype).to(DEV), residual="masked",
                                             attention_mask=mask.to(DEV), return_final_states=True)
        assert_parity(torch.cat([o.contiguous() for o in outs], dim=1), want, exact=True, what=f"parts/metric/full/{wt.dtype}")
        assert torch.equal(bits(fs), bits(want_state)), wt.dtype
    # unmasked with both states and SiLU: the slabs of four steps of the large unmasked launches
    init = torch.randn(B, C, 3, generator=g).bfloat16()
    want, want_state = co.conv1d_fwd(x, w, b, activation="silu", residual=1, initial_state=init, final_state_len=5)
    outs, fs = cc.causal_conv1d_fn_parts(xs, w.to(DEV), b.to(DEV), activation="silu", residual=True,
                                         initial_states=init.to(DEV), final_states_out=torch.empty(B, C, 5, dtype=torch.bfloat16, device=DEV))
    assert_parity(torch.cat([o.contiguous() for o in outs], dim=1), want, exact=False, what="parts/metric/states", res=x)
    assert torch.equal(bits(fs), bits(want_state))
    # views into one projection output are not dense: the launch over a table of parts
    assert cc.kernel_plan_fwd_parts(blc_parts(x, dims, "sliced"), w.to(DEV)) == "blc_vec_parts"


def test_prefill_parts_fall_back_to_one_launch_per_part(cc):
    g = torch.Generator().manual_seed(9)
    B, L = 2, 96
    cases = [
        ("time-contiguous parts", [40, 24], 4, torch.bfloat16, "bcl"),
        ("channel counts off the vector size", [36, 30], 4, torch.bfloat16, "blc"),
        ("width 3", [64, 32], 3, torch.float32, "blc"),
        ("a single part", [72], 4, torch.float16, "blc"),
        ("an empty part", [64, 0, 16], 4, torch.bfloat16, "blc"),
    ]
    for what, dims, W, dtype, layout in cases:
        C = sum(dims)
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        want, want_state = co.conv1d_fwd(x, w, b, activation="silu", final_state_len=W - 1)
        if layout == "bcl":
            xs = [t.contiguous().to(DEV) for t in x.split(dims, dim=1)]
        else:
            xs = blc_parts(x, dims, "separate")
        plan = cc.kernel_plan_fwd_parts(xs, w.to(DEV))
        assert plan == ("blc_vec_parts" if what == "an empty part" else "per_part"), what
        outs, fs = cc.causal_conv1d_fn_parts(xs, w.to(DEV), b.to(DEV), activation="silu", return_final_states=True)
        assert [o.shape[1] for o in outs] == dims
        assert_parity(torch.cat([o.contiguous() for o in outs], dim=1), want, exact=False, what=what)
        assert torch.equal(bits(fs), bits(want_state)), what


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("S", [3, 4, 8])
def test_update_parts_one_launch(cc, dtype, S):
    g = torch.Generator().manual_seed(S)
    for B, dims in [(16, (640, 160, 160)), (256, (1728, 1728)), (3, (8, 24, 16, 8))]:
        C = sum(dims)
        w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        st_ref = torch.randn(B, C, S, generator=g).to(dtype)
        st_gpu = st_ref.to(DEV)
        st_one = st_ref.to(DEV)
        for step in range(3):
            x = torch.randn(B, C, generator=g).to(dtype)
            want = co.conv1d_update(x, st_ref, w, b, activation="silu", residual=True)
            xs = [t.contiguous().to(DEV) for t in x.split(list(dims), dim=1)]
            assert cc.kernel_plan_update_parts(xs, st_gpu, w.to(DEV)) == "update_vec_parts"
            outs = cc.causal_conv1d_update_parts(xs, st_gpu, w.to(DEV), b.to(DEV), activation="silu", residual=True)
            got = torch.cat(outs, dim=1)
            what = f"update_parts/{dtype}/S{S}/B{B}/{dims}/step{step}"
            assert_parity(got, want, exact=False, what=what, res=x)
            assert torch.equal(bits(st_gpu), bits(st_ref)), what
            one = cc.causal_conv1d_update(x.to(DEV), st_one, w.to(DEV), b.to(DEV), activation="silu", residual=True)
            assert torch.equal(bits(got), bits(one)), what
            assert torch.equal(bits(st_gpu), bits(st_one)), what


def test_update_parts_token_mask_and_fallback(cc):
    g = torch.Generator().manual_seed(77)
    B, dims, S, dtype = 5, [12, 20], 6, torch.bfloat16      # state length 6 and odd widths: strided kernel, per part
    C = sum(dims)
    w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
    st = torch.randn(B, C, S, generator=g).to(dtype)
    x = torch.randn(B, C, generator=g).to(dtype)
    tm = torch.tensor([1, 0, 1, 1, 0])
    st_a, st_b = st.to(DEV), st.to(DEV)
    xs = [t.contiguous().to(DEV) for t in x.split(dims, dim=1)]
    assert cc.kernel_plan_update_parts(xs, st_a, w.to(DEV)) == "per_part"
    outs = cc.causal_conv1d_update_parts(xs, st_a, w.to(DEV), token_mask=tm.to(DEV), residual="unmasked")
    one = cc.causal_conv1d_update(x.to(DEV), st_b, w.to(DEV), token_mask=tm.to(DEV), residual="unmasked")
    assert torch.equal(bits(torch.cat(outs, dim=1)), bits(one))
    assert torch.equal(bits(st_a), bits(st_b))
    # and on the vector kernel
    dims, S = [16, 48], 8
    C = sum(dims)
    w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
    st = torch.randn(B, C, S, generator=g).to(dtype)
    x = torch.randn(B, C, generator=g).to(dtype)
    st_a, st_b = st.to(DEV), st.to(DEV)
    xs = [t.contiguous().to(DEV) for t in x.split(dims, dim=1)]
    assert cc.kernel_plan_update_parts(xs, st_a, w.to(DEV)) == "update_vec_parts"
    outs = cc.causal_conv1d_update_parts(xs, st_a, w.to(DEV), token_mask=tm.to(DEV), residual="masked")
    one = cc.causal_conv1d_update(x.to(DEV), st_b, w.to(DEV), token_mask=tm.to(DEV), residual="masked")
    assert torch.equal(bits(torch.cat(outs, dim=1)), bits(one))
    assert torch.equal(bits(st_a), bits(st_b))
    masked_rows = (tm == 0).nonzero().flatten()
    assert torch.all(st_a[masked_rows, :, -1] == 0)


class _Cfg:
    canon_kernel = 4
    canon_bias = True
    canon_activation = True


class _Cache:
    pass


def test_canon_layer_forward_parts_matches_forward_on_the_cat():
    """Canon-B through a prefill with padding, then decode steps: parts vs cat, same bits and same cached state."""
    from causal_conv1d.canon import CanonLayer
    torch.manual_seed(21)
    dims = [640, 160, 160]
    layer = CanonLayer(sum(dims), _Cfg, "b").to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        layer.weight.mul_(0.3)
        layer.bias_param.normal_(0, 0.1)
    B, T = 4, 37
    qkv = [torch.randn(B, T, d, device=DEV).bfloat16() for d in dims]
    mask = right_padded_mask([37, 20, 1, 30], T).to(DEV)
    c_parts, c_cat = _Cache(), _Cache()
    with torch.no_grad():
        ys = layer.forward_parts(qkv, attention_mask=mask, cache=c_parts, layer_idx=2)
        y = layer(torch.cat(qkv, dim=-1), attention_mask=mask, cache=c_cat, layer_idx=2)
        assert torch.equal(bits(torch.cat(ys, dim=-1)), bits(y))
        assert torch.equal(bits(c_parts.canon_cache_b[2]), bits(c_cat.canon_cache_b[2]))
        for step in range(5):
            tok = [torch.randn(B, 1, d, device=DEV).bfloat16() for d in dims]
            mask = torch.cat([mask, torch.ones(B, 1, dtype=mask.dtype, device=DEV)], dim=1)
            held = c_parts.canon_cache_b[2]
            ys = layer.forward_parts(tok, attention_mask=mask, cache=c_parts, layer_idx=2)
            y = layer(torch.cat(tok, dim=-1), attention_mask=mask, cache=c_cat, layer_idx=2)
            assert c_parts.canon_cache_b[2] is held
            assert torch.equal(bits(torch.cat(ys, dim=-1)), bits(y)), step
            assert torch.equal(bits(c_parts.canon_cache_b[2]), bits(c_cat.canon_cache_b[2])), step
        # no cache: plain block call
        ys = layer.forward_parts(qkv)
        assert torch.equal(bits(torch.cat(ys, dim=-1)), bits(layer(torch.cat(qkv, dim=-1))))


def test_parts_gradients_and_errors(cc):
    torch.manual_seed(4)
    dims = [16, 8]
    xs = [torch.randn(2, 24, d, device=DEV).transpose(1, 2).requires_grad_() for d in dims]
    w = (torch.randn(24, 4, device=DEV) * 0.3).requires_grad_()
    outs = cc.causal_conv1d_fn_parts(xs, w, activation="silu", residual=True)
    sum(o.square().sum() for o in outs).backward()
    x_cat = torch.cat([x.detach() for x in xs], dim=1).requires_grad_()
    w2 = w.detach().clone().requires_grad_()
    cc.causal_conv1d_fn(x_cat, w2, activation="silu", residual=True).square().sum().backward()
    torch.testing.assert_close(torch.cat([x.grad for x in xs], dim=1), x_cat.grad, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(w.grad, w2.grad, rtol=1e-6, atol=1e-6)

    assert "CanonConvPartsFn" in type(outs[0].grad_fn).__name__     # one node over the parts, no cat

    a = torch.randn(2, 16, 24, device=DEV)
    with pytest.raises(ValueError, match="Input dim 32 does not match weight dim 24"):
        cc.causal_conv1d_fn_parts([a, a], w.detach())
    with pytest.raises(ValueError, match="1..4 parts"):
        cc.causal_conv1d_fn_parts([a[:, :4]] * 5, w.detach())
    with pytest.raises(ValueError, match="differ in batch or seqlen"):
        cc.causal_conv1d_fn_parts([a[:, :16], a[:, :8, :20]], w.detach())
    with pytest.raises(ValueError, match="one dtype and device"):
        cc.causal_conv1d_fn_parts([a[:, :16], a[:, :8].half()], w.detach())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_parts_backward_runs_per_part_without_a_cat(cc, dtype):
    """Gate/up at the model's width: dx of every part is bit-identical to the matching channels of
    the single-tensor backward on the concatenation (same per-channel arithmetic), dweight / dbias
    agree to summation order, and against the float64 autograd of the eager formulation."""
    from oracle.canon_grad import conv1d_grads
    torch.manual_seed(11)
    B, L, dims = 4, 256, (1728, 1728)
    C = sum(dims)
    big = torch.randn(B, L, C).to(dtype)
    mask = torch.ones(B, L)
    mask[1, 200:] = 0
    mask[3, 31:] = 0
    w = torch.randn(C, 4) * 0.3
    bias = torch.randn(C) * 0.1
    dout = torch.randn(B, L, C).to(dtype)

    def leaf(t):
        return t.to(DEV).requires_grad_()

    xs = [leaf(big[..., c0:c0 + d].contiguous()) for c0, d in zip((0, dims[0]), dims)]
    wg, bg = leaf(w), leaf(bias)
    outs = cc.causal_conv1d_fn_parts([x.transpose(1, 2) for x in xs], wg, bg, activation="silu",
                                     attention_mask=mask.to(DEV), residual=True)
    douts = [dout[..., c0:c0 + d].to(DEV).transpose(1, 2) for c0, d in zip((0, dims[0]), dims)]
    torch.autograd.backward(outs, douts)

    xc = leaf(big)
    wc, bc = leaf(w), leaf(bias)
    yc = cc.causal_conv1d_fn(xc.transpose(1, 2), wc, bc, activation="silu", attention_mask=mask.to(DEV),
                             residual=True)
    yc.backward(dout.to(DEV).transpose(1, 2))
    torch.cuda.synchronize()
    assert torch.equal(bits(torch.cat([o.transpose(1, 2) for o in outs], dim=-1)), bits(yc.transpose(1, 2)))
    assert torch.equal(bits(torch.cat([x.grad for x in xs], dim=-1)), bits(xc.grad))
    torch.testing.assert_close(wg.grad, wc.grad, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(bg.grad, bc.grad, rtol=1e-5, atol=1e-4)

    _, dw64, db64, _ = conv1d_grads(big.transpose(1, 2), w, bias, dout.transpose(1, 2), mask=mask,
                                    activation="silu", residual="masked")
    assert (wg.grad.cpu().double() - dw64).abs().max().item() <= 1e-4 * dw64.abs().max().item()
    assert (bg.grad.cpu().double() - db64).abs().max().item() <= 1e-4 * db64.abs().max().item()
