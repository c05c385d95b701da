"""HIP kernels (through the C ABI, via the drop-in package) vs the CPU oracle.

Bar: conv_state bit exact; outputs bit exact without SiLU (same fma chain on
both sides), with SiLU within 1 bf16/fp16 ulp resp. 1e-5 relative for fp32
(the GPU uses v_exp_f32 / v_rcp_f32, the oracle libm).
"""
import itertools

import pytest
import torch

from helpers import assert_parity, bits, right_padded_mask, ulp_diff
from oracle import canon_oracle as co

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def cc():
    import causal_conv1d
    return causal_conv1d


def layouts(x_bcl_cpu):
    """The same logical [B,C,L] tensor on the GPU in both dense layouts."""
    xg = x_bcl_cpu.to(DEV)
    yield "bcl", xg
    yield "blc", xg.transpose(1, 2).contiguous().transpose(1, 2)


def run_fwd(cc, x, w, b, act=None, mask=None, residual=False, init=None, S_out=None, rounding="fused"):
    fs = None
    if S_out is not None:
        fs = torch.full((x.shape[0], x.shape[1], S_out), float("nan"), dtype=x.dtype, device=DEV)
    r = cc.causal_conv1d_fn(x, w.to(DEV), None if b is None else b.to(DEV), activation=act,
                            attention_mask=None if mask is None else mask.to(DEV), residual=residual,
                            initial_states=None if init is None else init.to(DEV),
                            final_states_out=fs, rounding=rounding)
    torch.cuda.synchronize()
    return r


# ---- benchmark configuration 1: fp32 x[1,640,1024], Canon-A ------------------------------------------------------
def test_config1_fp32_canon_a(cc):
    torch.manual_seed(0)
    x = torch.randn(1, 640, 1024)
    w = torch.randn(640, 4) * 0.02
    b = torch.zeros(640)
    want = co.conv1d_fwd(x, w, b, residual=1)
    for name, xg in layouts(x):
        assert cc.kernel_plan_fwd(xg, w.to(DEV)) == f"{name}_vec"
        got = run_fwd(cc, xg, w, b, residual=True)
        assert got.stride() == xg.stride()
        assert_parity(got, want, exact=True, what=f"config1/{name}")


# ---- benchmark configuration 2: bf16 B8 L1024, C in {640, 960, 3456} ------------------------------------------------------
@pytest.mark.parametrize("C", [640, 960, 3456])
@pytest.mark.parametrize("act", [None, "silu"])
def test_config2_bf16_prefill(cc, C, act):
    g = torch.Generator().manual_seed(C)
    x = torch.randn(8, C, 1024, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.02).bfloat16()
    b = (torch.randn(C, generator=g) * 0.01).bfloat16()
    want = co.conv1d_fwd(x, w, b, activation=act)
    for name, xg in layouts(x):
        assert cc.kernel_plan_fwd(xg, w.to(DEV)) == f"{name}_vec"
        got = run_fwd(cc, xg, w, b, act=act)
        assert_parity(got, want, exact=act is None, what=f"config2/C{C}/{act}/{name}")


# ---- unmasked channel-contiguous launches of 40 MB and more run slabs of four time steps per wave -----------------------
@pytest.mark.parametrize("dtype,B,C,L", [(torch.bfloat16, 4, 2048, 1723), (torch.float16, 3, 3456, 1030),
                                         (torch.float32, 2, 2600, 1029)])
def test_short_slab_launches_with_everything_on(cc, dtype, B, C, L):
    """The large unmasked launches (slabs of 4 steps, taps fetched first through the leading arguments): lengths that
    end inside a tile and inside a slab, a channel count that ends inside a 64-lane tile, initial and final states,
    SiLU, both residual settings, fp32 taps on 16-bit inputs, both rounding modes; the same call with an all-ones
    mask (slabs of 8 steps) gives the same bits."""
    g = torch.Generator().manual_seed(L)
    assert 2 * B * C * L * torch.empty(0, dtype=dtype).element_size() >= 40 << 20
    x = torch.randn(B, C, L, generator=g).to(dtype)
    w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype)
    init = torch.randn(B, C, 5, generator=g).to(dtype)
    xg = x.transpose(1, 2).contiguous().to(DEV).transpose(1, 2)
    ones = torch.ones(B, L, dtype=torch.bool)
    for act, residual, use_state, wt in [(None, True, True, dtype), ("silu", False, False, dtype),
                                         ("silu", True, True, torch.float32), (None, False, False, torch.float32)]:
        if wt != dtype and dtype == torch.float32:
            continue
        ww, bb = w.to(wt), b.to(wt)
        want = co.conv1d_fwd(x, ww, bb, activation=act, residual=1 if residual else 0,
                             initial_state=init if use_state else None, final_state_len=6 if use_state else None)
        want_out, want_fs = want if use_state else (want, None)
        r = run_fwd(cc, xg, ww, bb, act=act, residual=residual, init=init if use_state else None,
                    S_out=6 if use_state else None)
        got, fs = r if use_state else (r, None)
        what = f"short slabs/{dtype}/{act}/res{residual}/state{use_state}/taps {wt}"
        assert_parity(got, want_out, exact=act is None, what=what, res=x if residual else None)
        if use_state:
            assert torch.equal(bits(fs), bits(want_fs)), what
        r8 = run_fwd(cc, xg, ww, bb, act=act, residual=residual, mask=ones, init=init if use_state else None,
                     S_out=6 if use_state else None)
        got8 = r8[0] if use_state else r8
        assert torch.equal(bits(got), bits(got8)), what + ": slabs of 4 and of 8 steps differ"
    # the eager module's rounding points, against the C oracle's round_mode = 1
    want = co.conv1d_fwd(x, w, b, residual=1, round_mode=1)
    got = run_fwd(cc, xg, w, b, residual=True, rounding="eager")
    assert torch.equal(bits(got), bits(want)), f"short slabs/{dtype}/eager rounding"


# ---- benchmark configuration 3: ragged right-padded batch of 32 ------------------------------------------------------
@pytest.mark.parametrize("residual", ["masked", "unmasked"])
def test_config3_ragged_padded_prefill(cc, residual):
    g = torch.Generator().manual_seed(3)
    B, C, L = 32, 3456, 1024
    x = torch.randn(B, C, L, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.02).bfloat16()
    b = (torch.randn(C, generator=g) * 0.01).bfloat16()
    lens = torch.randint(128, 1025, (B,), generator=g).tolist()
    mask = right_padded_mask(lens, L)
    want, want_fs = co.conv1d_fwd(x, w, b, mask=mask, residual=residual, final_state_len=4)
    for name, xg in layouts(x):
        got, fs = run_fwd(cc, xg, w, b, mask=mask, residual=residual, S_out=4)
        assert_parity(got, want, exact=True, what=f"config3/{name}")
        assert torch.equal(bits(fs), bits(want_fs)), f"config3/{name}: state"
        del got, fs, xg
    # size-independent properties at full size: all-ones mask == no mask
    xg = x.to(DEV)
    ones = torch.ones(B, L, dtype=torch.bool)
    a = run_fwd(cc, xg, w, b, mask=ones, residual=residual)
    c = run_fwd(cc, xg, w, b, residual=residual)
    assert torch.equal(bits(a), bits(c))


# ---- benchmark configuration 4: decode, B256, state 3, 64 carried steps ------------------------------------------------------
@pytest.mark.parametrize("S", [3, 4, 8])
def test_config4_decode_64_steps(cc, S):
    g = torch.Generator().manual_seed(4)
    B, C, steps = 256, 3456, 64
    state0 = torch.randn(B, C, S, generator=g).bfloat16()
    xs = torch.randn(steps, B, C, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.02).bfloat16()
    b = (torch.randn(C, generator=g) * 0.01).bfloat16()
    st_ref = state0.clone()
    st_gpu = state0.to(DEV)
    ptr = st_gpu.data_ptr()
    wg, bg, xg = w.to(DEV), b.to(DEV), xs.to(DEV)
    assert cc.kernel_plan_update(xg[0], st_gpu, wg, bg) == "update_vec"
    for i in range(steps):
        want = co.conv1d_update(xs[i], st_ref, w, b)
        got = cc.causal_conv1d_update(xg[i], st_gpu, wg, bg)
        assert_parity(got, want, exact=True, what=f"config4/S{S}/step{i}")
    assert st_gpu.data_ptr() == ptr
    assert torch.equal(bits(st_gpu), bits(st_ref))
    # closed form: the state is the last S tokens (S <= steps)
    assert torch.equal(bits(st_gpu), bits(xs[-S:].permute(1, 2, 0)))


# ---- the reference's own grid (causal-conv1d-mps/test.py:110-146) -----------
@pytest.mark.parametrize("itype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("has_bias", [False, True])
def test_reference_grid(cc, itype, silu, has_bias):
    for dim, seqlen in itertools.product([64, 128, 256], [1, 2, 8, 16, 32, 64, 128, 256]):
        torch.manual_seed(42)
        x = torch.randn(2, dim, seqlen).to(itype)
        w = torch.randn(dim, 4)                      # fp32 weights, cast by the callee
        b = torch.randn(dim) if has_bias else None
        act = "silu" if silu else None
        want = co.conv1d_fwd(x, w, b, activation=act)
        for name, xg in layouts(x):
            got = run_fwd(cc, xg, w, b, act=act)
            assert_parity(got, want, exact=not silu, what=f"grid/{dim}/{seqlen}/{name}")
        # the reference's own tolerance, for the record (test.py:121-126)
        rtol, atol = {torch.float32: (3e-4, 1e-3), torch.bfloat16: (5e-3, 2e-2), torch.float16: (3e-3, 5e-3)}[itype]
        torch.testing.assert_close(got.cpu(), want, rtol=rtol, atol=atol)


# ---- fused mask + residual, the reference's fused test (test.py:149-197) ----
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("has_bias", [False, True])
def test_short_conv_fused_reference_case(cc, silu, has_bias):
    for dim, seqlen in itertools.product([64, 128], [8, 16, 32, 64]):
        torch.manual_seed(42)
        x = torch.randn(2, seqlen, dim)
        w = torch.randn(dim, 4)
        b = torch.randn(dim) if has_bias else None
        mask = torch.ones(2, seqlen)
        for i in range(2):
            mask[i, int(torch.randint(seqlen // 2, seqlen, (1,))):] = 0
        got = cc.short_conv_fused(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), mask.to(DEV),
                                  activation=silu, residual=True)
        want = co.conv1d_fwd(x.transpose(1, 2), w, b, mask=mask, activation="silu" if silu else None,
                             residual="unmasked").transpose(1, 2)
        assert_parity(got, want, exact=not silu, what=f"fused/{dim}/{seqlen}", res=x)


# ---- edge shapes, odd strides, every kernel family --------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_edge_shapes_and_strides(cc, dtype):
    g = torch.Generator().manual_seed(9)
    cases = [(1, 1, 1), (2, 3, 5), (1, 8, 3), (3, 7, 129), (2, 16, 128), (2, 24, 136), (1, 40, 1000),
             (2, 8, 2048 + 8), (1, 2, 8192), (5, 1000, 9)]
    for (B, C, L), W in itertools.product(cases, [2, 3, 4]):
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = torch.randn(C, W, generator=g).to(dtype)
        b = torch.randn(C, generator=g).to(dtype)
        lens = torch.randint(1, L + 1, (B,), generator=g).tolist()
        mask = right_padded_mask(lens, L, torch.int32)
        want, wfs = co.conv1d_fwd(x, w, b, mask=mask, residual=1, final_state_len=W)
        for name, xg in layouts(x):
            got, fs = run_fwd(cc, xg, w, b, mask=mask, residual=True, S_out=W)
            assert_parity(got, want, exact=True, what=f"edge/{B}x{C}x{L}/W{W}/{name}")
            assert torch.equal(bits(fs), bits(wfs))
    # views that are neither dense layout: slices in every dimension, misaligned base
    big = torch.randn(3, 37, 301, generator=g).to(dtype)
    w = torch.randn(20, 4, generator=g).to(dtype)
    xg = big.to(DEV)[1:3, 5:25, 3:280:2]
    want = co.conv1d_fwd(big[1:3, 5:25, 3:280:2], w, None, activation="silu")
    got = run_fwd(cc, xg, w, None, act="silu")
    assert_parity(got, want, exact=False, what="edge/strided view")
    # dense but misaligned (base pointer off by one element) -> scalar kernel, same answer
    flat = torch.randn(2 * 16 * 256 + 1, generator=g).to(dtype)
    xv = flat[1:].view(2, 16, 256)
    w = torch.randn(16, 4, generator=g).to(dtype)
    xg = flat.to(DEV)[1:].view(2, 16, 256)
    assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "generic"
    assert_parity(run_fwd(cc, xg, w, None), co.conv1d_fwd(xv, w), exact=True, what="edge/misaligned")


@pytest.mark.parametrize("xdtype", [torch.bfloat16, torch.float32])
def test_every_mask_dtype_and_alignment(cc, xdtype):
    g = torch.Generator().manual_seed(55)
    B, C, L = 3, 16, 640
    x = torch.randn(B, C, L, generator=g).to(xdtype)
    w = torch.randn(C, 4, generator=g).to(xdtype)
    keep = torch.rand(B, L, generator=g) > 0.3
    want, wfs = co.conv1d_fwd(x, w, None, mask=keep, residual=1, final_state_len=4)
    for mdtype in [torch.bool, torch.uint8, torch.int32, torch.int64, torch.float32, torch.bfloat16, torch.float16]:
        m = keep.to(mdtype)
        # contiguous (wide loads), a strided view and a misaligned view (narrow loads)
        wide = torch.zeros(B, 2 * L + 1, dtype=mdtype)
        wide[:, 1::2] = m
        shifted = torch.zeros(B * L + 1, dtype=mdtype)
        shifted[1:] = m.flatten()
        variants = {"contig": m.to(DEV), "strided": wide.to(DEV)[:, 1::2], "misaligned": shifted.to(DEV)[1:].view(B, L)}
        for vname, mg in variants.items():
            for name, xg in layouts(x):
                fs = torch.empty(B, C, 4, dtype=xdtype, device=DEV)
                got, fs = cc.causal_conv1d_fn(xg, w.to(DEV), attention_mask=mg, residual=True, final_states_out=fs)
                assert_parity(got, want, exact=True, what=f"mask {mdtype} {vname} {name}")
                assert torch.equal(bits(fs), bits(wfs))
    # non-0/1 values multiply in (and round to the storage type first)
    scale = (torch.rand(B, L, generator=g) * 3).to(torch.float32)
    want = co.conv1d_fwd(x, w, None, mask=scale, residual="unmasked")
    for name, xg in layouts(x):
        got = cc.causal_conv1d_fn(xg, w.to(DEV), attention_mask=scale.to(DEV), residual="unmasked")
        assert_parity(got, want, exact=True, what=f"scaled mask {name}")
    big = torch.tensor([[2 ** 40, -2 ** 33, 1, 0] * (L // 4)] * B, dtype=torch.int64)
    want = co.conv1d_fwd(x, w, None, mask=big)
    for name, xg in layouts(x):
        got = cc.causal_conv1d_fn(xg, w.to(DEV), attention_mask=big.to(DEV))
        assert_parity(got, want, exact=True, what=f"int64 mask beyond 32 bits {name}")


def test_empty_inputs(cc):
    w = torch.randn(8, 4, device=DEV)
    for shape in [(0, 8, 16), (2, 8, 0)]:
        out = cc.causal_conv1d_fn(torch.empty(shape, device=DEV), w)
        assert out.shape == shape
    st = torch.zeros(0, 8, 4, device=DEV)
    assert cc.causal_conv1d_update(torch.empty(0, 8, device=DEV), st, w).shape == (0, 8)


# ---- initial / final states, chunking, streaming ----------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_prefill_and_streaming_equivalence(cc, dtype):
    g = torch.Generator().manual_seed(21)
    B, C, L = 2, 64, 512
    x = torch.randn(B, C, L, generator=g).to(dtype)
    w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype)
    for name, xg in layouts(x):
        full, fs_full = run_fwd(cc, xg, w, b, S_out=8)
        # prefill in two pieces joined through a 3-slot state
        for cut in (8, 128, 264):
            first = xg[:, :, :cut]
            second = xg[:, :, cut:]
            if name == "bcl":
                first, second = first.contiguous(), second.contiguous()
            a, sa = run_fwd(cc, first, w, b, S_out=3)
            c, sc = run_fwd(cc, second, w, b, init=sa, S_out=8)
            assert torch.equal(bits(torch.cat([a, c], dim=-1)), bits(full)), (name, cut)
            assert torch.equal(bits(sc), bits(fs_full))
        # prefill then single-token updates == one prefill
        head = xg[:, :, :500].contiguous() if name == "bcl" else xg[:, :, :500]
        out_h, state = run_fwd(cc, head, w, b, S_out=4)
        cols = []
        for t in range(500, L):
            cols.append(cc.causal_conv1d_update(xg[:, :, t], state, w.to(DEV), b.to(DEV)))
        got = torch.cat([out_h, torch.stack(cols, dim=-1)], dim=-1)
        assert torch.equal(bits(got), bits(full)), name
        assert torch.equal(bits(state), bits(fs_full[:, :, -4:]))


def test_update_variants_vs_oracle(cc):
    g = torch.Generator().manual_seed(33)
    for dtype, W, S, (B, C), act, res in itertools.product(
            [torch.float32, torch.bfloat16, torch.float16], [2, 3, 4], [3, 4, 5, 8],
            [(1, 8), (3, 20), (5, 256), (2, 1000)], [None, "silu"], [False, "masked", "unmasked"]):
        x = torch.randn(B, C, generator=g).to(dtype)
        st = torch.randn(B, C, S, generator=g).to(dtype)
        w = torch.randn(C, W, generator=g)
        b = torch.randn(C, generator=g)
        tm = (torch.rand(B, generator=g) > 0.3).to(torch.int64)
        # oracle: masked token in, residual adds masked or raw token
        xt = (x * tm[:, None]).to(dtype)
        st_ref = st.clone()
        want = co.conv1d_update(xt, st_ref, w, b, activation=act, residual=(res == "masked"))
        if res == "unmasked":
            want = want.float() + x.float()      # rounded before this add: loose comparison below
        st_gpu = st.to(DEV)
        got = cc.causal_conv1d_update(x.to(DEV), st_gpu, w.to(DEV), b.to(DEV), activation=act,
                                      token_mask=tm.to(DEV), residual=res)
        assert torch.equal(bits(st_gpu), bits(st_ref)), (dtype, W, S, B, C)
        if res == "unmasked":
            torch.testing.assert_close(got.cpu().float(), want, rtol=2e-2, atol=2e-2)
        else:
            assert_parity(got, want, exact=act is None, what=f"update/{dtype}/W{W}/S{S}/{B}x{C}/{res}",
                          res=xt if res else None)


def test_update_residual_exact(cc):
    g = torch.Generator().manual_seed(34)
    for dtype, S in itertools.product([torch.float32, torch.bfloat16], [3, 4, 8, 6]):
        B, C = 4, 264
        x = torch.randn(B, C, generator=g).to(dtype)
        st = torch.randn(B, C, S, generator=g).to(dtype)
        w = torch.randn(C, 4, generator=g).to(dtype)
        st_ref = st.clone()
        want = co.conv1d_update(x, st_ref, w, None, residual=True)
        st_gpu = st.to(DEV)
        got = cc.short_conv_update(x.to(DEV), st_gpu, w.to(DEV), None, activation=False, residual=True)
        assert_parity(got, want, exact=True, what=f"update residual S{S}")
        assert torch.equal(bits(st_gpu), bits(st_ref))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_update_vector_kernel_on_buffers_aligned_to_4_bytes_only(cc, dtype):
    """State, token and weights carved out of larger buffers at 4-byte offsets: the vector kernel asks for no more."""
    g = torch.Generator().manual_seed(36)
    B, C = 5, 264
    es = torch.empty((), dtype=dtype).element_size()
    off = 4 // es                      # elements in 4 bytes
    for S in (3, 4, 8):
        st = torch.randn(B, C, S, generator=g).to(dtype)
        x = torch.randn(B, C, generator=g).to(dtype)
        w = (torch.randn(C, 4, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        flat = torch.zeros(B * C * S + 2 * off, dtype=dtype, device=DEV)
        st_gpu = flat[off:off + B * C * S].view(B, C, S)
        st_gpu.copy_(st.to(DEV))
        xflat = torch.zeros(B * C + 2 * off, dtype=dtype, device=DEV)
        x_gpu = xflat[off:off + B * C].view(B, C)
        x_gpu.copy_(x.to(DEV))
        assert st_gpu.data_ptr() % 16 == 4 and x_gpu.data_ptr() % 16 == 4
        assert cc.kernel_plan_update(x_gpu, st_gpu, w.to(DEV), b.to(DEV)) == "update_vec"
        st_ref = st.clone()
        want = co.conv1d_update(x, st_ref, w, b, activation="silu", residual=True)
        got = cc.causal_conv1d_update(x_gpu, st_gpu, w.to(DEV), b.to(DEV), activation="silu", residual=True)
        assert_parity(got, want, exact=False, what=f"4-byte aligned S{S}", res=x)
        assert torch.equal(bits(st_gpu), bits(st_ref))
        assert float(flat[:off].abs().sum()) == 0 and float(flat[off + B * C * S:].abs().sum()) == 0   # neighbours untouched


def test_noncontiguous_state_takes_strided_kernel_and_stays_in_place(cc):
    g = torch.Generator().manual_seed(35)
    B, C, S = 3, 64, 4
    big = torch.randn(B, C, 2 * S, generator=g).bfloat16()
    x = torch.randn(B, C, generator=g).bfloat16()
    w = torch.randn(C, 4, generator=g).bfloat16()
    big_g = big.to(DEV)
    view = big_g[:, :, ::2]
    assert cc.kernel_plan_update(x.to(DEV), view, w.to(DEV)) == "update_generic"
    st_ref = big[:, :, ::2].contiguous()
    want = co.conv1d_update(x, st_ref, w)
    got = cc.causal_conv1d_update(x.to(DEV), view, w.to(DEV))
    assert_parity(got, want, exact=True)
    assert torch.equal(bits(big_g[:, :, ::2]), bits(st_ref))
    assert torch.equal(bits(big_g[:, :, 1::2]), bits(big[:, :, 1::2]))   # untouched neighbours


# ---- eager rounding mode: bit parity with the eager module ------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act", [False, True])
def test_eager_rounding_matches_eager_module(cc, dtype, act):
    from oracle.canon_eager import EagerCanon
    torch.manual_seed(77)
    B, T, D = 4, 200, 96
    x = torch.randn(B, T, D).to(dtype)
    w = (torch.randn(D, 4) * 0.4).to(dtype)
    bias = (torch.randn(D) * 0.1).to(dtype)
    mask = right_padded_mask([200, 150, 64, 3], T)
    cache = {}
    want = EagerCanon(w, bias, act).forward(x, mask, cache, 0)
    fs = torch.empty(B, D, 8, dtype=dtype, device=DEV)
    got, fs = cc.causal_conv1d_fn(x.to(DEV).transpose(1, 2), w.to(DEV), bias.to(DEV),
                                  activation="silu" if act else None, attention_mask=mask.to(DEV),
                                  residual="masked", rounding="eager", final_states_out=fs)
    got = got.transpose(1, 2)
    assert torch.equal(bits(fs), bits(cache[0]))
    assert_parity(got, want, exact=(not act and dtype != torch.float32), what="eager mode", res=x)
    # decode steps in eager mode
    state = fs
    layer = EagerCanon(w, bias, act)
    for _ in range(4):
        xt = torch.randn(B, 1, D).to(dtype)
        want = layer.forward(xt, None, cache, 0)[:, 0]
        got = cc.causal_conv1d_update(xt[:, 0].to(DEV), state, w.to(DEV), bias.to(DEV),
                                      activation="silu" if act else None, residual="unmasked",
                                      rounding="eager")
        assert torch.equal(bits(state), bits(cache[0]))
        assert_parity(got, want, exact=(not act and dtype != torch.float32), what="eager step", res=xt[:, 0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_eager_rounding_with_silu_vs_the_c_oracle_in_both_layouts(cc, dtype, capsys):
    """rounding='eager' with SiLU and a residual against the C oracle's round_mode = 1 (rounds after the conv, after
    the activation and at the store), in the vector kernels of both layouts and with a padding mask: within one
    unit in the last place of the output itself (the GPU divides and exponentiates in fp32 like libm but not
    with libm's code), and the share of outputs that are bit equal is printed."""
    g = torch.Generator().manual_seed(131)
    B, C, L = 3, 264, 520
    x = torch.randn(B, C, L, generator=g).to(dtype)
    w = (torch.randn(C, 4, generator=g) * 0.4).to(dtype)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype)
    mask = right_padded_mask([520, 300, 7], L)
    for m, res in ((None, False), (None, "unmasked"), (mask, "masked")):
        want, want_state = co.conv1d_fwd(x, w, b, activation="silu", mask=m, residual=res, final_state_len=8, round_mode=1)
        for name, xg in layouts(x):
            assert cc.kernel_plan_fwd(xg, w.to(DEV), rounding="eager") == f"{name}_vec"
            got, state = run_fwd(cc, xg, w, b, act="silu", mask=m, residual=res, S_out=8, rounding="eager")
            assert torch.equal(bits(state), bits(want_state))
            d = ulp_diff(got, want)
            equal = (d == 0).float().mean().item()
            # the eager mode rounds the activation before the residual is added, so what reaches the sum is a
            # storage-type value on both sides: one step of it apart at most, which the sum's rounding may keep
            xm = x if m is None else x * m.unsqueeze(1).to(dtype)
            assert_parity(got, want, exact=False, what=f"eager silu/{name}/res{res}", res=xm if res else None)
            with capsys.disabled():
                print(f"\n[eager rounding + SiLU, {str(dtype)[6:]}, {name}, residual {res}] bit equal {equal * 100:.2f} %, "
                      f"largest distance {d.max().item()} ulp of the output")


def test_silu_with_residual_literal_ulp_distance(cc, capsys):
    """The optional-activation variant at configuration 2's largest shape: SiLU and a residual, one rounding.  The
    bar of this repository measures the 1 ulp against the larger of the output and the residual term (the sum
    cancels).  Reported here as well: the literal distance in units of the OUTPUT's last place, which is large
    exactly where x + silu(conv) cancels, and the same distance for the oracle evaluated with float32 libm against
    float64: any two correct evaluations of the activation differ there."""
    import numpy as np
    g = torch.Generator().manual_seed(3456)
    B, C, L = 8, 3456, 1024
    x = torch.randn(B, C, L, generator=g).bfloat16()
    w = (torch.randn(C, 4, generator=g) * 0.02).bfloat16()
    b = (torch.randn(C, generator=g) * 0.01).bfloat16()
    want = co.conv1d_fwd(x, w, b, activation="silu", residual=1)
    # the same in float64 (exact products and sums of bf16 values up to the activation)
    xd, wd = x.double(), w.double()
    xp = torch.nn.functional.pad(xd, (3, 0))
    z = b.double()[None, :, None] + sum(wd[None, :, k, None] * xp[:, :, k:k + L] for k in range(4))
    ref64 = (xd + z / (1 + torch.exp(-z))).bfloat16()
    for name, xg in layouts(x):
        got = run_fwd(cc, xg, w, b, act="silu", residual=True)
        assert_parity(got, want, exact=False, what=f"silu+residual/{name}", res=x)
        d = ulp_diff(got, want)
        d64 = ulp_diff(want, ref64)
        hist = np.bincount(d.flatten().numpy().clip(max=3), minlength=4)
        worst = d.max().item()
        at = tuple(int(i) for i in (d == worst).nonzero()[0])
        with capsys.disabled():
            print(f"\n[SiLU + residual, bf16 [8,3456,1024], {name}] literal distance to the oracle in ulp of the output: "
                  f"0: {hist[0]}, 1: {hist[1]}, 2: {hist[2]}, >= 3: {hist[3]} elements; largest {worst} at {at} where "
                  f"out = {want[at].item():.3e}, x = {x[at].item():.3e} (the sum cancels); the oracle itself is up to "
                  f"{d64.max().item()} ulp from a float64 evaluation")
        # away from cancellation (|out| at least half of |x|) the literal distance is within one ulp
        plain = want.float().abs() >= 0.5 * x.float().abs()
        assert d[plain].max().item() <= 1


def test_errors_surface(cc):
    x = torch.randn(2, 8, 16, device=DEV)
    w = torch.randn(8, 4, device=DEV)
    with pytest.raises(ValueError, match="does not match"):
        cc.causal_conv1d_fn(x, torch.randn(5, 4, device=DEV))
    with pytest.raises(NotImplementedError, match="width"):
        cc.causal_conv1d_fn(x, torch.randn(8, 5, device=DEV))
    with pytest.raises(ValueError, match="int32"):
        cc.causal_conv1d_fn(x, w, seq_idx=torch.zeros(2, 16, dtype=torch.int64, device=DEV))
    with pytest.raises(ValueError, match="shorter than width-1"):
        cc.causal_conv1d_update(x[:, :, 0], torch.zeros(2, 8, 2, device=DEV), w)


def test_integer_mask_narrowing_is_never_stale(cc):
    """Large problems convert an int64 mask to x.dtype once and reuse it while the same mask
    object comes back; a changed or different mask must never hit the cached copy."""
    g = torch.Generator().manual_seed(91)
    B, C, L = 4, 512, 1024          # 2M elements: above the narrowing threshold
    x = torch.randn(B, C, L, generator=g).bfloat16()
    w = torch.randn(C, 4, generator=g).bfloat16()
    xg, wg = x.to(DEV), w.to(DEV)
    m1 = right_padded_mask([1024, 700, 300, 5], L)
    m2 = right_padded_mask([10, 1024, 64, 999], L)
    mg = m1.to(DEV)
    for m_cpu in (m1, m1, m2):
        if m_cpu is m2:
            mg.copy_(m2.to(DEV))     # same tensor object and address, new content
        got = cc.causal_conv1d_fn(xg, wg, attention_mask=mg, residual=True)
        assert_parity(got, co.conv1d_fwd(x, w, None, mask=m_cpu, residual=1), exact=True, what="narrowed mask")
    del mg
    other = m1.to(DEV)               # may land on the freed address
    got = cc.causal_conv1d_fn(xg, wg, attention_mask=other, residual=True)
    assert_parity(got, co.conv1d_fwd(x, w, None, mask=m1, residual=1), exact=True, what="narrowed mask, new tensor")
    sliced = torch.cat([m2, m1], dim=1).to(DEV)[:, -L:]      # a view, as CanonLayer slices it
    got = cc.causal_conv1d_fn(xg, wg, attention_mask=sliced, residual=True)
    assert_parity(got, co.conv1d_fwd(x, w, None, mask=m1, residual=1), exact=True, what="narrowed mask view")


# ---- packed variable-length sequences (seq_idx) --------------------------------
def packed_seq_idx(B, L, gen, max_seqs=6):
    """Per batch row: L positions cut into 1..max_seqs consecutive sequences (some of length 1..3)."""
    seq = torch.zeros(B, L, dtype=torch.int32)
    for b in range(B):
        n = int(torch.randint(1, max_seqs + 1, (1,), generator=gen))
        cuts = sorted(set(torch.randint(1, max(L, 2), (n - 1,), generator=gen).tolist())) if L > 1 else []
        for i, c in enumerate(cuts):
            seq[b, c:] = i + 1
    return seq


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_seq_idx_matches_oracle_and_separate_calls(cc, dtype):
    g = torch.Generator().manual_seed(71)
    for (B, C, L), W in itertools.product([(3, 64, 100), (2, 520, 37), (1, 8, 5), (4, 24, 257)], [2, 3, 4]):
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        seq = packed_seq_idx(B, L, g)
        seq[0, :] = seq[0, :] * 7 + 3                    # the values only matter through equality
        mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
        for act, res, m in [(None, False, None), ("silu", "masked", mask), (None, "unmasked", mask)]:
            want = co.conv1d_fwd_seq(x, w, b, seq, mask=m, activation=act, residual=res)
            for name, xg in layouts(x):
                plan = cc.kernel_plan_fwd(xg, w.to(DEV), seq_idx=seq.to(DEV))
                assert plan == ("blc_vec_seq" if name == "blc" and C % (16 // x.element_size()) == 0 else "generic")
                got = cc.causal_conv1d_fn(xg, w.to(DEV), b.to(DEV), seq_idx=seq.to(DEV), activation=act,
                                          attention_mask=None if m is None else m.to(DEV), residual=res)
                xm = x if m is None else (x.float() * m[:, None, :].float()).to(dtype)
                assert_parity(got, want, exact=act is None, what=f"seq/{dtype}/{B}x{C}x{L}/W{W}/{act}/{res}/{name}",
                              res=xm if res else None)
        # the defining property: a packed row equals its sequences convolved one by one
        xg = x.to(DEV).transpose(1, 2).contiguous().transpose(1, 2)
        packed = cc.causal_conv1d_fn(xg, w.to(DEV), b.to(DEV), seq_idx=seq.to(DEV), activation="silu")
        for bi in range(B):
            bounds = [0] + [t for t in range(1, L) if seq[bi, t] != seq[bi, t - 1]] + [L]
            for lo, hi in zip(bounds[:-1], bounds[1:]):
                alone = cc.causal_conv1d_fn(xg[bi:bi + 1, :, lo:hi], w.to(DEV), b.to(DEV), activation="silu")
                assert torch.equal(bits(packed[bi:bi + 1, :, lo:hi]), bits(alone)), (bi, lo, hi)


def test_seq_idx_constant_is_no_seq_idx(cc):
    g = torch.Generator().manual_seed(72)
    x = torch.randn(8, 3456, 256, generator=g).bfloat16().to(DEV).transpose(1, 2).contiguous().transpose(1, 2)
    w = (torch.randn(3456, 4, generator=g) * 0.02).bfloat16().to(DEV)
    seq = torch.full((8, 256), 5, dtype=torch.int32, device=DEV)
    a = cc.causal_conv1d_fn(x, w, seq_idx=seq, residual=True)
    b = cc.causal_conv1d_fn(x, w, residual=True)
    assert torch.equal(bits(a), bits(b))


def test_more_than_2_31_elements(cc):
    """Index arithmetic past 32 bits: 2.26e9 elements per tensor (4.5 GB of bf16).  The CPU oracle is
    run on a few (batch, channel) rows only; the rest is covered by a size-independent property, a batch
    row convolved alone gives the bits it has inside the big call."""
    B, C, L = 64, 3456, 10240
    assert B * C * L > 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(99)
    w_cpu = (torch.randn(C, 4, generator=torch.Generator().manual_seed(98)) * 0.3).bfloat16()
    w = w_cpu.to(DEV)
    for layout in ("bcl", "blc"):
        if layout == "bcl":
            x = torch.empty(B, C, L, dtype=torch.bfloat16, device=DEV)
        else:
            x = torch.empty(B, L, C, dtype=torch.bfloat16, device=DEV).transpose(1, 2)
        for b in range(B):
            x[b].copy_(torch.randn(C, L, generator=g, device=DEV))
        assert cc.kernel_plan_fwd(x, w) == f"{layout}_vec"
        out, state = cc.causal_conv1d_fn(x, w, activation=None, residual=True, return_final_states=True)
        torch.cuda.synchronize()
        for b in (0, 31, 63):
            alone, st = cc.causal_conv1d_fn(x[b:b + 1], w, residual=True, return_final_states=True)
            assert torch.equal(bits(out[b:b + 1]), bits(alone)), (layout, b)
            assert torch.equal(bits(state[b:b + 1]), bits(st)), (layout, b)
        # the last rows in memory against the oracle
        xs = x[B - 1:, C - 8:, :].contiguous().cpu()
        want, want_state = co.conv1d_fwd(xs, w_cpu[C - 8:], None, residual=1, final_state_len=3)
        assert torch.equal(bits(out[B - 1:, C - 8:, :]), bits(want)), layout
        assert torch.equal(bits(state[B - 1:, C - 8:, :]), bits(want_state)), layout
        del x, out, state
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_time_contiguous_rows_off_the_16_byte_grid(cc, dtype):
    """Row lengths that are not a multiple of the vector size: every row starts at a different misalignment,
    the aligned middle takes the vector code, the few elements around it are computed one per lane."""
    g = torch.Generator().manual_seed(91)
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    for (B, C, L), W in itertools.product([(2, 24, 16 * E + 1), (3, 7, 1023), (1, 40, 16 * E + E - 1), (2, 5, 2049),
                                           (2, 16, 700)], [2, 3, 4]):
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
        init = torch.randn(B, C, 5, generator=g).to(dtype)
        for act, res, m, st in [(None, False, None, False), ("silu", "masked", mask, True), (None, "unmasked", mask, False),
                                ("silu", True, None, True)]:
            want = co.conv1d_fwd(x, w, b, mask=m, activation=act, residual=res,
                                 initial_state=init if st else None, final_state_len=8 if st else None)
            xg = x.to(DEV)
            assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "bcl_vec", (B, C, L)
            got = run_fwd(cc, xg, w, b, act=act, mask=m, residual=res, init=init if st else None, S_out=8 if st else None)
            what = f"edge/{dtype}/{B}x{C}x{L}/W{W}/{act}/{res}/mask{m is not None}/state{st}"
            xm = x if m is None else (x.float() * m[:, None, :].float()).to(dtype)
            if st:
                assert_parity(got[0], want[0], exact=act is None, what=what, res=xm if res else None)
                assert torch.equal(bits(got[1]), bits(want[1])), what
            else:
                assert_parity(got, want, exact=act is None, what=what, res=xm if res else None)


def test_large_time_contiguous_launches_in_blocks_of_eight_waves(cc):
    """Unmasked time-contiguous launches of 16384 waves or more run in blocks of eight waves: a last block that is
    not full, rows off the 16-byte grid, rows of two segments; and the same rows with a mask (single-wave blocks)."""
    g = torch.Generator().manual_seed(97)
    for (B, C, L) in [(7, 2403, 1023), (2, 4211, 4100)]:
        x = torch.randn(B, C, L, generator=g).bfloat16()
        w = (torch.randn(C, 4, generator=g) * 0.3).bfloat16()
        b = (torch.randn(C, generator=g) * 0.1).bfloat16()
        mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
        xg = x.to(DEV)
        assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "bcl_vec", (B, C, L)
        # the three regimes of the block size: eight waves here, one with a mask, four in a small launch
        assert cc.kernel_plan_fwd_waves(xg, w.to(DEV)) == 8, (B, C, L)
        assert cc.kernel_plan_fwd_waves(xg, w.to(DEV), attention_mask=mask.to(DEV)) == 1
        assert cc.kernel_plan_fwd_waves(xg[:1, :512], w[:512].to(DEV)) == 4
        for m, res in ((None, True), (mask, "masked")):
            want, want_state = co.conv1d_fwd(x, w, b, mask=m, residual=res, final_state_len=8)
            got, state = run_fwd(cc, xg, w, b, mask=m, residual=res, S_out=8)
            what = f"big/{B}x{C}x{L}/mask{m is not None}"
            assert_parity(got, want, exact=True, what=what)
            assert torch.equal(bits(state), bits(want_state)), what


@pytest.mark.parametrize("dtype,shape", [(torch.bfloat16, (2, 40, 4096)), (torch.bfloat16, (1, 24, 8192 + 64)),
                                         (torch.float32, (1, 16, 4096)), (torch.float16, (3, 8, 2048 + 512))])
def test_long_unmasked_time_contiguous_rows_of_several_segments(cc, dtype, shape):
    """Aligned rows longer than one wave covers, without a mask: every segment after a row's first takes its three
    inputs of history from the vector before it, which its first lane requests together with the segment.  Widths
    2-4, SiLU, both residual settings, initial and final states, both rounding modes."""
    g = torch.Generator().manual_seed(shape[2])
    B, C, L = shape
    x = torch.randn(B, C, L, generator=g).to(dtype)
    init = torch.randn(B, C, 4, generator=g).to(dtype)
    xg = x.to(DEV)
    for W in (2, 3, 4):
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "bcl_vec"
        for act, res, st in [(None, True, True), ("silu", False, False), ("silu", True, True)]:
            want = co.conv1d_fwd(x, w, b, activation=act, residual=1 if res else 0,
                                 initial_state=init if st else None, final_state_len=5 if st else None)
            want_out, want_fs = want if st else (want, None)
            r = run_fwd(cc, xg, w, b, act=act, residual=res, init=init if st else None, S_out=5 if st else None)
            got, fs = r if st else (r, None)
            what = f"long rows/{dtype}/{shape}/W{W}/{act}/res{res}/state{st}"
            assert_parity(got, want_out, exact=act is None, what=what, res=x if res else None)
            if st:
                assert torch.equal(bits(fs), bits(want_fs)), what
        want = co.conv1d_fwd(x, w, b, residual=1, round_mode=1)
        assert torch.equal(bits(run_fwd(cc, xg, w, b, residual=True, rounding="eager")), bits(want)), f"{shape}/W{W}/eager"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_short_time_contiguous_rows_share_a_wave(cc, dtype):
    """Rows of 1..32 whole vectors: 2..64 rows per wave (every power-of-two group size, vector counts on and
    off the powers of two, row counts that leave the last wave partly empty), all options, both state ends."""
    g = torch.Generator().manual_seed(92)
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    shapes = [(3, 7, 1), (2, 33, 2), (1, 5, 3), (2, 9, 5), (3, 16, 8), (1, 21, 13), (2, 6, 16), (1, 11, 17), (2, 3, 31), (1, 67, 32)]
    for (B, C, nvec), W in itertools.product(shapes, [2, 3, 4]):
        L = nvec * E
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        mask = right_padded_mask(torch.randint(1, L + 1, (B,), generator=g).tolist(), L)
        init = torch.randn(B, C, 5, generator=g).to(dtype)
        for act, res, m, st in [(None, False, None, False), ("silu", "masked", mask, True), (None, "unmasked", mask, False),
                                ("silu", True, None, True)]:
            want = co.conv1d_fwd(x, w, b, mask=m, activation=act, residual=res,
                                 initial_state=init if st else None, final_state_len=8 if st else None)
            xg = x.to(DEV)
            assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "bcl_vec_short", (B, C, L)
            got = run_fwd(cc, xg, w, b, act=act, mask=m, residual=res, init=init if st else None, S_out=8 if st else None)
            what = f"short/{dtype}/{B}x{C}x{L}/W{W}/{act}/{res}/mask{m is not None}/state{st}"
            xm = x if m is None else (x.float() * m[:, None, :].float()).to(dtype)
            if st:
                assert_parity(got[0], want[0], exact=act is None, what=what, res=xm if res else None)
                assert torch.equal(bits(got[1]), bits(want[1])), what
            else:
                assert_parity(got, want, exact=act is None, what=what, res=xm if res else None)
    # channel slices of a wider tensor keep the kernel as long as the rows stay on the 16-byte grid
    big = torch.randn(2, 40, 4 * E, generator=g).to(dtype)
    w = (torch.randn(24, 4, generator=g) * 0.3).to(dtype)
    xg = big.to(DEV)[:, 8:32]
    assert cc.kernel_plan_fwd(xg, w.to(DEV)) == "bcl_vec_short"
    assert_parity(run_fwd(cc, xg, w, None, residual=True), co.conv1d_fwd(big[:, 8:32].contiguous(), w, None, residual=1),
                  exact=True, what="short/slice")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_update_ring_buffer_and_state_pool(cc, dtype):
    """cache_seqlens (ring buffer) and conv_state_indices (rows of a state pool) against the oracle, whose
    two modes are pinned by their equivalence with the shift register."""
    g = torch.Generator().manual_seed(85)
    for (B, C), W, S in itertools.product([(4, 264), (3, 20), (64, 3456)], [2, 4], [3, 4, 8, 6]):
        if S < W - 1:
            continue
        rows = B + 3
        w = (torch.randn(C, W, generator=g) * 0.3).to(dtype)
        b = (torch.randn(C, generator=g) * 0.1).to(dtype)
        pool_ref = torch.randn(rows, C, S, generator=g).to(dtype)
        ring_ref = torch.randn(B, C, S, generator=g).to(dtype)
        idx = torch.randperm(rows, generator=g)[:B].to(torch.int32)
        # entries whose index lies outside the pool (upstream's padding slots) are skipped: nothing of them is touched
        idx[0] = -1
        if B > 2:
            idx[B - 1] = rows + 5
        pool_gpu, ring_gpu = pool_ref.to(DEV), ring_ref.to(DEV)
        lane_channels = 2 if (w.element_size() == 2 and S != 8) else 1     # a lane owns 12..16 bytes of state
        expect_plan = "update_vec" if (S in (3, 4, 8) and C % lane_channels == 0) else "update_generic"
        assert cc.kernel_plan_update(torch.empty(B, C, dtype=dtype, device=DEV), pool_gpu[:B], w.to(DEV)) == expect_plan
        for step in range(S + 2):
            x = torch.randn(B, C, generator=g).to(dtype)
            seqlens = torch.randint(0, 1000, (B,), generator=g).to(torch.int32) if step else torch.zeros(B, dtype=torch.int32)
            what = f"{dtype}/{B}x{C}/W{W}/S{S}/step{step}"
            want = co.conv1d_update_ext(x, pool_ref, w, b, activation="silu", residual=True, conv_state_indices=idx)
            got = cc.causal_conv1d_update(x.to(DEV), pool_gpu, w.to(DEV), b.to(DEV), activation="silu", residual=True,
                                          conv_state_indices=idx.to(DEV))
            assert_parity(got, want, exact=False, what="pool/" + what, res=x)
            assert torch.equal(bits(pool_gpu), bits(pool_ref)), what
            want = co.conv1d_update_ext(x, ring_ref, w, b, activation=None, residual=False, cache_seqlens=seqlens)
            got = cc.causal_conv1d_update(x.to(DEV), ring_gpu, w.to(DEV), b.to(DEV), cache_seqlens=seqlens.to(DEV))
            assert_parity(got, want, exact=True, what="ring/" + what)
            assert torch.equal(bits(ring_gpu), bits(ring_ref)), what


def test_randomised_shapes_layouts_and_options(cc):
    """300 seeded random calls across layouts (time-contiguous, channel-contiguous, both as slices of larger
    tensors), sizes around every vector / tile boundary, dtypes, widths and options, each against the oracle."""
    g = torch.Generator().manual_seed(2024)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    def pick(seq):
        return seq[ri(0, len(seq) - 1)]

    plans = {}
    for case in range(300):
        dtype = pick([torch.bfloat16, torch.float32, torch.float16])
        W = pick([2, 3, 4])
        B = ri(1, 3)
        C = pick([1, 3, 4, 8, 12, 20, 64, 100, 256, 260, 520])
        L = pick([1, 2, 3, 5, 8, 31, 32, 33, 64, 127, 128, 129, 136, 200, 255, 257, 515])
        layout = pick(["bcl", "blc", "bcl_slice", "blc_slice"])
        act = pick([None, "silu"])
        res = pick([False, "masked", "unmasked"])
        use_mask = ri(0, 1)
        use_bias = ri(0, 1)
        mode = pick(["plain", "plain", "state", "seq"])
        wdt = pick([dtype, dtype, torch.float32])      # x's own type, or fp32 master weights
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, W, generator=g) * 0.4).to(wdt)
        b = (torch.randn(C, generator=g) * 0.2).to(wdt) if use_bias else None
        mask = right_padded_mask([ri(1, L) for _ in range(B)], L, dtype=pick([torch.int64, torch.bool, torch.float32])) \
            if use_mask else None
        if layout == "bcl":
            xg = x.to(DEV)
        elif layout == "blc":
            xg = x.to(DEV).transpose(1, 2).contiguous().transpose(1, 2)
        elif layout == "bcl_slice":
            big = torch.zeros(B, C + 3, L + 8, dtype=dtype, device=DEV)
            big[:, 1:C + 1, 8:] = x.to(DEV)
            xg = big[:, 1:C + 1, 8:]
        else:
            big = torch.zeros(B, L + 2, C + 8, dtype=dtype, device=DEV)
            big[:, 1:L + 1, 8:] = x.to(DEV).transpose(1, 2)
            xg = big[:, 1:L + 1, 8:].transpose(1, 2)
        kw = dict(activation=act, residual=res, attention_mask=None if mask is None else mask.to(DEV))
        what = f"case {case}: {dtype} w{wdt} {layout} {B}x{C}x{L} W{W} {act} {res} mask{use_mask} bias{use_bias} {mode}"
        xm = x if mask is None else (x.float() * mask[:, None, :].float()).to(dtype)
        if mode == "seq":
            seq = packed_seq_idx(B, L, g)
            want = co.conv1d_fwd_seq(x, w, b, seq, mask=mask, activation=act, residual=res)
            got = cc.causal_conv1d_fn(xg, w.to(DEV), None if b is None else b.to(DEV), seq_idx=seq.to(DEV), **kw)
            plan = cc.kernel_plan_fwd(xg, w.to(DEV), seq_idx=seq.to(DEV))
        elif mode == "state":
            S_in, S_out = ri(W - 1, 9), ri(1, 9)
            init = torch.randn(B, C, S_in, generator=g).to(dtype)
            want, want_state = co.conv1d_fwd(x, w, b, mask=mask, activation=act, residual=res, initial_state=init,
                                             final_state_len=S_out)
            fs = torch.full((B, C, S_out), float("nan"), dtype=dtype, device=DEV)
            got, _ = cc.causal_conv1d_fn(xg, w.to(DEV), None if b is None else b.to(DEV), initial_states=init.to(DEV),
                                         final_states_out=fs, **kw)
            assert torch.equal(bits(fs), bits(want_state)), what
            plan = cc.kernel_plan_fwd(xg, w.to(DEV))
        else:
            want = co.conv1d_fwd(x, w, b, mask=mask, activation=act, residual=res)
            got = cc.causal_conv1d_fn(xg, w.to(DEV), None if b is None else b.to(DEV), **kw)
            plan = cc.kernel_plan_fwd(xg, w.to(DEV))
        plans[plan] = plans.get(plan, 0) + 1
        added = None if not res else (x if res == "unmasked" else xm)      # the term the sum may cancel against
        assert_parity(got, want, exact=act is None, what=what, res=added)
    # the draw reaches every kernel family
    assert set(plans) >= {"bcl_vec", "bcl_vec_short", "blc_vec", "blc_vec_seq", "generic"}, plans


def test_randomised_large_channel_contiguous_launches(cc):
    """Twelve seeded random channel-contiguous calls that move 40-90 MB (the launches with their own slab length,
    store policy and request order): one tensor or two equal dense parts, channel counts that end inside a tile,
    lengths that end inside a slab, with and without mask / SiLU / states, each against the oracle."""
    g = torch.Generator().manual_seed(4040)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    def pick(seq):
        return seq[ri(0, len(seq) - 1)]

    plans = {}
    for case in range(12):
        dtype = pick([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        es = torch.empty(0, dtype=dtype).element_size()
        pair = case % 2 == 1
        C = 8 * ri(60, 500)                                   # a multiple of 8, so that two equal parts stay whole lanes
        B = ri(1, 4)
        target = ri(42, 90) << 20
        L = max(40, target // (2 * B * C * es))
        act = pick([None, "silu"])
        res = pick([False, "masked", "unmasked"])
        use_mask, use_state = ri(0, 1), ri(0, 1)
        wdt = pick([dtype, torch.float32])
        x = torch.randn(B, C, L, generator=g).to(dtype)
        w = (torch.randn(C, 4, generator=g) * 0.4).to(wdt)
        b = (torch.randn(C, generator=g) * 0.2).to(wdt)
        mask = right_padded_mask([ri(1, L) for _ in range(B)], L, dtype=pick([torch.int64, torch.bool])) if use_mask else None
        init = torch.randn(B, C, 4, generator=g).to(dtype) if use_state else None
        want = co.conv1d_fwd(x, w, b, mask=mask, activation=act, residual=res, initial_state=init,
                             final_state_len=7 if use_state else None)
        want_out, want_state = want if use_state else (want, None)
        kw = dict(activation=act, residual=res, attention_mask=None if mask is None else mask.to(DEV),
                  initial_states=None if init is None else init.to(DEV),
                  final_states_out=torch.full((B, C, 7), float("nan"), dtype=dtype, device=DEV) if use_state else None)
        what = f"case {case}: {dtype} w{wdt} {'pair' if pair else 'one'} {B}x{C}x{L} {act} {res} mask{use_mask} state{use_state}"
        if pair:
            xs = [t.transpose(1, 2).contiguous().to(DEV).transpose(1, 2) for t in x.split([C // 2, C // 2], dim=1)]
            plan = cc.kernel_plan_fwd_parts(xs, w.to(DEV), attention_mask=kw["attention_mask"])
            r = cc.causal_conv1d_fn_parts(xs, w.to(DEV), b.to(DEV), **kw)
            outs, fs = r if use_state else (r, None)
            got = torch.cat([o.contiguous() for o in outs], dim=1)
        else:
            xg = x.transpose(1, 2).contiguous().to(DEV).transpose(1, 2)
            plan = cc.kernel_plan_fwd(xg, w.to(DEV))
            r = cc.causal_conv1d_fn(xg, w.to(DEV), b.to(DEV), **kw)
            got, fs = r if use_state else (r, None)
        plans[plan] = plans.get(plan, 0) + 1
        xm = x if mask is None else (x.float() * mask[:, None, :].float()).to(dtype)
        added = None if not res else (x if res == "unmasked" else xm)
        assert_parity(got, want_out, exact=act is None, what=what, res=added)
        if use_state:
            assert torch.equal(bits(fs), bits(want_state)), what
        del x, got, want, want_out
    assert set(plans) == {"blc_vec", "blc_vec_pair"}, plans


def test_randomised_decode_steps(cc):
    """200 seeded random decode calls: dtypes, widths, state lengths, strided states, token masks, residual
    modes, ring-buffer and state-pool addressing, each carried for three steps against the oracle."""
    g = torch.Generator().manual_seed(4048)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    def pick(seq):
        return seq[ri(0, len(seq) - 1)]

    for case in range(200):
        dtype = pick([torch.bfloat16, torch.float32, torch.float16])
        W = pick([2, 3, 4])
        S = pick([s for s in (1, 2, 3, 4, 5, 8, 9) if s >= W - 1])
        B, C = ri(1, 5), pick([1, 4, 8, 12, 24, 64, 264, 1032])
        act = pick([None, "silu"])
        mode = pick(["plain", "plain", "ring", "pool", "strided"])
        res = pick([False, True])
        wdt = pick([dtype, dtype, torch.float32])      # x's own type, or fp32 master weights
        w = (torch.randn(C, W, generator=g) * 0.4).to(wdt)
        b = (torch.randn(C, generator=g) * 0.2).to(wdt) if ri(0, 1) else None
        rows = B + 2 if mode == "pool" else B
        state_ref = torch.randn(rows, C, S, generator=g).to(dtype)
        if mode == "strided":
            big = torch.zeros(rows, C, S + 3, dtype=dtype, device=DEV)
            state_gpu = big[:, :, 1:S + 1]
            state_gpu.copy_(state_ref.to(DEV))
        else:
            state_gpu = state_ref.to(DEV)
        idx = torch.randperm(rows, generator=g)[:B].to(torch.int32) if mode == "pool" else None
        for step in range(3):
            x = torch.randn(B, C, generator=g).to(dtype)
            sl = torch.randint(0, 50, (B,), generator=g).to(torch.int32) if mode == "ring" else None
            want = co.conv1d_update_ext(x, state_ref, w, b, activation=act, residual=res, cache_seqlens=sl,
                                        conv_state_indices=idx)
            xg = x.to(DEV)
            if (case + step) % 3 == 0:      # the token as a slice of a wider tensor (odd offsets fail the alignment test)
                off = (case + step) % 4
                wide = torch.zeros(B, C + 5, dtype=dtype, device=DEV)
                wide[:, off:off + C] = xg
                xg = wide[:, off:off + C]
            got = cc.causal_conv1d_update(xg, state_gpu, w.to(DEV), None if b is None else b.to(DEV), activation=act,
                                          residual=res, cache_seqlens=None if sl is None else sl.to(DEV),
                                          conv_state_indices=None if idx is None else idx.to(DEV))
            what = f"case {case}: {dtype} w{wdt} {B}x{C} W{W} S{S} {act} res{res} {mode} step{step}"
            assert_parity(got, want, exact=act is None, what=what, res=x if res else None)
            assert torch.equal(bits(state_gpu), bits(state_ref)), what
