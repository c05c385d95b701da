"""canon_conv1d_bwd_static (the entry point for callers that cannot allocate device memory) against
canon_conv1d_bwd, through the C ABI: same dx / dweight / dbias bit for bit, on two calls in a row, the second
on a smaller input (the static scratch still holds the first call's partial sums then)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _params(_lib, x, dout, dx, weight, bias, mask, dweight, dbias, act, res):
    p = _lib.BwdParams()
    p.struct_size = ctypes.sizeof(_lib.BwdParams)
    p.x_dtype = _lib.DTYPE_CODE[x.dtype]
    p.w_dtype = _lib.DTYPE_CODE[weight.dtype]
    p.width = weight.shape[1]
    p.activation, p.residual_mode = act, res
    p.batch, p.channels, p.seqlen = x.shape
    p.x = x.data_ptr()
    p.x_stride_b, p.x_stride_c, p.x_stride_l = x.stride()
    p.dout = dout.data_ptr()
    p.dout_stride_b, p.dout_stride_c, p.dout_stride_l = dout.stride()
    p.dx = dx.data_ptr()
    p.dx_stride_b, p.dx_stride_c, p.dx_stride_l = dx.stride()
    p.weight = weight.data_ptr()
    p.w_stride_c, p.w_stride_k = weight.stride()
    p.bias = bias.data_ptr() if bias is not None else None
    if mask is not None:
        p.mask = mask.data_ptr()
        p.mask_dtype = _lib.MASK_CODE[mask.dtype]
        p.mask_stride_b, p.mask_stride_l = mask.stride()
    p.dweight = dweight.data_ptr()
    p.dbias = dbias.data_ptr() if dbias is not None else None
    return p


def _both(_lib, shape, layout, dtype, act, res, with_mask, seed):
    """(dx, dweight, dbias) of canon_conv1d_bwd and of canon_conv1d_bwd_static for one seeded problem."""
    L = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    B, C, T = shape
    x = torch.randn(B, C, T, generator=g).to(dtype).to(DEV)
    dout = torch.randn(B, C, T, generator=g).to(dtype).to(DEV)
    if layout == "blc":
        x = x.transpose(1, 2).contiguous().transpose(1, 2)
        dout = dout.transpose(1, 2).contiguous().transpose(1, 2)
    weight = (torch.randn(C, 4, generator=g) * 0.3).to(dtype).to(DEV)
    bias = (torch.randn(C, generator=g) * 0.1).to(dtype).to(DEV)
    mask = None
    if with_mask:
        mask = torch.ones(B, T, dtype=torch.int64)
        for b in range(B):
            mask[b, T - (b * 7) % (T // 2):] = 0
        mask = mask.to(DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    results = []
    for static in (False, True):
        dx = torch.full_like(x, float("nan"))
        dweight = torch.full((C, 4), float("nan"), dtype=torch.float32, device=DEV)
        dbias = torch.full((C,), float("nan"), dtype=torch.float32, device=DEV)
        p = _params(_lib, x, dout, dx, weight, bias, mask, dweight, dbias, act, res)
        if static:
            rc = L.canon_conv1d_bwd_static(ctypes.byref(p), stream)
        else:
            nbytes = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(p))
            assert 0 < nbytes <= 8 << 20
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
            p.workspace, p.workspace_bytes = workspace.data_ptr(), nbytes
            rc = L.canon_conv1d_bwd(ctypes.byref(p), stream)
        assert rc == 0, L.canon_conv1d_last_error().decode()
        torch.cuda.synchronize()
        results.append((dx, dweight, dbias))
    return results


def _same(a, b):
    for u, v, name in zip(a, b, ("dx", "dweight", "dbias")):
        assert not torch.isnan(u.float()).any() and not torch.isnan(v.float()).any(), name
        iu = u.contiguous().view(torch.int16 if u.element_size() == 2 else torch.int32)
        iv = v.contiguous().view(torch.int16 if v.element_size() == 2 else torch.int32)
        assert torch.equal(iu, iv), f"{name}: the static-scratch call differs from canon_conv1d_bwd"


@pytest.mark.parametrize("layout", ["blc", "bcl"])
def test_static_scratch_backward_equals_the_workspace_call(layout):
    from causal_conv1d import _lib
    # a larger problem first, then a smaller one: the scratch keeps the first call's partial sums
    big = _both(_lib, (4, 640, 1024), layout, torch.bfloat16, act=1, res=1, with_mask=True, seed=1)
    _same(*big)
    small = _both(_lib, (2, 96, 200), layout, torch.bfloat16, act=0, res=2, with_mask=False, seed=2)
    _same(*small)
    tiny = _both(_lib, (1, 8, 5), layout, torch.float32, act=1, res=0, with_mask=True, seed=3)   # strided kernel
    _same(*tiny)


def test_static_scratch_backward_rejects_what_does_not_fit():
    from causal_conv1d import _lib
    L = _lib.lib()
    # the strided kernel on a large odd shape needs more than the static buffer: sized on the host, no launch
    B, C, T = 256, 3457, 1024
    p = _lib.BwdParams()
    p.struct_size = ctypes.sizeof(_lib.BwdParams)
    p.x_dtype = p.w_dtype = 1
    p.width = 4
    p.batch, p.channels, p.seqlen = B, C, T
    fake = 1 << 20
    p.x, p.dout, p.dx, p.weight, p.dweight = fake, fake * 2, fake * 3, fake * 4, fake * 5
    for name in ("x", "dout", "dx"):
        setattr(p, name + "_stride_b", C * T)
        setattr(p, name + "_stride_c", 1)
        setattr(p, name + "_stride_l", C)
    p.w_stride_c, p.w_stride_k = 4, 1
    need = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(p))
    assert need > 8 << 20
    rc = L.canon_conv1d_bwd_static(ctypes.byref(p), None)
    assert rc == _lib.ERR_UNSUPPORTED
    assert "static buffer holds 8388608" in L.canon_conv1d_last_error().decode()


def _problem(_lib, shape, seed):
    """One channel-contiguous bf16 problem with its argument block (workspace fields unset)."""
    g = torch.Generator().manual_seed(seed)
    B, C, T = shape
    x = torch.randn(B, T, C, generator=g).bfloat16().to(DEV).transpose(1, 2)
    dout = torch.randn(B, T, C, generator=g).bfloat16().to(DEV).transpose(1, 2)
    weight = (torch.randn(C, 4, generator=g) * 0.3).bfloat16().to(DEV)
    bias = (torch.randn(C, generator=g) * 0.1).bfloat16().to(DEV)
    dx = torch.empty_like(x)
    dweight = torch.empty(C, 4, dtype=torch.float32, device=DEV)
    dbias = torch.empty(C, dtype=torch.float32, device=DEV)
    p = _params(_lib, x, dout, dx, weight, bias, None, dweight, dbias, 1, 1)
    return p, (x, dout, weight, bias), (dx, dweight, dbias)


def test_static_scratch_backward_allocates_nothing_after_the_device_is_set_up():
    """Free device memory as the driver reports it is the same before and after calls of the static-scratch entry
    point, once canon_conv1d_init has set the device up (the code objects and the scratch array are in place)."""
    from causal_conv1d import _lib
    L = _lib.lib()
    assert L.canon_conv1d_init() == 0, L.canon_conv1d_last_error().decode()
    assert L.canon_conv1d_init() == 0                       # idempotent
    p, keep, outs = _problem(_lib, (4, 640, 512), 11)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # one warm-up call: whatever the runtime sets up at a kernel's first launch is in place after it
    assert L.canon_conv1d_bwd_static(ctypes.byref(p), stream) == 0, L.canon_conv1d_last_error().decode()
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert L.canon_conv1d_bwd_static(ctypes.byref(p), stream) == 0, L.canon_conv1d_last_error().decode()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"free device memory changed by {free0 - free1} bytes across calls that must not allocate"


def test_static_scratch_backward_captured_in_a_hip_graph_replays_exactly():
    """The call recorded into a HIP graph (what it exists for) and replayed several times, with eager work and
    synchronisations in between and the inputs rewritten before every replay: each replay equals
    canon_conv1d_bwd on the same inputs bit for bit."""
    from causal_conv1d import _lib
    L = _lib.lib()
    assert L.canon_conv1d_init() == 0
    p, (x, dout, weight, bias), (dx, dweight, dbias) = _problem(_lib, (3, 960, 384), 12)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                           # warm-up outside the capture
        assert L.canon_conv1d_bwd_static(ctypes.byref(p), ctypes.c_void_p(side.cuda_stream)) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = L.canon_conv1d_bwd_static(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, L.canon_conv1d_last_error().decode()
    g = torch.Generator(device=DEV).manual_seed(13)
    for replay in range(3):
        x.copy_(torch.randn(x.shape, generator=g, device=DEV))          # new inputs in the captured buffers
        dout.copy_(torch.randn(dout.shape, generator=g, device=DEV))
        for t in (dx, dweight, dbias):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (dx, dweight, dbias)]
        # the reference: the workspace call, launched eagerly on the same inputs
        want = [torch.full_like(t, float("nan")) for t in (dx, dweight, dbias)]
        q = _params(_lib, x, dout, want[0], weight, bias, None, want[1], want[2], 1, 1)
        nbytes = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(q))
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        q.workspace, q.workspace_bytes = workspace.data_ptr(), nbytes
        assert L.canon_conv1d_bwd(ctypes.byref(q), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        torch.cuda.synchronize()
        _same(got, want)
