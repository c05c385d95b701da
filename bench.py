#!/usr/bin/env python3
"""Benchmark of the Canon causal depthwise conv1d hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one prefill launch over bf16 x[B=8, C=3456, L=1024] (bias, residual
add fused, no activation), inputs resident in HBM.  Launches rotate over
enough distinct (x, out) buffer pairs that the working set is several times
the 256 MB Infinity Cache, so the rate is an HBM rate, not a cache rate.
Launches go through the C ABI (canon_conv1d_fwd) with prebuilt argument
structs; time is taken with HIP events on the launch stream.

The one JSON line also carries: the decode update (B=256, C=3456, state 3,
64 carried steps) in microseconds per step, the same prefill in the
channel-contiguous layout (one tensor, and gate / up as two tensors through the
multi-part call), its backward, the roofline fraction, and a CPU baseline (the
eager PyTorch formulation of the reference on this box's host cores).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "viby-model_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, vendor figure
# HBM bytes per launch of the headline kernel as rocprofv3 counted them (FETCH_SIZE / WRITE_SIZE scaled by a plain
# copy of known size): read from the committed summary of that profile, not measured by this run
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "prefill_time_contiguous_bf16_B8_C3456_L1024.txt")


def profiled_traffic_bytes():
    """'traffic per launch N MB' of the committed profile of the headline kernel, in bytes (None if absent)."""
    import re
    try:
        m = re.search(r"traffic per launch ([0-9.]+) MB", open(TRAFFIC_PROFILE).read())
    except OSError:
        return None
    return float(m.group(1)) * 1e6 if m else None


B, C, L, W = 8, 3456, 1024, 4   # the configuration the metric is quoted on
DEC_B, DEC_S, DEC_STEPS = 256, 3, 64


def prefill_bytes(b, c, l, esize=2, wsize=2):
    # one read of x, one write of out, taps and bias once
    return 2 * b * c * l * esize + c * W * wsize + c * wsize


def decode_bytes(b, c, s, esize=2, wsize=2):
    # state read + written, token read, output written, taps and bias
    return b * c * (2 * s + 2) * esize + c * W * wsize + c * wsize


CLOCK_RAMP_S = 0.03   # untimed load before the warm-up steps: the first ~10 ms after idle run ~1 % slower (clocks ramping)


PREFILL_ACT = 0       # activation of the prefill legs (0 none, 1 SiLU: --activation silu)
REGIONS = 9           # back-to-back timed regions of `steps` launches each; the median region is the figure reported


def time_region(fn, steps, warmup, ramp=True, regions=None, stats=None):
    """ms per step: `regions` timed regions of exactly `steps` steps each, one after the other on the launch stream,
    each bracketed by events; the MEDIAN region is returned (a single region of 20 launches is 0.4 ms: one
    scheduling hiccup of the host moves it by several percent).  `stats`, a dict, receives min / max / regions."""
    import torch
    regions = regions or REGIONS
    t_end = time.perf_counter() + (CLOCK_RAMP_S if ramp else 0.0)
    i = 0
    while time.perf_counter() < t_end and i < 1500:   # bounded both ways: launches are slow under a profiler
        fn(i)
        i += 1
    torch.cuda.synchronize()
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True) for _ in range(regions + 1)]
    events[0].record()
    k = 0
    for r in range(regions):
        for _ in range(steps):
            fn(k)
            k += 1
        events[r + 1].record()
    torch.cuda.synchronize()
    times = sorted(events[r].elapsed_time(events[r + 1]) / steps for r in range(regions))
    if stats is not None:
        stats.update({"regions": regions, "min_ms_per_step": round(times[0], 6), "max_ms_per_step": round(times[-1], 6)})
    return times[len(times) // 2]  # ms per step


def graph_of(run):
    """`run(stream)` captured as one HIP graph on torch's current stream (after one uncaptured pass on a side
    stream, which loads what the launches need)."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(ctypes.c_void_p(side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return graph


def bench_prefill(layout, steps, warmup, nbuf, ramp=True, shape=None, dtype=None, rounding=0, with_mask=False,
                  as_graph=False, act=None, stats=None):
    """One prefill launch per step over `nbuf` rotating buffer pairs.  shape: (B, C, L), the metric's by default;
    dtype: torch.bfloat16 by default; rounding: 0 fused, 1 the eager module's rounding points; act: 1 = SiLU; with_mask: a
    right-padded padding mask of x's type and the masked residual (what CanonLayer passes); as_graph: the launches
    of one pass over the buffer pairs replayed as a HIP graph (for kernels shorter than the few microseconds this
    host needs to issue a launch from Python: back-to-back launches would measure the host)."""
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    Bx, Cx, Lx = shape or (B, C, L)
    dtype = dtype or torch.bfloat16
    act = PREFILL_ACT if act is None else act
    g = torch.Generator(device=dev).manual_seed(0)
    w = (torch.randn(Cx, W, generator=g, device=dev) * 0.02).to(dtype)
    bias = (torch.randn(Cx, generator=g, device=dev) * 0.01).to(dtype)
    mask = None
    if with_mask:
        lens = torch.randint(Lx // 8, Lx + 1, (Bx,), generator=g, device=dev)
        mask = (torch.arange(Lx, device=dev)[None, :] < lens[:, None]).to(dtype)
    # all buffer pairs are carved out of ONE allocation, as an arena-allocating runtime would hold them:
    # measured 1 % faster than separately allocated tensors (fewer, larger address-translation fragments)
    n = Bx * Cx * Lx
    pool = torch.empty(2 * nbuf * n, dtype=dtype, device=dev)
    xs, outs, params = [], [], []
    for i in range(nbuf):
        x, o = pool[2 * i * n:(2 * i + 1) * n], pool[(2 * i + 1) * n:(2 * i + 2) * n]
        if layout == "bcl":
            x, o = x.view(Bx, Cx, Lx), o.view(Bx, Cx, Lx)
        else:
            x, o = x.view(Bx, Lx, Cx).transpose(1, 2), o.view(Bx, Lx, Cx).transpose(1, 2)
        x.copy_(torch.randn(x.shape, generator=g, device=dev))
        xs.append(x)
        outs.append(o)
        params.append(cc._fill_fwd(x, o, w, bias, mask, None, None, act, 1, rounding))
    plan = _lib.lib().canon_conv1d_fwd_plan(ctypes.byref(params[0])).decode()
    fwd = _lib.lib().canon_conv1d_fwd
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    refs = [ctypes.byref(p) for p in params]

    def step(i):
        rc = fwd(refs[i % nbuf], stream)
        if rc:
            _lib.check(rc, "canon_conv1d_fwd")

    if as_graph:
        # at least 48 launches per replay, so that what a replay itself costs (about 10 us) is spread thin
        passes = max(1, -(-48 // nbuf))

        def some_passes(stream_):
            for _ in range(passes):
                for r in refs:
                    rc = fwd(r, stream_)
                    if rc:
                        _lib.check(rc, "canon_conv1d_fwd")
        graph = graph_of(some_passes)
        nodes = passes * nbuf
        ms = time_region(lambda i: graph.replay(), max(5, steps // nodes), 2, ramp, stats=stats) / nodes
        return ms, plan
    ms = time_region(step, steps, warmup, ramp, stats=stats)
    return ms, plan


def bench_ragged(layout, steps, warmup, nbuf, batch=32):
    """configs[2]: right-padded batch of 32, valid lengths uniform in [128, 1024], the padding mask multiplied
    in before the conv and the masked residual added (out = m*x + conv(m*x) + bias).  The mask is what the
    Python wrapper hands the kernel for a trainer's int64 mask on a problem of this size: narrowed to bf16."""
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(4)
    w = (torch.randn(C, W, generator=g, device=dev) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g, device=dev) * 0.01).bfloat16()
    lens = torch.randint(128, L + 1, (batch,), generator=g, device=dev)
    mask = (torch.arange(L, device=dev)[None, :] < lens[:, None]).to(torch.bfloat16)
    keep, refs = [], []
    for _ in range(nbuf):
        if layout == "bcl":
            x = torch.randn(batch, C, L, generator=g, device=dev).bfloat16()
        else:
            x = torch.randn(batch, L, C, generator=g, device=dev).bfloat16().transpose(1, 2)
        o = torch.empty_like(x)
        p = cc._fill_fwd(x, o, w, bias, mask, None, None, PREFILL_ACT, 1, 0)
        keep.append((x, o, p))
        refs.append(ctypes.byref(p))
    fwd = _lib.lib().canon_conv1d_fwd
    plan = _lib.lib().canon_conv1d_fwd_plan(refs[0]).decode()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        rc = fwd(refs[i % nbuf], stream)
        if rc:
            _lib.check(rc, "canon_conv1d_fwd")

    ms = time_region(step, steps, warmup)
    return ms, plan, prefill_bytes(batch, C, L) + batch * L * 2


def bench_copy(steps, warmup, nbuf):
    """What the runtime's own device-to-device copy of one x-sized buffer reaches on this GPU with the
    same buffer rotation: the same bytes as a kernel that reads x once and writes out once."""
    import torch
    n = B * C * L
    pool = torch.empty(2 * nbuf * n, dtype=torch.bfloat16, device="cuda:0").normal_()
    pairs = [(pool[2 * i * n:(2 * i + 1) * n], pool[(2 * i + 1) * n:(2 * i + 2) * n]) for i in range(nbuf)]

    def step(i):
        src, dst = pairs[i % nbuf]
        dst.copy_(src)

    return time_region(step, steps, warmup)


def bench_prefill_parts(steps, warmup, nbuf):
    """Canon-D as the model produces it: gate and up projections as two (B, L, C/2) tensors, convolved
    by one multi-part launch (no torch.cat, outputs stay split)."""
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(3)
    w = (torch.randn(C, W, generator=g, device=dev) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g, device=dev) * 0.01).bfloat16()
    keep, calls = [], []
    for _ in range(nbuf):
        xs = [torch.randn(B, L, C // 2, generator=g, device=dev).bfloat16().transpose(1, 2) for _ in range(2)]
        outs = [torch.empty_like(x) for x in xs]
        p = cc._fill_fwd(xs[0], outs[0], w, bias, None, None, None, PREFILL_ACT, 1, 0)
        p.channels = C
        p.x = p.out = None
        arr = cc._part_array(xs, outs)
        keep.append((xs, outs, p, arr))
        calls.append((ctypes.byref(p), arr))
    L_ = _lib.lib()
    plan = L_.canon_conv1d_fwd_parts_plan(calls[0][0], calls[0][1], 2).decode()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        ref, arr = calls[i % nbuf]
        rc = L_.canon_conv1d_fwd_parts(ref, arr, 2, stream)
        if rc:
            _lib.check(rc, "canon_conv1d_fwd_parts")

    ms = time_region(step, steps, warmup)
    return ms, plan


def bench_decode(reps, warmup):
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(1)
    w = (torch.randn(C, W, generator=g, device=dev) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g, device=dev) * 0.01).bfloat16()
    state = torch.randn(DEC_B, C, DEC_S, generator=g, device=dev).bfloat16()
    toks = torch.randn(DEC_STEPS, DEC_B, C, generator=g, device=dev).bfloat16()
    outs = torch.empty_like(toks)
    params = [cc._fill_update(toks[i], outs[i], state, w, bias, None, 0, 0, 0) for i in range(DEC_STEPS)]
    refs = [ctypes.byref(p) for p in params]
    upd = _lib.lib().canon_conv1d_update
    plan = _lib.lib().canon_conv1d_update_plan(refs[0]).decode()

    def run64(stream):
        for r in refs:
            rc = upd(r, stream)
            if rc:
                _lib.check(rc, "canon_conv1d_update")

    cur = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ms_eager = time_region(lambda i: run64(cur), reps, warmup) / DEC_STEPS

    # the same 64 carried steps as one HIP graph (what a decode loop would replay)
    graph = graph_of(run64)
    ms_graph = time_region(lambda i: graph.replay(), reps, warmup) / DEC_STEPS
    return ms_eager * 1e3, ms_graph * 1e3, plan


def bench_decode_backward(steps, warmup, nbuf=8):
    """Backward of one decode step at the decode configuration (with SiLU, state gradients both ways):
    token, saved state, dout and the updated state's gradient read; dx and the state's gradient written."""
    import torch
    from causal_conv1d import _lib
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(5)
    w = (torch.randn(C, W, generator=g, device=dev) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g, device=dev) * 0.01).bfloat16()
    dw = torch.empty(C, W, dtype=torch.float32, device=dev)
    db = torch.empty(C, dtype=torch.float32, device=dev)
    L_ = _lib.lib()
    keep, refs, ws = [], [], None
    for _ in range(nbuf):
        def t(*shape):
            return torch.randn(*shape, generator=g, device=dev).bfloat16()
        x, dout, dx = t(DEC_B, C), t(DEC_B, C), torch.empty(DEC_B, C, dtype=torch.bfloat16, device=dev)
        st, dso = t(DEC_B, C, DEC_S), t(DEC_B, C, DEC_S)
        ds = torch.empty_like(st)
        p = _lib.UpdateBwdParams()
        p.struct_size = ctypes.sizeof(_lib.UpdateBwdParams)
        p.x_dtype = p.w_dtype = 1
        p.width, p.activation, p.state_len = W, 1, DEC_S
        p.batch, p.channels = DEC_B, C
        for name, ten in (("x", x), ("dout", dout), ("dx", dx)):
            setattr(p, name, ten.data_ptr())
            setattr(p, name + "_stride_b", ten.stride(0))
            setattr(p, name + "_stride_c", ten.stride(1))
        p.conv_state = st.data_ptr()
        p.state_stride_b, p.state_stride_c, p.state_stride_s = st.stride()
        p.dstate_out = dso.data_ptr()
        p.dstate_out_stride_b, p.dstate_out_stride_c, p.dstate_out_stride_s = dso.stride()
        p.dstate = ds.data_ptr()
        p.dstate_stride_b, p.dstate_stride_c, p.dstate_stride_s = ds.stride()
        p.weight, p.w_stride_c, p.w_stride_k = w.data_ptr(), W, 1
        p.bias, p.dweight, p.dbias = bias.data_ptr(), dw.data_ptr(), db.data_ptr()
        if ws is None:
            ws = torch.empty(L_.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(p)), dtype=torch.uint8, device=dev)
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
        keep.append((x, dout, dx, st, dso, ds, p))
        refs.append(ctypes.byref(p))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        rc = L_.canon_conv1d_update_bwd(refs[i % nbuf], stream)
        if rc:
            _lib.check(rc, "canon_conv1d_update_bwd")

    ms = time_region(step, steps, warmup)
    elems = DEC_B * C
    return ms * 1e3, (3 * DEC_S + 3) * elems * 2, ws.numel()


def bench_backward(steps, warmup, nbuf, layout="channel_last"):
    """Backward of the same prefill step (channel-contiguous, as a training step through the model
    produces it, or time-contiguous): reads x and dout, writes dx, reduces dweight / dbias."""
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(2)
    w = (torch.randn(C, W, generator=g, device=dev) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g, device=dev) * 0.01).bfloat16()
    dw = torch.empty(C, W, dtype=torch.float32, device=dev)
    db = torch.empty(C, dtype=torch.float32, device=dev)
    keep, params = [], []
    for _ in range(nbuf):
        if layout == "channel_last":
            x = torch.randn(B, L, C, generator=g, device=dev).bfloat16().transpose(1, 2)
            dy = torch.randn(B, L, C, generator=g, device=dev).bfloat16().transpose(1, 2)
        else:
            x = torch.randn(B, C, L, generator=g, device=dev).bfloat16()
            dy = torch.randn(B, C, L, generator=g, device=dev).bfloat16()
        dx = torch.empty_like(x)
        p = _lib.BwdParams()
        p.struct_size = ctypes.sizeof(_lib.BwdParams)
        p.x_dtype = p.w_dtype = 1
        p.width, p.residual_mode = W, 1
        p.batch, p.channels, p.seqlen = B, C, L
        for name, t in (("x", x), ("dout", dy), ("dx", dx)):
            setattr(p, name, t.data_ptr())
            for sname, v in zip(("b", "c", "l"), t.stride()):
                setattr(p, f"{name}_stride_{sname}", v)
        p.weight, p.w_stride_c, p.w_stride_k, p.bias = w.data_ptr(), W, 1, bias.data_ptr()
        p.dweight, p.dbias = dw.data_ptr(), db.data_ptr()
        keep.append((x, dy, dx))
        params.append(p)
    L_ = _lib.lib()
    ws = torch.empty(L_.canon_conv1d_bwd_workspace_bytes(ctypes.byref(params[0])), dtype=torch.uint8, device=dev)
    for p in params:
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    plan = L_.canon_conv1d_bwd_plan(ctypes.byref(params[0])).decode()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    refs = [ctypes.byref(p) for p in params]

    def step(i):
        rc = L_.canon_conv1d_bwd(refs[i % nbuf], stream)
        if rc:
            _lib.check(rc, "canon_conv1d_bwd")

    ms = time_region(step, steps, warmup)
    return ms, plan, ws.numel()


def _shape_row(what, shape, dtype, masked, steps, warmup, act=0):
    """One shape in both layouts.  us_per_step (and the rates derived from it) is always the HIP-graph figure: the
    launches of one pass over the buffer pairs replayed as a graph, i.e. device time without the host's launch cost
    (the shortest of these kernels finish faster than Python issues the next launch).  us_per_step_host_issued,
    launches issued one by one from Python, is a side column."""
    import torch
    esize = 4 if dtype == torch.float32 else 2
    nbytes = prefill_bytes(*shape, esize, esize) + (shape[0] * shape[2] * esize if masked else 0)
    nbuf = max(3, min(48, int(700e6 / nbytes) + 1))
    row = {"workload": f"{what}: {'fp32' if esize == 4 else 'bf16'} x[{shape[0]},{shape[1]},{shape[2]}]", "bytes": nbytes}
    for layout, key in (("bcl", "time_contiguous"), ("blc", "channel_last")):
        ms_host, plan = bench_prefill(layout, steps, warmup, nbuf, shape=shape, dtype=dtype, with_mask=masked, act=act)
        ms, _ = bench_prefill(layout, steps, warmup, nbuf, shape=shape, dtype=dtype, with_mask=masked, as_graph=True, act=act)
        row[key] = {"kernel": plan, "us_per_step": round(ms * 1e3, 3), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "us_per_step_host_issued": round(ms_host * 1e3, 3)}
    return row


def bench_canon_shapes(steps, warmup):
    """The other shapes the Canon layers are called with (reference: causal-conv1d-mps/bench.py:89-164 benches
    Canon A/C, B and D): C = 640 (A, C), 960 (B), 3456 (D) at B8 L1024 bf16 in both layouts, the fp32 B1 C640
    case of configuration 1, and the masked B16 calls of configuration 5's prefill.  These are small: a launch
    moves 5-60 MB, so part of each figure is the cost of a launch itself (see launch_floor)."""
    import torch
    cases = [("configs[1] Canon-A/C", (8, 640, 1024), torch.bfloat16, False),
             ("configs[1] Canon-B", (8, 960, 1024), torch.bfloat16, False),
             ("configs[0] Canon-A fp32", (1, 640, 1024), torch.float32, False),
             ("configs[4] prefill Canon-A/C, padding mask", (16, 640, 1024), torch.bfloat16, True),
             ("configs[4] prefill Canon-B, padding mask", (16, 960, 1024), torch.bfloat16, True),
             ("configs[4] prefill Canon-D, padding mask", (16, 3456, 1024), torch.bfloat16, True)]
    return [_shape_row(what, shape, dtype, masked, steps, warmup) for what, shape, dtype, masked in cases]


def bench_silu(steps, warmup):
    """configs[1] with its optional SiLU (every Canon scenario of the reference's own bench runs with
    activation=True, causal-conv1d-mps/bench.py:106-123, 236-246): C = 640 and 3456 at B8 L1024 bf16, both
    layouts, and next to each the same launch without the activation, timed the same way in the same run."""
    import torch
    rows = []
    for what, shape in (("configs[1] Canon-A/C, SiLU", (8, 640, 1024)), ("configs[1] Canon-D, SiLU", (8, 3456, 1024))):
        row = _shape_row(what, shape, torch.bfloat16, False, steps, warmup, act=1)
        plain = _shape_row(what, shape, torch.bfloat16, False, steps, warmup, act=0)
        for key in ("time_contiguous", "channel_last"):
            row[key]["us_per_step_no_activation"] = plain[key]["us_per_step"]
            row[key]["silu_cost"] = round(row[key]["us_per_step"] / plain[key]["us_per_step"] - 1.0, 4)
        rows.append(row)
    return rows


COPY_LIB = os.path.join(ROOT, "tests", "copy_ceiling", "libcopy_ceiling.so")


def bench_copy_ceiling(steps, warmup):
    """Plain copies with the prefill kernels' access patterns (tests/copy_ceiling/copy_ceiling.hip): whole rows
    (every lane 16 bytes, 2 KB per wave: the time-contiguous kernel without its arithmetic) and 512-byte wide tiles
    of 16 rows (4 per wave, as the kernel's unmasked launches of 40 MB and more; 32 rows below that) through buffer
    accesses (the channel-contiguous kernel without history, taps and LDS), at the metric
    shape and at four times it, same buffer rotation as the kernels; and an empty launch.  The line through the
    two sizes separates what a launch costs from the rate the data moves at."""
    import torch
    if not os.path.exists(COPY_LIB):
        return None
    lib = ctypes.CDLL(COPY_LIB)
    lib.copy_rows.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
    lib.copy_tiles.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p]
    lib.empty_launch.argtypes = [ctypes.c_void_p]
    lib.copy_tile_shape.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                    ctypes.c_int, ctypes.c_void_p]
    shapes = ["32x512B_8B_lanes", "16x512B_8B_lanes", "16x1KB_16B_lanes", "32x1KB_16B_lanes", "64x256B_16B_lanes"]
    dev = "cuda:0"
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"what": "plain streamed copies of bf16 [B, 3456, 1024] each way in the access patterns of the two prefill "
                   "kernels, rotating buffers; intercept_us / GB/s_slope: the line through the two sizes"}
    times = {}
    for batch in (8, 32):
        nbytes = batch * C * L * 2
        nbuf = max(3, int(700e6 / (2 * nbytes)) + 1)
        pool = torch.empty(2 * nbuf * nbytes, dtype=torch.uint8, device=dev)
        pool.random_(0, 255)
        src = [pool.data_ptr() + 2 * i * nbytes for i in range(nbuf)]
        dst = [pool.data_ptr() + (2 * i + 1) * nbytes for i in range(nbuf)]

        def rows(i):
            if lib.copy_rows(src[i % nbuf], dst[i % nbuf], nbytes, stream):
                raise RuntimeError("copy_rows failed")

        def tiles(i):
            if lib.copy_tiles(src[i % nbuf], dst[i % nbuf], batch, L, C * 2, stream):
                raise RuntimeError("copy_tiles failed")

        k = max(20, steps * 8 // batch)
        times["rows", batch] = time_region(rows, k, warmup) * 1e3
        times["tiles", batch] = time_region(tiles, k, warmup) * 1e3
        for code, name in enumerate(shapes):
            def shaped(i, code=code):
                if lib.copy_tile_shape(src[i % nbuf], dst[i % nbuf], batch, L, C * 2, code, stream):
                    raise RuntimeError("copy_tile_shape failed")
            pool[nbytes:2 * nbytes].zero_()
            times[name, batch] = time_region(shaped, k, warmup) * 1e3
            torch.cuda.synchronize()
            if not torch.equal(pool[:nbytes], pool[nbytes:2 * nbytes]):
                raise RuntimeError(f"copy_tile_shape {name} did not copy")
        # the copies copy: spot check of the last destination
        torch.cuda.synchronize()
        i = (k - 1) % nbuf
        a = pool[2 * i * nbytes:(2 * i + 1) * nbytes]
        b = pool[(2 * i + 1) * nbytes:(2 * i + 2) * nbytes]
        if not torch.equal(a, b):
            raise RuntimeError("copy_tiles did not copy")
        del pool
    def line(kind):
        t8, t32 = times[kind, 8], times[kind, 32]
        per_entry = (t32 - t8) / 24.0
        return {"B8_us": round(t8, 3), "B32_us": round(t32, 3),
                "GB/s_slope": round(2 * C * L * 2 / (per_entry * 1e-6) / 1e9, 1),
                "intercept_us": round(t8 - 8 * per_entry, 3)}

    for kind in ("rows", "tiles"):
        out[kind] = line(kind)
    out["tile_shapes"] = dict({name: line(name) for name in shapes},
                              what="the channel-contiguous tensor copied in other tile shapes (rows x bytes per block of "
                                   "four waves, bytes per lane), blocks in address order, stores written through: no "
                                   "decomposition streams faster than the kernel's own by more than a few percent")

    def run64(stream_):
        for _ in range(64):
            lib.empty_launch(stream_)

    graph = graph_of(run64)
    out["empty_launch_us_hipgraph"] = round(time_region(lambda i: graph.replay(), max(4, steps // 16), 2) * 1e3 / 64, 3)
    return out


def bench_launch_floor(steps, warmup):
    """What one launch through this entry point costs when it moves next to nothing: canon_conv1d_update on a
    [1, 8] token (one wave), back to back on the stream every other leg uses."""
    import torch
    import causal_conv1d as cc
    from causal_conv1d import _lib
    dev = "cuda:0"
    x = torch.zeros(1, 8, dtype=torch.bfloat16, device=dev)
    out, state = torch.empty_like(x), torch.zeros(1, 8, 3, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(8, W, dtype=torch.bfloat16, device=dev)
    p = cc._fill_update(x, out, state, w, None, None, 0, 0, 0)
    ref, upd = ctypes.byref(p), _lib.lib().canon_conv1d_update
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        rc = upd(ref, stream)
        if rc:
            _lib.check(rc, "canon_conv1d_update")

    def run64(stream_):
        for _ in range(64):
            rc = upd(ref, stream_)
            if rc:
                _lib.check(rc, "canon_conv1d_update")

    graph = graph_of(run64)
    us_graph = time_region(lambda i: graph.replay(), max(4, steps // 64), 2) * 1e3 / 64
    return time_region(step, steps, warmup) * 1e3, us_graph


def bench_decode_host_cost(calls=5000):
    """Host time of one decode call through the Python API, no synchronisation inside the loop (the GPU side of
    these calls is ~3 us, so the queue never fills): causal_conv1d_update and one CanonLayer.forward step at the
    shapes of configuration 5 (B16, Canon-D, the eager module's 8-slot state)."""
    import types
    import torch
    import causal_conv1d as cc
    from causal_conv1d.canon import CanonLayer
    dev = "cuda:0"
    Bd, Cd = 16, C
    x = torch.randn(Bd, Cd, device=dev).bfloat16()
    state = torch.zeros(Bd, Cd, 8, dtype=torch.bfloat16, device=dev)
    w = torch.randn(Cd, W, device=dev).bfloat16()
    layer = CanonLayer(Cd, types.SimpleNamespace(canon_kernel=W, canon_bias=False, canon_activation=False), "d")
    layer = layer.to(dev).to(torch.bfloat16)
    cache = types.SimpleNamespace(_max_layers=1)
    xt = torch.randn(Bd, 1, Cd, device=dev).bfloat16()
    mask = torch.ones(Bd, 1100, dtype=torch.int64, device=dev)

    def per_call(fn):
        for _ in range(200):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            fn()
        dt = time.perf_counter() - t0
        torch.cuda.synchronize()
        return dt / calls * 1e6

    with torch.no_grad():
        layer(xt.expand(Bd, 16, Cd).contiguous(), attention_mask=mask[:, :16], cache=cache, layer_idx=0)
        return {"causal_conv1d_update": round(per_call(lambda: cc.causal_conv1d_update(x, state, w)), 2),
                "canon_layer_step": round(per_call(lambda: layer(xt, attention_mask=mask, cache=cache, layer_idx=0)), 2),
                "what": "host microseconds per call (time.perf_counter over %d calls, no sync), bf16 B16 C3456, "
                        "8-slot state; the layer step includes the token mask and nn.Module.__call__" % calls}


def bench_config5(steps=128):
    """configs[4]: the Viby-shaped 18-layer bf16 model (tests/viby_harness.py, a restatement of the reference
    forward, model/model.py:1115-1157, 1308-1327) with random weights: prefill of B16 x L1024 token ids, then
    `steps` greedy tokens through the conv caches.  Timed with the HIP Canon layers and with the Canon layers
    switched off (everything else identical), the decode both as a Python loop that launches kernel by kernel and
    with the whole step captured once as a HIP graph (causal_conv1d.canon.GraphedDecodeStep) and replayed per
    token: the difference between the two models is what the 72 Canon calls per forward cost."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from viby_harness import VibyShaped, generate_graphed, init_weights, viby_config
    from causal_conv1d.canon import CanonLayer

    class NoCanon(torch.nn.Module):
        def forward(self, x, attention_mask=None, cache=None, layer_idx=None):
            return x

    dev = "cuda:0"
    cfg = viby_config()
    Bm, Tm = 16, 1024
    ids = torch.randint(0, cfg.vocab_size, (Bm, Tm), generator=torch.Generator().manual_seed(5)).to(dev)
    out = {"workload": f"configs[4]: 18 layers, hidden 640, 4 q / 1 kv heads of 160, FFN 1728, vocab 25600, Canon A-D, "
                       f"bf16, random weights; prefill B{Bm} x L{Tm}, then {steps} greedy steps; wall clock around "
                       f"torch.cuda.synchronize()"}

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        r = fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, r

    for name, factory in (("hip_canon", lambda C, n: CanonLayer(C, cfg, n)), ("canon_off", lambda C, n: NoCanon())):
        model = init_weights(VibyShaped(cfg, factory), 11, torch.bfloat16, dev)
        with torch.no_grad():
            model.generate(ids[:2, :64], 2)                      # warm-up: library, allocator
            generate_graphed(model, ids[:2, :64], 3)
            mask = torch.ones(Bm, Tm, dtype=torch.int64, device=dev)
            t_prefill = min(timed(lambda: model.forward(ids, model.new_cache(), mask))[0] for _ in range(3))
            t_loop, _ = timed(lambda: model.generate(ids, steps))
            t_graph, _ = timed(lambda: generate_graphed(model, ids, steps))
        out[name] = {"prefill_ms": round(t_prefill * 1e3, 2),
                     "prefill_plus_decode_python_loop_s": round(t_loop, 4),
                     "prefill_plus_decode_hipgraph_s": round(t_graph, 4),
                     "decode_ms_per_token_python_loop": round((t_loop - t_prefill) / (steps - 1) * 1e3, 3),
                     "decode_ms_per_token_hipgraph": round((t_graph - t_prefill) / (steps - 1) * 1e3, 3)}
        del model
        torch.cuda.empty_cache()
    h, o = out["hip_canon"], out["canon_off"]
    out["canon_share"] = {
        "prefill": round(1.0 - o["prefill_ms"] / h["prefill_ms"], 4),
        "decode_python_loop": round(1.0 - o["decode_ms_per_token_python_loop"] / h["decode_ms_per_token_python_loop"], 4),
        "decode_hipgraph": round(1.0 - o["decode_ms_per_token_hipgraph"] / h["decode_ms_per_token_hipgraph"], 4),
        "what": "1 - time with the Canon layers off / time with the HIP Canon layers: under the graph it is device time "
                "(72 update launches per token), in the Python loop mostly the host's cost of issuing them"}
    return out


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _median_time(fn, budget_s, max_runs):
    fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < max_runs):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)


def cpu_baseline(budget_s=10.0):
    """The reference's eager formulation on the host cores, same shapes: the mask-free Canon-D
    block call (pad + grouped conv1d + residual, model/model.py:604-675) on all threads torch
    uses and on one, and the single-token step (roll + write + multiply + sum,
    model/model.py:372-398) at the decode shape."""
    import torch
    from oracle.canon_eager import EagerCanon
    cores = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, L, C, generator=g).bfloat16()
    w = (torch.randn(C, W, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(C, generator=g) * 0.01).bfloat16()
    layer = EagerCanon(w, bias, False)
    med, n = _median_time(lambda: layer.forward(x), 0.6 * budget_s, 300)

    cache = {}
    tok = torch.randn(DEC_B, 1, C, generator=g).bfloat16()
    layer.forward(tok, cache=cache, key=0)      # creates the 8-slot state the eager module keeps
    med_dec, n_dec = _median_time(lambda: layer.forward(tok, cache=cache, key=0), budget_s / 4, 1000)
    dec_bytes = decode_bytes(DEC_B, C, 8)

    torch.set_num_threads(1)
    try:
        med1, n1 = _median_time(lambda: layer.forward(x), budget_s / 2, 30)
    finally:
        torch.set_num_threads(cores)
    nbytes = prefill_bytes(B, C, L)
    return {
        "value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": cores,
        "kind": "port", "cpu": _cpu_model(), "torch": torch.__version__,
        "sample": f"{n} passes of the full bf16 [8,3456,1024] step, eager torch restatement "
                  f"(oracle/canon_eager.py), median {med * 1e3:.1f} ms",
        "ms": round(med * 1e3, 2), "tokens_per_s": round(B * L / med),
        "one_core": {"value": round(nbytes / med1 / 1e9, 3), "unit": "GB/s", "ms": round(med1 * 1e3, 1),
                     "sample": f"{n1} passes, torch.set_num_threads(1)"},
        "decode": {"us_per_step": round(med_dec * 1e6, 1), "GB/s": round(dec_bytes / med_dec / 1e9, 3),
                   "cores": cores,
                   "sample": f"{n_dec} single-token steps, bf16 [{DEC_B},{C}] token, 8-slot state "
                             f"(the eager module's), roll + write + multiply + sum"},
    }


def main():
    global REGIONS, PREFILL_ACT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the legs that run the headline kernels on other shapes (canon_shapes, launch_floor, "
                         "host cost, eager rounding): a profile of the command then has one workload per kernel name")
    ap.add_argument("--regions", type=int, default=REGIONS,
                    help="timed regions of --steps launches per leg; the median is reported (profiles use 1)")
    ap.add_argument("--activation", choices=("none", "silu"), default="none",
                    help="silu: the prefill legs run with the optional SiLU (for a profile of that variant; the metric is "
                         "quoted without it)")
    ap.add_argument("--copy-ceiling", action="store_true", help="with --no-extra: run the plain-copy leg all the same")
    ap.add_argument("--no-config5", action="store_true", help="skip the whole-model leg (configs[4])")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="also run this many plain device-to-device copies of one x-sized buffer "
                         "(a kernel of known traffic to scale profiler byte counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU by design (rows of the conv are independent; "
                 "there is no multi-GPU path to measure). Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    REGIONS = max(1, args.regions)
    PREFILL_ACT = 1 if args.activation == "silu" else 0

    if args.calibration_copies:
        src = torch.empty(B * C * L, dtype=torch.bfloat16, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(args.calibration_copies):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    nbuf = 6  # 6 x 113 MB = 680 MB of distinct traffic between reuses
    head_stats, blc_stats = {}, {}
    ms, plan = bench_prefill("bcl", args.steps, args.warmup, nbuf, stats=head_stats)
    # right after the headline leg (clocks are up) and short: its launches of the same kernel hardly move that
    # kernel's average duration in a profile of this command
    ms_warm, _ = bench_prefill("bcl", max(20, args.steps // 10), 5, 1, ramp=False)
    ms_copy = bench_copy(args.steps, args.warmup, nbuf)
    ms_blc, plan_blc = bench_prefill("blc", args.steps, args.warmup, nbuf, stats=blc_stats)
    if not args.no_extra:
        ms_blc_eager, plan_blc_eager = bench_prefill("blc", args.steps, args.warmup, nbuf, rounding=1)
    ms_parts, plan_parts = bench_prefill_parts(args.steps, args.warmup, nbuf)
    rag_steps, rag_warm = max(20, args.steps // 4), max(4, args.warmup // 4)
    ms_rag, plan_rag, rag_bytes = bench_ragged("blc", rag_steps, rag_warm, 3)     # 3 x 453 MB between reuses
    ms_rag_t, plan_rag_t, _ = bench_ragged("bcl", rag_steps, rag_warm, 3)
    dec_us, dec_graph_us, dec_plan = bench_decode(max(4, args.steps // 20), 2)
    ms_bwd, plan_bwd, ws_bwd = bench_backward(max(20, args.steps // 3), max(4, args.warmup // 3), 4)

    us_dbwd, dbwd_bytes, ws_dbwd = bench_decode_backward(max(50, args.steps), max(5, args.warmup))
    ms_bwd_t, plan_bwd_t, ws_bwd_t = bench_backward(max(20, args.steps // 3), max(4, args.warmup // 3), 4, "time_contiguous")
    ceiling = None
    if args.no_extra and args.copy_ceiling:
        ceiling = bench_copy_ceiling(args.steps, args.warmup)
    if not args.no_extra:
        shapes = bench_canon_shapes(max(50, args.steps // 2), max(5, args.warmup // 2))
        silu = bench_silu(max(50, args.steps // 2), max(5, args.warmup // 2))
        config5 = None if args.no_config5 else bench_config5()
        floor_us = bench_launch_floor(max(200, args.steps), max(20, args.warmup))
        ceiling = bench_copy_ceiling(args.steps, args.warmup)
        host_cost = bench_decode_host_cost()

    nbytes = prefill_bytes(B, C, L)
    gbps = nbytes / (ms * 1e-3) / 1e9
    out = {
        "metric": "Canon conv1d HBM GB/s (prefill B8 L1024 C3456 bf16); decode us/step B256",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "timing": dict(head_stats, what="ms_per_step is the median of `regions` back-to-back "
                                                    "timed regions of exactly `steps` launches each (HIP events)"),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1]: prefill bf16 x[B=8,C=3456,L=1024] time-contiguous, width 4, "
                               "bias, residual fused, " + ("SiLU" if PREFILL_ACT else "no activation"), "kernel": plan,
                   "storage": "bf16", "accumulate": "f32", "rotating_buffer_pairs": nbuf},
        "tokens_per_s": round(B * L / (ms * 1e-3)),
        "device_copy_same_bytes": {"ms_per_step": round(ms_copy, 6),
                                   "GB/s": round(2 * B * C * L * 2 / (ms_copy * 1e-3) / 1e9, 1),
                                   "what": "torch copy_ (the runtime's device-to-device copy) of one x-sized buffer, same rotation"},
        "prefill_same_buffers": {"ms_per_step": round(ms_warm, 6), "GB/s": round(nbytes / (ms_warm * 1e-3) / 1e9, 1),
                                 "what": "the headline launch repeated on ONE buffer pair (113 MB, inside the 256 MB "
                                         "Infinity Cache): a cache rate, reported beside the HBM rate, never as it"},
        "prefill_channel_last": {"kernel": plan_blc, "ms_per_step": round(ms_blc, 6), "timing": blc_stats,
                                 "GB/s": round(nbytes / (ms_blc * 1e-3) / 1e9, 1),
                                 "frac_of_hbm_peak": round(nbytes / (ms_blc * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
        "prefill_channel_last_parts": {"workload": "gate, up as two [8,1024,1728] tensors, one launch, no cat",
                                       "kernel": plan_parts, "ms_per_step": round(ms_parts, 6),
                                       "GB/s": round(nbytes / (ms_parts * 1e-3) / 1e9, 1)},
        "ragged_prefill_B32": {"workload": "configs[2]: bf16 x[32,3456,1024] right-padded, lengths U[128,1024], bf16 "
                                           "padding mask multiplied in, masked residual fused; rate over all "
                                           "B*C*L elements (the padded ones are read and written too)",
                               "channel_last": {"kernel": plan_rag, "ms_per_step": round(ms_rag, 6),
                                                "GB/s": round(rag_bytes / (ms_rag * 1e-3) / 1e9, 1)},
                               "time_contiguous": {"kernel": plan_rag_t, "ms_per_step": round(ms_rag_t, 6),
                                                   "GB/s": round(rag_bytes / (ms_rag_t * 1e-3) / 1e9, 1)}},
        "decode": {"workload": f"configs[3]: bf16 state[{DEC_B},{C},{DEC_S}], {DEC_STEPS} carried steps",
                   "kernel": dec_plan, "us_per_step_stream": round(dec_us, 3),
                   "us_per_step_hipgraph": round(dec_graph_us, 3),
                   "GB/s_hipgraph": round(decode_bytes(DEC_B, C, DEC_S) / (dec_graph_us * 1e-6) / 1e9, 1)},
        "backward_channel_last": {"kernel": plan_bwd, "ms_per_step": round(ms_bwd, 6),
                                  "GB/s": round(1.5 * nbytes / (ms_bwd * 1e-3) / 1e9, 1),
                                  "bytes": "x and dout read, dx written (3 tensor passes)",
                                  "scratch_bytes": ws_bwd},
        "backward_time_contiguous": {"kernel": plan_bwd_t, "ms_per_step": round(ms_bwd_t, 6),
                                     "GB/s": round(1.5 * nbytes / (ms_bwd_t * 1e-3) / 1e9, 1),
                                     "bytes": "x and dout read, dx written (3 tensor passes)",
                                     "scratch_bytes": ws_bwd_t},
        "decode_backward": {"workload": f"backward of one decode step, bf16 state[{DEC_B},{C},{DEC_S}], SiLU, state "
                                        "gradients in and out; two launches (step kernel + fixed-order reduction)",
                            "us_per_step": round(us_dbwd, 3),
                            "GB/s": round(dbwd_bytes / (us_dbwd * 1e-6) / 1e9, 1), "scratch_bytes": ws_dbwd},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": profiled_traffic_bytes(),
                     "traffic_source": "profiles/" + os.path.basename(TRAFFIC_PROFILE)},
    }
    if not args.no_extra:
        out["prefill_channel_last_eager_rounding"] = {
            "kernel": plan_blc_eager, "ms_per_step": round(ms_blc_eager, 6),
            "GB/s": round(nbytes / (ms_blc_eager * 1e-3) / 1e9, 1),
            "what": "prefill_channel_last with round_mode = eager (the eager module's rounding points: bit-identical "
                    "to the reference's CPU path)"}
        out["decode"]["host_us_per_call"] = host_cost
        out["canon_shapes"] = shapes
        out["prefill_silu"] = silu
        if config5 is not None:
            out["config5"] = config5
        out["copy_ceiling"] = ceiling
        if ceiling:
            out["roofline"]["frac_of_plain_copy"] = round(ceiling["rows"]["B8_us"] / (ms * 1e3), 4)
            out["prefill_channel_last"]["frac_of_plain_tile_copy"] = round(ceiling["tiles"]["B8_us"] / (ms_blc * 1e3), 4)
        out["launch_floor"] = {
            "us_per_launch": round(floor_us[0], 3), "us_per_launch_hipgraph": round(floor_us[1], 3),
            "what": "canon_conv1d_update on a [1, 8] token (one wave), back to back on the same stream: what a launch "
                    "costs before it moves any data, issued one by one from Python (host and device side together) "
                    "and as 64 nodes of a HIP graph (the device side alone)"}
    if args.no_extra and ceiling:
        out["copy_ceiling"] = ceiling
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
