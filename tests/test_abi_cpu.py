"""CPU-side checks of the C ABI and of the host logic (no kernel is launched).

  * the shared library loads and exports every function the header declares
  * the ctypes mirrors of the parameter structs match the C layout (checked
    against gcc's sizeof/offsetof of the real header)
  * argument validation and kernel-family planning (pure host code)
  * the Python wrappers raise the reference's error types / messages
    (causal-conv1d-mps/test.py:220-236) before touching a device
  * there is no fallback: a missing library is an ImportError
"""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "canon_conv1d.h")

import causal_conv1d as cc                      # noqa: E402
from causal_conv1d import _lib                  # noqa: E402
from causal_conv1d._lib import BwdParams, FwdParams, Part, UpdateBwdParams, UpdateParams  # noqa: E402


def test_library_exports_every_declared_function():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(canon_conv1d_[a-z_]+)\s*\(", text))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    L = _lib.lib()
    for name in declared:
        assert getattr(L, name) is not None
    assert L.canon_conv1d_abi_version() == _lib.ABI_VERSION
    assert L.canon_conv1d_last_error() is not None


def test_ctypes_structs_match_the_header(tmp_path):
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', 'int main(void){']
    structs = (("canon_conv1d_fwd_params", FwdParams), ("canon_conv1d_update_params", UpdateParams),
               ("canon_conv1d_bwd_params", BwdParams), ("canon_conv1d_update_bwd_params", UpdateBwdParams),
               ("canon_conv1d_part", Part))
    for cname, cls in structs:
        lines.append(f'printf("{cname} size %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'printf("{cname} {fname} %zu\\n", offsetof({cname}, {fname}));')
    lines.append('return 0;}')
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-o", str(exe), str(src)])
    out = subprocess.check_output([str(exe)], text=True).split("\n")
    got = {tuple(l.split()[:2]): int(l.split()[2]) for l in out if l}
    for cname, cls in structs:
        assert got[(cname, "size")] == ctypes.sizeof(cls)
        for fname, _ in cls._fields_:
            assert got[(cname, fname)] == getattr(cls, fname).offset, (cname, fname)


# ---------------------------------------------------------------------------
# planning / validation: fake (never dereferenced) device addresses
# ---------------------------------------------------------------------------
FAKE_X, FAKE_OUT, FAKE_W, FAKE_STATE = 0x10000000, 0x20000000, 0x30000000, 0x40000000


def fwd_params(B=8, C=3456, L=1024, layout="bcl", dtype=1, **over):
    p = FwdParams()
    p.struct_size = ctypes.sizeof(FwdParams)
    p.x_dtype = p.w_dtype = dtype
    p.width = 4
    p.batch, p.channels, p.seqlen = B, C, L
    p.x, p.out, p.weight = FAKE_X, FAKE_OUT, FAKE_W
    if layout == "bcl":
        strides = (C * L, L, 1)
    else:
        strides = (C * L, 1, C)
    p.x_stride_b, p.x_stride_c, p.x_stride_l = strides
    p.out_stride_b, p.out_stride_c, p.out_stride_l = strides
    p.w_stride_c, p.w_stride_k = 4, 1
    for k, v in over.items():
        setattr(p, k, v)
    return p


def plan(p):
    r = _lib.lib().canon_conv1d_fwd_plan(ctypes.byref(p))
    return r.decode() if r is not None else None


def last_error():
    return _lib.lib().canon_conv1d_last_error().decode()


def test_fwd_plan_picks_the_vector_kernels_for_dense_layouts():
    for C in (640, 960, 3456):
        assert plan(fwd_params(C=C, layout="bcl")) == "bcl_vec"
        assert plan(fwd_params(C=C, layout="blc")) == "blc_vec"
    assert plan(fwd_params(B=1, C=640, L=1024, dtype=0)) == "bcl_vec"     # benchmark configuration 1 (fp32, CPU-runnable)
    # time-contiguous rows that are not a whole number of vectors keep the vector kernel (edge elements aside)
    # as long as x and out share their strides
    assert plan(fwd_params(L=1023)) == "bcl_vec"
    assert plan(fwd_params(L=1023, out_stride_c=1024, out_stride_b=3456 * 1024)) == "generic"
    # ragged channel counts, misaligned base pointers -> strided kernel
    assert plan(fwd_params(C=3457, layout="blc")) == "generic"
    assert plan(fwd_params(x=FAKE_X + 2)) == "generic"
    # the channel-contiguous kernel takes the tap addresses (48 bits each), the batch stride in lane vectors (32 bits)
    # and the number of channel tiles (16 bits) among its leading scalar arguments: beyond those, the strided kernel
    assert plan(fwd_params(layout="blc", weight=FAKE_W | 1 << 48)) == "generic"
    assert plan(fwd_params(layout="blc", bias=FAKE_W + 4096)) == "blc_vec"
    assert plan(fwd_params(layout="blc", bias=1 << 50)) == "generic"
    assert plan(fwd_params(B=1, C=65535 * 256, L=8, layout="blc")) == "blc_vec"
    assert plan(fwd_params(B=1, C=65536 * 256, L=8, layout="blc")) == "generic"
    assert plan(fwd_params(B=2, C=8, L=8, layout="blc", x_stride_b=4 << 32, out_stride_b=4 << 32)) == "generic"
    # the eager module's rounding points are register arithmetic: the same kernels
    assert plan(fwd_params(round_mode=1)) == "bcl_vec"
    assert plan(fwd_params(round_mode=1, layout="blc")) == "blc_vec"
    # rows too short for a wave of their own: several rows per wave, as long as they are whole aligned vectors
    assert plan(fwd_params(L=64)) == "bcl_vec_short"
    assert plan(fwd_params(L=8)) == "bcl_vec_short"
    assert plan(fwd_params(L=120)) == "bcl_vec_short"
    assert plan(fwd_params(L=128)) == "bcl_vec_short" and plan(fwd_params(L=256)) == "bcl_vec_short"
    assert plan(fwd_params(L=264)) == "bcl_vec"
    assert plan(fwd_params(L=255)) == "bcl_vec"                            # ... not whole vectors, but long enough
    assert plan(fwd_params(L=60)) == "generic"                             # ... not whole vectors
    assert plan(fwd_params(L=4)) == "generic"
    assert plan(fwd_params(L=64, round_mode=1)) == "bcl_vec_short"
    # strided but aligned rows (a channel slice of a bigger tensor) stay vectorised
    assert plan(fwd_params(C=128, x_stride_b=4096 * 1024, x_stride_c=1024)) == "bcl_vec"


def test_fwd_plan_waves_per_block():
    """Waves per block of the time-contiguous prefill: 1 with a padding mask, 4 in small unmasked launches, 8 from
    16384 waves; the other kernels run blocks of four."""
    waves = lambda p: _lib.lib().canon_conv1d_fwd_plan_waves(ctypes.byref(p))
    assert waves(fwd_params()) == 8                                        # 8 * 3456 rows = 27648 waves
    assert waves(fwd_params(B=4)) == 4                                     # 13824 waves
    assert waves(fwd_params(B=4, C=4096)) == 8                             # exactly 16384
    assert waves(fwd_params(B=4, C=4095)) == 4
    assert waves(fwd_params(mask=FAKE_STATE, mask_dtype=2, mask_stride_b=1024, mask_stride_l=1)) == 1
    assert waves(fwd_params(B=32, mask=FAKE_STATE, mask_dtype=4, mask_stride_b=1024, mask_stride_l=1)) == 1
    assert waves(fwd_params(layout="blc")) == 4
    assert waves(fwd_params(L=64)) == 4                                    # rows sharing waves
    assert waves(fwd_params(B=0)) == 0
    assert waves(fwd_params(width=9)) == -1


def test_fwd_validation_messages():
    cases = [
        (dict(struct_size=8), "struct_size"),
        (dict(width=5), "width 5"),
        (dict(width=1), "width 1"),
        (dict(x_dtype=7), "x_dtype"),
        (dict(activation=3), "activation"),
        (dict(residual_mode=9), "residual_mode"),
        (dict(round_mode=2), "round_mode"),
        (dict(batch=-1), "negative"),
        (dict(out=FAKE_X), "alias"),
        (dict(out=FAKE_X + 4096), "ranges overlap"),                      # a shifted view of the same buffer
        (dict(x=0), "NULL"),
        (dict(mask=FAKE_STATE, mask_dtype=17), "mask_dtype"),
        (dict(initial_state=FAKE_STATE, initial_len=2), "initial_len"),
        (dict(final_state=FAKE_STATE, final_len=0), "final_len"),
        (dict(batch=1 << 20, channels=1 << 12), "2^31"),
    ]
    for over, needle in cases:
        assert plan(fwd_params(**over)) is None, over
        assert needle in last_error(), (over, last_error())
    assert _lib.lib().canon_conv1d_fwd_plan(None) is None
    # empty problems are accepted (and launch nothing)
    assert plan(fwd_params(B=0)) is not None
    assert plan(fwd_params(L=0, x=0, out=0)) is not None


def update_params(B=256, C=3456, S=3, dtype=1, **over):
    p = UpdateParams()
    p.struct_size = ctypes.sizeof(UpdateParams)
    p.x_dtype = p.w_dtype = dtype
    p.width, p.state_len = 4, S
    p.batch, p.channels = B, C
    p.x, p.out, p.conv_state, p.weight = FAKE_X, FAKE_OUT, FAKE_STATE, FAKE_W
    p.x_stride_b, p.x_stride_c = C, 1
    p.out_stride_b, p.out_stride_c = C, 1
    p.state_stride_b, p.state_stride_c, p.state_stride_s = C * S, S, 1
    p.w_stride_c, p.w_stride_k = 4, 1
    for k, v in over.items():
        setattr(p, k, v)
    return p


def uplan(p):
    r = _lib.lib().canon_conv1d_update_plan(ctypes.byref(p))
    return r.decode() if r is not None else None


def test_update_plan_and_validation():
    for S in (3, 4, 8):
        assert uplan(update_params(S=S)) == "update_vec"
    assert uplan(update_params(S=5)) == "update_generic"
    assert uplan(update_params(C=3457)) == "update_generic"
    # a lane of the vector kernel owns one 12..16-byte run of the state: two channels with 16-bit elements
    # and 3 or 4 slots (so the token is read as 4-byte words), one channel otherwise
    assert uplan(update_params(C=3457, S=8)) == "update_vec"
    assert uplan(update_params(C=3457, dtype=0)) == "update_vec"
    assert uplan(update_params(C=3458)) == "update_vec"
    assert uplan(update_params(x=FAKE_X + 2)) == "update_generic"                  # token off the 4-byte grid
    assert uplan(update_params(x=FAKE_X + 2, S=8)) == "update_vec"                 # ... one 16-bit channel per lane: fine
    assert uplan(update_params(x=FAKE_X + 4)) == "update_vec"
    assert uplan(update_params(x_stride_b=3457)) == "update_generic"               # odd row pitch
    assert uplan(update_params(out=FAKE_OUT + 2)) == "update_generic"
    assert uplan(update_params(conv_state=FAKE_STATE + 2)) == "update_generic"
    assert uplan(update_params(conv_state=FAKE_STATE + 4)) == "update_vec"
    assert uplan(update_params(state_stride_b=3456 * 3 + 1)) == "update_generic"   # rows of a state pool off the grid
    assert uplan(update_params(state_stride_b=3456 * 3 + 2)) == "update_vec"
    assert uplan(update_params(state_stride_s=2, state_stride_c=6, state_stride_b=3456 * 6)) == "update_generic"
    assert uplan(update_params(round_mode=1)) == "update_vec"        # eager rounding: the same kernel
    assert uplan(update_params(conv_state_indices=FAKE_STATE + 64)) == "update_vec"       # state pool: row indirection
    assert uplan(update_params(cache_seqlens=FAKE_STATE + 64)) == "update_generic"        # circular buffer
    for over, needle in [(dict(S=2), "state_len"), (dict(width=7), "width"),
                         (dict(cache_seqlens=FAKE_STATE + 2), "4-byte aligned"),
                         (dict(conv_state_indices=FAKE_STATE + 1), "4-byte aligned"),
                         (dict(conv_state=0), "NULL"), (dict(struct_size=4), "struct_size"),
                         # the state is rewritten in place: neither the token nor the output may lie inside it
                         (dict(x=FAKE_STATE + 4096), "overlap"), (dict(out=FAKE_STATE), "overlap"),
                         (dict(conv_state=FAKE_X - 64), "overlap")]:
        if "S" in over:
            p = update_params(S=over["S"])
        else:
            p = update_params(**over)
        assert uplan(p) is None, over
        assert needle in last_error(), (over, last_error())


# ---------------------------------------------------------------------------
# Python wrappers: the reference's error conventions, raised on the host
# ---------------------------------------------------------------------------
def test_wrapper_errors_match_reference_conventions():
    x = torch.randn(2, 4, 8)
    with pytest.raises(ValueError, match="does not match"):
        cc.causal_conv1d_fn(x, torch.randn(5, 4))
    with pytest.raises(ValueError, match="Expected 3D input tensor"):
        cc.causal_conv1d_fn(torch.randn(4, 8), torch.randn(4, 4))
    with pytest.raises(ValueError, match="Expected 2D weight tensor"):
        cc.causal_conv1d_fn(x, torch.randn(4, 1, 4))
    with pytest.raises(ValueError, match="Expected 1D bias tensor"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4), torch.randn(4, 1))
    with pytest.raises(ValueError, match="Bias dim 3 does not match"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4), torch.randn(3))
    with pytest.raises(NotImplementedError, match="activation must be None, silu, or swish"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4), activation="relu")
    with pytest.raises(ValueError, match="seq_idx shape"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4), seq_idx=torch.zeros(2, 9, dtype=torch.int32))
    with pytest.raises(ValueError, match="cannot be combined with seq_idx"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4), seq_idx=torch.zeros(2, 8, dtype=torch.int32), return_final_states=True)
    with pytest.raises(NotImplementedError, match="width 5"):
        cc.causal_conv1d_fn(x, torch.randn(4, 5))
    with pytest.raises(ValueError, match="Unsupported input dtype"):
        cc.causal_conv1d_fn(x.double(), torch.randn(4, 4))
    # a CPU tensor is an error, never a silent slow path
    with pytest.raises(ValueError, match="must be on a ROCm GPU device"):
        cc.causal_conv1d_fn(x, torch.randn(4, 4))
    with pytest.raises(ValueError, match="Expected 2D input tensor"):
        cc.causal_conv1d_update(torch.randn(4), torch.zeros(2, 4, 4), torch.randn(4, 4))
    with pytest.raises(ValueError, match="Expected 3D conv_state"):
        cc.causal_conv1d_update(torch.randn(2, 4), torch.zeros(2, 4), torch.randn(4, 4))
    with pytest.raises(ValueError, match="doesn't match conv_state"):
        cc.causal_conv1d_update(torch.randn(2, 4), torch.zeros(3, 4, 4), torch.randn(4, 4))
    with pytest.raises(ValueError, match="cache_seqlens must be a contiguous int32 tensor"):
        cc.causal_conv1d_update(torch.randn(2, 4), torch.zeros(2, 4, 4), torch.randn(4, 4),
                                cache_seqlens=torch.zeros(2, dtype=torch.int64))
    with pytest.raises(ValueError, match="conv_state_indices must be a contiguous int32 tensor"):
        cc.causal_conv1d_update(torch.randn(2, 4), torch.zeros(7, 4, 4), torch.randn(4, 4),
                                conv_state_indices=torch.zeros(3, dtype=torch.int32))
    with pytest.raises(ValueError, match="must be on a ROCm GPU device"):
        cc.causal_conv1d_update(torch.randn(2, 4), torch.zeros(2, 4, 4), torch.randn(4, 4))
    with pytest.raises(ValueError, match="Expected 3D input tensor"):
        cc.short_conv_fused(torch.randn(4, 8), torch.randn(8, 4))


def test_missing_library_is_an_import_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "does", "not", "exist.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "viby-model_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"oracle", text, flags=re.I), os.path.join(dirpath, f)


def test_canon_layer_module_mirrors_the_reference_class():
    """Same constructor, parameter names/shapes and cache attribute as model/model.py:201-241."""
    import types
    from causal_conv1d.canon import CanonLayer
    cfg = types.SimpleNamespace(canon_kernel=4, canon_bias=True, canon_activation=False)
    layer = CanonLayer(640, cfg, "b")
    sd = layer.state_dict()
    assert set(sd) == {"weight", "bias_param"}
    assert tuple(sd["weight"].shape) == (640, 1, 4) and tuple(sd["bias_param"].shape) == (640,)
    layer.reset_parameters()
    assert float(layer.weight.abs().max()) <= 0.5 + 1e-6          # kaiming-uniform(a=sqrt 5), fan_in 4
    nobias = CanonLayer(8, types.SimpleNamespace(canon_kernel=3, canon_bias=False, canon_activation=True), "a")
    assert nobias.bias_param is None and set(nobias.state_dict()) == {"weight"}
    cache = types.SimpleNamespace(_max_layers=18)
    assert nobias._slot(cache) is cache.canon_cache_a and len(cache.canon_cache_a) == 18
    with pytest.raises(ValueError, match="must be on a ROCm GPU device"):
        layer(torch.randn(1, 4, 640))


def bwd_params(B=8, C=3456, L=1024, layout="blc", dtype=1, **over):
    p = BwdParams()
    p.struct_size = ctypes.sizeof(BwdParams)
    p.x_dtype = p.w_dtype = dtype
    p.width = 4
    p.batch, p.channels, p.seqlen = B, C, L
    p.x, p.dout, p.dx, p.weight, p.dweight = FAKE_X, FAKE_OUT, FAKE_STATE, FAKE_W, FAKE_W + 0x100000
    strides = (C * L, L, 1) if layout == "bcl" else (C * L, 1, C)
    for name in ("x", "dout", "dx"):
        for s, v in zip(("b", "c", "l"), strides):
            setattr(p, f"{name}_stride_{s}", v)
    p.w_stride_c, p.w_stride_k = 4, 1
    for k, v in over.items():
        setattr(p, k, v)
    return p


def test_bwd_plan_and_workspace():
    L = _lib.lib()
    p = bwd_params()
    assert L.canon_conv1d_bwd_plan(ctypes.byref(p)) == b"bwd_blc_vec"
    ws = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(p))
    assert 0 < ws <= 20 << 20 and ws % (3456 * 5 * 4) == 0        # whole partial sets, bounded scratch
    assert L.canon_conv1d_bwd_plan(ctypes.byref(bwd_params(layout="bcl"))) == b"bwd_bcl_vec"
    assert L.canon_conv1d_bwd_plan(ctypes.byref(bwd_params(layout="bcl", L=1023))) == b"bwd_generic"
    assert L.canon_conv1d_bwd_plan(ctypes.byref(bwd_params(C=3457))) == b"bwd_generic"
    # packed sequences: only the walk kernel gates taps by sequence index
    for layout in ("blc", "bcl"):
        q = bwd_params(layout=layout, seq_idx=FAKE_X + 0x400000, seq_stride_b=1024, seq_stride_l=1)
        assert L.canon_conv1d_bwd_plan(ctypes.byref(q)) == b"bwd_generic"
    assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(bwd_params(seq_idx=FAKE_X + 2))) == -1
    assert "seq_idx must be 4-byte aligned" in last_error()
    # an initial state / the gradient of the captured final state: the channel-contiguous kernel handles both,
    # time-contiguous rows go to the walk kernel; its checks
    for layout, want in (("blc", b"bwd_blc_vec"), ("bcl", b"bwd_generic")):
        q = bwd_params(layout=layout, initial_state=FAKE_X + 0x800000, initial_len=3, init_stride_b=3456 * 3, init_stride_c=3,
                       init_stride_s=1)
        assert L.canon_conv1d_bwd_plan(ctypes.byref(q)) == want
        q = bwd_params(layout=layout, dfinal_state=FAKE_X + 0x900000, final_len=4)
        assert L.canon_conv1d_bwd_plan(ctypes.byref(q)) == want
    for over, msg in [(dict(initial_state=FAKE_X, initial_len=2), "shorter than width-1"),
                      (dict(dinitial_state=FAKE_X), "needs initial_state"),
                      (dict(dfinal_state=FAKE_X, final_len=0), "final_len 0"),
                      (dict(dfinal_state=FAKE_X, final_len=4, seq_idx=FAKE_X + 0x400000), "seq_idx"),
                      (dict(initial_state=FAKE_X, initial_len=3, seq_idx=FAKE_X + 0x400000), "seq_idx")]:
        assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(bwd_params(**over))) == -1, over
        assert msg in last_error(), (over, last_error())
    assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(bwd_params(width=9))) == -1
    assert "width 9" in last_error()
    assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(bwd_params(B=0))) == 0
    # the launching call validates what the planner cannot: pointers and the scratch itself
    assert L.canon_conv1d_bwd(ctypes.byref(bwd_params(workspace=0)), None) == _lib.ERR_INVALID_ARGUMENT
    assert "workspace" in last_error()
    assert L.canon_conv1d_bwd(ctypes.byref(bwd_params(dx=FAKE_X)), None) == _lib.ERR_INVALID_ARGUMENT
    assert "alias" in last_error()


def _demanded_workspace(p):
    """What canon_conv1d_bwd itself asks for: its complaint about a one-byte workspace names the size."""
    import re
    p.workspace, p.workspace_bytes = FAKE_W + 0x200000, 1
    assert _lib.lib().canon_conv1d_bwd(ctypes.byref(p), None) == _lib.ERR_INVALID_ARGUMENT
    m = re.search(r"at least (\d+) bytes", last_error())
    assert m, last_error()
    return int(m.group(1))


def test_bwd_workspace_query_covers_misaligned_pointers():
    L = _lib.lib()
    # time-contiguous rows with a padded row stride, x off by one element: the call takes the strided kernel,
    # which needs more scratch than the vector kernel an aligned x would get
    for over in (dict(x=FAKE_X + 2), dict(dout=FAKE_OUT + 2), dict(dx=FAKE_STATE + 2), dict()):
        q = bwd_params(layout="bcl", x_stride_c=1032, x_stride_b=3456 * 1032, **over)
        want_kernel = b"bwd_generic" if over else b"bwd_bcl_vec"
        assert L.canon_conv1d_bwd_plan(ctypes.byref(q)) == want_kernel, over
        assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(q)) == _demanded_workspace(q), over
    for over in (dict(x=FAKE_X + 4), dict(dx=FAKE_STATE + 2)):          # channel-contiguous: 8-byte lanes
        q = bwd_params(**over)
        assert L.canon_conv1d_bwd_plan(ctypes.byref(q)) == b"bwd_generic"
        assert L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(q)) == _demanded_workspace(q), over
    # sizes asked for before the tensors exist (NULL pointers): enough for whichever kernel the call will take
    for layout in ("bcl", "blc"):
        unknown = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(bwd_params(layout=layout, x=0, dout=0, dx=0)))
        for over in (dict(), dict(x=FAKE_X + 2)):
            assert unknown >= _demanded_workspace(bwd_params(layout=layout, **over)), (layout, over)


def test_static_scratch_backward_checks_on_the_host():
    L = _lib.lib()
    assert L.canon_conv1d_bwd_static(None, None) == _lib.ERR_INVALID_ARGUMENT
    assert L.canon_conv1d_bwd_static(ctypes.byref(bwd_params(struct_size=4)), None) == _lib.ERR_INVALID_ARGUMENT
    assert "struct_size" in last_error()


def test_mask_narrowing_works_on_inference_tensors():
    """An int64 padding mask is converted to x's type once and cached on its identity and version; tensors made
    under torch.inference_mode() have no version counter, so they are converted without the cache."""
    import causal_conv1d as cc
    x = torch.zeros(2, 4, 8, dtype=torch.bfloat16)
    big = cc._NARROW_MIN_ELEMENTS
    mask = torch.ones(2, 8, dtype=torch.int64)
    first = cc._narrow_mask(mask, x, big)
    assert first.dtype == torch.bfloat16 and cc._narrow_mask(mask, x, big) is first          # cached
    assert cc._narrow_mask(mask, x, big - 1) is mask                                         # small problems: as given
    with torch.inference_mode():
        imask = torch.ones(2, 8, dtype=torch.int64)
        got = cc._narrow_mask(imask, x, big)
        assert got.dtype == torch.bfloat16 and torch.equal(got.float(), imask.float())
    mask[0, 3] = 0                                                                           # a new version: converted again
    assert cc._narrow_mask(mask, x, big)[0, 3].item() == 0


def update_bwd_params(B=256, C=3456, S=3, dtype=1, **over):
    p = UpdateBwdParams()
    p.struct_size = ctypes.sizeof(UpdateBwdParams)
    p.x_dtype = p.w_dtype = dtype
    p.width, p.state_len = 4, S
    p.batch, p.channels = B, C
    p.x, p.dout, p.dx, p.weight, p.conv_state = FAKE_X, FAKE_OUT, FAKE_OUT + 0x4000000, FAKE_W, FAKE_STATE
    p.dweight, p.workspace, p.workspace_bytes = FAKE_W + 0x100000, FAKE_W + 0x200000, 1 << 30
    for name in ("x", "dout", "dx"):
        setattr(p, f"{name}_stride_b", C)
        setattr(p, f"{name}_stride_c", 1)
    for name in ("state", "dstate_out", "dstate"):
        for s, v in zip(("b", "c", "s"), (C * S, S, 1)):
            setattr(p, f"{name}_stride_{s}", v)
    p.w_stride_c, p.w_stride_k = 4, 1
    for k, v in over.items():
        setattr(p, k, v)
    return p


def test_update_bwd_validation_and_workspace():
    L = _lib.lib()
    ws = L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(update_bwd_params()))
    assert 0 < ws <= 8 << 20 and ws % (3456 * 5 * 4) == 0          # whole partial sets, one per batch group
    assert L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(update_bwd_params(dweight=0))) == 0
    assert L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(update_bwd_params(B=0))) == 0
    assert L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(update_bwd_params(B=1, C=8))) == 8 * 5 * 4
    for over, msg in [(dict(width=5), "width 5"), (dict(S=2), "shorter than width-1"), (dict(struct_size=4), "struct_size"),
                      (dict(x_dtype=7), "x_dtype 7"), (dict(activation=3), "activation 3"),
                      (dict(dweight=0, dbias=FAKE_W), "dbias needs dweight"),
                      (dict(token_mask=FAKE_X, mask_dtype=9), "mask_dtype 9")]:
        assert L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(update_bwd_params(**over))) == -1, over
        assert msg in last_error(), (over, last_error())
    # what only the launching call can check: pointers and the scratch
    for over, msg in [(dict(dout=0), "NULL"), (dict(workspace=0), "workspace"), (dict(workspace_bytes=16), "workspace"),
                      (dict(dstate=FAKE_X, dstate_out=FAKE_X), "alias")]:
        assert L.canon_conv1d_update_bwd(ctypes.byref(update_bwd_params(**over)), None) == _lib.ERR_INVALID_ARGUMENT, over
        assert msg in last_error(), (over, last_error())


def make_parts(dims, B=8, L=1024, layout="blc", elem=2, row=None):
    """Fake part descriptors: separate (B, L, C_i) allocations, or with ``row`` slices of one (B, L, row) tensor."""
    arr = (Part * len(dims))()
    c0 = 0
    for i, d in enumerate(dims):
        if row is not None:
            arr[i].x, arr[i].out = FAKE_X + c0 * elem, FAKE_OUT + c0 * elem
            strides = (row * L, 1, row)
        else:
            arr[i].x, arr[i].out = FAKE_X + i * 0x1000000, FAKE_OUT + i * 0x1000000
            strides = (d * L, 1, d) if layout == "blc" else (d * L, L, 1)
        arr[i].x_stride_b, arr[i].x_stride_c, arr[i].x_stride_l = strides
        arr[i].out_stride_b, arr[i].out_stride_c, arr[i].out_stride_l = strides
        arr[i].channels = d
        c0 += d
    return arr


def test_parts_plan_and_validation():
    L = _lib.lib()

    def fplan(p, arr, n=None):
        r = L.canon_conv1d_fwd_parts_plan(ctypes.byref(p), arr, len(arr) if n is None else n)
        return r.decode() if r is not None else None

    def uplan_parts(p, arr):
        r = L.canon_conv1d_update_parts_plan(ctypes.byref(p), arr, len(arr))
        return r.decode() if r is not None else None

    # Canon-B (q, k, v) and Canon-D (gate, up), separate tensors and slices of one projection output
    assert fplan(fwd_params(C=960, layout="blc"), make_parts([640, 160, 160])) == "blc_vec_parts"
    assert fplan(fwd_params(C=3456, layout="blc"), make_parts([1728, 1728])) == "blc_vec_pair"       # equal and dense
    assert fplan(fwd_params(C=3456, layout="blc"), make_parts([1728, 1728], row=3456)) == "blc_vec_parts"   # views of one tensor
    assert fplan(fwd_params(C=960, layout="blc"), make_parts([640, 160, 160], row=960)) == "blc_vec_parts"
    assert fplan(fwd_params(C=960, layout="blc", x=None, out=None), make_parts([640, 160, 160])) == "blc_vec_parts"
    # one launch per part: time-contiguous parts, a single part, other widths, channel counts off the vector size
    assert fplan(fwd_params(C=960), make_parts([640, 320], layout="bcl")) == "per_part"
    assert fplan(fwd_params(C=640, layout="blc"), make_parts([640])) == "per_part"
    assert fplan(fwd_params(C=960, layout="blc", width=3, w_stride_c=3), make_parts([640, 320])) == "per_part"
    assert fplan(fwd_params(C=100, layout="blc"), make_parts([60, 40])) == "blc_vec_parts"     # 8-byte channel groups
    assert fplan(fwd_params(C=102, layout="blc"), make_parts([62, 40])) == "per_part"
    # rejected
    assert fplan(fwd_params(C=961, layout="blc"), make_parts([640, 160, 160])) is None
    assert "960 channels" in last_error() and "961" in last_error()
    assert fplan(fwd_params(C=960, layout="blc"), make_parts([640, 160, 160]), n=0) is None
    assert "nparts" in last_error()
    assert fplan(fwd_params(C=5 * 64, layout="blc"), make_parts([64] * 5)) is None
    assert L.canon_conv1d_fwd_parts_plan(ctypes.byref(fwd_params()), None, 2) is None
    assert "parts is NULL" in last_error()
    bad = make_parts([640, 320])
    bad[1].x = None
    assert fplan(fwd_params(C=960, layout="blc"), bad) is None
    assert "must not be NULL" in last_error()

    assert uplan_parts(update_params(C=960, S=8), make_parts([640, 160, 160], L=1)) == "update_vec_parts"
    assert uplan_parts(update_params(C=3456, S=3), make_parts([1728, 1728], L=1)) == "update_vec_parts"
    assert uplan_parts(update_params(C=3456, S=5), make_parts([1728, 1728], L=1)) == "per_part"
    assert uplan_parts(update_params(C=3456, S=3), make_parts([3456], L=1)) == "per_part"
    assert uplan_parts(update_params(C=3457, S=3), make_parts([1728, 1728], L=1)) is None


def test_seq_idx_plan_and_validation():
    FAKE_SEQ = 0x50000000
    assert plan(fwd_params(layout="blc", seq_idx=FAKE_SEQ, seq_stride_b=1024, seq_stride_l=1)) == "blc_vec_seq"
    assert plan(fwd_params(layout="bcl", seq_idx=FAKE_SEQ, seq_stride_b=1024, seq_stride_l=1)) == "generic"
    assert plan(fwd_params(layout="blc", seq_idx=FAKE_SEQ + 2, seq_stride_b=1024, seq_stride_l=1)) is None
    assert "4-byte aligned" in last_error()
    assert plan(fwd_params(layout="blc", seq_idx=FAKE_SEQ, final_state=FAKE_STATE, final_len=3)) is None
    assert "seq_idx excludes" in last_error()


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "single-GPU" in (r.stderr + r.stdout)


def test_torch_operators_for_traced_graphs_have_shape_only_twins():
    """torch.compile traces the launches as operators of the canon_conv1d namespace; their shape-only
    implementations (what tracing runs) are checked here on meta tensors, no GPU involved."""
    import causal_conv1d  # noqa: F401  (registers the operators)
    ops = torch.ops.canon_conv1d
    x = torch.empty(2, 40, 16, device="meta", dtype=torch.bfloat16).transpose(1, 2)      # channel-contiguous view
    w = torch.empty(16, 4, device="meta", dtype=torch.float32)
    b = torch.empty(16, device="meta", dtype=torch.float32)
    y, fin = ops.fwd(x, w, b, None, None, None, 8, 1, 1, 0)
    assert y.shape == x.shape and y.stride() == x.stride() and y.dtype == x.dtype
    assert tuple(fin.shape) == (2, 16, 8) and fin.dtype == x.dtype
    assert tuple(ops.fwd(x, w, None, None, None, None, 0, 0, 0, 0)[1].shape) == (2, 16, 0)
    dx, dw, db, di = ops.bwd(x, x, w, b, None, None, None, None, 0, 1)
    assert tuple(di.shape) == (2, 16, 0)
    init = torch.empty(2, 16, 3, dtype=x.dtype, device="meta")
    assert tuple(ops.bwd(x, x, w, b, None, None, init, init, 0, 1)[3].shape) == (2, 16, 3)
    assert dx.stride() == x.stride() and tuple(dw.shape) == (16, 4) and dw.dtype == w.dtype and tuple(db.shape) == (16,)
    assert tuple(ops.bwd(x, x, w, None, None, None, None, None, 0, 1)[2].shape) == (0,)
    st = torch.empty(2, 16, 4, device="meta", dtype=torch.bfloat16)
    assert tuple(ops.update(x[:, :, 0], st, w, None, None, None, None, 0, 0, 0).shape) == (2, 16)
    outs = ops.fwd_parts([x[:, :12], x[:, 12:]], w, None, None, None, 3, 0, 0, 0)
    assert [tuple(t.shape) for t in outs] == [(2, 12, 40), (2, 4, 40), (2, 16, 3)]
    outs = ops.update_parts([x[:, :12, 0], x[:, 12:, 0]], st, w, None, None, 0, 0, 0)
    assert [tuple(t.shape) for t in outs] == [(2, 12), (2, 4)]
    # the decode step as a function (traced graphs with gradients): output and new state, nothing written to
    out, new = ops.update_step(x[:, :, 0], st, w, b, None, None, None, 1, 1, 0)
    assert tuple(out.shape) == (2, 16) and new.shape == st.shape and new.dtype == st.dtype
    assert "!" not in str(ops.update_step.default._schema)
    g = ops.update_bwd(x[:, :, 0], st, w, b, None, x[:, :, 0], st, None, None, 1, 1)
    assert [tuple(t.shape) for t in g] == [(2, 16), (2, 16, 4), (16, 4), (16,)] and g[2].dtype == w.dtype
    assert tuple(ops.update_bwd(x[:, :, 0], st, w, None, None, x[:, :, 0], st, None, None, 0, 0)[3].shape) == (0,)
    # the state arguments of the decode operators are declared as written to
    assert "Tensor(a1!) conv_state" in str(ops.update.default._schema)
    assert "Tensor(a1!) conv_state" in str(ops.update_parts.default._schema)


def test_copy_ceiling_library_exports_what_the_bench_times():
    """tests/copy_ceiling (plain copies in the kernels' access patterns, timed by bench.py beside the kernels):
    loads without a GPU and exports its three entry points."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "copy_ceiling", "libcopy_ceiling.so")
    if not os.path.exists(path):
        pytest.skip("not built (make -C tests/copy_ceiling)")
    lib = ctypes.CDLL(path)
    for name in ("copy_rows", "copy_tiles", "copy_tile_shape", "empty_launch"):
        assert getattr(lib, name) is not None
