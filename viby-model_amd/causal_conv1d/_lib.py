"""ctypes binding of ``libcanon_conv1d.so`` (the C ABI in ``include/canon_conv1d.h``).

No CPU path exists: if the shared library is missing or a call fails, an
exception is raised.
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcanon_conv1d.so")

ABI_VERSION = 9

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
MASK_CODE = {
    torch.bool: 0, torch.uint8: 0, torch.int32: 1, torch.int64: 2,
    torch.float32: 3, torch.bfloat16: 4, torch.float16: 5,
}
ROUND_CODE = {"fused": 0, "eager": 1}

OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_LAUNCH = 0, 1, 2, 3

_i32, _i64, _u32, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_uint32, ctypes.c_void_p


class FwdParams(ctypes.Structure):
    _fields_ = [
        ("struct_size", _u32),
        ("x_dtype", _i32), ("w_dtype", _i32), ("mask_dtype", _i32),
        ("width", _i32), ("activation", _i32), ("residual_mode", _i32), ("round_mode", _i32),
        ("batch", _i64), ("channels", _i64), ("seqlen", _i64),
        ("x", _vp), ("x_stride_b", _i64), ("x_stride_c", _i64), ("x_stride_l", _i64),
        ("out", _vp), ("out_stride_b", _i64), ("out_stride_c", _i64), ("out_stride_l", _i64),
        ("weight", _vp), ("w_stride_c", _i64), ("w_stride_k", _i64),
        ("bias", _vp),
        ("mask", _vp), ("mask_stride_b", _i64), ("mask_stride_l", _i64),
        ("initial_state", _vp), ("init_stride_b", _i64), ("init_stride_c", _i64), ("init_stride_s", _i64),
        ("initial_len", _i32), ("final_len", _i32),
        ("final_state", _vp), ("final_stride_b", _i64), ("final_stride_c", _i64), ("final_stride_s", _i64),
        ("seq_idx", _vp), ("seq_stride_b", _i64), ("seq_stride_l", _i64),
    ]


class UpdateParams(ctypes.Structure):
    _fields_ = [
        ("struct_size", _u32),
        ("x_dtype", _i32), ("w_dtype", _i32), ("mask_dtype", _i32),
        ("width", _i32), ("activation", _i32), ("residual_mode", _i32), ("round_mode", _i32),
        ("state_len", _i32), ("state_rows", _i32),
        ("batch", _i64), ("channels", _i64),
        ("x", _vp), ("x_stride_b", _i64), ("x_stride_c", _i64),
        ("out", _vp), ("out_stride_b", _i64), ("out_stride_c", _i64),
        ("conv_state", _vp), ("state_stride_b", _i64), ("state_stride_c", _i64), ("state_stride_s", _i64),
        ("weight", _vp), ("w_stride_c", _i64), ("w_stride_k", _i64),
        ("bias", _vp),
        ("token_mask", _vp), ("mask_stride_b", _i64),
        ("cache_seqlens", _vp), ("conv_state_indices", _vp),
    ]


class BwdParams(ctypes.Structure):
    _fields_ = [
        ("struct_size", _u32),
        ("x_dtype", _i32), ("w_dtype", _i32), ("mask_dtype", _i32),
        ("width", _i32), ("activation", _i32), ("residual_mode", _i32), ("reserved0", _i32),
        ("batch", _i64), ("channels", _i64), ("seqlen", _i64),
        ("x", _vp), ("x_stride_b", _i64), ("x_stride_c", _i64), ("x_stride_l", _i64),
        ("dout", _vp), ("dout_stride_b", _i64), ("dout_stride_c", _i64), ("dout_stride_l", _i64),
        ("dx", _vp), ("dx_stride_b", _i64), ("dx_stride_c", _i64), ("dx_stride_l", _i64),
        ("weight", _vp), ("w_stride_c", _i64), ("w_stride_k", _i64),
        ("bias", _vp),
        ("mask", _vp), ("mask_stride_b", _i64), ("mask_stride_l", _i64),
        ("dweight", _vp), ("dbias", _vp),
        ("workspace", _vp), ("workspace_bytes", _i64),
        ("seq_idx", _vp), ("seq_stride_b", _i64), ("seq_stride_l", _i64),
        ("initial_state", _vp), ("init_stride_b", _i64), ("init_stride_c", _i64), ("init_stride_s", _i64),
        ("initial_len", _i32), ("reserved1", _i32),
        ("dinitial_state", _vp), ("dinit_stride_b", _i64), ("dinit_stride_c", _i64), ("dinit_stride_s", _i64),
        ("dfinal_state", _vp), ("dfinal_stride_b", _i64), ("dfinal_stride_c", _i64), ("dfinal_stride_s", _i64),
        ("final_len", _i32), ("reserved2", _i32),
    ]


class UpdateBwdParams(ctypes.Structure):
    _fields_ = [
        ("struct_size", _u32),
        ("x_dtype", _i32), ("w_dtype", _i32), ("mask_dtype", _i32),
        ("width", _i32), ("activation", _i32), ("residual_mode", _i32), ("state_len", _i32),
        ("batch", _i64), ("channels", _i64),
        ("x", _vp), ("x_stride_b", _i64), ("x_stride_c", _i64),
        ("conv_state", _vp), ("state_stride_b", _i64), ("state_stride_c", _i64), ("state_stride_s", _i64),
        ("weight", _vp), ("w_stride_c", _i64), ("w_stride_k", _i64),
        ("bias", _vp),
        ("token_mask", _vp), ("mask_stride_b", _i64),
        ("dout", _vp), ("dout_stride_b", _i64), ("dout_stride_c", _i64),
        ("dstate_out", _vp), ("dstate_out_stride_b", _i64), ("dstate_out_stride_c", _i64), ("dstate_out_stride_s", _i64),
        ("dx", _vp), ("dx_stride_b", _i64), ("dx_stride_c", _i64),
        ("dstate", _vp), ("dstate_stride_b", _i64), ("dstate_stride_c", _i64), ("dstate_stride_s", _i64),
        ("dweight", _vp), ("dbias", _vp),
        ("workspace", _vp), ("workspace_bytes", _i64),
        ("cache_seqlens", _vp), ("conv_state_indices", _vp), ("state_rows", _i64),
    ]


class Part(ctypes.Structure):
    _fields_ = [
        ("x", _vp), ("x_stride_b", _i64), ("x_stride_c", _i64), ("x_stride_l", _i64),
        ("out", _vp), ("out_stride_b", _i64), ("out_stride_c", _i64), ("out_stride_l", _i64),
        ("channels", _i64),
    ]


MAX_PARTS = 4

EXPORTS = (
    "canon_conv1d_abi_version",
    "canon_conv1d_last_error",
    "canon_conv1d_fwd",
    "canon_conv1d_update",
    "canon_conv1d_init",
    "canon_conv1d_fwd_plan",
    "canon_conv1d_fwd_plan_waves",
    "canon_conv1d_update_plan",
    "canon_conv1d_bwd",
    "canon_conv1d_bwd_static",
    "canon_conv1d_bwd_workspace_bytes",
    "canon_conv1d_bwd_plan",
    "canon_conv1d_update_bwd",
    "canon_conv1d_update_bwd_workspace_bytes",
    "canon_conv1d_fwd_parts",
    "canon_conv1d_update_parts",
    "canon_conv1d_fwd_parts_plan",
    "canon_conv1d_update_parts_plan",
)

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `make -j4 -C viby-model_amd/csrc` "
                "(hipcc, --offload-arch=gfx950). There is no fallback implementation.")
        L = ctypes.CDLL(LIB_PATH)
        L.canon_conv1d_abi_version.restype = ctypes.c_int
        L.canon_conv1d_abi_version.argtypes = []
        L.canon_conv1d_last_error.restype = ctypes.c_char_p
        L.canon_conv1d_last_error.argtypes = []
        L.canon_conv1d_fwd.restype = ctypes.c_int
        L.canon_conv1d_fwd.argtypes = [ctypes.POINTER(FwdParams), _vp]
        L.canon_conv1d_update.restype = ctypes.c_int
        L.canon_conv1d_update.argtypes = [ctypes.POINTER(UpdateParams), _vp]
        L.canon_conv1d_init.restype = ctypes.c_int
        L.canon_conv1d_init.argtypes = []
        L.canon_conv1d_fwd_plan_waves.restype = ctypes.c_int
        L.canon_conv1d_fwd_plan_waves.argtypes = [ctypes.POINTER(FwdParams)]
        L.canon_conv1d_fwd_plan.restype = ctypes.c_char_p
        L.canon_conv1d_fwd_plan.argtypes = [ctypes.POINTER(FwdParams)]
        L.canon_conv1d_update_plan.restype = ctypes.c_char_p
        L.canon_conv1d_update_plan.argtypes = [ctypes.POINTER(UpdateParams)]
        L.canon_conv1d_bwd.restype = ctypes.c_int
        L.canon_conv1d_bwd.argtypes = [ctypes.POINTER(BwdParams), _vp]
        L.canon_conv1d_bwd_static.restype = ctypes.c_int
        L.canon_conv1d_bwd_static.argtypes = [ctypes.POINTER(BwdParams), _vp]
        L.canon_conv1d_bwd_workspace_bytes.restype = ctypes.c_int64
        L.canon_conv1d_bwd_workspace_bytes.argtypes = [ctypes.POINTER(BwdParams)]
        L.canon_conv1d_bwd_plan.restype = ctypes.c_char_p
        L.canon_conv1d_bwd_plan.argtypes = [ctypes.POINTER(BwdParams)]
        L.canon_conv1d_update_bwd.restype = ctypes.c_int
        L.canon_conv1d_update_bwd.argtypes = [ctypes.POINTER(UpdateBwdParams), _vp]
        L.canon_conv1d_update_bwd_workspace_bytes.restype = ctypes.c_int64
        L.canon_conv1d_update_bwd_workspace_bytes.argtypes = [ctypes.POINTER(UpdateBwdParams)]
        L.canon_conv1d_fwd_parts.restype = ctypes.c_int
        L.canon_conv1d_fwd_parts.argtypes = [ctypes.POINTER(FwdParams), ctypes.POINTER(Part), _i32, _vp]
        L.canon_conv1d_update_parts.restype = ctypes.c_int
        L.canon_conv1d_update_parts.argtypes = [ctypes.POINTER(UpdateParams), ctypes.POINTER(Part), _i32, _vp]
        L.canon_conv1d_fwd_parts_plan.restype = ctypes.c_char_p
        L.canon_conv1d_fwd_parts_plan.argtypes = [ctypes.POINTER(FwdParams), ctypes.POINTER(Part), _i32]
        L.canon_conv1d_update_parts_plan.restype = ctypes.c_char_p
        L.canon_conv1d_update_parts_plan.argtypes = [ctypes.POINTER(UpdateParams), ctypes.POINTER(Part), _i32]
        got = L.canon_conv1d_abi_version()
        if got != ABI_VERSION:
            raise ImportError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}")
        _lib = L
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a status code into the exception the Python API documents."""
    if rc == OK:
        return
    msg = lib().canon_conv1d_last_error().decode("utf-8", "replace")
    if rc == ERR_INVALID_ARGUMENT:
        raise ValueError(f"{what}: {msg}")
    if rc == ERR_UNSUPPORTED:
        raise NotImplementedError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg}")
