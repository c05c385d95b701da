"""ctypes front end of the C oracle in ``canon_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by
the CPU-baseline leg of the benchmark, never by the shipped package.

All functions take and return CPU torch tensors.  ``x`` may have any strides;
it is made contiguous ``[B, C, L]`` before it is handed to C.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple, Union

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcanon_oracle.so")

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def build(force: bool = False) -> str:
    """Compile ``canon_oracle.c`` with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        L.canon_oracle_fwd.restype = i32
        L.canon_oracle_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64,
                                       i32, i32, i32, i32, i32, i32, i32, i32]
        L.canon_oracle_fwd_seq.restype = i32
        L.canon_oracle_fwd_seq.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i32, i32, i32, i32, i32]
        L.canon_oracle_update_ext.restype = i32
        L.canon_oracle_update_ext.argtypes = [vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i32, i32, i32, vp, vp, i64]
        L.canon_oracle_update.restype = i32
        L.canon_oracle_update.argtypes = [vp, vp, vp, vp, vp, i64, i64, i32, i32,
                                          i32, i32, i32, i32, i32]
        L.canon_oracle_float_to_bf16.restype = ctypes.c_uint16
        L.canon_oracle_float_to_bf16.argtypes = [ctypes.c_float]
        L.canon_oracle_float_to_f16.restype = ctypes.c_uint16
        L.canon_oracle_float_to_f16.argtypes = [ctypes.c_float]
        L.canon_oracle_bf16_to_float.restype = ctypes.c_float
        L.canon_oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.canon_oracle_f16_to_float.restype = ctypes.c_float
        L.canon_oracle_f16_to_float.argtypes = [ctypes.c_uint16]
        _lib = L
    return _lib


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _act(activation) -> int:
    if activation in (None, False):
        return 0
    if activation in (True, "silu", "swish"):
        return 1
    raise NotImplementedError("activation must be None, silu, or swish")


def _res_mode(residual) -> int:
    if residual in (None, False, 0):
        return 0
    if residual in (True, 1, "masked"):
        return 1
    if residual in (2, "unmasked"):
        return 2
    raise ValueError(f"bad residual mode {residual!r}")


def conv1d_fwd(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    mask: Optional[torch.Tensor] = None,
    initial_state: Optional[torch.Tensor] = None,
    final_state_len: Optional[int] = None,
    activation=None,
    residual=0,
    round_mode: int = 0,
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Prefill oracle over logical ``[B, C, L]``; see ``canon_oracle_fwd``."""
    assert x.dim() == 3 and weight.dim() == 2 and x.device.type == "cpu"
    B, C, L = x.shape
    W = weight.shape[1]
    assert weight.shape[0] == C
    xc = x.contiguous()
    wc = weight.contiguous()
    bc = None
    if bias is not None:
        bc = bias.to(weight.dtype).contiguous()
    mc = None
    if mask is not None:
        assert tuple(mask.shape) == (B, L)
        mc = mask.to(torch.float32).contiguous()
    ic = None
    s_in = 0
    if initial_state is not None:
        assert initial_state.shape[:2] == (B, C) and initial_state.dtype == x.dtype
        ic = initial_state.contiguous()
        s_in = ic.shape[2]
    out = torch.empty_like(xc)
    fs = None
    s_out = 0
    if final_state_len is not None:
        s_out = int(final_state_len)
        fs = torch.empty(B, C, s_out, dtype=x.dtype)
    rc = lib().canon_oracle_fwd(
        _ptr(xc), _ptr(wc), _ptr(bc), _ptr(mc), _ptr(ic), _ptr(out), _ptr(fs),
        B, C, L, W, s_in, s_out, _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype],
        _act(activation), _res_mode(residual), int(round_mode))
    if rc != 0:
        raise ValueError("canon_oracle_fwd rejected its arguments")
    return out if fs is None else (out, fs)


def conv1d_fwd_seq(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    seq_idx: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
    activation=None,
    residual=0,
) -> torch.Tensor:
    """Prefill oracle over packed sequences (``seq_idx`` [B, L] int32); see ``canon_oracle_fwd_seq``."""
    assert x.dim() == 3 and weight.dim() == 2 and x.device.type == "cpu"
    B, C, L = x.shape
    assert weight.shape[0] == C and tuple(seq_idx.shape) == (B, L)
    xc, wc = x.contiguous(), weight.contiguous()
    bc = bias.to(weight.dtype).contiguous() if bias is not None else None
    mc = mask.to(torch.float32).contiguous() if mask is not None else None
    sc = seq_idx.to(torch.int32).contiguous()
    out = torch.empty_like(xc)
    rc = lib().canon_oracle_fwd_seq(
        _ptr(xc), _ptr(wc), _ptr(bc), _ptr(mc), _ptr(sc), _ptr(out), B, C, L, weight.shape[1],
        _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype], _act(activation), _res_mode(residual))
    if rc != 0:
        raise ValueError("canon_oracle_fwd_seq rejected its arguments")
    return out


def conv1d_update(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    activation=None,
    residual: bool = False,
    round_mode: int = 0,
) -> torch.Tensor:
    """Decode-step oracle; ``conv_state`` (contiguous) is updated in place."""
    assert x.dim() == 2 and conv_state.dim() == 3 and conv_state.is_contiguous()
    assert x.device.type == "cpu" and conv_state.dtype == x.dtype
    B, C = x.shape
    S = conv_state.shape[2]
    W = weight.shape[1]
    assert conv_state.shape[:2] == (B, C) and weight.shape[0] == C
    xc = x.contiguous()
    wc = weight.contiguous()
    bc = None if bias is None else bias.to(weight.dtype).contiguous()
    out = torch.empty_like(xc)
    rc = lib().canon_oracle_update(
        _ptr(xc), _ptr(conv_state), _ptr(wc), _ptr(bc), _ptr(out), B, C, W, S,
        _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype], _act(activation),
        int(bool(residual)), int(round_mode))
    if rc != 0:
        raise ValueError("canon_oracle_update rejected its arguments")
    return out


def conv1d_update_ext(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    activation=None,
    residual: bool = False,
    cache_seqlens: Optional[torch.Tensor] = None,
    conv_state_indices: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Decode-step oracle with circular-buffer (``cache_seqlens``) and state-pool (``conv_state_indices``)
    addressing; ``conv_state`` (rows, C, S), contiguous, is updated in place.  Entries whose index lies outside
    the pool are skipped: their output rows are zero.  See ``canon_oracle_update_ext``."""
    assert x.dim() == 2 and conv_state.dim() == 3 and conv_state.is_contiguous() and x.device.type == "cpu"
    B, C = x.shape
    assert conv_state.shape[1] == C and conv_state.dtype == x.dtype
    S = conv_state.shape[2]
    xc, wc = x.contiguous(), weight.contiguous()
    bc = bias.to(weight.dtype).contiguous() if bias is not None else None
    sl = cache_seqlens.to(torch.int32).contiguous() if cache_seqlens is not None else None
    ix = conv_state_indices.to(torch.int32).contiguous() if conv_state_indices is not None else None
    if ix is None:
        assert conv_state.shape[0] == B
    out = torch.zeros_like(xc)
    rc = lib().canon_oracle_update_ext(
        _ptr(xc), _ptr(conv_state), _ptr(wc), _ptr(bc), _ptr(out), B, C, weight.shape[1], S,
        _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype], _act(activation), int(bool(residual)), _ptr(sl), _ptr(ix),
        conv_state.shape[0])
    if rc != 0:
        raise ValueError("canon_oracle_update_ext rejected its arguments")
    return out
