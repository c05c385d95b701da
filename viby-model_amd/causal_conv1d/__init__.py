"""MI355X (gfx950) causal depthwise conv1d, importable as ``causal_conv1d``.

This is the package name Viby's ``model/model.py:21-25`` imports, so with this
directory's parent on ``sys.path`` the Canon layers take this implementation
on ROCm devices without any change to the model code::

    from causal_conv1d import causal_conv1d_fn, causal_conv1d_update

``causal_conv1d_fn`` / ``causal_conv1d_update`` keep the upstream call
signatures used at ``model/model.py:460-466`` and ``:305-311`` (keyword set as
mirrored in ``causal-conv1d-mps/causal_conv1d_mps/autograd.py:501-510``).
Keyword-only extras fuse what CanonLayer does around those calls
(``attention_mask``, ``residual``), modelled on the reference's own fused API
``short_conv_fused`` / ``short_conv_update``
(``causal_conv1d_mps/__init__.py:154-161`` and ``:304-312``), which is also
exported here with the same argument meaning.

Everything runs in hand-written HIP kernels behind a C ABI
(``include/canon_conv1d.h``); there is no PyTorch fallback: a missing library
or a rejected call raises.
"""
from __future__ import annotations

import ctypes
import threading
from typing import List, Optional, Tuple, Union

import torch

from . import _lib
from ._lib import FwdParams, UpdateParams

__version__ = "0.1.0"

__all__ = [
    "causal_conv1d_fn",
    "causal_conv1d_update",
    "causal_conv1d_fn_parts",
    "causal_conv1d_update_parts",
    "short_conv_fused",
    "short_conv_update",
    "prepare_device",
    "kernel_plan_fwd",
    "kernel_plan_fwd_waves",
    "kernel_plan_update",
    "kernel_plan_fwd_parts",
    "kernel_plan_update_parts",
]

MIN_WIDTH, MAX_WIDTH = 2, 4   # CANON_CONV1D_MIN_WIDTH / _MAX_WIDTH

_RESIDUAL = {False: 0, None: 0, 0: 0, True: 1, 1: 1, "masked": 1, 2: 2, "unmasked": 2}


def _activation_flag(activation) -> int:
    if activation not in (None, "silu", "swish"):
        raise NotImplementedError("activation must be None, silu, or swish")
    return 0 if activation is None else 1


def _residual_mode(residual) -> int:
    try:
        return _RESIDUAL[residual]
    except (KeyError, TypeError):
        raise ValueError(f"residual must be False, True/'masked' or 'unmasked', got {residual!r}") from None


def _round_mode(rounding: str) -> int:
    try:
        return _lib.ROUND_CODE[rounding]
    except KeyError:
        raise ValueError(f"rounding must be 'fused' or 'eager', got {rounding!r}") from None


def _require_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise ValueError(f"{what} must be on a ROCm GPU device (device type 'cuda'), got {t.device}")


def _check_shapes(x_dim: int, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> None:
    """Shape / dtype errors first (they do not depend on where the tensors live)."""
    if weight.dim() != 2:
        raise ValueError(f"Expected 2D weight tensor (dim, width), got {weight.dim()}D")
    if x_dim != weight.shape[0]:
        raise ValueError(f"Input dim {x_dim} does not match weight dim {weight.shape[0]}")
    if not MIN_WIDTH <= weight.shape[1] <= MAX_WIDTH:
        raise NotImplementedError(f"width {weight.shape[1]} not supported (only widths 2..4)")
    if weight.dtype not in _lib.DTYPE_CODE:
        raise ValueError(f"Unsupported weight dtype {weight.dtype}")
    if bias is not None:
        if bias.dim() != 1:
            raise ValueError(f"Expected 1D bias tensor, got {bias.dim()}D")
        if bias.shape[0] != x_dim:
            raise ValueError(f"Bias dim {bias.shape[0]} does not match input dim {x_dim}")


def _check_devices(weight: torch.Tensor, bias: Optional[torch.Tensor], dev) -> None:
    _require_gpu(weight, "Weight tensor")
    if bias is not None:
        _require_gpu(bias, "Bias tensor")
    if weight.device != dev or (bias is not None and bias.device != dev):
        raise ValueError("weight and bias must be on the same device as x")


def _prep_bias(weight: torch.Tensor, bias: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    # the kernels read weight and bias with one element type
    if bias is None:
        return None
    if bias.dtype != weight.dtype or not bias.is_contiguous():
        bias = bias.to(weight.dtype).contiguous()
    return bias


_NARROW_MIN_ELEMENTS = 1 << 20
# (key, the source mask (kept alive so its address stays unique), converted mask); replaced as one object, so
# threads that race here each see a consistent entry
_narrow_cache = (None, None, None)


def _narrow_mask(mask: torch.Tensor, x: torch.Tensor, numel: int) -> torch.Tensor:
    """An integer mask wider than x's element type is converted to x.dtype once.

    Every (batch, channel) row re-reads its batch row of the mask, so an int64
    mask moves four times the bytes of bf16 data through the caches.  The
    conversion is what the multiply does anyway (``x * mask`` promotes the
    integer to x.dtype, ``model/model.py:455``; the reference wrapper casts the
    mask the same way, ``causal_conv1d_mps/__init__.py:244-247``).  The result
    is cached on the mask's identity because a model passes one mask to every
    Canon call of a forward.  Small problems keep the caller's mask as is.
    """
    if (mask.dtype.is_floating_point or mask.element_size() <= x.element_size()
            or numel < _NARROW_MIN_ELEMENTS):
        return mask
    if torch.compiler.is_compiling():
        return mask.to(x.dtype)      # one node of the traced graph; identical conversions are merged there
    if mask.is_inference():
        return mask.to(x.dtype)      # tensors made under torch.inference_mode() carry no version counter to key on
    global _narrow_cache
    key = (mask.data_ptr(), mask._version, tuple(mask.shape), mask.stride(), mask.dtype, x.dtype, mask.device)
    entry = _narrow_cache
    if entry[0] != key:
        entry = (key, mask, mask.to(x.dtype))
        _narrow_cache = entry
    return entry[2]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle without building a Stream object


def _stream(dev: torch.device) -> ctypes.c_void_p:
    if _raw_stream is not None and dev.index is not None:
        return ctypes.c_void_p(_raw_stream(dev.index))
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _call(fn, dev: torch.device, *args) -> int:
    """Launch on the current stream of ``dev`` with ``dev`` current (switching only if it is not already)."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return fn(*args, _stream(dev))
    with torch.cuda.device(dev):
        return fn(*args, _stream(dev))


def _fill_fwd(x, out, weight, bias, mask, initial_states, final_states, act, res, rnd, seq_idx=None) -> FwdParams:
    p = FwdParams()
    p.struct_size = ctypes.sizeof(FwdParams)
    p.x_dtype = _lib.DTYPE_CODE[x.dtype]
    p.w_dtype = _lib.DTYPE_CODE[weight.dtype]
    p.width = weight.shape[1]
    p.activation, p.residual_mode, p.round_mode = act, res, rnd
    p.batch, p.channels, p.seqlen = x.shape
    p.x = x.data_ptr()
    p.x_stride_b, p.x_stride_c, p.x_stride_l = x.stride()
    p.out = out.data_ptr()
    p.out_stride_b, p.out_stride_c, p.out_stride_l = out.stride()
    p.weight = weight.data_ptr()
    p.w_stride_c, p.w_stride_k = weight.stride()
    p.bias = bias.data_ptr() if bias is not None else None
    if mask is not None:
        p.mask = mask.data_ptr()
        p.mask_dtype = _lib.MASK_CODE[mask.dtype]
        p.mask_stride_b, p.mask_stride_l = mask.stride()
    if initial_states is not None:
        p.initial_state = initial_states.data_ptr()
        p.init_stride_b, p.init_stride_c, p.init_stride_s = initial_states.stride()
        p.initial_len = initial_states.shape[2]
    if final_states is not None:
        p.final_state = final_states.data_ptr()
        p.final_stride_b, p.final_stride_c, p.final_stride_s = final_states.stride()
        p.final_len = final_states.shape[2]
    if seq_idx is not None:
        p.seq_idx = seq_idx.data_ptr()
        p.seq_stride_b, p.seq_stride_l = seq_idx.stride()
    return p


def _check_fwd_args(x, shape, weight, bias, attention_mask, initial_states, return_final_states, final_states_out):
    """Checks shared by the single-tensor and the multi-part prefill; ``x`` is (one of) the input tensor(s),
    ``shape`` the logical (batch, dim, seqlen).  Returns (bias, attention_mask, final_states) as launched."""
    if x.dtype not in _lib.DTYPE_CODE:
        raise ValueError(f"Unsupported input dtype {x.dtype}; expected float32, bfloat16 or float16")
    batch, dim, seqlen = shape
    _check_shapes(dim, weight, bias)
    _require_gpu(x, "Input tensor")
    _check_devices(weight, bias, x.device)
    bias = _prep_bias(weight, bias)

    if attention_mask is not None:
        if attention_mask.dim() != 2:
            raise ValueError(f"Expected 2D attention mask, got {attention_mask.dim()}D")
        if tuple(attention_mask.shape) != (batch, seqlen):
            raise ValueError(
                f"Attention mask shape {tuple(attention_mask.shape)} does not match input shape ({batch}, {seqlen})")
        if attention_mask.dtype not in _lib.MASK_CODE:
            raise ValueError(f"Unsupported attention mask dtype {attention_mask.dtype}")
        if attention_mask.device != x.device:
            raise ValueError("Attention mask must be on the same device as x")
        attention_mask = _narrow_mask(attention_mask, x, batch * dim * seqlen)
    width = weight.shape[1]
    if initial_states is not None:
        if initial_states.dim() != 3 or tuple(initial_states.shape[:2]) != (batch, dim):
            raise ValueError(f"initial_states shape {tuple(initial_states.shape)} does not match (batch, dim, >=width-1)")
        if initial_states.dtype != x.dtype or initial_states.device != x.device:
            raise ValueError("initial_states must have the dtype and device of x")
    final_states = None
    if return_final_states or final_states_out is not None:
        if final_states_out is not None:
            if final_states_out.dim() != 3 or tuple(final_states_out.shape[:2]) != (batch, dim):
                raise ValueError(
                    f"final_states_out shape {tuple(final_states_out.shape)} does not match (batch, dim, state_len)")
            if final_states_out.dtype != x.dtype or final_states_out.device != x.device:
                raise ValueError("final_states_out must have the dtype and device of x")
            final_states = final_states_out
        else:
            final_states = torch.empty(batch, dim, width - 1, dtype=x.dtype, device=x.device)
    return bias, attention_mask, final_states


def causal_conv1d_fn(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    seq_idx: Optional[torch.Tensor] = None,
    initial_states: Optional[torch.Tensor] = None,
    return_final_states: bool = False,
    final_states_out: Optional[torch.Tensor] = None,
    activation: Optional[str] = None,
    *,
    attention_mask: Optional[torch.Tensor] = None,
    residual: Union[bool, str] = False,
    rounding: str = "fused",
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Causal depthwise conv over ``x`` of shape (batch, dim, seqlen).

    ``out[b,c,t] = act(bias[c] + sum_k weight[c,k] * x[b,c,t-(W-1)+k])`` with
    fp32 accumulation and one rounding to ``x.dtype``.  ``x`` may be time
    contiguous or channel contiguous (a transposed (batch, seqlen, dim) tensor,
    which is what ``model/model.py:459`` passes): both run vectorised kernels.
    Any other strides are read as they are by a strided kernel (several times
    slower; nothing is copied).  The output is ``torch.empty_like(x)``: x's
    strides when x is dense in some order of its dimensions, contiguous
    (batch, dim, seqlen) otherwise.

    seq_idx          (batch, seqlen) int32: packed variable-length sequences; positions
                     with different values do not see each other (the slot the
                     reference leaves at None, ``model/model.py:465``).  Inference
                     only, without initial / final states.
    initial_states   (batch, dim, >= W-1): history before t = 0 instead of zeros (differentiable).
    return_final_states / final_states_out (batch, dim, S): receives the last S
                     inputs (S = W-1 when allocated here; any S >= 1 when
                     given, e.g. the 4- or 8-slot conv_state of CanonLayer,
                     ``model/model.py:470-489``); the result is then
                     ``(out, final_states)``.
    attention_mask   (batch, seqlen) 0/1 of any dtype: inputs are multiplied by
                     it before the conv (``model/model.py:454-457``) and the
                     captured state holds the masked inputs.
    residual         False | True ('masked': ``out += x*mask``, the eager
                     CanonLayer, ``model/model.py:595,675``) | 'unmasked'
                     (``out += x``, ``model/model.py:491``).
    rounding         'fused' (one rounding) | 'eager' (also rounds after the
                     conv, after SiLU and after the residual add, which
                     reproduces the eager bf16/fp16 module bit for bit).
    """
    act = _activation_flag(activation)
    res = _residual_mode(residual)
    rnd = _round_mode(rounding)
    if x.dim() != 3:
        raise ValueError(f"Expected 3D input tensor (batch, dim, seqlen), got {x.dim()}D")
    if seq_idx is not None:
        if initial_states is not None or return_final_states or final_states_out is not None:
            raise ValueError("initial_states / final states cannot be combined with seq_idx")
        if seq_idx.dim() != 2 or tuple(seq_idx.shape) != (x.shape[0], x.shape[2]):
            raise ValueError(f"seq_idx shape {tuple(seq_idx.shape)} does not match (batch, seqlen) = "
                             f"({x.shape[0]}, {x.shape[2]})")
        if seq_idx.dtype != torch.int32 or seq_idx.device != x.device:
            raise ValueError("seq_idx must be an int32 tensor on the device of x")
    bias, attention_mask, final_states = _check_fwd_args(
        x, tuple(x.shape), weight, bias, attention_mask, initial_states, return_final_states, final_states_out)

    if x.numel() == 0 and final_states is not None and final_states.numel():
        raise ValueError("cannot produce final states from an empty input")

    if torch.compiler.is_compiling():
        # under torch.compile the launch is one opaque operator of the traced graph (trainer/train_pretrain.py:39
        # and eval_model.py:157 compile the whole model, the latter with fullgraph=True)
        result, fin = torch.ops.canon_conv1d.fwd(x, weight, bias, attention_mask, initial_states, seq_idx,
                                                 final_states.shape[2] if final_states is not None else 0,
                                                 act, res, rnd)
        if final_states is None:
            return result
        final_states.copy_(fin)
        return result, final_states
    if _wants_grad(x, weight, bias, initial_states):
        result = _CanonConvFn.apply(x, weight, bias, attention_mask, final_states, act, res, rnd, seq_idx,
                                    initial_states)
    else:
        result = _launch_fwd(x, weight, bias, attention_mask, initial_states, final_states, act, res, rnd, seq_idx)
        if final_states is not None:
            result = (result, final_states)
    return result


def _launch_fwd(x, weight, bias, mask, initial_states, final_states, act, res, rnd, seq_idx=None) -> torch.Tensor:
    out = torch.empty_like(x)
    if x.numel() == 0:
        return out
    p = _fill_fwd(x, out, weight, bias, mask, initial_states, final_states, act, res, rnd, seq_idx)
    rc = _call(_lib.lib().canon_conv1d_fwd, x.device, ctypes.byref(p))
    _lib.check(rc, "causal_conv1d_fn")
    return out


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class _CanonConvFn(torch.autograd.Function):
    """Autograd node of the prefill: forward and backward are one fused launch each
    (the backward recomputes the pre-activation from x, nothing but the inputs is saved).
    Mirrors the role of CausalConv1dMPSFunction / ShortConvFusedMPSFunction
    (causal_conv1d_mps/autograd.py:13-160, 162-338)."""

    @staticmethod
    def forward(ctx, x, weight, bias, mask, final_states, act, res, rnd, seq_idx=None, initial_states=None):
        out = _launch_fwd(x, weight, bias, mask, initial_states, final_states, act, res, rnd, seq_idx)
        # a copy of the (small) initial state: callers keep it in a cache tensor they overwrite right after
        # the call (CanonLayer copies the new state into it, decode steps shift it in place)
        ctx.save_for_backward(x, weight, bias, mask, seq_idx,
                              initial_states.detach().clone() if initial_states is not None else None)
        ctx.flags = (act, res)
        ctx.set_materialize_grads(False)
        if final_states is not None:
            # filled in place and differentiable: a gradient that arrives through the captured state (the next
            # chunk's initial_states, a decode step reading the cache) flows back into this call's inputs
            ctx.mark_dirty(final_states)
            return out, final_states
        return out

    @staticmethod
    def backward(ctx, dout, dfinal=None):
        x, weight, bias, mask, seq_idx, initial_states = ctx.saved_tensors
        if dout is None:
            dout = torch.zeros_like(x)
        act, res = ctx.flags
        channels, width = weight.shape
        dweight = torch.empty(channels, width, dtype=torch.float32, device=x.device)
        dbias = torch.empty(channels, dtype=torch.float32, device=x.device) if bias is not None else None
        dinit = None
        if initial_states is not None and ctx.needs_input_grad[9]:
            dinit = torch.empty_like(initial_states)
        dx = _launch_bwd(x, dout, weight, bias, mask, dweight, dbias, act, res, seq_idx, initial_states, dinit, dfinal)
        return (dx, dweight.to(weight.dtype), dbias.to(bias.dtype) if bias is not None else None,
                None, None, None, None, None, None, dinit)


def _launch_bwd(x, dout, weight, bias, mask, dweight, dbias, act, res, seq_idx=None, initial_states=None,
                dinit=None, dfinal=None) -> torch.Tensor:
    """One backward launch (+ the fixed-order reduction): returns dx with x's strides and fills the
    fp32 ``dweight`` (channels, W) / ``dbias`` (channels,) given (rows of larger tensors are fine)."""
    if dout.dtype != x.dtype:
        dout = dout.to(x.dtype)
    if dout.stride() != x.stride():
        dout = torch.empty_like(x).copy_(dout)       # same layout as x: keeps the vector kernel
    dx = torch.empty_like(x)
    width = weight.shape[1]
    p = _lib.BwdParams()
    p.struct_size = ctypes.sizeof(_lib.BwdParams)
    p.x_dtype = _lib.DTYPE_CODE[x.dtype]
    p.w_dtype = _lib.DTYPE_CODE[weight.dtype]
    p.width = width
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
    if seq_idx is not None:
        p.seq_idx = seq_idx.data_ptr()
        p.seq_stride_b, p.seq_stride_l = seq_idx.stride()
    if initial_states is not None:
        p.initial_state = initial_states.data_ptr()
        p.init_stride_b, p.init_stride_c, p.init_stride_s = initial_states.stride()
        p.initial_len = initial_states.shape[2]
        if dinit is not None:
            if x.numel() == 0:
                dinit.zero_()
            else:
                p.dinitial_state = dinit.data_ptr()
                p.dinit_stride_b, p.dinit_stride_c, p.dinit_stride_s = dinit.stride()
    if dfinal is not None and x.numel():
        if dfinal.dtype != x.dtype:
            dfinal = dfinal.to(x.dtype)
        p.dfinal_state = dfinal.data_ptr()
        p.dfinal_stride_b, p.dfinal_stride_c, p.dfinal_stride_s = dfinal.stride()
        p.final_len = dfinal.shape[2]
    p.dweight = dweight.data_ptr()
    p.dbias = dbias.data_ptr() if dbias is not None else None
    L = _lib.lib()
    nbytes = L.canon_conv1d_bwd_workspace_bytes(ctypes.byref(p))
    if nbytes < 0:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "causal_conv1d_fn backward")
    workspace = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=x.device)
    p.workspace = workspace.data_ptr()
    p.workspace_bytes = workspace.numel()
    rc = _call(L.canon_conv1d_bwd, x.device, ctypes.byref(p))
    _lib.check(rc, "causal_conv1d_fn backward")
    return dx


def _fill_update(x2, out2, conv_state, weight, bias, token_mask, act, res, rnd) -> UpdateParams:
    p = UpdateParams()
    p.struct_size = ctypes.sizeof(UpdateParams)
    p.x_dtype = _lib.DTYPE_CODE[x2.dtype]
    p.w_dtype = _lib.DTYPE_CODE[weight.dtype]
    p.width = weight.shape[1]
    p.activation, p.residual_mode, p.round_mode = act, res, rnd
    p.state_len = conv_state.shape[2]
    p.batch, p.channels = x2.shape
    p.x = x2.data_ptr()
    p.x_stride_b, p.x_stride_c = x2.stride()
    p.out = out2.data_ptr()
    p.out_stride_b, p.out_stride_c = out2.stride()
    p.conv_state = conv_state.data_ptr()
    p.state_stride_b, p.state_stride_c, p.state_stride_s = conv_state.stride()
    p.weight = weight.data_ptr()
    p.w_stride_c, p.w_stride_k = weight.stride()
    p.bias = bias.data_ptr() if bias is not None else None
    if token_mask is not None:
        p.token_mask = token_mask.data_ptr()
        p.mask_dtype = _lib.MASK_CODE[token_mask.dtype]
        p.mask_stride_b = token_mask.stride(0)
    return p


def causal_conv1d_update(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    activation: Optional[str] = None,
    cache_seqlens: Optional[torch.Tensor] = None,
    conv_state_indices: Optional[torch.Tensor] = None,
    *,
    token_mask: Optional[torch.Tensor] = None,
    residual: Union[bool, str] = False,
    rounding: str = "fused",
) -> torch.Tensor:
    """One decode step: ``x`` (batch, dim) or (batch, dim, 1); ``conv_state``
    (batch, dim, state_len >= W-1) is updated IN PLACE (shifted left by one,
    the token appended), so the caller's tensor object keeps holding the state
    (``model/model.py:305-313`` relies on that).

    ``out = act(bias + sum_{k<W-1} w[k]*state[S-(W-1)+k] + w[W-1]*x)``.

    cache_seqlens       (batch,) int32: upstream's circular-buffer mode.  ``conv_state`` is not
                shifted; the token is written to slot ``cache_seqlens % state_len`` and the W-1
                slots before it (cyclically) are the history.
    conv_state_indices  (batch,) int32: batch entry b uses row ``conv_state_indices[b]`` of
                ``conv_state`` (a pool of any number of rows).  An entry whose index is negative
                or not below the pool's size is skipped (upstream's padding slots): no state row
                is touched and its output row is zero.
    token_mask  (batch,) multiplies the token before everything else
                (``model/model.py:277-282``).
    residual    False | True ('masked': adds the masked token,
                ``model/model.py:313``) | 'unmasked' (``model/model.py:370``).
    rounding    'fused' | 'eager' (the rounding points of
                ``model/model.py:385-396``).
    """
    # A serving loop makes this call 72 times per generated token with the same shapes, strides, types and flags:
    # such a call, once it has passed every check below, is recognised by that signature and launched from a
    # prepared argument block with only the five addresses filled in.
    if cache_seqlens is None and conv_state_indices is None and not (
            torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad or conv_state.requires_grad
                                         or (bias is not None and bias.requires_grad)
                                         or (token_mask is not None and token_mask.requires_grad))):
        key = (x.shape, x.stride(), x.dtype, x.device, conv_state.shape, conv_state.stride(), conv_state.dtype,
               conv_state.device, weight.shape, weight.stride(), weight.dtype, weight.device,
               None if bias is None else (bias.shape, bias.stride(), bias.dtype, bias.device),
               None if token_mask is None else (token_mask.shape, token_mask.stride(), token_mask.dtype, token_mask.device),
               activation, residual, rounding)
        known = _known_updates()
        p = known.get(key)
        if p is not None and not torch.compiler.is_compiling():
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
            p.x, p.out, p.conv_state, p.weight = x.data_ptr(), out.data_ptr(), conv_state.data_ptr(), weight.data_ptr()
            if bias is not None:
                p.bias = bias.data_ptr()
            if token_mask is not None:
                p.token_mask = token_mask.data_ptr()
            rc = _call(_lib.lib().canon_conv1d_update, x.device, ctypes.byref(p))
            if rc:
                _lib.check(rc, "causal_conv1d_update")
            return out
    else:
        key = None
    act = _activation_flag(activation)
    res = _residual_mode(residual)
    rnd = _round_mode(rounding)
    squeeze_back = False
    if x.dim() == 3:
        if x.shape[2] != 1:
            raise NotImplementedError("causal_conv1d_update handles one token per call (seqlen 1)")
        x2 = x[:, :, 0]
        squeeze_back = True
    elif x.dim() == 2:
        x2 = x
    else:
        raise ValueError(f"Expected 2D input tensor (batch, dim), got {x.dim()}D")
    if x.dtype not in _lib.DTYPE_CODE:
        raise ValueError(f"Unsupported input dtype {x.dtype}; expected float32, bfloat16 or float16")
    if conv_state.dim() != 3:
        raise ValueError(f"Expected 3D conv_state tensor (batch, dim, state_len), got {conv_state.dim()}D")
    batch, dim = x2.shape
    if conv_state_indices is None and tuple(conv_state.shape[:2]) != (batch, dim):
        raise ValueError(
            f"Input shape {tuple(x2.shape)} doesn't match conv_state batch/dim {tuple(conv_state.shape[:2])}")
    if conv_state_indices is not None and conv_state.shape[1] != dim:
        raise ValueError(f"Input dim {dim} doesn't match conv_state dim {conv_state.shape[1]}")
    if conv_state.dtype != x.dtype or conv_state.device != x.device:
        raise ValueError("conv_state must have the dtype and device of x")
    for name, t in (("cache_seqlens", cache_seqlens), ("conv_state_indices", conv_state_indices)):
        if t is not None and (t.dim() != 1 or t.shape[0] != batch or t.dtype != torch.int32 or t.device != x.device
                              or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous int32 tensor of shape (batch,) = ({batch},) on the device of x")
    _check_shapes(dim, weight, bias)
    _require_gpu(x, "Input tensor")
    _check_devices(weight, bias, x.device)
    if conv_state.shape[2] < weight.shape[1] - 1:
        raise ValueError(f"conv_state length {conv_state.shape[2]} is shorter than width-1 = {weight.shape[1] - 1}")
    wants_grad = _wants_grad(x, weight, bias, conv_state)
    bias = _prep_bias(weight, bias)
    if token_mask is not None:
        if token_mask.dim() != 1 or token_mask.shape[0] != batch:
            raise ValueError(f"token_mask shape {tuple(token_mask.shape)} does not match (batch,) = ({batch},)")
        if token_mask.dtype not in _lib.MASK_CODE or token_mask.device != x.device:
            raise ValueError("token_mask must be a bool/int/float tensor on the device of x")

    if wants_grad and torch.compiler.is_compiling():
        # a traced graph with gradients: the step as a function (token, state) -> (output, new state) with its
        # backward registered, and the caller's state tensor overwritten by an ordinary copy the tracer understands
        # (the operator keeps its state argument for the backward, so it is handed a copy that the write below does
        # not touch)
        out, new_state = torch.ops.canon_conv1d.update_step(x2, conv_state.clone(), weight, bias, token_mask,
                                                            cache_seqlens, conv_state_indices, act, res, rnd)
        conv_state.copy_(new_state)
    elif wants_grad:
        out, _ = _CanonUpdateFn.apply(x2, conv_state, weight, bias, token_mask, act, res, cache_seqlens, conv_state_indices,
                                      rnd)
    elif torch.compiler.is_compiling():
        out = torch.ops.canon_conv1d.update(x2, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices,
                                            act, res, rnd)
    else:
        out = _launch_update(x2, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd)
        if (key is not None and not squeeze_back and out.numel()
                and (bias is None or (bias.dtype == weight.dtype and bias.is_contiguous()))):
            # the call went through: remember its signature with an argument block whose sizes, strides and flags are set
            _remember_update(key, _fill_update(x2, out, conv_state, weight, bias, token_mask, act, res, rnd))
    return out.unsqueeze(-1) if squeeze_back else out


def _canon_decode_step(x: torch.Tensor, conv_state: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor],
                       attention_mask: Optional[torch.Tensor], activation: Optional[str], rounding: str) -> torch.Tensor:
    """The single-token call of ``canon.CanonLayer`` (inference): ``x`` is the layer's (batch, 1, dim) input as it
    is, ``attention_mask`` the whole-history (batch, >= 1) mask whose LAST column scales the token, the residual
    is the unmasked token; returns (batch, 1, dim).  Same kernel and same checks as ``causal_conv1d_update`` on
    ``x[:, 0]`` / ``attention_mask[:, -1]``, without building those views and the output's: a signature that
    has been through ``causal_conv1d_update`` once is launched from its prepared argument block."""
    if torch.compiler.is_compiling():
        token_mask = attention_mask[:, -1] if attention_mask is not None else None
        return causal_conv1d_update(x[:, 0], conv_state, taps, bias, activation=activation, token_mask=token_mask,
                                    residual="unmasked", rounding=rounding).unsqueeze(1)
    key = (x.shape, x.stride(), x.dtype, x.device, conv_state.shape, conv_state.stride(), conv_state.dtype,
           conv_state.device, taps.shape, taps.stride(), taps.dtype, taps.device,
           None if bias is None else (bias.shape, bias.stride(), bias.dtype, bias.device),
           None if attention_mask is None else (attention_mask.dim(), attention_mask.shape[0], attention_mask.stride(1),
                                                attention_mask.dtype, attention_mask.device),
           activation, rounding)
    known = _known_updates()
    p = known.get(key)
    if p is None:
        token_mask = attention_mask[:, -1] if attention_mask is not None else None
        y = causal_conv1d_update(x[:, 0], conv_state, taps, bias, activation=activation, token_mask=token_mask,
                                 residual="unmasked", rounding=rounding)
        if y.numel() and (bias is None or (bias.dtype == taps.dtype and bias.is_contiguous())):
            # x[:, 0] and a contiguous (batch, dim) output: the strides of every later call with this signature
            _remember_update(key, _fill_update(x[:, 0], y, conv_state, taps, bias, token_mask, _activation_flag(activation),
                                               _residual_mode("unmasked"), _round_mode(rounding)))
        return y.unsqueeze(1)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    p.x, p.out, p.conv_state, p.weight = x.data_ptr(), out.data_ptr(), conv_state.data_ptr(), taps.data_ptr()
    if bias is not None:
        p.bias = bias.data_ptr()
    if attention_mask is not None:
        p.token_mask = attention_mask.data_ptr() + (attention_mask.shape[1] - 1) * attention_mask.stride(1) * attention_mask.element_size()
        p.mask_stride_b = attention_mask.stride(0)
    rc = _call(_lib.lib().canon_conv1d_update, x.device, ctypes.byref(p))
    if rc:
        _lib.check(rc, "causal_conv1d_update")
    return out


# signature of a checked decode call -> its prepared argument block; per thread, because the block is written to
_KNOWN_UPDATES_MAX = 256
_update_tls = threading.local()


def _known_updates() -> dict:
    try:
        return _update_tls.known
    except AttributeError:
        _update_tls.known = {}
        return _update_tls.known


def _remember_update(key, block) -> None:
    """Keep at most _KNOWN_UPDATES_MAX signatures per thread: the oldest one makes room (a model has a handful of
    distinct decode calls; a program that keeps producing new ones must not lose the fast path for good)."""
    known = _known_updates()
    if len(known) >= _KNOWN_UPDATES_MAX:
        known.pop(next(iter(known)))
    known[key] = block


def _launch_update(x2, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd):
    # entries of a state pool whose index lies outside the pool are skipped by the kernel: their output rows are zeros
    alloc = torch.empty if conv_state_indices is None else torch.zeros
    out = alloc(tuple(x2.shape), dtype=x2.dtype, device=x2.device)
    if out.numel():
        p = _fill_update(x2, out, conv_state, weight, bias, token_mask, act, res, rnd)
        if cache_seqlens is not None:
            p.cache_seqlens = cache_seqlens.data_ptr()
        if conv_state_indices is not None:
            p.conv_state_indices = conv_state_indices.data_ptr()
            p.state_rows = conv_state.shape[0]
        rc = _call(_lib.lib().canon_conv1d_update, x2.device, ctypes.byref(p))
        _lib.check(rc, "causal_conv1d_update")
    return out


class _CanonUpdateFn(torch.autograd.Function):
    """Autograd node of one decode step.  The forward overwrites ``conv_state``, so a copy of the
    state as it was is kept for the backward (as ShortConvUpdateMPSFunction does,
    causal_conv1d_mps/autograd.py:452-453); ``conv_state`` is declared modified in place and
    returned, so a gradient that arrives through the updated state (the next decode step reading
    it) flows back into this step's token and into the state before it.  The ring-buffer mode
    (``cache_seqlens``, the mode of the reference's own update autograd, causal_conv1d_mps/autograd.py:341-498) and
    the state-pool mode (``conv_state_indices``) differentiate the same way; in pool mode ``conv_state`` is the
    whole pool, and rows that no batch entry names pass their gradient through unchanged.  With
    ``rounding='eager'`` the forward rounds where the eager module does and the backward is that of the unrounded
    step, as for the prefill."""

    @staticmethod
    def forward(ctx, x2, conv_state, weight, bias, token_mask, act, res, cache_seqlens=None, conv_state_indices=None,
                rnd=0):
        before = conv_state.detach().clone()
        out = _launch_update(x2, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd)
        ctx.mark_dirty(conv_state)
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(x2, before, weight, bias, token_mask, cache_seqlens, conv_state_indices)
        ctx.flags = (act, res)
        return out, conv_state

    @staticmethod
    def backward(ctx, dout, dstate_out):
        x2, before, weight, bias, token_mask, cache_seqlens, conv_state_indices = ctx.saved_tensors
        act, res = ctx.flags
        if dout is None:
            dout = torch.zeros_like(x2)
        want_state = ctx.needs_input_grad[1]
        want_params = ctx.needs_input_grad[2] or (bias is not None and ctx.needs_input_grad[3])
        dx, dstate, dweight, dbias = _launch_update_bwd(x2, before, weight, bias, token_mask, dout, dstate_out, act, res,
                                                        want_state, want_params, cache_seqlens, conv_state_indices)
        return (dx, dstate, dweight.to(weight.dtype) if dweight is not None else None,
                dbias.to(bias.dtype) if dbias is not None else None, None, None, None, None, None, None)


def _launch_update_bwd(x2, before, weight, bias, token_mask, dout, dstate_out, act, res, want_state=True,
                       want_params=True, cache_seqlens=None, conv_state_indices=None):
    """One launch (+ the fixed-order reduction over the batch): (dx, dstate | None, dweight | None, dbias | None),
    the parameter gradients in fp32.  With ``conv_state_indices`` the state tensors are pools: the kernel writes the
    rows the batch entries name, the others carry ``dstate_out`` through."""
    if dout.dtype != x2.dtype:
        dout = dout.to(x2.dtype)
    if dstate_out is not None and dstate_out.dtype != x2.dtype:
        dstate_out = dstate_out.to(x2.dtype)
    batch, channels = x2.shape
    width = weight.shape[1]
    dev = x2.device
    dx = torch.empty(batch, channels, dtype=x2.dtype, device=dev)
    if not want_state:
        dstate = None
    elif conv_state_indices is None:
        dstate = torch.empty(tuple(before.shape), dtype=x2.dtype, device=dev)
    elif dstate_out is not None:
        dstate = dstate_out.clone(memory_format=torch.contiguous_format)
    else:
        dstate = torch.zeros(tuple(before.shape), dtype=x2.dtype, device=dev)
    dweight = torch.empty(channels, width, dtype=torch.float32, device=dev) if want_params else None
    dbias = torch.empty(channels, dtype=torch.float32, device=dev) if want_params and bias is not None else None
    p = _lib.UpdateBwdParams()
    p.struct_size = ctypes.sizeof(_lib.UpdateBwdParams)
    p.x_dtype = _lib.DTYPE_CODE[x2.dtype]
    p.w_dtype = _lib.DTYPE_CODE[weight.dtype]
    p.width = width
    p.activation, p.residual_mode = act, res
    p.state_len = before.shape[2]
    p.batch, p.channels = batch, channels
    p.x = x2.data_ptr()
    p.x_stride_b, p.x_stride_c = x2.stride()
    p.conv_state = before.data_ptr()
    p.state_stride_b, p.state_stride_c, p.state_stride_s = before.stride()
    p.weight = weight.data_ptr()
    p.w_stride_c, p.w_stride_k = weight.stride()
    p.bias = bias.data_ptr() if bias is not None else None
    if token_mask is not None:
        p.token_mask = token_mask.data_ptr()
        p.mask_dtype = _lib.MASK_CODE[token_mask.dtype]
        p.mask_stride_b = token_mask.stride(0)
    p.dout = dout.data_ptr()
    p.dout_stride_b, p.dout_stride_c = dout.stride()
    if dstate_out is not None:
        p.dstate_out = dstate_out.data_ptr()
        p.dstate_out_stride_b, p.dstate_out_stride_c, p.dstate_out_stride_s = dstate_out.stride()
    p.dx = dx.data_ptr()
    p.dx_stride_b, p.dx_stride_c = dx.stride()
    if dstate is not None:
        p.dstate = dstate.data_ptr()
        p.dstate_stride_b, p.dstate_stride_c, p.dstate_stride_s = dstate.stride()
    p.dweight = dweight.data_ptr() if dweight is not None else None
    p.dbias = dbias.data_ptr() if dbias is not None else None
    if cache_seqlens is not None:
        p.cache_seqlens = cache_seqlens.data_ptr()
    if conv_state_indices is not None:
        p.conv_state_indices = conv_state_indices.data_ptr()
        p.state_rows = before.shape[0]
    L = _lib.lib()
    nbytes = L.canon_conv1d_update_bwd_workspace_bytes(ctypes.byref(p))
    if nbytes < 0:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "causal_conv1d_update backward")
    workspace = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=dev)
    p.workspace = workspace.data_ptr()
    p.workspace_bytes = workspace.numel()
    rc = _call(L.canon_conv1d_update_bwd, dev, ctypes.byref(p))
    _lib.check(rc, "causal_conv1d_update backward")
    return dx, dstate, dweight, dbias


# ---------------------------------------------------------------------------
# Channel ranges given as separate tensors (Canon-B: q, k, v; Canon-D: gate, up)
# ---------------------------------------------------------------------------
def _part_array(xs, outs):
    arr = (_lib.Part * len(xs))()
    for i, (x, o) in enumerate(zip(xs, outs)):
        p = arr[i]
        p.x = x.data_ptr()
        p.out = o.data_ptr()
        p.channels = x.shape[1]
        if x.dim() == 3:
            p.x_stride_b, p.x_stride_c, p.x_stride_l = x.stride()
            p.out_stride_b, p.out_stride_c, p.out_stride_l = o.stride()
        else:
            p.x_stride_b, p.x_stride_c = x.stride()
            p.out_stride_b, p.out_stride_c = o.stride()
    return arr


def _check_parts(xs, ndim: int, what: str):
    xs = list(xs)
    if not 1 <= len(xs) <= _lib.MAX_PARTS:
        raise ValueError(f"{what}: expected 1..{_lib.MAX_PARTS} parts, got {len(xs)}")
    first = xs[0]
    for x in xs:
        if x.dim() != ndim:
            raise ValueError(f"{what}: expected {ndim}D parts, got {x.dim()}D")
        if x.dtype != first.dtype or x.device != first.device:
            raise ValueError(f"{what}: all parts must have one dtype and device")
        if x.shape[0] != first.shape[0] or tuple(x.shape[2:]) != tuple(first.shape[2:]):
            raise ValueError(f"{what}: parts differ in batch or seqlen: {tuple(x.shape)} vs {tuple(first.shape)}")
    return xs


def causal_conv1d_fn_parts(
    xs,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    initial_states: Optional[torch.Tensor] = None,
    return_final_states: bool = False,
    final_states_out: Optional[torch.Tensor] = None,
    activation: Optional[str] = None,
    attention_mask: Optional[torch.Tensor] = None,
    residual: Union[bool, str] = False,
    rounding: str = "fused",
):
    """``causal_conv1d_fn`` on ``torch.cat(xs, dim=1)`` without making the cat.

    ``xs``: 1..4 tensors (batch, dim_i, seqlen); ``weight`` (sum dim_i, W), ``bias`` and the
    states cover all channels in the order of the parts.  Returns the tuple of outputs, one per
    part with that part's strides (and the final states when asked for).  This is what Canon-B /
    Canon-D need (``model/model.py:772-789, 962-971`` concatenate q/k/v and gate/up only to call
    the conv once); results equal the call on the concatenation bit for bit.  Differentiable:
    the backward runs once per part on that part's rows of the weights (no cat there either).
    """
    act = _activation_flag(activation)
    res = _residual_mode(residual)
    rnd = _round_mode(rounding)
    xs = _check_parts(xs, 3, "causal_conv1d_fn_parts")
    batch, seqlen = xs[0].shape[0], xs[0].shape[2]
    dims = [x.shape[1] for x in xs]
    dim = sum(dims)
    bias, attention_mask, final_states = _check_fwd_args(
        xs[0], (batch, dim, seqlen), weight, bias, attention_mask, initial_states, return_final_states,
        final_states_out)
    if batch * dim * seqlen == 0 and final_states is not None and final_states.numel():
        raise ValueError("cannot produce final states from an empty input")

    wants_grad = _wants_grad(*xs, weight, bias, initial_states)
    if wants_grad and initial_states is not None and torch.compiler.is_compiling():
        raise NotImplementedError("causal_conv1d_fn_parts (gfx950): gradients through a call with initial_states are "
                                  "implemented outside torch.compile")
    if torch.compiler.is_compiling():
        *outs, fin = torch.ops.canon_conv1d.fwd_parts(xs, weight, bias, attention_mask, initial_states,
                                                      final_states.shape[2] if final_states is not None else 0,
                                                      act, res, rnd)
        outs = tuple(outs)
        if final_states is not None:
            final_states.copy_(fin)
    elif wants_grad:
        result = _CanonConvPartsFn.apply(weight, bias, attention_mask, final_states, act, res, rnd, initial_states, *xs)
        outs = tuple(result[:len(xs)])
    else:
        outs = _launch_fwd_parts(xs, weight, bias, attention_mask, initial_states, final_states, act, res, rnd)
    return (outs, final_states) if final_states is not None else outs


def _launch_fwd_parts(xs, weight, bias, mask, initial_states, final_states, act, res, rnd):
    outs = tuple(torch.empty_like(x) for x in xs)
    dim = sum(x.shape[1] for x in xs)
    if xs[0].shape[0] * dim * xs[0].shape[2]:
        p = _fill_fwd(xs[0], outs[0], weight, bias, mask, initial_states, final_states, act, res, rnd)
        p.channels = dim
        p.x = p.out = None
        arr = _part_array(xs, outs)
        rc = _call(_lib.lib().canon_conv1d_fwd_parts, xs[0].device, ctypes.byref(p), arr, len(xs))
        _lib.check(rc, "causal_conv1d_fn_parts")
    return outs


class _CanonConvPartsFn(torch.autograd.Function):
    """Autograd node of the multi-part prefill: one forward launch over all parts; the backward
    runs the fused backward once per part, on that part's rows of weight / bias and that part's channels of the
    states, so neither direction concatenates anything.  As in the single-tensor node the captured final state is
    differentiable (a gradient arriving through it flows back into the inputs) and so is the initial state."""

    @staticmethod
    def forward(ctx, weight, bias, mask, final_states, act, res, rnd, initial_states, *xs):
        outs = _launch_fwd_parts(xs, weight, bias, mask, initial_states, final_states, act, res, rnd)
        # (a copy of the small initial state: callers keep it in a cache tensor they overwrite right after the call)
        ctx.save_for_backward(weight, bias, mask, initial_states.detach().clone() if initial_states is not None else None,
                              *xs)
        ctx.flags = (act, res, final_states is not None)
        ctx.set_materialize_grads(False)
        if final_states is not None:
            ctx.mark_dirty(final_states)
            return (*outs, final_states)
        return outs

    @staticmethod
    def backward(ctx, *grads):
        weight, bias, mask, initial_states, *xs = ctx.saved_tensors
        act, res, has_final = ctx.flags
        douts = grads[:len(xs)]
        dfinal = grads[len(xs)] if has_final else None
        channels, width = weight.shape
        dev = xs[0].device
        dweight = torch.empty(channels, width, dtype=torch.float32, device=dev)
        dbias = torch.empty(channels, dtype=torch.float32, device=dev) if bias is not None else None
        dinit = None
        if initial_states is not None and ctx.needs_input_grad[7]:
            dinit = torch.empty_like(initial_states)
        dxs, c0 = [], 0
        for x, dout in zip(xs, douts):
            c1 = c0 + x.shape[1]
            if dout is None:
                dout = torch.zeros_like(x)
            dxs.append(_launch_bwd(x, dout, weight[c0:c1], bias[c0:c1] if bias is not None else None, mask,
                                   dweight[c0:c1], dbias[c0:c1] if dbias is not None else None, act, res, None,
                                   initial_states[:, c0:c1] if initial_states is not None else None,
                                   dinit[:, c0:c1] if dinit is not None else None,
                                   dfinal[:, c0:c1] if dfinal is not None else None))
            c0 = c1
        return (dweight.to(weight.dtype), dbias.to(bias.dtype) if bias is not None else None,
                None, None, None, None, None, dinit, *dxs)


def causal_conv1d_update_parts(
    xs,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    activation: Optional[str] = None,
    *,
    token_mask: Optional[torch.Tensor] = None,
    residual: Union[bool, str] = False,
    rounding: str = "fused",
):
    """``causal_conv1d_update`` on ``torch.cat(xs, dim=1)`` without making the cat: ``xs`` are 1..4
    tokens (batch, dim_i); ``conv_state`` (batch, sum dim_i, state_len) is the one state of the layer,
    updated in place.  Returns the tuple of outputs."""
    act = _activation_flag(activation)
    res = _residual_mode(residual)
    rnd = _round_mode(rounding)
    xs = _check_parts(xs, 2, "causal_conv1d_update_parts")
    x0 = xs[0]
    if x0.dtype not in _lib.DTYPE_CODE:
        raise ValueError(f"Unsupported input dtype {x0.dtype}; expected float32, bfloat16 or float16")
    batch = x0.shape[0]
    dims = [x.shape[1] for x in xs]
    dim = sum(dims)
    if conv_state.dim() != 3:
        raise ValueError(f"Expected 3D conv_state tensor (batch, dim, state_len), got {conv_state.dim()}D")
    if tuple(conv_state.shape[:2]) != (batch, dim):
        raise ValueError(
            f"Input shape {(batch, dim)} doesn't match conv_state batch/dim {tuple(conv_state.shape[:2])}")
    if conv_state.dtype != x0.dtype or conv_state.device != x0.device:
        raise ValueError("conv_state must have the dtype and device of x")
    _check_shapes(dim, weight, bias)
    _require_gpu(x0, "Input tensor")
    _check_devices(weight, bias, x0.device)
    if conv_state.shape[2] < weight.shape[1] - 1:
        raise ValueError(f"conv_state length {conv_state.shape[2]} is shorter than width-1 = {weight.shape[1] - 1}")
    wants_grad = _wants_grad(*xs, weight, bias, conv_state)
    if wants_grad and torch.compiler.is_compiling():
        raise NotImplementedError(
            "causal_conv1d_update_parts (gfx950): the backward of the multi-part decode step is implemented outside "
            "torch.compile; call under torch.no_grad() or detach the inputs")
    bias = _prep_bias(weight, bias)
    if token_mask is not None:
        if token_mask.dim() != 1 or token_mask.shape[0] != batch:
            raise ValueError(f"token_mask shape {tuple(token_mask.shape)} does not match (batch,) = ({batch},)")
        if token_mask.dtype not in _lib.MASK_CODE or token_mask.device != x0.device:
            raise ValueError("token_mask must be a bool/int/float tensor on the device of x")
    if torch.compiler.is_compiling():
        return tuple(torch.ops.canon_conv1d.update_parts(xs, conv_state, weight, bias, token_mask, act, res, rnd))
    if wants_grad:
        return tuple(_CanonUpdatePartsFn.apply(conv_state, weight, bias, token_mask, act, res, rnd, *xs)[:len(xs)])
    return _launch_update_parts(xs, conv_state, weight, bias, token_mask, act, res, rnd)


class _CanonUpdatePartsFn(torch.autograd.Function):
    """Autograd node of the multi-part decode step: one forward launch over all parts; the backward runs the decode
    step's backward once per part, on that part's channels of the saved state and of the state gradients and on its
    rows of weight / bias.  The state is modified in place and differentiable, as in ``_CanonUpdateFn``."""

    @staticmethod
    def forward(ctx, conv_state, weight, bias, token_mask, act, res, rnd, *xs):
        before = conv_state.detach().clone()
        outs = _launch_update_parts(xs, conv_state, weight, bias, token_mask, act, res, rnd)
        ctx.mark_dirty(conv_state)
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(before, weight, bias, token_mask, *xs)
        ctx.flags = (act, res)
        return (*outs, conv_state)

    @staticmethod
    def backward(ctx, *grads):
        before, weight, bias, token_mask, *xs = ctx.saved_tensors
        act, res = ctx.flags
        douts, dstate_out = grads[:len(xs)], grads[len(xs)]
        want_state = ctx.needs_input_grad[0]
        want_params = ctx.needs_input_grad[1] or (bias is not None and ctx.needs_input_grad[2])
        dstate = torch.empty_like(before) if want_state else None
        dws, dbs, dxs, c0 = [], [], [], 0
        for x, dout in zip(xs, douts):
            c1 = c0 + x.shape[1]
            if dout is None:
                dout = torch.zeros_like(x)
            dx, ds, dw, db = _launch_update_bwd(x, before[:, c0:c1], weight[c0:c1], bias[c0:c1] if bias is not None else None,
                                                token_mask, dout, dstate_out[:, c0:c1] if dstate_out is not None else None,
                                                act, res, want_state, want_params)
            if want_state:
                dstate[:, c0:c1] = ds
            dxs.append(dx)
            dws.append(dw)
            dbs.append(db)
            c0 = c1
        dweight = torch.cat(dws, dim=0).to(weight.dtype) if want_params else None
        dbias = torch.cat(dbs, dim=0).to(bias.dtype) if want_params and bias is not None else None
        return (dstate, dweight, dbias, None, None, None, None, *dxs)


def _launch_update_parts(xs, conv_state, weight, bias, token_mask, act, res, rnd):
    outs = tuple(torch.empty_like(x, memory_format=torch.contiguous_format) for x in xs)
    dim = sum(x.shape[1] for x in xs)
    if xs[0].shape[0] * dim:
        p = _fill_update(xs[0], outs[0], conv_state, weight, bias, token_mask, act, res, rnd)
        p.channels = dim
        p.x = p.out = None
        arr = _part_array(xs, outs)
        rc = _call(_lib.lib().canon_conv1d_update_parts, xs[0].device, ctypes.byref(p), arr, len(xs))
        _lib.check(rc, "causal_conv1d_update_parts")
    return outs


# ---------------------------------------------------------------------------
# The launches as torch operators, for traced graphs (torch.compile).  Eager calls do not go through them
# (operator dispatch costs more than the launch); a function being traced does, because ctypes calls
# cannot be traced and the reference compiles its model (trainer/train_pretrain.py:39, train_full_sft.py:54,
# eval_model.py:157 with fullgraph=True).  Each has a shape-only twin for tracing, and the prefill has its
# backward registered, so compiled training graphs differentiate through it.
# ---------------------------------------------------------------------------
def _new_state(x, channels: int, state_len: int) -> Optional[torch.Tensor]:
    return torch.empty(x.shape[0], channels, state_len, dtype=x.dtype, device=x.device) if state_len > 0 else None


@torch.library.custom_op("canon_conv1d::fwd", mutates_args=(), device_types="cuda")
def _op_fwd(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], mask: Optional[torch.Tensor],
            initial_states: Optional[torch.Tensor], seq_idx: Optional[torch.Tensor], state_len: int,
            act: int, res: int, rnd: int) -> Tuple[torch.Tensor, torch.Tensor]:
    # functional (an operator with an autograd formula must be): the final states are a second result,
    # of zero length when none are wanted
    fin = _new_state(x, x.shape[1], state_len)
    out = _launch_fwd(x, weight, bias, mask, initial_states, fin, act, res, rnd, seq_idx)
    return out, fin if fin is not None else x.new_empty((x.shape[0], x.shape[1], 0))


@_op_fwd.register_fake
def _(x, weight, bias, mask, initial_states, seq_idx, state_len, act, res, rnd):
    return torch.empty_like(x), x.new_empty((x.shape[0], x.shape[1], state_len))


@torch.library.custom_op("canon_conv1d::bwd", mutates_args=(), device_types="cuda")
def _op_bwd(x: torch.Tensor, dout: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
            mask: Optional[torch.Tensor], seq_idx: Optional[torch.Tensor], initial_states: Optional[torch.Tensor],
            dfinal: Optional[torch.Tensor], act: int, res: int
            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    channels, width = weight.shape
    dweight = torch.empty(channels, width, dtype=torch.float32, device=x.device)
    dbias = torch.empty(channels if bias is not None else 0, dtype=torch.float32, device=x.device)
    dinit = torch.empty_like(initial_states) if initial_states is not None else x.new_empty((x.shape[0], channels, 0))
    dx = _launch_bwd(x, dout, weight, bias, mask, dweight, dbias if bias is not None else None, act, res, seq_idx,
                     initial_states, dinit if initial_states is not None else None, dfinal)
    return dx, dweight.to(weight.dtype), dbias.to(bias.dtype if bias is not None else weight.dtype), dinit


@_op_bwd.register_fake
def _(x, dout, weight, bias, mask, seq_idx, initial_states, dfinal, act, res):
    return (torch.empty_like(x), torch.empty_like(weight, memory_format=torch.contiguous_format),
            weight.new_empty((weight.shape[0] if bias is not None else 0,),
                             dtype=bias.dtype if bias is not None else weight.dtype),
            torch.empty_like(initial_states) if initial_states is not None
            else x.new_empty((x.shape[0], weight.shape[0], 0)))


def _op_fwd_setup(ctx, inputs, output):
    x, weight, bias, mask, initial, seq_idx, state_len, act, res, _rnd = inputs
    ctx.save_for_backward(x, weight, bias, mask, seq_idx, initial)
    ctx.flags = (act, res, bias is not None, state_len)


def _op_fwd_backward(ctx, dout, dstate):
    x, weight, bias, mask, seq_idx, initial = ctx.saved_tensors
    act, res, has_bias, state_len = ctx.flags
    # the captured state is a result of the operator: whatever gradient reaches it is passed on (a traced graph
    # cannot tell an unused state from one whose gradient happens to be zero)
    dfinal = dstate if state_len > 0 else None
    dx, dweight, dbias, dinit = torch.ops.canon_conv1d.bwd(x, dout, weight, bias, mask, seq_idx, initial, dfinal,
                                                           act, res)
    return (dx, dweight, (dbias if has_bias else None), None, (dinit if initial is not None else None),
            None, None, None, None, None)


_op_fwd.register_autograd(_op_fwd_backward, setup_context=_op_fwd_setup)


@torch.library.custom_op("canon_conv1d::update", mutates_args=("conv_state",), device_types="cuda")
def _op_update(x: torch.Tensor, conv_state: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               token_mask: Optional[torch.Tensor], cache_seqlens: Optional[torch.Tensor],
               conv_state_indices: Optional[torch.Tensor], act: int, res: int, rnd: int) -> torch.Tensor:
    return _launch_update(x, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd)


@_op_update.register_fake
def _(x, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd):
    return x.new_empty(tuple(x.shape))


# The decode step as a function, for traced graphs that need its gradient: the state is not overwritten but returned
# (an operator that mutates an argument cannot carry a gradient through that argument).
@torch.library.custom_op("canon_conv1d::update_step", mutates_args=(), device_types="cuda")
def _op_update_step(x: torch.Tensor, conv_state: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                    token_mask: Optional[torch.Tensor], cache_seqlens: Optional[torch.Tensor],
                    conv_state_indices: Optional[torch.Tensor], act: int, res: int, rnd: int
                    ) -> Tuple[torch.Tensor, torch.Tensor]:
    new_state = conv_state.clone(memory_format=torch.contiguous_format)
    out = _launch_update(x, new_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd)
    return out, new_state


@_op_update_step.register_fake
def _(x, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, rnd):
    return x.new_empty(tuple(x.shape)), torch.empty_like(conv_state, memory_format=torch.contiguous_format)


@torch.library.custom_op("canon_conv1d::update_bwd", mutates_args=(), device_types="cuda")
def _op_update_bwd(x: torch.Tensor, before: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                   token_mask: Optional[torch.Tensor], dout: torch.Tensor, dstate_out: torch.Tensor,
                   cache_seqlens: Optional[torch.Tensor], conv_state_indices: Optional[torch.Tensor], act: int, res: int
                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    dx, dstate, dweight, dbias = _launch_update_bwd(x, before, weight, bias, token_mask, dout, dstate_out, act, res,
                                                    True, True, cache_seqlens, conv_state_indices)
    return (dx, dstate, dweight.to(weight.dtype),
            dbias.to(bias.dtype) if dbias is not None else weight.new_empty((0,)))


@_op_update_bwd.register_fake
def _(x, before, weight, bias, token_mask, dout, dstate_out, cache_seqlens, conv_state_indices, act, res):
    return (x.new_empty(tuple(x.shape)), torch.empty_like(before, memory_format=torch.contiguous_format),
            torch.empty_like(weight, memory_format=torch.contiguous_format),
            weight.new_empty((weight.shape[0],), dtype=bias.dtype) if bias is not None else weight.new_empty((0,)))


def _op_update_step_setup(ctx, inputs, output):
    x, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices, act, res, _rnd = inputs
    ctx.save_for_backward(x, conv_state, weight, bias, token_mask, cache_seqlens, conv_state_indices)
    ctx.flags = (act, res, bias is not None)


def _op_update_step_backward(ctx, dout, dnew_state):
    x, before, weight, bias, token_mask, cache_seqlens, conv_state_indices = ctx.saved_tensors
    act, res, has_bias = ctx.flags
    dx, dstate, dweight, dbias = torch.ops.canon_conv1d.update_bwd(
        x, before, weight, bias, token_mask, dout.contiguous(), dnew_state, cache_seqlens, conv_state_indices, act, res)
    return dx, dstate, dweight, (dbias if has_bias else None), None, None, None, None, None, None


_op_update_step.register_autograd(_op_update_step_backward, setup_context=_op_update_step_setup)


@torch.library.custom_op("canon_conv1d::fwd_parts", mutates_args=(), device_types="cuda")
def _op_fwd_parts(xs: List[torch.Tensor], weight: torch.Tensor, bias: Optional[torch.Tensor],
                  mask: Optional[torch.Tensor], initial_states: Optional[torch.Tensor],
                  state_len: int, act: int, res: int, rnd: int) -> List[torch.Tensor]:
    # one output per part, then the final states (zero length when none are wanted)
    channels = sum(x.shape[1] for x in xs)
    fin = _new_state(xs[0], channels, state_len)
    outs = list(_launch_fwd_parts(xs, weight, bias, mask, initial_states, fin, act, res, rnd))
    return outs + [fin if fin is not None else xs[0].new_empty((xs[0].shape[0], channels, 0))]


@_op_fwd_parts.register_fake
def _(xs, weight, bias, mask, initial_states, state_len, act, res, rnd):
    channels = sum(x.shape[1] for x in xs)
    return [torch.empty_like(x) for x in xs] + [xs[0].new_empty((xs[0].shape[0], channels, state_len))]


def _op_fwd_parts_setup(ctx, inputs, output):
    xs, weight, bias, mask, _initial, _state_len, act, res, _rnd = inputs
    ctx.save_for_backward(weight, bias, mask, *xs)
    ctx.flags = (act, res, bias is not None)


def _op_fwd_parts_backward(ctx, grads):
    # one fused backward per part, on that part's rows of the weights (no cat here either)
    weight, bias, mask, *xs = ctx.saved_tensors
    act, res, has_bias = ctx.flags
    dxs, dws, dbs, c0 = [], [], [], 0
    for x, dout in zip(xs, grads):
        c1 = c0 + x.shape[1]
        dx, dw, db, _ = torch.ops.canon_conv1d.bwd(x, dout, weight[c0:c1], bias[c0:c1] if has_bias else None,
                                                   mask, None, None, None, act, res)
        dxs.append(dx)
        dws.append(dw)
        dbs.append(db)
        c0 = c1
    return dxs, torch.cat(dws, dim=0), (torch.cat(dbs, dim=0) if has_bias else None), None, None, None, None, None, None


_op_fwd_parts.register_autograd(_op_fwd_parts_backward, setup_context=_op_fwd_parts_setup)


@torch.library.custom_op("canon_conv1d::update_parts", mutates_args=("conv_state",), device_types="cuda")
def _op_update_parts(xs: List[torch.Tensor], conv_state: torch.Tensor, weight: torch.Tensor,
                     bias: Optional[torch.Tensor], token_mask: Optional[torch.Tensor], act: int, res: int,
                     rnd: int) -> List[torch.Tensor]:
    return list(_launch_update_parts(xs, conv_state, weight, bias, token_mask, act, res, rnd))


@_op_update_parts.register_fake
def _(xs, conv_state, weight, bias, token_mask, act, res, rnd):
    return [torch.empty_like(x, memory_format=torch.contiguous_format) for x in xs]


# ---------------------------------------------------------------------------
# The reference's fused (batch, seqlen, dim) API, same argument meaning.
# ---------------------------------------------------------------------------
def short_conv_fused(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    attention_mask: Optional[torch.Tensor] = None,
    activation: bool = True,
    residual: bool = True,
) -> torch.Tensor:
    """``x`` (batch, seqlen, dim) -> ``(x if residual) + act(conv(x * mask) + bias)``.

    Same contract as ``causal_conv1d_mps.short_conv_fused``
    (``causal_conv1d_mps/__init__.py:154-301``, kernel
    ``causal_conv1d.metal:530-580``): the mask multiplies the conv inputs, the
    residual term is the unmasked ``x``.
    """
    if x.dim() != 3:
        raise ValueError(f"Expected 3D input tensor (batch, seqlen, dim), got {x.dim()}D")
    y = causal_conv1d_fn(
        x.transpose(1, 2), weight, bias, activation="silu" if activation else None,
        attention_mask=attention_mask, residual="unmasked" if residual else False)
    return y.transpose(1, 2)


def short_conv_update(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    cache_seqlens: Optional[torch.Tensor] = None,
    activation: bool = True,
    residual: bool = True,
) -> torch.Tensor:
    """Single-token step with the argument order of
    ``causal_conv1d_mps.short_conv_update`` (``causal_conv1d_mps/__init__.py:304-419``).

    Without ``cache_seqlens`` the state is a shift register (newest token last), the layout the
    prefill path and the eager step (``model/model.py:385-386``) use.  With it the state is a ring
    written at ``cache_seqlens % state_len``, as in the reference's Metal kernel
    (``causal_conv1d.metal:755-775``); a state filled by the prefill is right-aligned, so the
    first ring position consistent with it is ``cache_seqlens = 0 (mod state_len)``.
    """
    return causal_conv1d_update(x, conv_state, weight, bias, activation="silu" if activation else None,
                                cache_seqlens=cache_seqlens, residual="masked" if residual else False)


# ---------------------------------------------------------------------------
# introspection (lets callers and tests assert that a layout takes a fast path)
# ---------------------------------------------------------------------------
def kernel_plan_fwd(x, weight, bias=None, activation=None, attention_mask=None, residual=False,
                    rounding="fused", initial_states=None, final_states_out=None, seq_idx=None) -> str:
    """Kernel family ``causal_conv1d_fn`` would launch: 'bcl_vec', 'blc_vec', 'blc_vec_seq' or 'generic'."""
    out = torch.empty_like(x)
    p = _fill_fwd(x, out, weight, _prep_bias(weight, bias), attention_mask, initial_states, final_states_out,
                  _activation_flag(activation), _residual_mode(residual), _round_mode(rounding), seq_idx)
    name = _lib.lib().canon_conv1d_fwd_plan(ctypes.byref(p))
    if name is None:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "kernel_plan_fwd")
    return name.decode()


def kernel_plan_fwd_waves(x, weight, bias=None, activation=None, attention_mask=None, residual=False,
                          rounding="fused") -> int:
    """Waves per block of the launch ``causal_conv1d_fn`` would make (1, 4 or 8 for time-contiguous rows, else 4)."""
    out = torch.empty_like(x)
    p = _fill_fwd(x, out, weight, _prep_bias(weight, bias), attention_mask, None, None,
                  _activation_flag(activation), _residual_mode(residual), _round_mode(rounding))
    n = _lib.lib().canon_conv1d_fwd_plan_waves(ctypes.byref(p))
    if n < 0:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "kernel_plan_fwd_waves")
    return n


def prepare_device(device=None) -> None:
    """Set the library up on ``device`` (default: the current one): loads its code objects and resolves the static
    scratch buffer, so that nothing of that is left to the first launches.  Call it before capturing launches
    into a HIP graph or entering a section that must not allocate device memory."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().canon_conv1d_init(), "prepare_device")


def kernel_plan_update(x, conv_state, weight, bias=None, activation=None, residual=False, rounding="fused") -> str:
    """Kernel family ``causal_conv1d_update`` would launch: 'update_vec' or 'update_generic'."""
    out = torch.empty_like(x)
    p = _fill_update(x, out, conv_state, weight, _prep_bias(weight, bias), None,
                     _activation_flag(activation), _residual_mode(residual), _round_mode(rounding))
    name = _lib.lib().canon_conv1d_update_plan(ctypes.byref(p))
    if name is None:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "kernel_plan_update")
    return name.decode()


def kernel_plan_fwd_parts(xs, weight, bias=None, activation=None, attention_mask=None, residual=False) -> str:
    """'blc_vec_pair' (two dense tensors of one shape) or 'blc_vec_parts' if ``causal_conv1d_fn_parts`` would run
    these parts as one launch, else 'per_part'."""
    xs = list(xs)
    outs = [torch.empty_like(x) for x in xs]
    p = _fill_fwd(xs[0], outs[0], weight, _prep_bias(weight, bias), attention_mask, None, None,
                  _activation_flag(activation), _residual_mode(residual), 0)
    p.channels = sum(x.shape[1] for x in xs)
    name = _lib.lib().canon_conv1d_fwd_parts_plan(ctypes.byref(p), _part_array(xs, outs), len(xs))
    if name is None:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "kernel_plan_fwd_parts")
    return name.decode()


def kernel_plan_update_parts(xs, conv_state, weight, bias=None, activation=None, residual=False) -> str:
    """'update_vec_parts' if ``causal_conv1d_update_parts`` would run as one launch, else 'per_part'."""
    xs = list(xs)
    outs = [torch.empty_like(x) for x in xs]
    p = _fill_update(xs[0], outs[0], conv_state, weight, _prep_bias(weight, bias), None,
                     _activation_flag(activation), _residual_mode(residual), 0)
    p.channels = sum(x.shape[1] for x in xs)
    name = _lib.lib().canon_conv1d_update_parts_plan(ctypes.byref(p), _part_array(xs, outs), len(xs))
    if name is None:
        _lib.check(_lib.ERR_INVALID_ARGUMENT, "kernel_plan_update_parts")
    return name.decode()
