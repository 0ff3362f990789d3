"""ctypes binding of the C ABI declared in include/dmf_attn.h.

The library is loaded from ``dmf_amd/libdmf_attn.so`` (built in-tree by
``python -m dmf_amd.build``).  There is deliberately no fallback: a missing
library raises ``RuntimeError`` at the first call.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p, POINTER

import torch
from torch._C import _functorch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdmf_attn.so")

DMF_ATTN_F32, DMF_ATTN_BF16 = 0, 1
SUPPORTED_HEAD_DIMS = (32, 64, 72, 80, 96, 128)

# name -> (restype, argtypes): the complete exported surface of include/dmf_attn.h
_P, _I, _F = c_void_p, c_int, c_float
_S = POINTER(c_int64)
SIGNATURES = {
    "dmf_attn_version": (c_int, []),
    "dmf_attn_strerror": (c_char_p, [c_int]),
    "dmf_attn_fwd_jvp": (c_int, [_P] * 10 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_fwd": (c_int, [_P] * 5 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_bwd": (c_int, [_P] * 10 + [_S] + [_I] * 5 + [_F, _I, _P]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load (once) and return the library with argtypes/restypes set."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m dmf_amd.build` "
                "(the HIP kernels are the only implementation; there is no fallback)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {load().dmf_attn_strerror(rc).decode()} (code {rc})")


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DMF_ATTN_F32
    if t.dtype == torch.bfloat16:
        return DMF_ATTN_BF16
    raise TypeError(f"dmf_amd attention supports float32 and bfloat16, got {t.dtype}")


def _raw(t):
    """Strip functorch wrappers.  Inside a functorch transform (e.g. the ``jvp``
    staticmethod of an autograd.Function under ``torch.func.jvp``) saved tensors
    and even freshly allocated ones are wrapper tensors without storage."""
    while t is not None and _functorch.is_functorch_wrapped_tensor(t):
        t = _functorch.get_unwrapped(t)
    return t


def _empty(shape, dtype, device) -> torch.Tensor:
    return _raw(torch.empty(shape, dtype=dtype, device=device))


def _prep(t: torch.Tensor) -> torch.Tensor:
    """Kernels need unit last-dim stride and 16-byte aligned rows; views into a
    packed qkv buffer already satisfy this and are passed through untouched."""
    t = _raw(t)
    eb = t.element_size()
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * eb) % 16 == 0 for s in t.stride()[:-1])
    return t if ok else _raw(t.contiguous())


def _strides(*tensors) -> ctypes.Array:
    flat = []
    for t in tensors:
        flat.extend(t.stride())
    return (c_int64 * len(flat))(*flat)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _check_inputs(ref: torch.Tensor, *others: torch.Tensor) -> None:
    if not ref.is_cuda:
        raise RuntimeError("dmf_amd attention runs on the GPU only (tensor is on %s)" % ref.device)
    if ref.dim() != 4:
        raise ValueError(f"expected (B, L, H, D) tensors, got shape {tuple(ref.shape)}")
    for o in others:
        if o.device != ref.device or o.dtype != ref.dtype:
            raise ValueError("all attention operands must share device and dtype")


def fwd_jvp(q, k, v, tq, tk, tv, scale: float, need_dlse: bool = False):
    """Fused forward + JVP.  Returns (o, to, lse) -- or (o, to, lse, dlse) with
    ``need_dlse`` -- o/to contiguous (B, Lq, H, D), lse/dlse (B, H, Lq) fp32."""
    _check_inputs(q, k, v, tq, tk, tv)
    q, k, v, tq, tk, tv = map(_prep, (q, k, v, tq, tk, tv))
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    o = _empty((B, Lq, H, D), q.dtype, q.device)
    to = _empty((B, Lq, H, D), q.dtype, q.device)
    lse = _empty((B, H, Lq), torch.float32, q.device)
    dlse = _empty((B, H, Lq), torch.float32, q.device) if need_dlse else None
    with torch.cuda.device(q.device):
        rc = load().dmf_attn_fwd_jvp(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
            o.data_ptr(), to.data_ptr(), lse.data_ptr(), dlse.data_ptr() if need_dlse else None,
            _strides(q, k, v, tq, tk, tv, o, to),
            B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    _check(rc, "dmf_attn_fwd_jvp")
    return (o, to, lse, dlse) if need_dlse else (o, to, lse)


def fwd(q, k, v, scale: float, need_lse: bool = True):
    """Primal-only forward.  Returns (o, lse) (lse is None when not requested)."""
    _check_inputs(q, k, v)
    q, k, v = map(_prep, (q, k, v))
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    o = _empty((B, Lq, H, D), q.dtype, q.device)
    lse = _empty((B, H, Lq), torch.float32, q.device) if need_lse else None
    with torch.cuda.device(q.device):
        rc = load().dmf_attn_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr() if need_lse else None,
            _strides(q, k, v, o), B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    _check(rc, "dmf_attn_fwd")
    return o, lse


def bwd(dout, q, k, v, o, lse, scale: float):
    """Backward on the primal output.  Returns (dq, dk, dv), contiguous."""
    _check_inputs(q, k, v, o, dout)
    dout, q, k, v, o = map(_prep, (dout, q, k, v, o))
    lse = _raw(_raw(lse).contiguous())
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    dq = _empty((B, Lq, H, D), q.dtype, q.device)
    dk = _empty((B, Lkv, H, D), q.dtype, q.device)
    dv = _empty((B, Lkv, H, D), q.dtype, q.device)
    delta = _empty((B, H, Lq), torch.float32, q.device)
    with torch.cuda.device(q.device):
        rc = load().dmf_attn_bwd(
            dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(),
            _strides(dout, q, k, v, o, dq, dk, dv), B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    _check(rc, "dmf_attn_bwd")
    return dq, dk, dv
