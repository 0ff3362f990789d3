"""ctypes binding of the C ABI declared in include/dmf_attn.h and include/dmf_block.h.

The library is loaded from ``dmf_amd/libdmf_attn.so`` (built in-tree by
``python -m dmf_amd.build``).  There is deliberately no fallback: a missing
library raises ``RuntimeError`` at the first call.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import warnings
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p, POINTER

import torch
from torch._C import _functorch
from torch._functorch.pyfunctorch import retrieve_all_functorch_interpreters as _interpreters
try:   # private helpers of functorch: without them the operators go through functorch's own dispatch
    from torch._functorch.pyfunctorch import temporarily_pop_interpreter_stack as _pop_interpreter
    _HAVE_LEVEL_TOOLS = hasattr(_functorch, "_wrap_for_grad")
except ImportError:
    _pop_interpreter, _HAVE_LEVEL_TOOLS = None, False

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdmf_attn.so")

DMF_ATTN_F32, DMF_ATTN_BF16 = 0, 1
SUPPORTED_HEAD_DIMS = (32, 64, 72, 80, 96, 128)

# name -> (restype, argtypes): the complete exported surface of include/dmf_attn.h and include/dmf_block.h
_P, _I, _F, _L = c_void_p, c_int, c_float, c_int64
_S = POINTER(c_int64)
SIGNATURES = {
    "dmf_attn_version": (c_int, []),
    "dmf_attn_strerror": (c_char_p, [c_int]),
    "dmf_attn_fwd_jvp": (c_int, [_P] * 10 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_fwd": (c_int, [_P] * 5 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_fwd_qnorm": (c_int, [_P] * 7 + [_F] + [_P] * 4 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_fwd_qknorm": (c_int, [_P] * 8 + [_F] + [_P] * 6 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_bwd": (c_int, [_P] * 10 + [_S] + [_I] * 5 + [_F, _I, _P]),
    "dmf_attn_plan": (c_int, [_I] * 7 + [ctypes.c_char_p, _I]),
    "dmf_block_workspace_floats": (c_int64, [_I] * 4),
    "dmf_ln_modulate_fwd": (c_int, [_P] * 8 + [_S] + [_I] * 3 + [_F] + [_I] * 3 + [_P]),
    "dmf_ln_modulate_bwd": (c_int, [_P] * 8 + [_L] + [_I] * 3 + [_F] + [_I] * 3 + [_P]),
    "dmf_gate_residual_fwd": (c_int, [_P] * 8 + [_S] + [_I] * 3 + [_I] * 3 + [_P]),
    "dmf_gate_residual_bwd": (c_int, [_P] * 6 + [_L] + [_I] * 3 + [_I] * 3 + [_P]),
    "dmf_gelu_tanh_fwd": (c_int, [_P] * 4 + [_L, _I, _P]),
    "dmf_gelu_tanh_bwd": (c_int, [_P] * 3 + [_L, _I, _P]),
    "dmf_rmsnorm_fwd": (c_int, [_P] * 5 + [_S] + [_I] * 4 + [_F, _I, _I, _P]),
    "dmf_rmsnorm_bwd": (c_int, [_P] * 6 + [_S] + [_I] * 4 + [_F, _I, _I, _P]),
    "dmf_colsum": (c_int, [_P] * 3 + [_L, _I, _I, _I, _P]),
    "dmf_colsum_static": (c_int, [_P] * 2 + [_L, _I, _I, _I, _P]),
    "dmf_residual_ln_modulate_fwd": (c_int, [_P] * 14 + [_S] + [_I] * 3 + [_F] + [_I] * 4 + [_P]),
    "dmf_silu_fwd": (c_int, [_P] * 4 + [_L, _I, _I, _P]),
    "dmf_silu_bwd": (c_int, [_P] * 3 + [_L, _I, _I, _P]),
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


PLAN_ENTRIES = {"fwd": 0, "fwd_jvp": 1, "bwd": 2, "fwd_qnorm_jvp": 3, "fwd_qknorm_jvp": 4}


def plan(entry: str, B: int, H: int, Lq: int, Lkv: int, D: int, dtype=torch.bfloat16) -> str:
    """Name(s) of the kernel(s) the entry point ``entry`` launches for this shape on the current
    device, as profilers print them (``dmf_attn_plan``; host-only, launches nothing)."""
    buf = ctypes.create_string_buffer(256)
    code = DMF_ATTN_BF16 if dtype == torch.bfloat16 else DMF_ATTN_F32
    _check(load().dmf_attn_plan(PLAN_ENTRIES[entry], B, H, Lq, Lkv, D, code, buf, len(buf)), "dmf_attn_plan")
    return buf.value.decode()


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


def _apply(fn_cls, args):
    """``fn_cls.apply(*args)`` minus what ``torch.autograd.Function.apply`` does in Python
    before handing over to the C++ node constructor: binding the arguments against
    ``inspect.signature(forward)`` (~40 us per call; every caller in this package passes
    all arguments positionally) and the functorch check (the caller has made sure that
    no transform is active)."""
    return super(torch.autograd.Function, fn_cls).apply(*args)


# Call custom Functions below a single torch.func.jvp level instead of through it (module switch for A/B timing and tests).
BASE_LEVEL_UNDER_JVP = _HAVE_LEVEL_TOOLS


def run_function(fn_cls, *args):
    """``fn_cls.apply(*args)`` without functorch's custom-Function dispatch where that
    is sound.  The operators of this package unpack forward-AD duals themselves and
    pass primals and tangents as separate arguments, so inside ``torch.func.jvp`` the
    dispatch adds nothing but its (considerable, ~0.2-0.4 ms) per-call cost:

    * nothing needs a gradient and only ``jvp`` levels are active: ``fn_cls.forward``
      is called directly;
    * a gradient is needed and exactly one ``jvp`` level is active: the arguments are
      unwrapped, ``apply`` runs below the level like the ordinary autograd node it is,
      and the outputs are wrapped for the level again (what functorch does for every
      built-in operator);
    * otherwise (no transform, nested levels, ``vmap`` / ``grad``): plain ``apply``.

    Under ``torch.compile`` (the reference compiles the model it calls without JVP,
    train_dmf.py:269-275) the call is a graph break: the kernels are reached through
    ctypes, which a tracer cannot follow, so the operator runs eagerly between the
    compiled pieces."""
    if torch.compiler.is_compiling():
        return _run_function_eagerly(fn_cls, *args)
    stack = _interpreters()
    if not stack:
        return _apply(fn_cls, args)
    # (inside a functorch level the wrapper tensors do not report requires_grad; the wrapped values do)
    needs_grad = torch.is_grad_enabled() and any(isinstance(a, torch.Tensor) and (a.requires_grad or _raw(a).requires_grad)
                                                 for a in args)
    only_jvp = all(i.key() == _functorch.TransformType.Jvp for i in stack)
    if not needs_grad and only_jvp:
        return fn_cls.forward(*args)
    if BASE_LEVEL_UNDER_JVP and only_jvp and len(stack) == 1:
        level = stack[0].level()
        raw_args = [_raw(a) if isinstance(a, torch.Tensor) else a for a in args]
        with _pop_interpreter():
            outs = _apply(fn_cls, raw_args)
        wrap = lambda o: _functorch._wrap_for_grad(o, level) if isinstance(o, torch.Tensor) else o
        return tuple(wrap(o) for o in outs) if isinstance(outs, tuple) else wrap(outs)
    return fn_cls.apply(*args)


def plain_inference(*tensors) -> bool:
    """True when a primal-only call needs nothing kept for later: no gradient can be asked for (grad mode off, or no
    operand requires one) and no functorch transform is active.  Such calls (sampling, guidance targets) run the
    kernels directly -- no autograd node, no log-sum-exp output."""
    if torch.compiler.is_compiling() or _interpreters():
        return False
    return not (torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors))


@torch.compiler.disable
def _run_function_eagerly(fn_cls, *args):
    return run_function(fn_cls, *args)


_SIDE_STREAMS = {}


def side_stream(device) -> torch.cuda.Stream:
    """One extra stream per device (default priority) for fork / join of independent
    kernels; a stream capture records such a fork as parallel graph branches."""
    key = torch.device(device).index
    if key is None:
        key = torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


_NO_GUARD = contextlib.nullcontext()


def _on(device):
    """Context that makes ``device`` current for the launch -- nothing at all when it already is."""
    return _NO_GUARD if device.index == torch.cuda.current_device() else torch.cuda.device(device)


def _empty(shape, dtype, device) -> torch.Tensor:
    return _raw(torch.empty(shape, dtype=dtype, device=device))


def _prep(t: torch.Tensor) -> torch.Tensor:
    """Kernels need unit last-dim stride and 16-byte aligned rows; views into a
    packed qkv buffer already satisfy this and are passed through untouched."""
    t = _raw(t)
    eb = t.element_size()
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * eb) % 16 == 0 for s in t.stride()[:-1])
    if ok:
        return t
    # A layout the kernels cannot read in place costs a full extra HBM round trip per operand: count it and say so once.
    global relayout_copies
    relayout_copies += 1
    if relayout_copies == 1:
        warnings.warn(
            f"dmf_amd: operand with shape {tuple(t.shape)}, strides {tuple(t.stride())} and data pointer "
            f"{'aligned' if t.data_ptr() % 16 == 0 else 'not aligned'} to 16 bytes is copied to a contiguous buffer before "
            "the kernel runs (needs unit last-dim stride and 16-byte aligned rows); further copies are counted in "
            "dmf_amd._lib.relayout_copies without a warning", RuntimeWarning, stacklevel=3)
    return _raw(t.contiguous())


# Number of operands _prep had to copy because of their layout since import (0 on the model path: packed-qkv views are read in place).
relayout_copies = 0


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
    with _on(q.device):
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
    with _on(q.device):
        rc = load().dmf_attn_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr() if need_lse else None,
            _strides(q, k, v, o), B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    _check(rc, "dmf_attn_fwd")
    return o, lse


ENOKERNEL = -8   # DMF_ATTN_ENOKERNEL


def fwd_qnorm(q, k, v, tq, tk, tv, q_gain, eps: float, scale: float, need_lse: bool = True):
    """Forward (+ JVP when ``tq`` is given) with the per-head RMS norm of q (gain
    ``q_gain``, (D), fp32 or exactly representable in it) applied inside the attention kernel.  Returns (o, to, lse)
    (``to`` None without tangents), or None when no kernel implements the variant for
    this shape / dtype -- the caller then normalises q itself."""
    jvp = tq is not None
    if jvp:
        _check_inputs(q, k, v, tq, tk, tv)
        q, k, v, tq, tk, tv = map(_prep, (q, k, v, tq, tk, tv))
    else:
        _check_inputs(q, k, v)
        q, k, v = map(_prep, (q, k, v))
    gain = _raw(q_gain)
    if gain.dim() != 1 or gain.shape[0] != q.shape[-1] or gain.device != q.device:
        raise ValueError("fwd_qnorm: q_gain must be a (D) tensor on the device of q")
    if q.dtype != torch.bfloat16:
        return None
    gain = _raw(gain.float().contiguous())   # exact for a bf16 gain (a model cast to bf16 as a whole)
    if gain.data_ptr() % 16:
        return None
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    o = _empty((B, Lq, H, D), q.dtype, q.device)
    to = _empty((B, Lq, H, D), q.dtype, q.device) if jvp else None
    lse = _empty((B, H, Lq), torch.float32, q.device) if (need_lse or jvp) else None
    z = q   # stands in for absent tangents in the stride table (ignored by the library)
    with _on(q.device):
        rc = load().dmf_attn_fwd_qnorm(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _ptr(tq), _ptr(tk), _ptr(tv), gain.data_ptr(), float(eps),
            o.data_ptr(), _ptr(to), _ptr(lse), None,
            _strides(q, k, v, tq if jvp else z, tk if jvp else z, tv if jvp else z, o, to if jvp else o),
            B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    if rc == ENOKERNEL:
        return None
    _check(rc, "dmf_attn_fwd_qnorm")
    return o, to, lse


def fwd_qknorm(q, k, v, tq, tk, tv, q_gain, k_gain, eps: float, scale: float, need_lse: bool = True, save_normed: bool = False):
    """Forward (+ JVP when ``tq`` is given) on the raw q and k projections: the per-head RMS norms of q and of k (gains
    ``q_gain``, ``k_gain``, (D); ``k_gain`` None: k is already normalised) are applied inside the attention kernel.  Returns (o, to, lse, q_hat, k_hat) -- ``to``
    None without tangents, ``q_hat`` / ``k_hat`` the normalised primal rows when ``save_normed`` (a backward pass
    follows), else None -- or None when no kernel implements the variant for this shape / dtype."""
    jvp = tq is not None
    if jvp:
        _check_inputs(q, k, v, tq, tk, tv)
        q, k, v, tq, tk, tv = map(_prep, (q, k, v, tq, tk, tv))
    else:
        _check_inputs(q, k, v)
        q, k, v = map(_prep, (q, k, v))
    gains = []
    for name, gn in (("q_gain", q_gain), ("k_gain", k_gain)):
        if gn is None and name == "k_gain":   # k is already normalised
            gains.append(None)
            continue
        gn = _raw(gn)
        if gn.dim() != 1 or gn.shape[0] != q.shape[-1] or gn.device != q.device:
            raise ValueError(f"fwd_qknorm: {name} must be a (D) tensor on the device of q")
        gains.append(_raw(gn.float().contiguous()))   # exact for a bf16 gain (a model cast to bf16 as a whole)
    if q.dtype != torch.bfloat16 or any(gn is not None and gn.data_ptr() % 16 for gn in gains):
        return None
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    o = _empty((B, Lq, H, D), q.dtype, q.device)
    to = _empty((B, Lq, H, D), q.dtype, q.device) if jvp else None
    lse = _empty((B, H, Lq), torch.float32, q.device) if (need_lse or jvp) else None
    qh = _empty((B, Lq, H, D), q.dtype, q.device) if save_normed else None
    kh = _empty((B, Lkv, H, D), q.dtype, q.device) if save_normed and gains[1] is not None else None
    z = q   # stands in for absent tangents in the stride table (ignored by the library)
    with _on(q.device):
        rc = load().dmf_attn_fwd_qknorm(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _ptr(tq), _ptr(tk), _ptr(tv), gains[0].data_ptr(), _ptr(gains[1]), float(eps),
            o.data_ptr(), _ptr(to), _ptr(lse), None, _ptr(qh), _ptr(kh),
            _strides(q, k, v, tq if jvp else z, tk if jvp else z, tv if jvp else z, o, to if jvp else o),
            B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    if rc == ENOKERNEL:
        return None
    _check(rc, "dmf_attn_fwd_qknorm")
    return o, to, lse, qh, kh


def bwd(dout, q, k, v, o, lse, scale: float, out=None):
    """Backward on the primal output.  Returns (dq, dk, dv): freshly allocated
    contiguous tensors, or the three tensors given as ``out`` (any (B, L, H, D)
    views with unit last-dim stride and 16-byte aligned rows, e.g. the three slots
    of one packed (B, L, 3, H, D) gradient buffer), which the kernels fill in place."""
    _check_inputs(q, k, v, o, dout)
    dout, q, k, v, o = map(_prep, (dout, q, k, v, o))
    lse = _raw(_raw(lse).contiguous())
    B, Lq, H, D = q.shape
    Lkv = k.shape[1]
    if out is None:
        dq = _empty((B, Lq, H, D), q.dtype, q.device)
        dk = _empty((B, Lkv, H, D), q.dtype, q.device)
        dv = _empty((B, Lkv, H, D), q.dtype, q.device)
    else:
        dq, dk, dv = map(_raw, out)
        _check_inputs(q, dq, dk, dv)
        if dq.shape != q.shape or dk.shape != k.shape or dv.shape != v.shape:
            raise ValueError("bwd: `out` tensors must have the shapes of q, k, v")
    delta = _empty((B, H, Lq), torch.float32, q.device)
    with _on(q.device):
        rc = load().dmf_attn_bwd(
            dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(),
            _strides(dout, q, k, v, o, dq, dk, dv), B, H, Lq, Lkv, D, float(scale), _dtype_code(q), _stream(q))
    _check(rc, "dmf_attn_bwd")
    return dq, dk, dv


# ---- fused block glue (include/dmf_block.h) -----------------------------------------------------------------------

def _ptr(t):
    return None if t is None else t.data_ptr()


def _dense(t):
    """Contiguous, functorch-unwrapped (None passes through)."""
    if t is None:
        return None
    t = _raw(t)
    return t if t.is_contiguous() else _raw(t.contiguous())


def _mod(t, B: int, C: int):
    """A per-sample modulation vector, (B, C) or (B, 1, C) with unit channel
    stride -> (tensor, batch stride in elements); chunks of a wider adaLN output
    are passed through without a copy."""
    if t is None:
        return None, 0
    t = _raw(t)
    if t.numel() != B * C or t.shape[0] != B or t.shape[-1] != C:
        raise ValueError(f"expected a (B, C) or (B, 1, C) modulation tensor with B={B}, C={C}, got {tuple(t.shape)}")
    eb = t.element_size()
    if t.stride(-1) != 1 or t.data_ptr() % 16 or (t.stride(0) * eb) % 16:
        t = _raw(t.contiguous())
    return t, (t.stride(0) if B > 1 else C)


def _same_dtype(what: str, *ts):
    ts = [t for t in ts if t is not None]
    for t in ts[1:]:
        if t.dtype != ts[0].dtype or t.device != ts[0].device:
            raise ValueError(f"{what}: operands must share dtype and device")


def _blc(x):
    if not x.is_cuda:
        raise RuntimeError("dmf_amd block kernels run on the GPU only (tensor is on %s)" % x.device)
    if x.dim() != 3:
        raise ValueError(f"expected a (B, L, C) tensor, got shape {tuple(x.shape)}")
    return x.shape


def _workspace(which: int, B: int, L: int, dim: int, device) -> torch.Tensor:
    n = load().dmf_block_workspace_floats(which, B, L, dim)
    return _empty((max(int(n), 1),), torch.float32, device)


def ln_modulate_fwd(x, shift, scale, tx=None, tshift=None, tscale=None, eps: float = 1e-6, out_dtype=None, jvp=False):
    """(y, ty) of LayerNorm(x)*(1+scale)+shift; ty is None unless ``jvp``."""
    B, L, C = _blc(x)
    _same_dtype("ln_modulate x", x, tx)
    _same_dtype("ln_modulate shift/scale", shift, scale, tshift, tscale)
    x, tx = _dense(x), _dense(tx)
    (shift, s0), (scale, s1), (tshift, s2), (tscale, s3) = (_mod(t, B, C) for t in (shift, scale, tshift, tscale))
    out_dtype = out_dtype or x.dtype
    y = _empty((B, L, C), out_dtype, x.device)
    ty = _empty((B, L, C), out_dtype, x.device) if jvp else None
    with _on(x.device):
        rc = load().dmf_ln_modulate_fwd(
            x.data_ptr(), _ptr(tx), shift.data_ptr(), scale.data_ptr(), _ptr(tshift), _ptr(tscale), y.data_ptr(), _ptr(ty),
            (c_int64 * 4)(s0, s1, s2, s3), B, L, C, float(eps), _dtype_code(x), _dtype_code(shift), _dtype_code(y), _stream(x))
    _check(rc, "dmf_ln_modulate_fwd")
    return y, ty


def ln_modulate_bwd(gy, x, scale, eps: float = 1e-6, gres=None):
    """(gx, gshift, gscale); gshift / gscale are dense (B, C) of scale's dtype.
    ``gres`` (like x) is added to gx: the gradient x receives from elsewhere."""
    B, L, C = _blc(x)
    _same_dtype("ln_modulate_bwd x", x, gres)
    gy, x, gres = _dense(gy), _dense(x), _dense(gres)
    scale, ss = _mod(scale, B, C)
    gx = _empty((B, L, C), x.dtype, x.device)
    gshift = _empty((B, C), scale.dtype, x.device)
    gscale = _empty((B, C), scale.dtype, x.device)
    ws = _workspace(0, B, L, C, x.device)
    with _on(x.device):
        rc = load().dmf_ln_modulate_bwd(
            gy.data_ptr(), x.data_ptr(), scale.data_ptr(), _ptr(gres), gx.data_ptr(), gshift.data_ptr(), gscale.data_ptr(),
            ws.data_ptr(), ss, B, L, C, float(eps), _dtype_code(x), _dtype_code(scale), _dtype_code(gy), _stream(x))
    _check(rc, "dmf_ln_modulate_bwd")
    return gx, gshift, gscale


def gate_residual_fwd(x, gate, h, tx=None, tgate=None, th=None, jvp=False):
    """(y, ty) of x + gate*h, dtype of x; ty is None unless ``jvp``."""
    B, L, C = _blc(x)
    _same_dtype("gate_residual x", x, tx)
    _same_dtype("gate_residual h", h, th)
    _same_dtype("gate_residual gate", gate, tgate)
    if h.shape != x.shape:
        raise ValueError("gate_residual: x and h must have the same shape")
    x, tx, h, th = _dense(x), _dense(tx), _dense(h), _dense(th)
    (gate, g0), (tgate, g1) = _mod(gate, B, C), _mod(tgate, B, C)
    y = _empty((B, L, C), x.dtype, x.device)
    ty = _empty((B, L, C), x.dtype, x.device) if jvp else None
    with _on(x.device):
        rc = load().dmf_gate_residual_fwd(
            x.data_ptr(), _ptr(tx), gate.data_ptr(), _ptr(tgate), h.data_ptr(), _ptr(th), y.data_ptr(), _ptr(ty),
            (c_int64 * 2)(g0, g1), B, L, C, _dtype_code(x), _dtype_code(gate), _dtype_code(h), _stream(x))
    _check(rc, "dmf_gate_residual_fwd")
    return y, ty


def gate_residual_bwd(gy, gate, h):
    """(gh, ggate): gh like h, ggate dense (B, C) of gate's dtype."""
    B, L, C = _blc(h)
    gy, h = _dense(gy), _dense(h)
    gate, gs = _mod(gate, B, C)
    gh = _empty((B, L, C), h.dtype, h.device)
    ggate = _empty((B, C), gate.dtype, h.device)
    ws = _workspace(1, B, L, C, h.device)
    with _on(h.device):
        rc = load().dmf_gate_residual_bwd(
            gy.data_ptr(), gate.data_ptr(), h.data_ptr(), gh.data_ptr(), ggate.data_ptr(), ws.data_ptr(),
            gs, B, L, C, _dtype_code(gy), _dtype_code(gate), _dtype_code(h), _stream(h))
    _check(rc, "dmf_gate_residual_bwd")
    return gh, ggate


def gelu_tanh_fwd(x, tx=None):
    """(y, ty) of tanh-GELU; ty is None when ``tx`` is None."""
    if not x.is_cuda:
        raise RuntimeError("dmf_amd block kernels run on the GPU only (tensor is on %s)" % x.device)
    _same_dtype("gelu_tanh", x, tx)
    x, tx = _dense(x), _dense(tx)
    y = _empty(x.shape, x.dtype, x.device)
    ty = _empty(x.shape, x.dtype, x.device) if tx is not None else None
    with _on(x.device):
        rc = load().dmf_gelu_tanh_fwd(x.data_ptr(), _ptr(tx), y.data_ptr(), _ptr(ty), x.numel(), _dtype_code(x), _stream(x))
    _check(rc, "dmf_gelu_tanh_fwd")
    return y, ty


def gelu_tanh_bwd(gy, x):
    _same_dtype("gelu_tanh_bwd", x, gy)
    gy, x = _dense(gy), _dense(x)
    gx = _empty(x.shape, x.dtype, x.device)
    with _on(x.device):
        rc = load().dmf_gelu_tanh_bwd(gy.data_ptr(), x.data_ptr(), gx.data_ptr(), x.numel(), _dtype_code(x), _stream(x))
    _check(rc, "dmf_gelu_tanh_bwd")
    return gx


def rmsnorm_fwd(x, gain, tx=None, eps: float = 1e-6, jvp=False):
    """(y, ty) of the per-head RMS norm of a (B, L, H, D) tensor (strided views are
    read in place); outputs are contiguous."""
    _check_inputs(x, *([tx] if tx is not None else []))
    x, tx = _prep(x), (None if tx is None else _prep(tx))
    gain = _dense(gain)
    B, L, H, D = x.shape
    y = _empty((B, L, H, D), x.dtype, x.device)
    ty = _empty((B, L, H, D), x.dtype, x.device) if jvp else None
    with _on(x.device):
        rc = load().dmf_rmsnorm_fwd(
            x.data_ptr(), _ptr(tx), gain.data_ptr(), y.data_ptr(), _ptr(ty), _strides(x, tx if tx is not None else x),
            B, L, H, D, float(eps), _dtype_code(x), _dtype_code(gain), _stream(x))
    _check(rc, "dmf_rmsnorm_fwd")
    return y, ty


def rmsnorm_bwd(gy, x, gain, eps: float = 1e-6, out=None):
    """(gx, ggain): gx a fresh contiguous (B, L, H, D) tensor -- or ``out``, any
    (B, L, H, D) view with unit last-dim stride and 16-byte aligned rows (e.g. one
    slot of a packed qkv gradient buffer), filled in place; ggain (D) of gain's dtype."""
    _check_inputs(x, gy)
    x, gy, gain = _prep(x), _dense(gy), _dense(gain)
    B, L, H, D = x.shape
    if out is None:
        gx = _empty((B, L, H, D), x.dtype, x.device)
    else:
        gx = _raw(out)
        _check_inputs(x, gx)
        if gx.shape != x.shape:
            raise ValueError("rmsnorm_bwd: `out` must have the shape of x")
    ggain = _empty((D,), gain.dtype, x.device)
    ws = _workspace(2, B, L, D, x.device)
    with _on(x.device):
        rc = load().dmf_rmsnorm_bwd(
            gy.data_ptr(), x.data_ptr(), gain.data_ptr(), gx.data_ptr(), ggain.data_ptr(), ws.data_ptr(), _strides(x, gx),
            B, L, H, D, float(eps), _dtype_code(x), _dtype_code(gain), _stream(x))
    _check(rc, "dmf_rmsnorm_bwd")
    return gx, ggain


def colsum(x, out_dtype=None):
    """Column sums of a dense 2-D tensor (rows, C) -> (C,), fixed summation order."""
    if not x.is_cuda:
        raise RuntimeError("dmf_amd block kernels run on the GPU only (tensor is on %s)" % x.device)
    if x.dim() != 2:
        raise ValueError(f"expected a (rows, C) matrix, got shape {tuple(x.shape)}")
    x = _dense(x)
    rows, C = x.shape
    out = _empty((C,), out_dtype or x.dtype, x.device)
    n = load().dmf_block_workspace_floats(3, 1, min(rows, 2 ** 31 - 1), C)
    ws = _empty((max(int(n), 1),), torch.float32, x.device)
    with _on(x.device):
        rc = load().dmf_colsum(x.data_ptr(), out.data_ptr(), ws.data_ptr(), rows, C, _dtype_code(x), _dtype_code(out), _stream(x))
    _check(rc, "dmf_colsum")
    return out


def silu_fwd(x, tx=None, out_dtype=None):
    """(y, ty) of SiLU in ``out_dtype`` (default: x's); ty is None when ``tx`` is None."""
    if not x.is_cuda:
        raise RuntimeError("dmf_amd block kernels run on the GPU only (tensor is on %s)" % x.device)
    _same_dtype("silu", x, tx)
    x, tx = _dense(x), _dense(tx)
    out_dtype = out_dtype or x.dtype
    y = _empty(x.shape, out_dtype, x.device)
    ty = _empty(x.shape, out_dtype, x.device) if tx is not None else None
    with _on(x.device):
        rc = load().dmf_silu_fwd(x.data_ptr(), _ptr(tx), y.data_ptr(), _ptr(ty), x.numel(), _dtype_code(x), _dtype_code(y), _stream(x))
    _check(rc, "dmf_silu_fwd")
    return y, ty


def silu_bwd(gy, x):
    gy, x = _dense(gy), _dense(x)
    gx = _empty(x.shape, x.dtype, x.device)
    with _on(x.device):
        rc = load().dmf_silu_bwd(gy.data_ptr(), x.data_ptr(), gx.data_ptr(), x.numel(), _dtype_code(x), _dtype_code(gy), _stream(x))
    _check(rc, "dmf_silu_bwd")
    return gx


def residual_ln_modulate_fwd(x, gate, h, shift, scale, tx=None, tgate=None, th=None, tshift=None, tscale=None,
                             eps: float = 1e-6, out_dtype=None, jvp=False):
    """(y, z, ty, tz): y = x + gate*h (dtype of x), z = LayerNorm(y)*(1+scale)+shift
    (``out_dtype``); the tangents are None unless ``jvp``."""
    B, L, C = _blc(x)
    _same_dtype("residual_ln_modulate x", x, tx)
    _same_dtype("residual_ln_modulate h", h, th)
    _same_dtype("residual_ln_modulate modulation", gate, tgate, shift, scale, tshift, tscale)
    if h.shape != x.shape:
        raise ValueError("residual_ln_modulate: x and h must have the same shape")
    x, tx, h, th = _dense(x), _dense(tx), _dense(h), _dense(th)
    mods = [_mod(t, B, C) for t in (gate, tgate, shift, scale, tshift, tscale)]
    out_dtype = out_dtype or x.dtype
    y = _empty((B, L, C), x.dtype, x.device)
    z = _empty((B, L, C), out_dtype, x.device)
    ty = _empty((B, L, C), x.dtype, x.device) if jvp else None
    tz = _empty((B, L, C), out_dtype, x.device) if jvp else None
    with _on(x.device):
        rc = load().dmf_residual_ln_modulate_fwd(
            x.data_ptr(), _ptr(tx), mods[0][0].data_ptr(), _ptr(mods[1][0]), h.data_ptr(), _ptr(th),
            mods[2][0].data_ptr(), mods[3][0].data_ptr(), _ptr(mods[4][0]), _ptr(mods[5][0]),
            y.data_ptr(), _ptr(ty), z.data_ptr(), _ptr(tz), (c_int64 * 6)(*[m[1] for m in mods]), B, L, C, float(eps),
            _dtype_code(x), _dtype_code(mods[0][0]), _dtype_code(h), _dtype_code(z), _stream(x))
    _check(rc, "dmf_residual_ln_modulate_fwd")
    return y, z, ty, tz


def residual_ln_modulate_bwd(gy, gz, y, h, gate, scale, eps: float = 1e-6):
    """(gx, gh, ggate, gshift, gscale); ``gy`` (gradient of y from its other
    consumers) may be None.  Two launches: the LayerNorm backward with ``gy`` folded
    in, then the gated-residual backward on the total."""
    gx, gshift, gscale = ln_modulate_bwd(gz, y, scale, eps, gres=gy)
    gh, ggate = gate_residual_bwd(gx, gate, h)
    return gx, gh, ggate, gshift, gscale
