"""Forward-mode attention operator on hand-written gfx950 kernels.

Host-side mirror of the reference's operator module
(models/flash_attention_2_jvp.py:177-319): the same ``FlashAttnFunc`` protocol
(new-style ``forward`` without ctx + ``setup_context``, as ``torch.func.jvp``
requires) and the same ``flash_attn_func`` dual-tensor wrapper, but every
device computation goes through the C ABI in ``dmf_amd._lib``:

* dual inputs  -> one fused forward+JVP kernel (replaces the Triton
  ``_attn_fwd_dual[_split]`` launch, reference :196-230),
* plain inputs -> primal-only forward kernel (replaces ``flash_attn_2_cuda.fwd``,
  reference :233-243),
* ``backward`` -> dQ/dK/dV kernels (replaces ``flash_attn_2_cuda.bwd``,
  reference :260-276).

Unlike the reference, ``jvp`` is functional: when ``FlashAttnFunc.apply`` is
handed dual tensors directly, the tangents of ``o`` and ``lse`` are computed by
a second pass of the fused kernel over the saved primals.
"""
from __future__ import annotations

import warnings

import torch
import torch.autograd.forward_ad as fwAD

from . import _lib


def _default_scale(q: torch.Tensor, softmax_scale):
    return q.shape[-1] ** (-0.5) if softmax_scale is None else softmax_scale


class FlashAttnFunc(torch.autograd.Function):
    """(q, k, v, tq, tk, tv, softmax_scale) -> (o, lse, to); tensors are (B, L, H, D).

    ``lse`` is the natural-log logsumexp of the scaled scores, (B, H, Lq) fp32.
    ``to`` is None when any tangent is None.
    """

    @staticmethod
    def forward(q, k, v, tq, tk, tv, softmax_scale):
        scale = _default_scale(q, softmax_scale)
        enable_jvp = (tq is not None) and (tk is not None) and (tv is not None)
        if enable_jvp:
            o, to, lse = _lib.fwd_jvp(q, k, v, tq, tk, tv, scale)
        else:
            o, lse = _lib.fwd(q, k, v, scale, need_lse=True)
            to = None
        return o, lse, to

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        q, k, v, tq, tk, tv, softmax_scale = inputs
        o, lse, to = outputs
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.save_for_forward(q, k, v)
        ctx.softmax_scale = _default_scale(q, softmax_scale)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, dout, *ignored):
        # Gradients flow through the primal output only: cotangents of ``lse``
        # and ``to`` are dropped and the tangent inputs get no gradient, exactly
        # as in the reference (flash_attention_2_jvp.py:260-276) -- valid for the
        # MeanFlow loss because its JVP target is detached (loss.py:171-172).
        q, k, v, o, lse = ctx.saved_tensors
        if dout is None:
            return None, None, None, None, None, None, None
        dq, dk, dv = _lib.bwd(dout, q, k, v, o, lse, ctx.softmax_scale)
        return dq, dk, dv, None, None, None, None

    @staticmethod
    def jvp(ctx, gq, gk, gv, *ignored):
        # Tangents of ``o`` and ``lse`` along (gq, gk, gv) from a second pass of
        # the fused kernel.  ``to`` (if any) gets no tangent: that would be a
        # second-order quantity, which the reference does not provide either.
        if gq is None and gk is None and gv is None:
            return None, None, None
        # (saved tensors and tangents arrive functorch-wrapped here; _lib unwraps them)
        q, k, v = ctx.saved_tensors[:3]
        gq = torch.zeros_like(q) if gq is None else gq
        gk = torch.zeros_like(k) if gk is None else gk
        gv = torch.zeros_like(v) if gv is None else gv
        _, to, _, dlse = _lib.fwd_jvp(q, k, v, gq, gk, gv, ctx.softmax_scale, need_dlse=True)
        return to, dlse, None


def _is_dual_mode(*tensors) -> bool:
    """True if any tensor carries a forward-AD tangent (reference :285-291)."""
    return any(fwAD.unpack_dual(t).tangent is not None for t in tensors)


# ---- the primal operator as a registered custom op: what torch.compile traces instead of the ctypes calls ------------
# (forward + backward on the primal output, no tangents: the reference compiles only the model it calls without JVP,
#  train_dmf.py:269-275; in eager mode nothing goes through here)

@torch.library.custom_op("dmf_amd::attn_fwd", mutates_args=())
def _attn_fwd_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> tuple[torch.Tensor, torch.Tensor]:
    return _lib.fwd(q, k, v, scale, need_lse=True)


@_attn_fwd_op.register_fake
def _(q, k, v, scale):
    B, Lq, H, D = q.shape
    return q.new_empty((B, Lq, H, D)), q.new_empty((B, H, Lq), dtype=torch.float32)


@torch.library.custom_op("dmf_amd::attn_bwd", mutates_args=())
def _attn_bwd_op(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
                 scale: float) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _lib.bwd(dout, q, k, v, o, lse, scale)


@_attn_bwd_op.register_fake
def _(dout, q, k, v, o, lse, scale):
    return tuple(t.new_empty(t.shape) for t in (q, k, v))


def _attn_op_setup(ctx, inputs, output):
    q, k, v, scale = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, o, lse)
    ctx.scale = scale


def _attn_op_backward(ctx, dout, dlse_unused):
    q, k, v, o, lse = ctx.saved_tensors
    dq, dk, dv = torch.ops.dmf_amd.attn_bwd(dout, q, k, v, o, lse, ctx.scale)
    return dq, dk, dv, None


_attn_fwd_op.register_autograd(_attn_op_backward, setup_context=_attn_op_setup)


_warned_fp16 = False


def _padded_head_dim(d: int) -> int:
    """The kernels' head dim that serves head dim ``d``: itself, or the next larger one."""
    for n in _lib.SUPPORTED_HEAD_DIMS:
        if n >= d:
            return n
    raise ValueError(f"head dim {d} exceeds the largest supported one ({_lib.SUPPORTED_HEAD_DIMS[-1]})")


def flash_attn_func(q, k, v, softmax_scale=None):
    """Attention on (B, L, H, D) tensors; dual tensors in -> dual tensor out.

    Same contract as the reference's ``flash_attn_func``
    (models/flash_attention_2_jvp.py:294-319): under forward-mode AD the
    primals and tangents are unpacked (a missing tangent becomes zeros, :303-304),
    pushed through one fused kernel, and re-packed with ``fwAD.make_dual``.
    Head dims without a kernel of their own (the reference covers them by splitting
    and masking, models/triton_utils.py:22-45) are zero-padded to the next one that
    has -- exact, since zero columns add nothing to the scores and give zero output
    columns -- at the price of a padded copy of every operand.  fp16 operands (the
    reference's ``--mixed-precision fp16`` / ``--dtype fp16``) have no kernels of their
    own either: they are computed by the fp32 kernels and rounded back to fp16, which
    is exact to fp16 rounding but an order of magnitude slower than bf16 (warned once).
    """
    if q.dtype == torch.float16:
        global _warned_fp16
        if not _warned_fp16:
            _warned_fp16 = True
            warnings.warn("dmf_amd attention: fp16 operands are computed by the fp32 kernels (correct, but about ten times "
                          "slower than bf16 on this device); use bf16 for speed", stacklevel=2)
        return flash_attn_func(q.float(), k.float(), v.float(), _default_scale(q, softmax_scale)).to(torch.float16)
    d = q.shape[-1]
    dp = _padded_head_dim(d)
    if dp != d:
        scale = _default_scale(q, softmax_scale)
        pad = lambda t: torch.nn.functional.pad(t, (0, dp - d))
        return flash_attn_func(pad(q), pad(k), pad(v), scale)[..., :d]
    if torch.compiler.is_compiling():
        # traced by torch.compile: one opaque operator in the graph (no forward-AD inside compiled code)
        return torch.ops.dmf_amd.attn_fwd(q, k, v, float(_default_scale(q, softmax_scale)))[0]
    if _is_dual_mode(q, k, v):
        primals, tangents = [], []
        for t in (q, k, v):
            p, tg = fwAD.unpack_dual(t)
            primals.append(p)
            tangents.append(torch.zeros_like(p) if tg is None else tg)
        out, _, t_out = _lib.run_function(FlashAttnFunc, *primals, *tangents, softmax_scale)
        return fwAD.make_dual(out, t_out)
    if _lib.plain_inference(q, k, v):
        return _lib.fwd(q, k, v, _default_scale(q, softmax_scale), need_lse=False)[0]
    out, _, _ = _lib.run_function(FlashAttnFunc, q, k, v, None, None, None, softmax_scale)
    return out


class FlashAttnQKVPackedFunc(torch.autograd.Function):
    """(qkv, tqkv, softmax_scale) -> (o, lse, to) for a packed (B, L, 3, H, D)
    projection output -- the buffer ``Attention.forward`` slices q, k, v from
    (reference models/layers.py:143-147).  Same kernels as ``FlashAttnFunc`` (the
    slices are read in place); ``backward`` has the kernels write dq, dk, dv into
    the three slots of one packed gradient buffer, so autograd never has to stack
    and re-lay-out three separate gradients."""

    @staticmethod
    def forward(qkv, tqkv, softmax_scale):
        q, k, v = qkv.unbind(2)
        scale = _default_scale(q, softmax_scale)
        if tqkv is not None:
            o, to, lse = _lib.fwd_jvp(q, k, v, *tqkv.unbind(2), scale)
        else:
            o, lse = _lib.fwd(q, k, v, scale, need_lse=True)
            to = None
        return o, lse, to

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        qkv, _, softmax_scale = inputs
        o, lse, _ = outputs
        ctx.save_for_backward(qkv, o, lse)
        ctx.save_for_forward(qkv)
        ctx.softmax_scale = _default_scale(qkv, softmax_scale)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, dout, *ignored):
        qkv, o, lse = ctx.saved_tensors
        if dout is None:
            return None, None, None
        gqkv = torch.empty(qkv.shape, dtype=qkv.dtype, device=qkv.device)
        _lib.bwd(dout, *qkv.unbind(2), o, lse, ctx.softmax_scale, out=gqkv.unbind(2))
        return gqkv, None, None

    @staticmethod
    def jvp(ctx, gqkv, *ignored):
        if gqkv is None:
            return None, None, None
        qkv = ctx.saved_tensors[0]
        q, k, v = _lib._raw(qkv).unbind(2)
        tq, tk, tv = _lib._raw(gqkv).unbind(2)
        _, to, _, dlse = _lib.fwd_jvp(q, k, v, tq, tk, tv, ctx.softmax_scale, need_dlse=True)
        return to, dlse, None


def flash_attn_qkvpacked_func(qkv, softmax_scale=None):
    """Attention on a packed (B, L, 3, H, D) tensor, returns (B, L, H, D); dual in
    -> dual out, like ``flash_attn_func``."""
    if qkv.dim() != 5 or qkv.shape[2] != 3:
        raise ValueError(f"expected a packed (B, L, 3, H, D) tensor, got shape {tuple(qkv.shape)}")
    p, tg = fwAD.unpack_dual(qkv)
    if tg is None and _lib.plain_inference(p):
        q, k, v = p.unbind(2)
        return _lib.fwd(q, k, v, _default_scale(q, softmax_scale), need_lse=False)[0]
    out, _, t_out = _lib.run_function(FlashAttnQKVPackedFunc, p, tg, softmax_scale)
    return out if tg is None else fwAD.make_dual(out, t_out)


# Normalise q / q and k inside the attention kernel where a kernel offers it (module switches for A/B timing and tests).
IN_KERNEL_Q_NORM = True
IN_KERNEL_K_NORM = True
# A work-group of the tuned kernels covers 256 query rows and normalises the key tiles it consumes, so beyond that
# length a head's keys would be normalised once per query block: measured slower than one stand-alone pass over k
# (47.2 vs 46.7 ms on the DMFT-XL/2 512px forward+JVP step), so longer sequences keep that pass.
K_NORM_IN_KERNEL_MAX_LQ = 256


class QKNormAttnQKVPackedFunc(torch.autograd.Function):
    """(qkv, tqkv, q_gain, k_gain, eps, softmax_scale) -> (o, lse, to): per-head RMS
    norm of the q and k slots of a packed (B, L, 3, H, D) projection output followed
    by attention -- ``q, k = self.q_norm(q), self.k_norm(k); x = self.attn(q, k, v)``
    (reference models/layers.py:147-151) -- as one autograd node.  Forward is ONE
    launch where a tuned kernel exists: the attention kernel reads the raw q, k, v
    slots in place, normalises q (and its tangent) while loading it and every key
    tile once it sits in on-chip memory, and hands the normalised primal rows to
    the backward pass as two extra outputs.  Otherwise (fp32, untuned shapes, or the
    module switches above) the k slot / both slots go through the stand-alone
    RMS-norm kernel first.  Backward sends dv and the two norm gradients straight
    into the three slots of one packed gradient buffer.  ``qn`` is None only when q
    was normalised inside the kernel without being saved (backward then recomputes it)."""

    @staticmethod
    def forward(qkv, tqkv, q_gain, k_gain, eps, softmax_scale):
        q, k, v = qkv.unbind(2)
        scale = _default_scale(q, softmax_scale)
        jvp = tqkv is not None
        tq, tk, tv = tqkv.unbind(2) if jvp else (None, None, None)
        # the normalised rows are written only when a backward pass can follow
        save = any(isinstance(t, torch.Tensor) and t.requires_grad for t in (qkv, q_gain, k_gain))
        if IN_KERNEL_Q_NORM and IN_KERNEL_K_NORM and q.shape[1] <= K_NORM_IN_KERNEL_MAX_LQ:
            fused = _lib.fwd_qknorm(q, k, v, tq, tk, tv, q_gain, k_gain, eps, scale, save_normed=save)
            if fused is not None:
                o, to, lse, qn, kn = fused
                return o, lse, to, qn, kn
        kn, tkn = _lib.rmsnorm_fwd(k, k_gain, tk, eps, jvp)
        fused = _lib.fwd_qknorm(q, kn, v, tq, tkn, tv, q_gain, None, eps, scale, save_normed=save) if IN_KERNEL_Q_NORM else None
        if fused is not None:
            o, to, lse, qn, _ = fused
            return o, lse, to, qn, kn
        qn, tqn = _lib.rmsnorm_fwd(q, q_gain, tq, eps, jvp)
        if jvp:
            o, to, lse = _lib.fwd_jvp(qn, kn, v, tqn, tkn, tv, scale)
        else:
            o, lse = _lib.fwd(qn, kn, v, scale, need_lse=True)
            to = None
        return o, lse, to, qn, kn

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        qkv, _, q_gain, k_gain, eps, softmax_scale = inputs
        o, lse, _, qn, kn = outputs
        ctx.save_for_backward(qkv, q_gain, k_gain, qn, kn, o, lse)
        ctx.mark_non_differentiable(*(t for t in (qn, kn) if t is not None))
        ctx.eps, ctx.softmax_scale = eps, _default_scale(qkv, softmax_scale)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, dout, *ignored):
        if dout is None:
            return (None,) * 6
        qkv, q_gain, k_gain, qn, kn, o, lse = ctx.saved_tensors
        q, k, v = qkv.unbind(2)
        if qn is None:   # normalised in the kernel without being saved (no input asked for a gradient at forward time)
            qn, _ = _lib.rmsnorm_fwd(q, q_gain, None, ctx.eps, False)
        if kn is None:
            kn, _ = _lib.rmsnorm_fwd(k, k_gain, None, ctx.eps, False)
        gqkv = torch.empty(qkv.shape, dtype=qkv.dtype, device=qkv.device)
        gq, gk, gv = gqkv.unbind(2)
        dqn = torch.empty(qn.shape, dtype=qn.dtype, device=qn.device)
        dkn = torch.empty(kn.shape, dtype=kn.dtype, device=kn.device)
        _lib.bwd(dout, qn, kn, v, o, lse, ctx.softmax_scale, out=(dqn, dkn, gv))
        _, gq_gain = _lib.rmsnorm_bwd(dqn, q, q_gain, ctx.eps, out=gq)
        _, gk_gain = _lib.rmsnorm_bwd(dkn, k, k_gain, ctx.eps, out=gk)
        return gqkv, None, gq_gain, gk_gain, None, None


def flash_attn_qknorm_qkvpacked_func(qkv, q_gain, k_gain, eps: float = 1e-6, softmax_scale=None):
    """RMS-normalise the q and k slots of a packed (B, L, 3, H, D) tensor per head
    (gains ``q_gain``, ``k_gain`` of shape (D)) and attend; returns (B, L, H, D).
    Dual in -> dual out; the gains are constants of the tangent map."""
    if qkv.dim() != 5 or qkv.shape[2] != 3:
        raise ValueError(f"expected a packed (B, L, 3, H, D) tensor, got shape {tuple(qkv.shape)}")
    p, tg = fwAD.unpack_dual(qkv)
    if tg is None and _lib.plain_inference(p, q_gain, k_gain):
        q, k, v = p.unbind(2)
        scale = _default_scale(q, softmax_scale)
        if IN_KERNEL_Q_NORM and IN_KERNEL_K_NORM and q.shape[1] <= K_NORM_IN_KERNEL_MAX_LQ:
            fused = _lib.fwd_qknorm(q, k, v, None, None, None, q_gain, k_gain, eps, scale, need_lse=False)
            if fused is not None:
                return fused[0]
        kn, _ = _lib.rmsnorm_fwd(k, k_gain, None, eps, False)
        fused = _lib.fwd_qnorm(q, kn, v, None, None, None, q_gain, eps, scale, need_lse=False) if IN_KERNEL_Q_NORM else None
        if fused is not None:
            return fused[0]
        qn, _ = _lib.rmsnorm_fwd(q, q_gain, None, eps, False)
        return _lib.fwd(qn, kn, v, scale, need_lse=False)[0]
    out, _, t_out, _, _ = _lib.run_function(QKNormAttnQKVPackedFunc, p, tg, q_gain, k_gain, eps, softmax_scale)
    return out if tg is None else fwAD.make_dual(out, t_out)
