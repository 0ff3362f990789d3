"""Fused DiT-block glue operators with forward-mode (JVP) support.

Host-side counterparts of the small tensor expressions that surround the
attention operator in the reference's block (models/layers.py):

* ``ln_modulate(x, shift, scale)``  = ``modulate(LayerNorm(x), shift, scale)``   (:28-29, :198, :200, :219)
* ``gate_residual(x, gate, h)``     = ``x + gate * h``                           (:198, :200)
* ``residual_ln_modulate(x, gate, h, shift, scale)`` = the two above back to back (:198-200)
* ``gelu_tanh(x)``                  = ``nn.GELU(approximate="tanh")(x)``         (:162, :166)
* ``rms_norm(x, gain)``             = ``RMSNorm.forward``                        (:33-42, :148)
* ``silu(x)``                       = ``nn.SiLU()`` of the adaLN branch          (:185-188, :211-214)
* ``dual_linear(x, weight, bias)``  = ``nn.Linear`` (:131,137,161-165,...) -- library GEMMs, see ``DualLinearFunc``
* ``linear_gelu_tanh(x, weight, bias)`` = ``act(fc1(x))`` of the MLP (:166) -- GELU in the GEMM epilogue when nothing is differentiated

Each follows the protocol of the attention operator (flash_attention_hip_jvp):
a wrapper unpacks forward-AD duals, one ``torch.autograd.Function`` call pushes
primal and tangent through a single fused kernel (C ABI: include/dmf_block.h),
and the result is re-packed with ``fwAD.make_dual``.  ``backward`` propagates
through the primal output only: tangent inputs get no gradient and the
cotangent of the tangent output is dropped -- exact for the MeanFlow loss, whose
JVP target is detached (loss.py:171-172), and the same convention as the
reference's attention ``backward`` (flash_attention_2_jvp.py:260-276).
There is no fallback: without the HIP library every call raises.
"""
from __future__ import annotations

import torch
import torch.autograd.forward_ad as fwAD

from . import _lib


def _unpack(*tensors):
    primals, tangents = [], []
    for t in tensors:
        p, tg = fwAD.unpack_dual(t)
        primals.append(p)
        tangents.append(tg)
    return primals, tangents, any(tg is not None for tg in tangents)


def _primal_only(*tangent_cotangents):
    """These operators differentiate through their primal output only.  A loss that keeps the JVP output attached
    (unlike the MeanFlow loss, loss.py:171-172) would need the second-order terms the reference's tensor expressions
    carry; say so instead of returning gradients that silently lack them."""
    if any(g is not None for g in tangent_cotangents):
        raise NotImplementedError(
            "dmf_amd.block_ops: a gradient arrived at the tangent (JVP) output of a fused block operator; these operators "
            "back-propagate through the primal output only -- detach the JVP output (as DMFLoss does) or build the model "
            "with block_ops='torch'")


def _like(g, ref):
    """Gradient of a (B, C) modulation operand reshaped to the operand's shape."""
    return g.reshape(ref)


class LNModulateFunc(torch.autograd.Function):
    """(x, shift, scale, tx, tshift, tscale, eps, out_dtype, jvp) -> (y, ty)."""

    @staticmethod
    def forward(x, shift, scale, tx, tshift, tscale, eps, out_dtype, jvp):
        return _lib.ln_modulate_fwd(x, shift, scale, tx, tshift, tscale, eps, out_dtype, jvp)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        x, shift, scale, _, _, _, eps, _, _ = inputs
        ctx.save_for_backward(x, scale)
        ctx.eps, ctx.mod_shape = eps, (shift.shape, scale.shape)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty):
        _primal_only(gty)
        if gy is None:
            return (None,) * 9
        x, scale = ctx.saved_tensors
        gx, gshift, gscale = _lib.ln_modulate_bwd(gy, x, scale, ctx.eps)
        return gx, _like(gshift, ctx.mod_shape[0]), _like(gscale, ctx.mod_shape[1]), None, None, None, None, None, None


class GateResidualFunc(torch.autograd.Function):
    """(x, gate, h, tx, tgate, th, jvp) -> (y, ty)."""

    @staticmethod
    def forward(x, gate, h, tx, tgate, th, jvp):
        return _lib.gate_residual_fwd(x, gate, h, tx, tgate, th, jvp)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        x, gate, h = inputs[:3]
        ctx.save_for_backward(gate, h)
        ctx.gate_shape, ctx.x_dtype = gate.shape, x.dtype
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty):
        _primal_only(gty)
        if gy is None:
            return (None,) * 7
        gate, h = ctx.saved_tensors
        gh, ggate = _lib.gate_residual_bwd(gy, gate, h)
        return gy, _like(ggate, ctx.gate_shape), gh, None, None, None, None


class ResidualLNModulateFunc(torch.autograd.Function):
    """(x, gate, h, shift, scale, tx, tgate, th, tshift, tscale, eps, out_dtype, jvp) -> (y, z, ty, tz)."""

    @staticmethod
    def forward(x, gate, h, shift, scale, tx, tgate, th, tshift, tscale, eps, out_dtype, jvp):
        return _lib.residual_ln_modulate_fwd(x, gate, h, shift, scale, tx, tgate, th, tshift, tscale, eps, out_dtype, jvp)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        x, gate, h, shift, scale = inputs[:5]
        ctx.save_for_backward(outputs[0], h, gate, scale)
        ctx.eps, ctx.shapes = inputs[10], (gate.shape, shift.shape, scale.shape)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gz, gty, gtz):
        _primal_only(gty, gtz)
        if gy is None and gz is None:
            return (None,) * 13
        y, h, gate, scale = ctx.saved_tensors
        if gz is None:   # only the residual output was used
            gh, ggate = _lib.gate_residual_bwd(gy, gate, h)
            return (gy, _like(ggate, ctx.shapes[0]), gh) + (None,) * 10
        gx, gh, ggate, gshift, gscale = _lib.residual_ln_modulate_bwd(gy, gz, y, h, gate, scale, ctx.eps)
        return (gx, _like(ggate, ctx.shapes[0]), gh, _like(gshift, ctx.shapes[1]), _like(gscale, ctx.shapes[2])) + (None,) * 8


class GeluTanhFunc(torch.autograd.Function):
    """(x, tx) -> (y, ty)."""

    @staticmethod
    def forward(x, tx):
        return _lib.gelu_tanh_fwd(x, tx)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        ctx.save_for_backward(inputs[0])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty):
        _primal_only(gty)
        if gy is None:
            return None, None
        (x,) = ctx.saved_tensors
        return _lib.gelu_tanh_bwd(gy.to(x.dtype), x), None


class SiluFunc(torch.autograd.Function):
    """(x, tx, out_dtype) -> (y, ty)."""

    @staticmethod
    def forward(x, tx, out_dtype):
        return _lib.silu_fwd(x, tx, out_dtype)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        ctx.save_for_backward(inputs[0])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty):
        _primal_only(gty)
        if gy is None:
            return None, None, None
        (x,) = ctx.saved_tensors
        return _lib.silu_bwd(gy, x), None, None


class RMSNormFunc(torch.autograd.Function):
    """(x, gain, tx, eps, jvp) -> (y, ty); x is (B, L, H, D), normalised over D."""

    @staticmethod
    def forward(x, gain, tx, eps, jvp):
        return _lib.rmsnorm_fwd(x, gain, tx, eps, jvp)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        x, gain, _, eps, _ = inputs
        ctx.save_for_backward(x, gain)
        ctx.eps = eps
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty):
        _primal_only(gty)
        if gy is None:
            return (None,) * 5
        x, gain = ctx.saved_tensors
        gx, ggain = _lib.rmsnorm_bwd(gy.to(x.dtype), x, gain, ctx.eps)
        return gx, ggain, None, None, None


class DualLinearFunc(torch.autograd.Function):
    """(x, tx, weight, bias, w_lp, b_lp) -> (y, ty, w) with y = x W^T + b, ty = tx W^T: exactly
    one library GEMM per stream.  torch's own forward-mode rule for ``linear``
    also multiplies the primal input by a materialised all-zero weight tangent
    and adds the two products (three GEMMs, two fills, a copy and an add per
    layer); parameters carry no tangent in the MeanFlow JVP (loss.py:165-170), so
    that work is skipped here.  Under autocast the operands are cast once (``w``,
    the cast weight, is returned so that ``backward`` can reuse it)."""

    @staticmethod
    def forward(x, tx, weight, bias, w_lp, b_lp):
        linear = torch.nn.functional.linear
        if x.is_cuda and torch.is_autocast_enabled("cuda"):
            dt = torch.get_autocast_dtype("cuda")
            cached = w_lp is not None and w_lp.dtype == dt
            w = w_lp if cached else weight.to(dt)
            b = None if bias is None else (b_lp if cached and b_lp is not None else bias.to(dt))
            with torch.autocast("cuda", enabled=False):
                y = linear(x.to(dt), w, b)
                ty = None if tx is None else linear(tx.to(dt), w)
            # (an input is never handed back as an output: a cached copy reaches backward through the inputs)
            return y, ty, (w if not cached and w is not weight else None)
        return linear(x, weight, bias), (None if tx is None else linear(tx, weight)), None

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        x, _, weight, bias, w_lp, _ = inputs
        w = outputs[2]
        if w is not None:
            ctx.mark_non_differentiable(w)
        elif w_lp is not None and x.is_cuda and torch.is_autocast_enabled("cuda") and w_lp.dtype == torch.get_autocast_dtype("cuda"):
            w = w_lp
        else:
            w = weight
        ctx.save_for_backward(x, w)
        ctx.weight_dtype = weight.dtype
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, gy, gty, gw_unused):
        _primal_only(gty)
        if gy is None:
            return (None,) * 6
        x, w = ctx.saved_tensors
        g2 = gy.reshape(-1, gy.shape[-1]).to(w.dtype)
        want_gx, want_gw = ctx.needs_input_grad[0], ctx.needs_input_grad[2]
        want_gb = ctx.bias_dtype is not None and ctx.needs_input_grad[3]
        gx = gw = gb = None
        # The input gradient and the parameter gradients are independent and the weight-gradient GEMM (small
        # output, long contraction) does not fill the device, so on the GPU they are issued on two streams: a
        # fork/join that a stream capture records as two parallel branches (-4 % on the XL/2 train step; the same
        # trick for the primal / tangent GEMMs of the forward pass measured neutral to negative and is not used).
        fork = g2.is_cuda and want_gx and (want_gw or want_gb)
        if fork:
            main, side = torch.cuda.current_stream(g2.device), _lib.side_stream(g2.device)
            side.wait_stream(main)
            torch.cuda.set_stream(side)
        try:
            if want_gw:
                x2 = x.reshape(-1, x.shape[-1]).to(w.dtype)
                if g2.is_cuda and g2.dtype != ctx.weight_dtype and ctx.weight_dtype == torch.float32:
                    gw = torch.mm(g2.t(), x2, out_dtype=torch.float32)   # the GEMM stores its fp32 accumulators: no cast kernel
                else:
                    gw = (g2.t() @ x2).to(ctx.weight_dtype)
            if want_gb:
                # torch's multi-block column reduction clears its scratch with a memset node, which does not survive
                # HIP-graph replay; the library's two-stage sum has no such node
                if g2.is_cuda and g2.shape[1] % 8 == 0:
                    gb = _lib.colsum(g2.contiguous(), ctx.bias_dtype)
                else:
                    if g2.is_cuda and torch.cuda.is_current_stream_capturing():
                        raise RuntimeError("dual_linear: the bias gradient of a layer whose output width is not a multiple of 8 falls back "
                                           "to torch's column sum, which does not replay correctly from a captured graph")
                    gb = g2.sum(0).to(ctx.bias_dtype)
        finally:
            if fork:
                torch.cuda.set_stream(main)
        if want_gx:
            gx = (g2 @ w).reshape(x.shape).to(x.dtype)
        if fork:
            main.wait_stream(side)
            for t in (gw, gb):   # allocated on the side stream, consumed (and later freed) on the main one
                if t is not None:
                    t.record_stream(main)
        return gx, None, gw, gb, None, None


def dual_linear(x, weight, bias=None, w_lp=None, b_lp=None):
    """``F.linear(x, weight, bias)``; a forward-AD dual ``x`` gives a dual result
    (weight and bias are constants of the tangent map).  ``w_lp`` / ``b_lp``: optional
    copies of the parameters in the autocast dtype, used instead of casting per call
    (the caller guarantees they are current)."""
    (xp,), (tx,), dual = _unpack(x)
    y, ty, _ = _lib.run_function(DualLinearFunc, xp, tx, weight, bias, w_lp, b_lp)
    return fwAD.make_dual(y, ty) if dual else y


def linear_gelu_tanh(x, weight, bias, w_lp=None, b_lp=None):
    """``gelu_tanh(F.linear(x, weight, bias))`` -- the first half of the MLP
    (reference models/layers.py:161-166).  Without gradients and without a tangent
    the activation rides in the GEMM's epilogue (one library call, the pre-activation
    never reaches HBM); otherwise the pre-activation is needed for the tangent and for
    the backward pass and this is ``dual_linear`` followed by ``gelu_tanh``."""
    if torch.is_grad_enabled() or bias is None or not x.is_cuda or fwAD.unpack_dual(x).tangent is not None:
        return gelu_tanh(dual_linear(x, weight, bias, w_lp, b_lp))
    dt = _autocast_dtype(x)
    cached = w_lp is not None and w_lp.dtype == dt
    w = w_lp if cached else weight.to(dt)
    b = b_lp if cached and b_lp is not None else bias.to(dt)
    x2 = _lib._raw(x).reshape(-1, x.shape[-1]).to(dt)
    return torch._addmm_activation(b, x2, _lib._raw(w).t(), use_gelu=True).reshape(*x.shape[:-1], w.shape[0])


def _autocast_dtype(x: torch.Tensor):
    if x.is_cuda and torch.is_autocast_enabled("cuda"):
        return torch.get_autocast_dtype("cuda")
    return x.dtype


def ln_modulate(x, shift, scale, eps: float = 1e-6):
    """``LayerNorm(x) * (1 + scale) + shift`` for x (B, L, C) and shift / scale
    (B, C) or (B, 1, C); LayerNorm over C without affine parameters.  Under
    autocast the result is produced directly in the autocast dtype (it only ever
    feeds a Linear, which would cast it)."""
    (xp, shp, scp), (tx, tsh, tsc), dual = _unpack(x, shift, scale)
    y, ty = _lib.run_function(LNModulateFunc, xp, shp, scp, tx, tsh, tsc, eps, _autocast_dtype(xp), dual)
    return fwAD.make_dual(y, ty) if dual else y


def gate_residual(x, gate, h):
    """``x + gate * h`` for x, h (B, L, C) and gate (B, C) or (B, 1, C); the result
    has the promoted dtype of x and h (the fp32 residual stream under autocast)."""
    (xp, gp, hp), (tx, tg, th), dual = _unpack(x, gate, h)
    dt = torch.promote_types(xp.dtype, hp.dtype)
    if xp.dtype != dt:
        xp, tx = xp.to(dt), (None if tx is None else tx.to(dt))
    y, ty = _lib.run_function(GateResidualFunc, xp, gp, hp, tx, tg, th, dual)
    return fwAD.make_dual(y, ty) if dual else y


def residual_ln_modulate(x, gate, h, shift, scale, eps: float = 1e-6):
    """``y = x + gate * h`` and ``z = LayerNorm(y) * (1 + scale) + shift`` in one pass;
    returns ``(y, z)`` with the dtypes ``gate_residual`` and ``ln_modulate`` would give."""
    (xp, gp, hp, shp, scp), (tx, tg, th, tsh, tsc), dual = _unpack(x, gate, h, shift, scale)
    dt = torch.promote_types(xp.dtype, hp.dtype)
    if xp.dtype != dt:
        xp, tx = xp.to(dt), (None if tx is None else tx.to(dt))
    y, z, ty, tz = _lib.run_function(ResidualLNModulateFunc, xp, gp, hp, shp, scp, tx, tg, th, tsh, tsc, eps, _autocast_dtype(xp), dual)
    return (fwAD.make_dual(y, ty), fwAD.make_dual(z, tz)) if dual else (y, z)


def gelu_tanh(x):
    """tanh-approximated GELU."""
    (xp,), (tx,), dual = _unpack(x)
    y, ty = _lib.run_function(GeluTanhFunc, xp, tx)
    return fwAD.make_dual(y, ty) if dual else y


def silu(x):
    """``x * sigmoid(x)``; under autocast the result is produced in the autocast
    dtype (it feeds the adaLN projection, which would cast it)."""
    (xp,), (tx,), dual = _unpack(x)
    y, ty = _lib.run_function(SiluFunc, xp, tx, _autocast_dtype(xp))
    return fwAD.make_dual(y, ty) if dual else y


def rms_norm(x, gain, eps: float = 1e-6):
    """Per-head RMS norm of a (B, L, H, D) tensor over D (strided views into a
    packed qkv buffer are read in place); returns a contiguous tensor.  The gain
    is treated as a constant by forward-mode AD (parameters carry no tangent)."""
    (xp,), (tx,), dual = _unpack(x)
    y, ty = _lib.run_function(RMSNormFunc, xp, gain, tx, eps, dual)
    return fwAD.make_dual(y, ty) if dual else y
