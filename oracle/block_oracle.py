"""CPU restatement of the DiT-block glue around the attention operator.  TEST INFRASTRUCTURE ONLY.

Each function restates a few lines of the reference's models/layers.py in plain
torch ops (any float dtype, CPU); tangents come from ``torch.func.jvp`` and
gradients from autograd of these same functions.  Parity status, i.e. which
independent checks in ``tests/test_block_oracle.py`` pin each function:

* ``layer_norm``     -- pinned: ``torch.nn.functional.layer_norm`` (library
                        routine; the reference uses ``nn.LayerNorm(..., elementwise_affine=False,
                        eps=1e-6)``, models/layers.py:174,180,208) and the invariants
                        mean = 0, biased variance = 1 - eps*rstd^2.
* ``modulate``       -- models/layers.py:28-29, one line of arithmetic; pinned by
                        the special cases scale = 0, shift = 0 (identity).
* ``ln_modulate``    -- composition of the two; its JVP and gradients are pinned
                        by numpy fp64 closed forms (``ln_modulate_closed_fp64``),
                        central finite differences, and the adjoint identity.
* ``gate_residual``  -- models/layers.py:198,200; pinned by closed forms.
* ``gelu_tanh``      -- pinned: ``torch.nn.functional.gelu(approximate="tanh")``
                        (the reference's ``nn.GELU(approximate="tanh")``,
                        models/layers.py:162) and finite differences for the derivative.
* ``silu``           -- pinned: ``torch.nn.functional.silu`` and finite differences.
* ``rms_norm``       -- models/layers.py:33-42 (rounding points included);
                        pinned by the closed form x / sqrt(mean x^2 + eps) * gain, finite
                        differences and the closed-form tangent / gradient
                        (``rms_norm_closed_fp64``).
"""
from __future__ import annotations

import math

import numpy as np
import torch


def layer_norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """LayerNorm over the last dim without affine parameters (biased variance),
    as ``nn.LayerNorm(C, elementwise_affine=False, eps=1e-6)`` (models/layers.py:174)."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) * torch.rsqrt(var + eps)


def modulate(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """models/layers.py:28-29."""
    return x * (1 + scale) + shift


def ln_modulate(x, shift, scale, eps: float = 1e-6):
    """``modulate(self.norm1(x), shift_msa, scale_msa)`` (models/layers.py:198); x is
    (B, L, C), shift / scale (B, 1, C)."""
    return modulate(layer_norm(x, eps), shift, scale)


def gate_residual(x, gate, h):
    """``x + gate * branch`` (models/layers.py:198,200); gate is (B, 1, C)."""
    return x + gate * h


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """``nn.GELU(approximate="tanh")`` (models/layers.py:162), written out."""
    return 0.5 * x * (1 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def silu(x: torch.Tensor) -> torch.Tensor:
    """``nn.SiLU()`` (models/layers.py:186,212), written out."""
    return x * torch.sigmoid(x)


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``RMSNorm.forward`` (models/layers.py:39-42): the mean of squares is taken
    in fp32, the rsqrt is cast back to x's dtype before the two multiplies."""
    norm_x = torch.rsqrt(x.pow(2).mean(-1, keepdim=True, dtype=torch.float32 if x.dtype != torch.float64 else None) + eps)
    return x * norm_x.to(dtype=x.dtype) * gain.to(dtype=x.dtype)


def jvp(fn, primals, tangents):
    """(out, tangent_out) of ``fn`` by torch forward-mode AD."""
    return torch.func.jvp(fn, tuple(primals), tuple(tangents))


def grads(fn, inputs, gout):
    """Gradients of <fn(*inputs), gout> w.r.t. every input, by autograd."""
    inputs = [t.detach().clone().requires_grad_(True) for t in inputs]
    out = fn(*inputs)
    return torch.autograd.grad(out, inputs, gout)


# --------------------------------------------------------------------------
# numpy fp64 closed forms (independent statements used to pin the above)
# --------------------------------------------------------------------------
def ln_modulate_closed_fp64(x, shift, scale, tx=None, tshift=None, tscale=None, gy=None, eps=1e-6):
    """Textbook formulas.  Returns dict with y and, if tangents given, ty, and, if
    gy given, gx, gshift, gscale.  Shapes: x (B, L, C); shift, scale (B, 1, C)."""
    f = lambda a: None if a is None else np.asarray(a, dtype=np.float64)
    x, shift, scale, tx, tshift, tscale, gy = map(f, (x, shift, scale, tx, tshift, tscale, gy))
    mean = x.mean(-1, keepdims=True)
    rstd = 1.0 / np.sqrt(((x - mean) ** 2).mean(-1, keepdims=True) + eps)
    xh = (x - mean) * rstd
    out = {"y": xh * (1 + scale) + shift}
    if tx is not None:
        dxh = rstd * (tx - tx.mean(-1, keepdims=True) - xh * (xh * tx).mean(-1, keepdims=True))
        out["ty"] = dxh * (1 + scale) + xh * tscale + tshift
    if gy is not None:
        g = gy * (1 + scale)
        out["gx"] = rstd * (g - g.mean(-1, keepdims=True) - xh * (g * xh).mean(-1, keepdims=True))
        out["gshift"] = gy.sum(1, keepdims=True)
        out["gscale"] = (gy * xh).sum(1, keepdims=True)
    return out


def rms_norm_closed_fp64(x, gain, tx=None, gy=None, eps=1e-6):
    """y = x r g, r = (mean x^2 + eps)^-1/2; ty = (tx r + x dr) g with
    dr = -r^3 mean(x tx); gx = r gy g - x r^3 mean(x gy g); ggain = sum gy x r."""
    f = lambda a: None if a is None else np.asarray(a, dtype=np.float64)
    x, gain, tx, gy = map(f, (x, gain, tx, gy))
    r = 1.0 / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)
    out = {"y": x * r * gain}
    if tx is not None:
        dr = -(r ** 3) * (x * tx).mean(-1, keepdims=True)
        out["ty"] = (tx * r + x * dr) * gain
    if gy is not None:
        g = gy * gain
        out["gx"] = r * g - x * r ** 3 * (x * g).mean(-1, keepdims=True)
        out["ggain"] = (gy * x * r).reshape(-1, x.shape[-1]).sum(0)
    return out


def gelu_tanh_grad_fp64(x):
    """d/dx of the tanh-GELU, written out."""
    x = np.asarray(x, dtype=np.float64)
    a, b = math.sqrt(2.0 / math.pi), 0.044715
    t = np.tanh(a * (x + b * x ** 3))
    return 0.5 * (1 + t) + 0.5 * x * (1 - t * t) * a * (1 + 3 * b * x * x)


def make_block_inputs(B, L, C, seed, dtype=torch.float32):
    """Seeded CPU inputs in a fixed draw order: x, tx, h, th, gy (B, L, C);
    shift, scale, gate and their tangents (B, 1, C), the modulation vectors at the
    0.1-0.5 magnitudes adaLN outputs have."""
    g = torch.Generator().manual_seed(seed)
    big = [torch.randn(B, L, C, generator=g) for _ in range(5)]
    mods = [0.3 * torch.randn(B, 1, C, generator=g) for _ in range(6)]
    x, tx, h, th, gy = (t.to(dtype) for t in big)
    shift, scale, gate, tshift, tscale, tgate = (t.to(dtype) for t in mods)
    return dict(x=x, tx=tx, h=h, th=th, gy=gy, shift=shift, scale=scale, gate=gate, tshift=tshift, tscale=tscale, tgate=tgate)
