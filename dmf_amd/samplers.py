"""Few-step flow-map sampling: the no-grad caller of the attention operator.

What the harness needs from the reference's sampler (samplers.py:60-100) is its
call pattern, not its code: a short schedule of (t, r) pairs from t = 1 down to
t = 0, one primal-only model call per pair without gradients -- the mode in which
the attention kernel skips the log-sum-exp output and the block kernels their
tangent streams -- and, inside the guidance window, a batch of twice the size
(labels + null class) whose two halves are blended.  The state is advanced in
fp64 by ``x += (r - t) * u(x, t, r)``; model inputs are cast to the sampling
dtype (``generate.py:84,115`` casts the model itself rather than using autocast).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


def get_tsteps(num_steps: int, t_start: float = 1.0, t_end: float = 0.0, shift: float = 1.0) -> torch.Tensor:
    """The ``num_steps + 1`` fp64 time knots: uniform from ``t_start`` to ``t_end``, then warped by
    ``t -> shift t / (1 + (shift - 1) t)`` (the identity for ``shift = 1``); samplers.py:60-66."""
    knots = torch.linspace(t_start, t_end, num_steps + 1, dtype=torch.float64)
    return knots if shift == 1.0 else knots * shift / ((shift - 1.0) * knots + 1.0)


@dataclass(frozen=True)
class _Hop:
    t: float        # time the state is at
    r: float        # time the flow map jumps to
    guided: bool    # classifier-free guidance applies on this hop


def _schedule(num_steps: int, shift: float, cfg_scale: float, g_min: float, g_max: float) -> list[_Hop]:
    knots = get_tsteps(num_steps, shift=shift).tolist()
    use_cfg = cfg_scale > 1.0
    return [_Hop(t, r, use_cfg and g_min <= t <= g_max) for t, r in zip(knots, knots[1:])]


def _times(value: float, n: int, like: torch.Tensor) -> torch.Tensor:
    # an fp64 scalar times fp32 ones in the reference: rounded to fp32 first, then to the sampling dtype
    return torch.full((n,), value, device=like.device, dtype=torch.float32).to(like.dtype)


def _mean_velocity(call, x64: torch.Tensor, hop: _Hop, y, y_null, cfg_scale: float, dtype) -> torch.Tensor:
    """u(x, t, r) in fp64; on a guided hop one call on the doubled batch, blended as uncond + w (cond - uncond)."""
    x = x64.to(dtype)
    if not hop.guided:
        return call(x, _times(hop.t, x.shape[0], x), _times(hop.r, x.shape[0], x), y).to(torch.float64)
    both = torch.cat((x, x), dim=0)
    u = call(both, _times(hop.t, both.shape[0], x), _times(hop.r, both.shape[0], x), torch.cat((y, y_null), dim=0))
    cond, uncond = u.to(torch.float64).chunk(2)
    return torch.lerp(uncond, cond, cfg_scale)


@torch.no_grad()
def euler_sampler(model, latents, y, num_steps: int = 4, cfg_scale: float = 1.0, g_min: float = 0.0, g_max: float = 1.0,
                  shift: float = 1.0, null_class: int = 1000, model_call=None, **kwargs):
    """Same arguments and result as the reference's ``euler_sampler`` (samplers.py:69-100).  ``model_call(x, t, r, y)``
    replaces ``model(x, t, r, y)`` when given (e.g. a captured graph of the model at the batch sizes the loop uses)."""
    call = model if model_call is None else model_call
    hops = _schedule(num_steps, shift, cfg_scale, g_min, g_max)
    y_null = torch.full_like(y, null_class) if any(h.guided for h in hops) else None
    x = latents.to(torch.float64)
    for hop in hops:
        x = x + (hop.r - hop.t) * _mean_velocity(call, x, hop, y, y_null, cfg_scale, latents.dtype)
    return x
