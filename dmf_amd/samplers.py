"""Few-step sampling loop: the no-grad caller of the operator.

Host-side mirror of the reference's ``get_tsteps`` and ``euler_sampler``
(samplers.py:60-100): ``num_steps`` calls ``model(x, t_cur, t_nxt, y)`` from t = 1
down to t = 0, each followed by the update ``x += (t_nxt - t_cur) * d`` in fp64;
with ``cfg_scale > 1`` the batch is doubled (labels + null class) inside the
guidance window and the two halves are combined.  Every model call is a
primal-only forward without gradients -- the mode in which the attention kernel
skips the log-sum-exp output and the block kernels their tangent streams.
``generate.py:84,115`` runs it on a model cast to the sampling dtype
(``model.to(dtype)``), not under autocast.
"""
from __future__ import annotations

import torch


def get_tsteps(num_steps: int, t_start: float = 1.0, t_end: float = 0.0, shift: float = 1.0) -> torch.Tensor:
    """``num_steps + 1`` fp64 times from ``t_start`` to ``t_end``, warped by
    ``shift * t / (1 + (shift - 1) * t)`` (samplers.py:60-66)."""
    t_steps = torch.linspace(t_start, t_end, num_steps + 1, dtype=torch.float64)
    if shift == 1.0:
        return t_steps
    return shift * t_steps / (1 + (shift - 1.0) * t_steps)


@torch.no_grad()
def euler_sampler(model, latents, y, num_steps: int = 4, cfg_scale: float = 1.0, g_min: float = 0.0, g_max: float = 1.0,
                  shift: float = 1.0, null_class: int = 1000, model_call=None, **kwargs):
    """samplers.py:69-100.  ``model_call(x, t, r, y)`` replaces ``model(x, t, r, y)``
    when given (e.g. a captured graph of the model at the batch sizes the loop uses)."""
    call = model if model_call is None else model_call
    dtype, device = latents.dtype, latents.device
    guided = cfg_scale > 1.0
    y_null = torch.full_like(y, null_class) if guided else None
    t_steps = get_tsteps(num_steps=num_steps, shift=shift)
    x_nxt = latents.to(torch.float64)
    for t_cur, t_nxt in zip(t_steps[:-1], t_steps[1:]):
        x_cur, y_cur, model_input = x_nxt, y, x_nxt
        in_window = guided and bool(g_min <= t_cur <= g_max)
        if in_window:
            model_input = torch.cat([model_input] * 2, dim=0)
            y_cur = torch.cat([y_cur, y_null], dim=0)
        model_input = model_input.to(dtype=dtype)
        n = model_input.shape[0]
        # the reference forms these as fp64 scalar * fp32 ones, i.e. rounded to fp32 first, then to the sampling dtype
        t_input = torch.full((n,), float(t_cur), device=device, dtype=torch.float32).to(dtype)
        r_input = torch.full((n,), float(t_nxt), device=device, dtype=torch.float32).to(dtype)
        d_cur = call(model_input, t_input, r_input, y_cur).to(torch.float64)
        if in_window:
            d_cond, d_uncond = d_cur.chunk(2)
            d_cur = d_uncond + cfg_scale * (d_cond - d_uncond)
        x_nxt = x_cur + (t_nxt - t_cur) * d_cur
    return x_nxt
