"""MeanFlow JVP step and end-to-end timing of the DMFT harness.

``meanflow_jvp`` restates the JVP call site of the reference's loss
(loss.py:165-173): ``torch.func.jvp`` through the whole model with tangents
(v, 1, 0) for (x_t, t, r), target ``u_tgt = v + (r - t) * du/dt`` detached.
``train_step`` adds the backward on the primal output only, as
train_dmf.py:325-330 does under bf16 autocast.
"""
from __future__ import annotations

import contextlib
import time
from functools import partial

import torch
import torch.autograd.forward_ad as fwAD

from .dmft import DMFT_models
from .layers import frozen_low_precision_params


def synthetic_batch(batch: int, device, seed: int = 2, input_size: int = 32, channels: int = 4, num_classes: int = 1000):
    """z ~ N(0,1) (B,4,S,S); t, r ~ U(0,1) with r <= t, shaped (B,1,1,1) as the
    reference's samplers produce them; labels uniform; tangent v ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(batch, channels, input_size, input_size, generator=g)
    v = torch.randn(batch, channels, input_size, input_size, generator=g)
    a, b = torch.rand(batch, 1, 1, 1, generator=g), torch.rand(batch, 1, 1, 1, generator=g)
    t, r = torch.maximum(a, b), torch.minimum(a, b)
    y = torch.randint(0, num_classes, (batch,), generator=g)
    return tuple(x.to(device) for x in (z, t, r, y, v))


def meanflow_jvp(model, x_t, t, r, y, v, functorch: bool = True):
    """(u, du_dt) = jvp(model(., ., ., y), (x_t, t, r), (v, 1, 0)) -- loss.py:165-170.

    ``functorch=True`` is the reference's call, ``torch.func.jvp``.  ``False`` opens
    the forward-AD dual level directly (``torch.autograd.forward_ad``), which is what
    ``torch.func.jvp`` does underneath minus functorch's interpreter: same values,
    but every custom autograd Function on the way costs ~20 us of host time instead
    of ~200 us, which matters for the eagerly launched training step."""
    if functorch:
        return torch.func.jvp(partial(model, y=y), (x_t, t, r), (v, torch.ones_like(t), torch.zeros_like(r)))
    with fwAD.dual_level():
        out = model(fwAD.make_dual(x_t, v), fwAD.make_dual(t, torch.ones_like(t)), fwAD.make_dual(r, torch.zeros_like(r)), y)
        return fwAD.unpack_dual(out)


def meanflow_loss(model, x_t, t, r, y, v, functorch: bool = True):
    """MeanFlow regression loss with the JVP target detached (loss.py:171-172);
    plain mean-squared error (the log-variance weighting is not part of the path)."""
    u, du_dt = meanflow_jvp(model, x_t, t, r, y, v, functorch)
    u_tgt = (v + (r - t) * du_dt).detach()
    return ((u - u_tgt) ** 2).mean(), u, du_dt


def train_step(model, batch, autocast: bool = True, functorch: bool = True):
    """Forward + JVP, then backward on the primal output only."""
    x_t, t, r, y, v = batch
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        loss, _, _ = meanflow_loss(model, x_t, t, r, y, v, functorch)
    loss.backward()
    return loss


def build_model(name: str, attn_func: str, device, qk_norm: bool = False, input_size: int = 32, dmf_depth=None, seed: int = 0,
                block_ops: str = "torch"):
    kw = {"attn_func": attn_func, "qk_norm": qk_norm, "input_size": input_size, "block_ops": block_ops}
    if dmf_depth is not None:
        kw["dmf_depth"] = dmf_depth
    return DMFT_models[name](**kw).init_trunc_normal_(0.02, seed).to(device)


class GraphedStep:
    """A step function captured once into a HIP graph and replayed.

    The uncompiled JVP pass issues roughly a thousand small launches per step
    from Python (loss.py:165 runs the eager module), which leaves the GPU idle
    more than half of the time once the kernels themselves are fused; replaying
    a captured graph removes the host from the loop.  ``fn(*inputs)`` must be a
    pure function of its tensor arguments (and of module parameters, which are
    read in place at replay time); its outputs live in the graph's memory pool
    and are overwritten by the next call.  Capture happens on a side stream at
    the default priority after ``warmup`` eager calls.
    """

    def __init__(self, fn, *example_inputs, warmup: int = 3):
        self.static_inputs = [x.clone() if isinstance(x, torch.Tensor) else x for x in example_inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                fn(*self.static_inputs)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_outputs = fn(*self.static_inputs)

    def __call__(self, *inputs):
        for dst, src in zip(self.static_inputs, inputs):
            if isinstance(dst, torch.Tensor) and dst is not src:
                dst.copy_(src)
        self.graph.replay()
        return self.static_outputs


def _time(fn, steps: int, warmup: int = 2) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_dmft(steps: int = 5, device="cuda:0", compare_base: bool = True, only=None, variants=None) -> dict:
    """images/s for (a) DMFT-B/2 256px forward+JVP, batch 64, bf16 autocast,
    (b) DMFT-XL/2 256px forward+JVP+backward, batch 32, and (c) DMFT-B/2 primal-only
    no-grad forward at batch 128 -- the call mode of the guidance branch
    (loss.py:64-69, a 2B batch) and of a sampler step (samplers.py:69-100) -- and
    (d) DMFT-XL/2 at 512px (1024 tokens) with qk-norm, forward+JVP, batch 16: the
    caller of the headline attention shape.  Variants:
    ``hip_fused_graph`` -- 'hip' attention + fused block glue, replayed as a HIP graph,
    ``hip_fused_fwad``  -- the same, launched eagerly with the forward-AD dual level opened directly,
    ``hip_fused``       -- the same, launched eagerly through ``torch.func.jvp`` (the reference's call),
    ``hip``             -- 'hip' attention inside the reference's tensor expressions,
    ``base``            -- naive attention (the reference's own CPU-runnable operator).
    ``only`` / ``variants`` restrict the model / the variants that are run."""
    out = {}
    # (key, model, batch, dmf_depth, mode, latent size, qk_norm)
    all_cases = [("DMFT-B/2", "DMFT-B/2", 64, 8, "jvp", 32, False), ("DMFT-XL/2", "DMFT-XL/2", 32, 20, "train", 32, False),
                 ("DMFT-B/2 no-grad", "DMFT-B/2", 128, 8, "nograd", 32, False),
                 ("DMFT-XL/2 512px qk-norm", "DMFT-XL/2", 16, 20, "jvp", 64, True)]
    cases = [c for c in all_cases if only in (None, c[0])]
    all_variants = [("hip_fused_graph", "hip", "hip", True), ("hip_fused_fwad", "hip", "hip", False), ("hip_fused", "hip", "hip", False),
                    ("hip", "hip", "torch", False)]
    if compare_base:
        all_variants.append(("base", "base", "torch", False))
    variants = [v for v in all_variants if variants is None or v[0] in variants]
    modes = {"jvp": "fwd+jvp", "train": "fwd+jvp+bwd", "nograd": "primal-only forward, no grad (guidance / sampler call)"}
    for key, name, batch, dmf_depth, mode, input_size, qk_norm in cases:
        row = {"batch": batch, "mode": modes[mode], "dtype": "bf16 autocast", "tokens": (input_size // 2) ** 2, "qk_norm": qk_norm}
        data = synthetic_batch(batch, device, input_size=input_size)
        for label, op, block_ops, graphed in variants:
            if mode == "nograd" and label == "hip_fused_fwad":
                continue   # no JVP in this mode
            model = build_model(name, op, device, qk_norm=qk_norm, input_size=input_size, dmf_depth=dmf_depth, block_ops=block_ops)
            functorch = label != "hip_fused_fwad"
            if mode == "train":
                def step(*batch_tensors):
                    model.zero_grad(set_to_none=True)
                    return train_step(model, batch_tensors, functorch=functorch).detach()
            elif mode == "jvp":
                model.requires_grad_(False)

                def step(*batch_tensors):
                    with torch.autocast("cuda", dtype=torch.bfloat16):
                        return meanflow_jvp(model, *batch_tensors, functorch=functorch)
            else:
                model.requires_grad_(False)

                def step(z, t, r, y, v):
                    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                        return model(z, t, r, y)
            # the forward+JVP-only and no-grad passes run over frozen weights: cast them once, not per call
            frozen = frozen_low_precision_params(model) if (mode != "train" and block_ops == "hip") else contextlib.nullcontext()
            with frozen:
                run = GraphedStep(step, *data) if graphed else step
                sec = _time(lambda: run(*data), steps * 4 if graphed else (steps if op == "hip" else max(2, steps // 2)))
            row[f"{label}_ms_per_step"] = sec * 1e3
            row[f"{label}_images_per_s"] = batch / sec
            del model, run, step
            torch.cuda.empty_cache()
        out[key] = row
    return out
