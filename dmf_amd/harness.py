"""MeanFlow JVP step and end-to-end timing of the DMFT harness.

``meanflow_jvp`` restates the JVP call site of the reference's loss
(loss.py:165-173): ``torch.func.jvp`` through the whole model with tangents
(v, 1, 0) for (x_t, t, r), target ``u_tgt = v + (r - t) * du/dt`` detached.
``train_step`` adds the backward on the primal output only, as
train_dmf.py:325-330 does under bf16 autocast.  ``dmf_loss`` restates the whole
training loss around that site (loss.py:142-181: the flow-matching branch with
gradients, the guidance calls without, the JVP branch, log-variance weighting),
``fm_loss`` the flow-matching loss that ``train_fm.py`` trains SiT with
(loss.py:208-231); both take their random draws as arguments, so a step is a pure
function of tensors and can be captured into a HIP graph.
"""
from __future__ import annotations

import contextlib
import math
import time
from functools import partial

import torch
import torch.autograd.forward_ad as fwAD

from .dmft import DMFT_models
from .layers import frozen_low_precision_params
from .samplers import euler_sampler
from .sit import SiT_models


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


def interpolant(x, t, eps, path_type: str = "linear"):
    """(x_t, v_t) of the noising path (loss.py:7-23) for the noise ``eps``."""
    if path_type == "linear":
        alpha, sigma, d_alpha, d_sigma = 1 - t, t, -1, 1
    elif path_type == "cosine":
        alpha, sigma = torch.cos(t * math.pi / 2), torch.sin(t * math.pi / 2)
        d_alpha, d_sigma = (-math.pi / 2) * torch.sin(t * math.pi / 2), (math.pi / 2) * torch.cos(t * math.pi / 2)
    else:
        raise NotImplementedError(path_type)
    return alpha * x + sigma * eps, d_alpha * x + d_sigma * eps


def _per_sample(err, reduce):
    return reduce(err, dim=list(range(1, err.dim())))


def log_lv_loss(x, y, lv, eps: float = 0.01):
    """(sum of squares, log-variance weighted loss) per sample -- loss.py:30-35."""
    err = (x - y) ** 2
    mean = _per_sample(err, torch.mean)
    return _per_sample(err, torch.sum), torch.log((1 / lv.exp()) * mean + eps) + lv


def mse_loss(x, y):
    """(sum of squares, mean of squares) per sample -- loss.py:38-42."""
    err = (x - y) ** 2
    return _per_sample(err, torch.sum), _per_sample(err, torch.mean)


def compute_guidance(model, x, t, y, v_t, drop_ids, omega: float = 0.5, g_min: float = 0.0, g_max: float = 1.0,
                     g_type: str = "default", null_class: int = 1000):
    """Guided regression target (loss.py:57-86).  ``"mg"`` calls the trained model
    itself as ``model(x, t, t, y)``, ``"distill"`` a frozen single-time teacher as
    ``model(x, t, y)`` -- both without gradients on a 2B batch (conditional and
    unconditional halves), which is the primal-only, lse-free mode of the operator."""
    if g_type == "default":
        return v_t
    if g_type not in ("mg", "distill"):
        raise NotImplementedError(f"Unknown guidance type: {g_type}")
    in_range = (t >= g_min) & (t <= g_max)
    with torch.no_grad():
        x_2, t_2 = torch.cat([x, x], dim=0), torch.cat([t, t], dim=0)
        y_2 = torch.cat([y, torch.full_like(y, null_class)], dim=0)
        v = (model(x_2, t_2, t_2, y_2) if g_type == "mg" else model(x_2, t_2, y_2)).to(torch.float32)
        v_cond, v_uncond = v.chunk(2, dim=0)
    if g_type == "mg":
        return torch.where(in_range & (~drop_ids.reshape(-1, 1, 1, 1)), v_t + omega * (v_cond - v_uncond), v_t)
    return torch.where(in_range, v_uncond + omega * (v_cond - v_uncond), v_cond)   # no class dropout for distillation


def dmf_loss(model, x, y, drop_ids, t_fm, t_mf, r_mf, eps_fm, eps_mf, model_t=None, functorch: bool = True,
             path_type: str = "linear", **guidance):
    """Per-sample training loss of ``DMFLoss.__call__`` (loss.py:142-181) and its
    dictionary of parts.  ``y`` already carries the dropped labels and ``drop_ids``
    says which (``cond_drop``, loss.py:129-133); times are (B, 1, 1, 1) and the two
    noise tensors shaped like ``x`` (``sample_times`` / ``interpolant`` draw them in
    the reference).  ``model`` must have a log-variance head.  Four model calls:
    flow-matching branch with gradients, two guidance evaluations without (on
    ``model_t``, default ``model``), and the MeanFlow branch under forward-mode AD
    with tangents (v_tgt, 1, 0), whose target is detached."""
    model_t = model if model_t is None else model_t
    x_t_fm, v_t_fm = interpolant(x, t_fm, eps_fm, path_type)
    v_fm, lv_fm = model(x_t_fm, t_fm, t_fm, y, return_logvar=True)
    v_tgt_fm = compute_guidance(model_t, x_t_fm, t_fm, y, v_t_fm, drop_ids, **guidance).detach()
    fm_mse, fm_lp = log_lv_loss(v_fm, v_tgt_fm, lv_fm)

    x_t_mf, v_t_mf = interpolant(x, t_mf, eps_mf, path_type)
    v_tgt_mf = compute_guidance(model_t, x_t_mf, t_mf, y, v_t_mf, drop_ids, **guidance).detach()
    tangents = (v_tgt_mf, torch.ones_like(t_mf), torch.zeros_like(r_mf))
    if functorch:
        (u, lv_mf), (du_dt, _) = torch.func.jvp(partial(model, y=y, return_logvar=True), (x_t_mf, t_mf, r_mf), tangents)
    else:
        with fwAD.dual_level():
            out, lv = model(*(fwAD.make_dual(p, tg) for p, tg in zip((x_t_mf, t_mf, r_mf), tangents)), y, return_logvar=True)
            (u, du_dt), lv_mf = fwAD.unpack_dual(out), fwAD.unpack_dual(lv).primal
    u_tgt = (v_tgt_mf + (r_mf - t_mf) * du_dt).detach()
    mf_mse, mf_lp = log_lv_loss(u, u_tgt, lv_mf)
    return 0.5 * (fm_lp + mf_lp), {"fm_loss": fm_mse, "fm_p_loss": fm_lp, "mf_p_loss": mf_lp, "mf_loss": mf_mse}


def fm_loss(model, x, y, t, eps, path_type: str = "linear"):
    """Per-sample flow-matching loss of ``FMLoss.__call__`` without the projection
    term (loss.py:224-230): ``model`` is a single-time (SiT) model."""
    x_t, v_t = interpolant(x, t, eps, path_type)
    fm, loss = mse_loss(model(x_t, t, y), v_t)
    return loss, {"fm_loss": fm}


def dmf_train_step(model, batch, model_t=None, functorch: bool = True, autocast: bool = True, **guidance):
    """One optimisation step's forward and backward as train_dmf.py:325-330 runs
    them: ``dmf_loss`` under bf16 autocast, mean over the batch, backward.  The
    parameters do not change between the (up to four) model calls of one step, so
    the fused Linear layers share one bf16 copy of their weights per step instead
    of casting them in every call; gradients still reach the fp32 parameters."""
    with contextlib.ExitStack() as stack:
        if autocast:   # (``autocast=False``: the same step in the parameters' own precision, e.g. an fp32 yardstick)
            stack.enter_context(frozen_low_precision_params(model))
            stack.enter_context(torch.autocast("cuda", dtype=torch.bfloat16))
        loss, _ = dmf_loss(model, *batch, model_t=model_t, functorch=functorch, **guidance)
        loss = loss.mean()
        loss.backward()
    return loss


def fm_train_step(model, batch, autocast: bool = True):
    """train_fm.py:347-352: ``fm_loss`` under bf16 autocast, mean, backward."""
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        loss, _ = fm_loss(model, *batch)
    loss = loss.mean()
    loss.backward()
    return loss


def synthetic_loss_batch(batch: int, device, seed: int = 3, input_size: int = 32, channels: int = 4, num_classes: int = 1000,
                         cfg_prob: float = 0.1):
    """(x, y, drop_ids, t_fm, t_mf, r_mf, eps_fm, eps_mf) for ``dmf_loss``: latents and
    noises ~ N(0,1), labels uniform with a fraction ``cfg_prob`` replaced by the null
    class, times logit-normal with the reference's defaults (loss.py:100-140), r <= t."""
    g = torch.Generator().manual_seed(seed)
    x, eps_fm, eps_mf = (torch.randn(batch, channels, input_size, input_size, generator=g) for _ in range(3))
    y = torch.randint(0, num_classes, (batch,), generator=g)
    drop_ids = torch.rand(batch, generator=g) < cfg_prob
    y = torch.where(drop_ids, num_classes, y)
    ln = lambda mean: torch.sigmoid(torch.randn(batch, 1, 1, 1, generator=g) + mean)
    t_fm, a, b = ln(-0.4), ln(-0.2), ln(0.2)
    return tuple(v.to(device) for v in (x, y, drop_ids, t_fm, torch.maximum(a, b), torch.minimum(a, b), eps_fm, eps_mf))


def build_model(name: str, attn_func: str, device, qk_norm: bool = False, input_size: int = 32, dmf_depth=None, seed: int = 0,
                block_ops: str = "torch", **extra):
    """A DMFT (``"DMFT-*"``) or SiT (``"SiT-*"``) of the reference's size registry with truncated-normal weights,
    constructed and initialised directly on ``device``."""
    kw = {"attn_func": attn_func, "qk_norm": qk_norm, "input_size": input_size, "block_ops": block_ops, **extra}
    if dmf_depth is not None:
        kw["dmf_depth"] = dmf_depth
    registry = SiT_models if name.startswith("SiT") else DMFT_models
    with torch.device(device):
        model = registry[name](**kw)
    return model.init_trunc_normal_(0.02, seed)


def stale_grad_accumulator(p: torch.Tensor) -> bool:
    """True if an autograd graph that is still alive refers to ``p``'s gradient accumulator.  The accumulator node is
    created on first use and freed with the last graph that points at it; asking for it twice returns the same
    object only while something else keeps it alive.  Anything else that legitimately holds the accumulator --
    a post-accumulate-grad hook, a DDP-style reducer -- reads as "stale" too.  Works under ``torch.no_grad()``
    (the probe switches gradient mode on for itself); a tensor that does not require a gradient has no accumulator."""
    if not p.requires_grad:
        return False
    key = "dmf_amd.stale_probe"
    with torch.enable_grad():
        node = p.view_as(p).grad_fn.next_functions[0][0]
        node.metadata[key] = True          # lives on the node itself, not on this Python wrapper
        del node
        node = p.view_as(p).grad_fn.next_functions[0][0]
    alive = bool(node.metadata.pop(key, False))
    return alive


class GraphedStep:
    """A step function captured once into a HIP graph and replayed.

    The uncompiled JVP pass issues roughly a thousand small launches per step
    from Python (loss.py:165 runs the eager module), which leaves the GPU idle
    more than half of the time once the kernels themselves are fused; replaying
    a captured graph removes the host from the loop.  ``fn(*inputs)`` must be a
    pure function of its tensor arguments (and of module parameters, which are
    read in place at replay time); its outputs live in the graph's memory pool
    and are overwritten by the next call.  The ``warmup`` eager calls and the
    capture run on ONE side stream at the default priority: a parameter's gradient
    accumulator is bound to the stream it was created on, so the accumulators
    that the warm-up creates are the ones the captured backward uses.  What the
    class cannot see is an autograd graph of an EARLIER step that the caller still
    holds (``loss`` kept instead of ``float(loss)`` / ``loss.detach()``): it keeps
    older accumulators alive, bound to the caller's stream, and the captured
    backward would then be sent to a stream that is not capturing.  ``parameters``
    (optional) lets the constructor refuse that case before capturing: it raises
    if any of them still has a gradient accumulator from before the warm-up.
    """

    def __init__(self, fn, *example_inputs, warmup: int = 3, parameters=None):
        self.static_inputs = [x.clone() if isinstance(x, torch.Tensor) else x for x in example_inputs]
        stale = [p for p in (parameters or ()) if p.requires_grad and stale_grad_accumulator(p)]
        if stale:
            raise RuntimeError(f"GraphedStep: {len(stale)} parameter(s) still have a gradient accumulator from an earlier step "
                               "(an autograd graph of that step is alive: drop it, e.g. keep float(loss) instead of loss) -- a "
                               "backward captured now would run on the stream that accumulator was created on")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                fn(*self.static_inputs)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
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


def bench_dmft(steps: int = 5, device="cuda:0", compare_base: bool = True, only=None, variants=None, log=None) -> dict:
    """images/s for (a) DMFT-B/2 256px forward+JVP, batch 64, bf16 autocast,
    (b) DMFT-XL/2 256px forward+JVP+backward, batch 32, and (c) DMFT-B/2 primal-only
    no-grad forward at batch 128 -- the call mode of the guidance branch
    (loss.py:64-69, a 2B batch) and of a sampler step (samplers.py:69-100) -- and
    (d) DMFT-XL/2 at 512px (1024 tokens) with qk-norm, forward+JVP, batch 16: the
    caller of the headline attention shape, (e) the whole DMF training step of
    train_dmf.py on DMFT-XL/2 with model guidance (``dmf_train_step``: four model
    calls, two of them no-grad on a 2B batch), batch 16, and (f) the flow-matching
    training step of train_fm.py on SiT-XL/2 (``fm_train_step``), batch 32, and (g)
    generate.py's sampling loop: ``euler_sampler``, 4 steps with classifier-free
    guidance 1.5 on t in [0, 0.8], DMFT-XL/2 cast to bf16, batch 64 (images/s counts
    finished latents).  Variants:
    ``hip_fused_graph`` -- 'hip' attention + fused block glue, replayed as a HIP graph,
    ``hip_fused_fwad``  -- the same, launched eagerly with the forward-AD dual level opened directly,
    ``hip_fused``       -- the same, launched eagerly through ``torch.func.jvp`` (the reference's call),
    ``hip``             -- 'hip' attention inside the reference's tensor expressions,
    ``base``            -- naive attention (the reference's own CPU-runnable operator).
    ``only`` (a key or a collection of keys) / ``variants`` restrict the cases / the variants that are run; ``log(text)``
    is called after every measurement."""
    out = {}
    # (key, model, batch, dmf_depth, mode, latent size, qk_norm)
    all_cases = [("DMFT-B/2", "DMFT-B/2", 64, 8, "jvp", 32, False), ("DMFT-XL/2", "DMFT-XL/2", 32, 20, "train", 32, False),
                 ("DMFT-B/2 no-grad", "DMFT-B/2", 128, 8, "nograd", 32, False),
                 ("DMFT-XL/2 512px qk-norm", "DMFT-XL/2", 16, 20, "jvp", 64, True),
                 ("DMFT-XL/2 512px qk-norm train", "DMFT-XL/2", 8, 20, "train", 64, True),
                 ("DMFT-XL/2 DMF loss step (mg)", "DMFT-XL/2", 16, 20, "dmf_loss", 32, False),
                 ("SiT-XL/2 FM train step", "SiT-XL/2", 32, None, "fm", 32, False),
                 ("DMFT-XL/2 4-step sampling cfg 1.5", "DMFT-XL/2", 64, 20, "sample", 32, False)]
    wanted = None if only is None else ({only} if isinstance(only, str) else set(only))
    cases = [c for c in all_cases if wanted is None or c[0] in wanted]
    all_variants = [("hip_fused_graph", "hip", "hip", True), ("hip_fused_fwad", "hip", "hip", False), ("hip_fused", "hip", "hip", False),
                    ("hip", "hip", "torch", False)]
    if compare_base:
        all_variants.append(("base", "base", "torch", False))
    if variants is not None and "torch_sdpa" in variants:   # the reference's third operator value, only on request
        all_variants.append(("torch_sdpa", "torch_sdpa", "torch", False))
    variants = [v for v in all_variants if variants is None or v[0] in variants]
    modes = {"jvp": "fwd+jvp", "train": "fwd+jvp+bwd", "nograd": "primal-only forward, no grad (guidance / sampler call)",
             "dmf_loss": "fwd(grad) + 2x guidance fwd (no grad, 2B) + fwd+jvp, then bwd", "fm": "fwd+bwd (no jvp)",
             "sample": "4 no-grad forwards (3 of them on a 2B batch) + fp64 Euler updates"}
    for key, name, batch, dmf_depth, mode, input_size, qk_norm in cases:
        row = {"batch": batch, "mode": modes[mode], "dtype": "bf16 model" if mode == "sample" else "bf16 autocast",
               "tokens": (input_size // 2) ** 2, "qk_norm": qk_norm}
        if mode == "dmf_loss":
            data = synthetic_loss_batch(batch, device, input_size=input_size)
        elif mode == "fm":
            x, y, _, t_fm, _, _, eps, _ = synthetic_loss_batch(batch, device, input_size=input_size)
            data = (x, y, t_fm, eps)
        elif mode == "sample":
            z, _, _, y, _ = synthetic_batch(batch, device, input_size=input_size)
            data = (z.to(torch.bfloat16), y)
        else:
            data = synthetic_batch(batch, device, input_size=input_size)
        for label, op, block_ops, graphed in variants:
            if mode in ("nograd", "fm", "sample") and label == "hip_fused_fwad":
                continue   # no JVP in this mode
            extra = {"use_logvar": True} if mode == "dmf_loss" else {}
            model = build_model(name, op, device, qk_norm=qk_norm, input_size=input_size, dmf_depth=dmf_depth, block_ops=block_ops,
                                **extra)
            functorch = label != "hip_fused_fwad"
            if mode == "sample":
                model = model.to(torch.bfloat16).eval().requires_grad_(False)     # generate.py:84-85

                def step(z, y):
                    return euler_sampler(model, z, y, num_steps=4, cfg_scale=1.5, g_min=0.0, g_max=0.8)
            elif mode == "dmf_loss":
                def step(*batch_tensors):
                    model.zero_grad(set_to_none=True)
                    return dmf_train_step(model, batch_tensors, functorch=functorch, g_type="mg", omega=0.5).detach()
            elif mode == "fm":
                def step(*batch_tensors):
                    model.zero_grad(set_to_none=True)
                    return fm_train_step(model, batch_tensors).detach()
            elif mode == "train":
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
            frozen = frozen_low_precision_params(model) if (mode in ("jvp", "nograd") and block_ops == "hip") else contextlib.nullcontext()
            with frozen:
                run = GraphedStep(step, *data, parameters=list(model.parameters())) if graphed else step
                sec = _time(lambda: run(*data), steps * 4 if graphed else (steps if op == "hip" else max(2, steps // 2)))
            row[f"{label}_ms_per_step"] = sec * 1e3
            row[f"{label}_images_per_s"] = batch / sec
            if log is not None:
                log(f"{key} [{label}]: {sec * 1e3:.2f} ms/step, {batch / sec:.1f} images/s")
            del model, run, step
            torch.cuda.empty_cache()
        out[key] = row
    return out
