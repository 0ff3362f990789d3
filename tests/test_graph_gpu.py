"""HIP-graph replay of the fused MeanFlow step (dmf_amd.harness.GraphedStep).

A captured graph must give, on every replay, what the eager step gives on the
same inputs -- with unrelated eager work and host synchronisation between
replays, and with inputs that change from replay to replay.  (A reduction that
clears scratch memory through a memset node passes the first replay and fails
later ones, by factors of 1 to 1000 relative; this is the test that catches it.)
The kernels are the same on both routes, so results normally agree bit for bit;
the assertions allow rounding-level differences (a library GEMM may pick a
different accumulation order from one launch to the next) and nothing more."""
import pytest
import torch

from dmf_amd import harness
from dmf_amd.dmft import DMFT
from oracle import attn_oracle as ao

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3   # relative L2; bf16 rounding of one GEMM output is ~4e-3 per element


def _same(a, b):
    return torch.equal(a, b) or ao.rel_l2(a.float().cpu(), b.float().cpu()) <= TOL


def _model(**kw):
    cfg = dict(input_size=32, patch_size=2, hidden_size=576, depth=3, num_heads=8, dmf_depth=2, attn_func="hip", block_ops="hip")
    cfg.update(kw)
    return DMFT(**cfg).init_trunc_normal_(0.02, seed=1).to(DEV)


def _eager_noise():
    a = torch.randn(512, 512, device=DEV)
    return float((a @ a).sum())


def test_graphed_jvp_step_replays_match_eager():
    model = _model(qk_norm=True)
    model.requires_grad_(False)

    def fn(z, t, r, y, v):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return harness.meanflow_jvp(model, z, t, r, y, v)

    batches = [harness.synthetic_batch(8, DEV, seed=s) for s in (2, 3, 4)]
    eager = [tuple(o.clone() for o in fn(*b)) for b in batches]
    step = harness.GraphedStep(fn, *batches[0])
    for rep in range(2):
        for b, (u_ref, du_ref) in zip(batches, eager):
            u, du = step(*b)
            torch.cuda.synchronize()
            assert _same(u, u_ref) and _same(du, du_ref), f"replay {rep} differs from eager"
            _eager_noise()


def test_graphed_train_step_replays_match_eager():
    model = _model(hidden_size=2304 // 4, depth=2, dmf_depth=1)   # qkv width 1728, fc1 width 2304: multi-block bias sums
    params = dict(model.named_parameters())
    # the strided-convolution weight gradient (MIOpen) is not run-to-run reproducible even in eager mode
    exact = [n for n in params if n != "x_embedder.proj.weight"]

    def fn(z, t, r, y, v):
        model.zero_grad(set_to_none=True)
        return harness.train_step(model, (z, t, r, y, v)).detach()

    batches = [harness.synthetic_batch(16, DEV, seed=s) for s in (2, 3, 4)]
    eager = []
    for b in batches:
        loss = fn(*b)
        eager.append((loss.clone(), {n: params[n].grad.clone() for n in exact if params[n].grad is not None}))
    del loss
    model.zero_grad(set_to_none=True)
    step = harness.GraphedStep(fn, *batches[0])
    for rep in range(2):
        for b, (loss_ref, grads_ref) in zip(batches, eager):
            loss = step(*b)
            torch.cuda.synchronize()
            assert _same(loss, loss_ref)
            bad = [n for n, g in grads_ref.items() if not _same(params[n].grad, g)]
            assert not bad, f"replay {rep}: gradients differ from eager for {bad[:6]}"
            _eager_noise()


def test_graphed_step_refuses_capture_while_an_earlier_graph_is_alive():
    """A backward captured while an earlier step's autograd graph is alive would use gradient accumulators bound to
    another stream (a runtime crash, not an error): the constructor refuses it on the host when it is given the parameters."""
    model = harness.build_model("DMFT-B/2", "hip", DEV, dmf_depth=8, block_ops="hip")
    batch = harness.synthetic_batch(2, DEV, seed=5)

    def fn(z, t, r, y, v):
        model.zero_grad(set_to_none=True)
        return harness.train_step(model, (z, t, r, y, v)).detach()

    kept = harness.train_step(model, batch)           # an attached loss: its graph stays alive
    with pytest.raises(RuntimeError, match="gradient accumulator from an earlier step"):
        harness.GraphedStep(fn, *batch, parameters=list(model.parameters()))
    del kept
    model.zero_grad(set_to_none=True)
    step = harness.GraphedStep(fn, *batch, parameters=list(model.parameters()))
    assert torch.isfinite(step(*batch)).all()
