"""DMFT harness (dmf_amd/dmft.py, dmf_amd/harness.py): structure checks on the
CPU with the 'base' operator, and on the GPU the judged end-to-end parity --
the model with the 'hip' attention against the same model (same weights, same
inputs) with the restated 'base' attention, through the MeanFlow JVP call
(reference loss.py:165-173) and the backward on the primal output."""
import pytest
import torch

from dmf_amd import harness
from dmf_amd.dmft import DMFT, DMFT_models
from oracle import attn_oracle as ao
from parity_util import grads, no_worse_than_base


def _small(attn_func, **kw):
    cfg = dict(input_size=8, patch_size=2, hidden_size=64, depth=3, num_heads=4, dmf_depth=2, attn_func=attn_func)
    cfg.update(kw)
    return DMFT(**cfg).init_trunc_normal_(0.02, seed=1)


def test_registry_matches_reference_sizes():
    # models/dmft.py:154-175: depth / hidden / heads per size, patch in {2,4,8}
    assert len(DMFT_models) == 15
    m = DMFT_models["DMFT-B/2"](attn_func="base")
    assert (len(m.blocks), m.num_heads, m.pos_embed.shape) == (12, 12, (1, 256, 768))
    assert sum(p.numel() for p in DMFT_models["DMFT-XL/2"](attn_func="base").parameters()) == 675_111_184 + 0


def test_reference_init_gives_zero_output_and_trunc_normal_does_not():
    """The reference zero-initialises the adaLN gates and the output layer
    (models/dmft.py:102-111), so its step-0 output is identically zero; the
    benchmark initialisation must not be."""
    z, t, r, y, v = harness.synthetic_batch(2, "cpu", input_size=8)
    m = DMFT(input_size=8, hidden_size=64, depth=2, num_heads=4, dmf_depth=1, attn_func="base")
    assert m(z, t, r, y).abs().max() == 0
    assert _small("base")(z, t, r, y).abs().max() > 0


def test_meanflow_jvp_matches_finite_differences_and_r_t_split():
    m = _small("base").double()
    z, t, r, y, v = (x.double() if x.is_floating_point() else x for x in harness.synthetic_batch(2, "cpu", input_size=8))
    u, du = harness.meanflow_jvp(m, z, t, r, y, v)
    h = 1e-6
    fd = (m(z + h * v, t + h, r, y) - m(z - h * v, t - h, r, y)) / (2 * h)
    assert ao.rel_l2(du, fd) < 1e-4   # the sinusoidal time embedding is computed in fp32 (models/layers.py:51)
    assert ao.rel_l2(u, m(z, t, r, y)) < 1e-14
    # encoder blocks see only t, decoder blocks and the final layer only r (models/dmft.py:134-141)
    seen = []
    hooks = [b.register_forward_hook(lambda mod, inp, out: seen.append(inp[1])) for b in m.blocks]
    m(z, t, r, y)
    for hk in hooks:
        hk.remove()
    assert torch.equal(seen[0], seen[1]) and not torch.equal(seen[1], seen[2])
    # loss target is detached: no gradient flows through du_dt
    loss, _, _ = harness.meanflow_loss(m, z, t, r, y, v)
    loss.backward()
    assert all(p.grad is not None for n, p in m.named_parameters() if p.requires_grad and "logvar" not in n)


@pytest.mark.gpu
@pytest.mark.parametrize("autocast,tol", [(False, 2e-4), (True, 3e-2)])
def test_dmft_hip_vs_base_jvp_and_grads(autocast, tol):
    """Head dim 72 (hidden 288 / 4 heads), N = 256 tokens, 4 blocks."""
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=4, num_heads=4, dmf_depth=3)
    m_hip, m_base = _small("hip", **kw).to(dev), _small("base", **kw).to(dev)
    m_base.load_state_dict(m_hip.state_dict())
    data = harness.synthetic_batch(4, dev)
    outs = []
    for m in (m_hip, m_base):
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            loss, u, du = harness.meanflow_loss(m, *data)
        loss.backward()
        outs.append((u.float().cpu(), du.float().cpu()))
    (u, du), (u_ref, du_ref) = outs
    assert ao.rel_l2(u, u_ref) <= tol, ao.rel_l2(u, u_ref)
    assert ao.rel_l2(du, du_ref) <= tol, ao.rel_l2(du, du_ref)
    worst = max(ao.rel_l2(p.grad.cpu(), q.grad.cpu()) for (n, p), (_, q) in zip(m_hip.named_parameters(), m_base.named_parameters())
                if p.grad is not None and float(q.grad.abs().max()) > 0)
    assert worst <= 5 * tol, worst


@pytest.mark.gpu
def test_dmft_hip_qk_norm_no_grad_sampling_path():
    """Primal-only, no-grad call (the sampler's mode, samplers.py:69-100) with qk-norm."""
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=2, num_heads=4, dmf_depth=1, qk_norm=True)
    m_hip, m_base = _small("hip", **kw).to(dev), _small("base", **kw).to(dev)
    m_base.load_state_dict(m_hip.state_dict())
    z, t, r, y, _ = harness.synthetic_batch(2, dev)
    with torch.no_grad():
        assert ao.rel_l2(m_hip(z, t, r, y).cpu(), m_base(z, t, r, y).cpu()) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("autocast,tol", [(False, 2e-4), (True, 3e-2)])
@pytest.mark.parametrize("qk_norm", [False, True])
def test_dmft_fused_block_ops_vs_torch_block_ops(autocast, tol, qk_norm):
    """Same model, weights and inputs; block glue (norm+modulate, gated residual,
    GELU, qk RMSNorm) through the fused kernels vs the reference's tensor
    expressions, both around the naive 'base' attention and around the 'hip' one.
    Under autocast the reference expressions round intermediate products to bf16
    (models/layers.py:29,42,198) where the fused kernels round once, hence the
    bf16-level tolerance there."""
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=4, num_heads=4, dmf_depth=3, qk_norm=qk_norm)
    m_ref = _small("base", **kw).to(dev)
    with torch.no_grad():   # non-trivial RMSNorm gains
        for n, p in m_ref.named_parameters():
            if n.endswith("_norm.scale"):
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=torch.Generator().manual_seed(7)).to(dev))
    data = harness.synthetic_batch(4, dev)

    def run(m):
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            loss, u, du = harness.meanflow_loss(m, *data)
        loss.backward()
        return u.float().cpu(), du.float().cpu()

    u_ref, du_ref = run(m_ref)
    for attn in ("base", "hip"):
        m = _small(attn, block_ops="hip", **kw).to(dev)
        m.load_state_dict(m_ref.state_dict())
        u, du = run(m)
        assert ao.rel_l2(u, u_ref) <= tol, (attn, ao.rel_l2(u, u_ref))
        assert ao.rel_l2(du, du_ref) <= tol, (attn, ao.rel_l2(du, du_ref))
        worst = max((ao.rel_l2(p.grad.cpu(), q.grad.cpu()), n) for (n, p), (_, q) in zip(m.named_parameters(), m_ref.named_parameters())
                    if q.grad is not None and float(q.grad.abs().max()) > 0)
        assert all(p.grad is not None for (n, p), (_, q) in zip(m.named_parameters(), m_ref.named_parameters()) if q.grad is not None)
        assert worst[0] <= 5 * tol, (attn, worst)


@pytest.mark.gpu
def test_dmft_fused_block_ops_no_grad_and_plain_forward():
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=2, num_heads=4, dmf_depth=1, qk_norm=True)
    m_f, m_ref = _small("hip", block_ops="hip", **kw).to(dev), _small("base", **kw).to(dev)
    m_ref.load_state_dict(m_f.state_dict())
    z, t, r, y, _ = harness.synthetic_batch(2, dev)
    with torch.no_grad():
        assert ao.rel_l2(m_f(z, t, r, y).cpu(), m_ref(z, t, r, y).cpu()) < 1e-4


def test_unknown_block_ops_raises():
    with pytest.raises(ValueError):
        _small("base", block_ops="nope")


def test_patch_embed_equals_strided_convolution():
    """models/dmft.py:54-56 uses timm's PatchEmbed (a kernel=stride convolution); the
    harness evaluates it as a Linear over flattened patches with the same parameters."""
    from dmf_amd.dmft import PatchEmbed
    pe = PatchEmbed(16, 4, 3, 40, block_ops="hip").double()
    x = torch.randn(2, 3, 16, 16, dtype=torch.float64)
    ref = pe.proj(x).flatten(2).transpose(1, 2)
    assert torch.allclose(pe(x), ref, atol=1e-12)
    pe.fused = False
    assert torch.equal(pe(x), ref)
    assert pe.proj.weight.shape == (40, 3, 4, 4)


def test_meanflow_jvp_direct_dual_level_equals_func_jvp():
    m = _small("base").double()
    z, t, r, y, v = (x.double() if x.is_floating_point() else x for x in harness.synthetic_batch(2, "cpu", input_size=8))
    u1, du1 = harness.meanflow_jvp(m, z, t, r, y, v, functorch=True)
    u2, du2 = harness.meanflow_jvp(m, z, t, r, y, v, functorch=False)
    # same formulas; functorch decomposes a few ATen ops differently, so agreement is to rounding, not bitwise
    assert torch.equal(u1, u2) and ao.rel_l2(du2, du1) < 1e-13


@pytest.mark.gpu
def test_fused_train_step_direct_dual_level_equals_func_jvp():
    dev = "cuda:0"
    m = _small("hip", block_ops="hip", input_size=32, hidden_size=288, depth=3, num_heads=4, dmf_depth=2).to(dev)
    data = harness.synthetic_batch(4, dev)
    grads = []
    for functorch in (True, False):
        m.zero_grad(set_to_none=True)
        loss = harness.train_step(m, data, functorch=functorch)
        grads.append((loss.detach().clone(), {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}))
    # same kernels on both routes; the ATen ops around them may round differently under bf16 autocast
    assert abs(float(grads[0][0]) - float(grads[1][0])) <= 1e-3 * abs(float(grads[0][0]))
    assert grads[0][1].keys() == grads[1][1].keys()
    worst = max(ao.rel_l2(grads[1][1][n].cpu(), grads[0][1][n].cpu()) for n in grads[0][1] if float(grads[0][1][n].abs().max()) > 0)
    assert worst <= 2e-2, worst


@pytest.mark.gpu
def test_dmft_b2_full_architecture_fused_graph_vs_base():
    """The DMFT-B/2 forward+JVP benchmark model at its real architecture (DMFT-B/2: 12 blocks, hidden 768, 12 heads of 64, 256 tokens,
    dmf_depth 8), reduced batch: forward+JVP under bf16 autocast through the fused path replayed as a HIP graph,
    against the same weights with the naive attention and the reference's expressions run eagerly."""
    dev = "cuda:0"
    m_ref = harness.build_model("DMFT-B/2", "base", dev, dmf_depth=8)
    m = harness.build_model("DMFT-B/2", "hip", dev, dmf_depth=8, block_ops="hip")
    m.load_state_dict(m_ref.state_dict())
    m.requires_grad_(False)
    m_ref.requires_grad_(False)
    data = harness.synthetic_batch(8, dev)

    def step(z, t, r, y, v):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return harness.meanflow_jvp(m, z, t, r, y, v)

    graphed = harness.GraphedStep(step, *data)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        u_ref, du_ref = harness.meanflow_jvp(m_ref, *data)
    for _ in range(2):
        u, du = graphed(*data)
        assert ao.rel_l2(u.float().cpu(), u_ref.float().cpu()) <= 3e-2
        assert ao.rel_l2(du.float().cpu(), du_ref.float().cpu()) <= 3e-2


@pytest.mark.gpu
def test_dmft_xl2_config5_train_step_fused_and_graph_vs_base():
    """The full DMFT-XL/2 256px training step at its real architecture (models/dmft.py:170: 28 blocks, hidden 1152,
    16 heads of 72, 256 tokens; dmf_depth 20), random trunc-normal weights, reduced batch: forward + JVP through the new
    attention and the fused block glue, then backward on the primal output with the JVP target detached
    (loss.py:165-173, train_dmf.py:320-335), eagerly and replayed as a HIP graph.  Yardstick: the same weights and
    inputs through the naive attention and the reference's expressions in fp32; the bf16-autocast reference path
    measures how far rounding alone moves u, du/dt, the loss and every parameter gradient, and the fused path may
    move them at most 1.5 times as far."""
    dev = "cuda:0"
    m_ref = harness.build_model("DMFT-XL/2", "base", dev, dmf_depth=20)
    assert (len(m_ref.blocks), m_ref.num_heads, m_ref.pos_embed.shape, m_ref.dmf_depth) == (28, 16, (1, 256, 1152), 20)
    data = harness.synthetic_batch(2, dev)

    def run(model, autocast):
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            loss, u, du = harness.meanflow_loss(model, *data)
        loss.backward()
        return float(loss), u.detach().float().cpu(), du.detach().float().cpu(), grads(model)

    l32, u32, du32, g32 = run(m_ref, False)
    lb, ub, dub, gb = run(m_ref, True)
    m = harness.build_model("DMFT-XL/2", "hip", dev, dmf_depth=20, block_ops="hip")
    m.load_state_dict(m_ref.state_dict())
    del m_ref
    lf, uf, duf, gf = run(m, True)
    eu, edu = ao.rel_l2(ub, u32), ao.rel_l2(dub, du32)
    print(f"base-bf16 vs fp32: u {eu:.3e} du {edu:.3e} loss {abs(lb - l32) / abs(l32):.3e}; "
          f"fused: u {ao.rel_l2(uf, u32):.3e} du {ao.rel_l2(duf, du32):.3e} loss {abs(lf - l32) / abs(l32):.3e}", flush=True)
    assert ao.rel_l2(uf, u32) <= 1.5 * eu + 2e-3 and ao.rel_l2(duf, du32) <= 1.5 * edu + 2e-3
    assert abs(lf - l32) <= 1.5 * abs(lb - l32) + 2e-3 * abs(l32)
    no_worse_than_base(gf, gb, g32)
    del gb, g32

    # the same step captured once and replayed: same loss and gradients as the eager fused step, to rounding
    def step(*b):
        m.zero_grad(set_to_none=True)
        return harness.train_step(m, b, functorch=False).detach()

    m.zero_grad(set_to_none=True)
    eager_loss = float(step(*data))
    eager = grads(m)
    m.zero_grad(set_to_none=True)
    graphed = harness.GraphedStep(step, *data)
    for _ in range(2):
        out = graphed(*data)
        torch.cuda.synchronize()
        assert abs(float(out) - eager_loss) <= 1e-3 * abs(eager_loss)
        got = grads(m)
        worst = max((ao.rel_l2(got[n], eager[n]), n) for n in eager if float(eager[n].abs().max()) > 0)
        assert worst[0] <= 2e-3, worst


@pytest.mark.gpu
@pytest.mark.parametrize("name,qk_norm", [("DMFT-S/2", False), ("DMFT-B/4", True), ("DMFT-L/8", False), ("DMFT-M/4", True)])
def test_registry_models_fused_vs_base(name, qk_norm):
    """Other sizes of the reference's registry (models/dmft.py:154-175): head dim 64, hidden 384 / 768 / 1024,
    64 and 16 tokens (patch 4 and 8): forward+JVP and gradients, fused path vs the reference expressions, fp32."""
    dev = "cuda:0"
    m_ref = harness.build_model(name, "base", dev, qk_norm=qk_norm, dmf_depth=2)
    m = harness.build_model(name, "hip", dev, qk_norm=qk_norm, dmf_depth=2, block_ops="hip")
    m.load_state_dict(m_ref.state_dict())
    data = harness.synthetic_batch(2, dev)
    outs = []
    for mod in (m, m_ref):
        loss, u, du = harness.meanflow_loss(mod, *data)
        loss.backward()
        outs.append((u.detach().cpu(), du.detach().cpu()))
    assert ao.rel_l2(outs[0][0], outs[1][0]) <= 2e-4 and ao.rel_l2(outs[0][1], outs[1][1]) <= 2e-4
    worst = max(ao.rel_l2(p.grad.cpu(), q.grad.cpu()) for (n, p), (_, q) in zip(m.named_parameters(), m_ref.named_parameters())
                if q.grad is not None and float(q.grad.abs().max()) > 0)
    assert worst <= 1e-3, worst


@pytest.mark.gpu
def test_frozen_low_precision_params_give_the_same_bits():
    """Cached bf16 parameter copies are exactly what autocast would cast per call."""
    from dmf_amd.layers import frozen_low_precision_params
    dev = "cuda:0"
    m = _small("hip", block_ops="hip", input_size=32, hidden_size=288, depth=2, num_heads=4, dmf_depth=1).to(dev)
    m.requires_grad_(False)
    data = harness.synthetic_batch(4, dev)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        u0, du0 = harness.meanflow_jvp(m, *data)
        with frozen_low_precision_params(m):
            assert m.blocks[0].attn.qkv.lp_weight.dtype == torch.bfloat16
            u1, du1 = harness.meanflow_jvp(m, *data)
        assert m.blocks[0].attn.qkv.lp_weight is None
    assert torch.equal(u0, u1) and torch.equal(du0, du1)
    # and training through cached copies still sends gradients to the fp32 parameters
    m.requires_grad_(True)
    with frozen_low_precision_params(m):
        harness.train_step(m, data)
    assert m.blocks[0].attn.qkv.weight.grad is not None and m.blocks[0].attn.qkv.weight.grad.dtype == torch.float32


@pytest.mark.gpu
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("block_ops", ["torch", "hip"])
def test_torch_compile(backend, block_ops):
    """The reference compiles the model it calls without JVP (train_dmf.py:269-275).
    With the reference's own block expressions the 'hip' attention is traced as one
    registered operator (``dmf_amd::attn_fwd`` / ``attn_bwd``), so even
    ``fullgraph=True`` works; the fused block glue is reached through ctypes and runs
    eagerly between compiled pieces (graph breaks).  Same outputs and gradients as the
    eager model either way."""
    dev = "cuda:0"
    m = _small("hip", input_size=16, hidden_size=128, num_heads=2, qk_norm=True, block_ops=block_ops).to(dev)
    z, t, r, y, _ = harness.synthetic_batch(4, dev, input_size=16)
    ref = m(z, t, r, y)
    ref.square().mean().backward()
    g_ref = {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}
    m.zero_grad(set_to_none=True)
    torch._dynamo.reset()
    cm = torch.compile(m, backend=backend, dynamic=True, fullgraph=block_ops == "torch")
    out = cm(z, t, r, y)
    out.square().mean().backward()
    assert ao.rel_l2(out, ref) <= 1e-5
    for n, p in m.named_parameters():
        if n in g_ref and float(g_ref[n].abs().max()) > 0:
            assert ao.rel_l2(p.grad, g_ref[n]) <= 1e-4, n
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert ao.rel_l2(cm(z, t, r, y).float(), ref) <= 3e-2
    torch._dynamo.reset()
