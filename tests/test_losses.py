"""The training-loss call sites around the operator (dmf_amd/harness.py:
``interpolant``, ``compute_guidance``, ``log_lv_loss``, ``dmf_loss``, ``fm_loss``)
and the single-time SiT model (dmf_amd/sit.py).  On the CPU: closed forms and
invariants that a dropped term, a wrong sign or a swapped argument breaks.  On the
GPU: the whole DMF / flow-matching training step with the 'hip' attention and the
fused block glue against the same weights with the naive 'base' attention and the
reference's tensor expressions (reference loss.py:142-181, 208-231)."""
import math

import pytest
import torch

from dmf_amd import harness
from dmf_amd.dmft import DMFT
from dmf_amd.sit import SiT, SiT_models
from oracle import attn_oracle as ao
from parity_util import no_worse_than_base


def _dmft(attn_func, **kw):
    cfg = dict(input_size=8, patch_size=2, hidden_size=64, depth=3, num_heads=4, dmf_depth=2, attn_func=attn_func, use_logvar=True)
    cfg.update(kw)
    m = DMFT(**cfg).init_trunc_normal_(0.02, seed=1)
    if not m.use_logvar:
        return m
    with torch.no_grad():   # a log-variance head that is not identically zero
        m.logvar_linear.weight.copy_(0.05 * torch.randn(m.logvar_linear.weight.shape, generator=torch.Generator().manual_seed(3)))
        m.logvar_linear.bias.fill_(0.1)
    return m


def _sit(attn_func, **kw):
    cfg = dict(input_size=8, patch_size=2, hidden_size=64, depth=3, num_heads=4, attn_func=attn_func)
    cfg.update(kw)
    return SiT(**cfg).init_trunc_normal_(0.02, seed=2)


def test_interpolant_closed_forms():
    g = torch.Generator().manual_seed(0)
    x, eps = torch.randn(3, 4, 8, 8, generator=g).double(), torch.randn(3, 4, 8, 8, generator=g).double()
    t = torch.rand(3, 1, 1, 1, generator=g).double()
    for path in ("linear", "cosine"):
        x0, _ = harness.interpolant(x, torch.zeros_like(t), eps, path)
        x1, _ = harness.interpolant(x, torch.ones_like(t), eps, path)
        assert torch.allclose(x0, x) and torch.allclose(x1, eps, atol=1e-15)          # data at t=0, noise at t=1
        h = 1e-6
        xt, vt = harness.interpolant(x, t, eps, path)
        fd = (harness.interpolant(x, t + h, eps, path)[0] - harness.interpolant(x, t - h, eps, path)[0]) / (2 * h)
        assert ao.rel_l2(vt, fd) < 1e-8                                                # v_t = d x_t / dt
    _, v_lin = harness.interpolant(x, t, eps, "linear")
    assert torch.equal(v_lin, eps - x)
    a, s = torch.cos(t * math.pi / 2), torch.sin(t * math.pi / 2)
    assert torch.allclose(harness.interpolant(x, t, eps, "cosine")[0], a * x + s * eps)
    with pytest.raises(NotImplementedError):
        harness.interpolant(x, t, eps, "vp")


def test_log_lv_loss_known_values_and_reference_broadcast():
    x, y = torch.zeros(2, 1, 2, 2), torch.ones(2, 1, 2, 2)
    y[1] *= 3
    lv = torch.zeros(2, 1, 1, 1)
    sq, lp = harness.log_lv_loss(x, y, lv)
    assert sq.tolist() == [4.0, 36.0]
    # lv is (B,1,1,1) and the per-sample mean (B,), so the reference's expression (loss.py:34) is an outer
    # broadcast to (B,1,1,B); with lv = 0 every row holds log(mean + 0.01)
    assert lp.shape == (2, 1, 1, 2)
    assert torch.allclose(lp[0, 0, 0], torch.log(torch.tensor([1.01, 9.01])))
    lv2 = torch.tensor([0.5, -1.0]).view(2, 1, 1, 1)
    _, lp2 = harness.log_lv_loss(x, y, lv2)
    assert math.isclose(float(lp2[1, 0, 0, 0]), math.log(math.e * 1.0 + 0.01) - 1.0, abs_tol=1e-6)
    sq2, m2 = harness.mse_loss(x, y)
    assert sq2.tolist() == [4.0, 36.0] and m2.tolist() == [1.0, 9.0]


class _Stub(torch.nn.Module):
    """Returns +1 on rows with a real label and -2 on null-class rows; records its call."""

    def __init__(self, single_time):
        super().__init__()
        self.single_time, self.calls = single_time, []

    def forward(self, x, t, *rest):
        y = rest[-1]
        assert len(rest) == (1 if self.single_time else 2)
        if not self.single_time:
            assert torch.equal(rest[0], t)                       # model(x, t, t, y): r = t in the guidance call
        self.calls.append((x.shape[0], y.clone(), torch.is_grad_enabled()))
        return torch.where(y == 1000, -2.0, 1.0).view(-1, 1, 1, 1).expand_as(x).clone()


def test_compute_guidance_modes():
    B = 4
    x, v_t = torch.zeros(B, 1, 2, 2), torch.full((B, 1, 2, 2), 10.0)
    t = torch.tensor([0.1, 0.5, 0.5, 0.9]).view(B, 1, 1, 1)
    y = torch.tensor([3, 7, 1000, 5])
    drop = torch.tensor([False, False, True, False])
    assert harness.compute_guidance(None, x, t, y, v_t, drop) is v_t                       # default: no model call
    stub = _Stub(single_time=False)
    out = harness.compute_guidance(stub, x, t, y, v_t, drop, omega=0.5, g_min=0.3, g_max=1.0, g_type="mg")
    n, y2, grad = stub.calls[0]
    assert n == 2 * B and not grad and y2.tolist() == [3, 7, 1000, 5, 1000, 1000, 1000, 1000]
    # v_t + omega (v_cond - v_uncond) = 10 + 0.5 * 3 where t in range and the label was kept; else v_t
    assert out[:, 0, 0, 0].tolist() == [10.0, 11.5, 10.0, 11.5]
    stub = _Stub(single_time=True)
    out = harness.compute_guidance(stub, x, t, y, v_t, drop, omega=2.0, g_min=0.3, g_max=0.6, g_type="distill")
    # in range: v_uncond + omega (v_cond - v_uncond) = -2 + 2 * 3 = 4 (row 2: its own label is the null class -> -2);
    # out of range: v_cond; class dropout is ignored (loss.py:83)
    assert out[:, 0, 0, 0].tolist() == [1.0, 4.0, -2.0, 1.0]
    with pytest.raises(NotImplementedError):
        harness.compute_guidance(stub, x, t, y, v_t, drop, g_type="cfg")


def test_dmf_loss_invariants_cpu():
    m = _dmft("base").double()
    m.logvar_linear.float()     # its input, the sinusoidal embedding, is fp32 whatever the model's dtype (models/layers.py:51)
    batch = [v.double() if v.is_floating_point() else v for v in harness.synthetic_loss_batch(3, "cpu", input_size=8)]
    x, y, drop, t_fm, t_mf, r_mf, e_fm, e_mf = batch
    loss, parts = harness.dmf_loss(m, *batch)
    assert loss.shape == (3, 1, 1, 3) and set(parts) == {"fm_loss", "fm_p_loss", "mf_p_loss", "mf_loss"}
    assert torch.equal(loss, 0.5 * (parts["fm_p_loss"] + parts["mf_p_loss"]))
    # forward-AD dual level opened directly = torch.func.jvp
    loss2, _ = harness.dmf_loss(m, *batch, functorch=False)
    assert ao.rel_l2(loss2, loss) < 1e-12
    # r = t removes the tangent from the target (u_tgt = v + (r - t) du/dt), and the model is then called exactly
    # as in the flow-matching branch: same times and noise in both branches -> the two halves of the loss coincide
    _, p = harness.dmf_loss(m, x, y, drop, t_fm, t_fm, t_fm, e_fm, e_fm)
    assert ao.rel_l2(p["mf_p_loss"], p["fm_p_loss"]) < 1e-12 and ao.rel_l2(p["mf_loss"], p["fm_loss"]) < 1e-12
    # the MeanFlow target against central differences of the model along (v, 1, 0)
    h = 1e-6
    x_t, v_t = harness.interpolant(x, t_mf, e_mf)
    with torch.no_grad():
        fd = (m(x_t + h * v_t, t_mf + h, r_mf, y) - m(x_t - h * v_t, t_mf - h, r_mf, y)) / (2 * h)
        u, lv = m(x_t, t_mf, r_mf, y, return_logvar=True)
        want = harness.log_lv_loss(u, v_t + (r_mf - t_mf) * fd, lv)[0]
    assert ao.rel_l2(parts["mf_loss"], want) < 1e-4      # the time embedding is computed in fp32 (models/layers.py:51)
    # gradients reach every parameter, the log-variance head included; none flows through the targets
    loss.mean().backward()
    assert all(q.grad is not None and float(q.grad.abs().max()) > 0 for n, q in m.named_parameters() if q.requires_grad)


def test_dmf_loss_guidance_uses_the_teacher_without_grad():
    m, teacher = _dmft("base"), _sit("base")
    batch = harness.synthetic_loss_batch(3, "cpu", input_size=8, cfg_prob=0.5)
    loss, _ = harness.dmf_loss(m, *batch, model_t=teacher, g_type="distill", omega=1.5)
    loss.mean().backward()
    assert all(q.grad is None for q in teacher.parameters())
    loss_mg, _ = harness.dmf_loss(m, *batch, g_type="mg", omega=0.7)
    loss_plain, _ = harness.dmf_loss(m, *batch)
    assert not torch.allclose(loss_mg, loss_plain) and not torch.allclose(loss, loss_plain)
    # omega = 0 switches model guidance off
    assert torch.equal(harness.dmf_loss(m, *batch, g_type="mg", omega=0.0)[0], loss_plain)


def test_sit_structure_matches_reference():
    # models/sit.py:149-175: depth / hidden / heads per size, patch in {2,4,8}
    assert len(SiT_models) == 15
    m = SiT_models["SiT-B/2"](attn_func="base")
    assert (len(m.blocks), m.num_heads, m.pos_embed.shape) == (12, 12, (1, 256, 768))
    keys = set(SiT_models["SiT-S/8"](attn_func="base", repa_depth=2, z_dims=(32, 48), projector_dim=64).state_dict())
    for k in ("pos_embed", "x_embedder.proj.weight", "t_embedder.mlp.0.weight", "t_embedder.mlp.2.bias",
              "y_embedder.embedding_table.weight", "projectors.0.0.weight", "projectors.1.4.bias", "blocks.0.attn.qkv.weight",
              "blocks.11.attn.proj.bias", "blocks.0.mlp.fc1.weight", "blocks.0.mlp.fc2.bias", "blocks.0.adaLN_modulation.1.weight",
              "final_layer.linear.weight", "final_layer.adaLN_modulation.1.bias"):
        assert k in keys, k
    # the reference's initialisation zeroes the gates and the output layer (models/sit.py:110-120)
    x, y, _, t, *_ = harness.synthetic_loss_batch(2, "cpu", input_size=8)
    assert SiT(input_size=8, hidden_size=64, depth=2, num_heads=4, attn_func="base")(x, t, y).abs().max() == 0
    s = _sit("base", repa_depth=2, z_dims=(32,), projector_dim=48)
    out, feats = s(x, t, y, return_feat=True)
    assert out.shape == x.shape and len(feats) == 1 and feats[0].shape == (2, 16, 32)
    assert torch.equal(s(x, t, y), out)
    # the projector taps the residual stream after block `repa_depth` (models/sit.py:141-142)
    seen = []
    hk = s.blocks[1].register_forward_hook(lambda mod, inp, o: seen.append(o))
    s(x, t, y)
    hk.remove()
    assert torch.allclose(feats[0], s.projectors[0](seen[0].reshape(-1, 64)).reshape(2, 16, -1))
    # a DMFT whose two times coincide conditions every block on the same vector, as SiT does: same weights -> same output
    d = DMFT(input_size=8, patch_size=2, hidden_size=64, depth=3, num_heads=4, dmf_depth=2, attn_func="base")
    d.load_state_dict(_sit("base").state_dict())
    assert torch.allclose(d(x, t, t, y), _sit("base")(x, t, y), atol=1e-6)


def _grads(m):
    return {n: p.grad.float().cpu() for n, p in m.named_parameters() if p.grad is not None}


def _worst(ga, gb):
    assert ga.keys() == gb.keys()
    return max((ao.rel_l2(ga[n], gb[n]), n) for n in ga if float(gb[n].abs().max()) > 0)


@pytest.mark.gpu
@pytest.mark.parametrize("g_type", ["default", "mg", "distill"])
def test_dmf_train_step_fused_vs_base(g_type):
    """The whole DMF training step (four model calls) under bf16 autocast: 'hip'
    attention + fused block glue, eager through ``torch.func.jvp``, eager with the
    dual level opened directly, and replayed as a HIP graph, against the same
    weights with the naive attention and the reference's expressions."""
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=4, num_heads=4, dmf_depth=3)
    m_ref = _dmft("base", **kw).to(dev)
    m = _dmft("hip", block_ops="hip", **kw).to(dev)
    m.load_state_dict(m_ref.state_dict())
    t_ref = t_hip = None
    if g_type == "distill":
        t_ref = _sit("base", input_size=32, hidden_size=288, depth=3, num_heads=4).to(dev).requires_grad_(False)
        t_hip = _sit("hip", block_ops="hip", input_size=32, hidden_size=288, depth=3, num_heads=4).to(dev).requires_grad_(False)
        t_hip.load_state_dict(t_ref.state_dict())
    batch = harness.synthetic_loss_batch(4, dev, cfg_prob=0.25)
    guidance = dict(g_type=g_type, omega=0.6, g_min=0.0, g_max=1.0)
    fp32_loss = float(harness.dmf_train_step(m_ref, batch, model_t=t_ref, autocast=False, **guidance))
    g_fp32 = _grads(m_ref)
    m_ref.zero_grad(set_to_none=True)
    ref_loss = float(harness.dmf_train_step(m_ref, batch, model_t=t_ref, **guidance))
    g_ref = _grads(m_ref)
    for functorch in (True, False):
        m.zero_grad(set_to_none=True)
        loss = float(harness.dmf_train_step(m, batch, model_t=t_hip, functorch=functorch, **guidance))
        assert abs(loss - fp32_loss) <= 1.5 * abs(ref_loss - fp32_loss) + 2e-3 * abs(fp32_loss), (functorch, loss, ref_loss, fp32_loss)
        no_worse_than_base(_grads(m), g_ref, g_fp32)
    eager = _grads(m)
    # (no autograd graph of an earlier step may be alive while the step is captured: only floats are kept above)

    def step(*b):
        m.zero_grad(set_to_none=True)
        return harness.dmf_train_step(m, b, model_t=t_hip, functorch=False, **guidance).detach()

    m.zero_grad(set_to_none=True)
    graphed = harness.GraphedStep(step, *batch)
    for _ in range(3):
        out = graphed(*batch)
        torch.cuda.synchronize()
        assert abs(float(out) - loss) <= 1e-3 * abs(loss) + 1e-5
        worst = _worst(_grads(m), eager)
        assert worst[0] <= 2e-3, worst


@pytest.mark.gpu
def test_fm_train_step_sit_fused_vs_base():
    """Flow-matching training step of a SiT (plain forward + backward: the primal
    forward kernel with lse, the backward kernels, the primal-only block glue)."""
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=4, num_heads=4, qk_norm=True)
    m_ref = _sit("base", **kw).to(dev)
    m = _sit("hip", block_ops="hip", **kw).to(dev)
    m.load_state_dict(m_ref.state_dict())
    x, y, _, t, _, _, eps, _ = harness.synthetic_loss_batch(4, dev)
    fp32 = float(harness.fm_train_step(m_ref, (x, y, t, eps), autocast=False))
    g_fp32 = _grads(m_ref)
    m_ref.zero_grad(set_to_none=True)
    ref = float(harness.fm_train_step(m_ref, (x, y, t, eps)))
    got = float(harness.fm_train_step(m, (x, y, t, eps)))
    assert abs(got - fp32) <= 1.5 * abs(ref - fp32) + 2e-3 * abs(fp32), (got, ref, fp32)
    no_worse_than_base(_grads(m), _grads(m_ref), g_fp32)
    # fp32 (no autocast): tight
    m.zero_grad(set_to_none=True)
    m_ref.zero_grad(set_to_none=True)
    for mod in (m, m_ref):
        loss, _ = harness.fm_loss(mod, x, y, t, eps)
        loss.mean().backward()
    worst = _worst(_grads(m), _grads(m_ref))
    assert worst[0] <= 2e-3, worst


@pytest.mark.gpu
def test_sit_projector_features_fused_vs_torch_under_jvp():
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=3, num_heads=4, repa_depth=2, z_dims=(64,), projector_dim=96)
    m_ref = _sit("base", **kw).to(dev)
    m = _sit("hip", block_ops="hip", **kw).to(dev)
    m.load_state_dict(m_ref.state_dict())
    x, y, _, t, _, _, eps, _ = harness.synthetic_loss_batch(4, dev)
    f = lambda mod: torch.func.jvp(lambda a, b: mod(a, b, y, return_feat=True), (x, t), (eps, torch.ones_like(t)))
    (o1, z1), (to1, tz1) = f(m)
    (o2, z2), (to2, tz2) = f(m_ref)
    for a, b in ((o1, o2), (z1[0], z2[0]), (to1, to2), (tz1[0], tz2[0])):
        assert ao.rel_l2(a, b) <= 2e-4


# ---- sampling loop (dmf_amd/samplers.py) ---------------------------------------------------------------------------

def test_get_tsteps_closed_form():
    from dmf_amd.samplers import get_tsteps
    t = get_tsteps(4)
    assert t.dtype == torch.float64 and t.tolist() == [1.0, 0.75, 0.5, 0.25, 0.0]
    s = get_tsteps(4, shift=3.0)
    assert torch.allclose(s, 3 * t / (1 + 2 * t)) and s[0] == 1.0 and s[-1] == 0.0 and float(s[2]) == 0.75


class _Field(torch.nn.Module):
    """d(x, t, r, y) = a(y) * x + t - 2 r with a = 1 for real labels and 3 for the null class; records (n, t, r)."""

    def __init__(self):
        super().__init__()
        self.calls = []

    def forward(self, x, t, r, y):
        assert not torch.is_grad_enabled()
        self.calls.append((x.shape[0], float(t[0]), float(r[0]), x.dtype))
        a = torch.where(y == 1000, 3.0, 1.0).view(-1, 1, 1, 1).to(x.dtype)
        return a * x + (t - 2 * r).view(-1, 1, 1, 1)


def test_euler_sampler_known_answers():
    from dmf_amd.samplers import euler_sampler
    x0 = torch.randn(3, 4, 2, 2, generator=torch.Generator().manual_seed(5))
    y = torch.tensor([1, 2, 3])
    f = _Field()
    out = euler_sampler(f, x0, y, num_steps=2)
    # two explicit Euler steps of x' = x + t - 2 r from t = 1 to 0.5 to 0, by hand in fp64 (r = next time)
    x = x0.double()
    x = x + (0.5 - 1.0) * (x + 1.0 - 2 * 0.5)
    x = x + (0.0 - 0.5) * (x + 0.5 - 0.0)
    assert out.dtype == torch.float64 and torch.allclose(out, x, atol=1e-6)
    assert [(n, t, r) for n, t, r, _ in f.calls] == [(3, 1.0, 0.5), (3, 0.5, 0.0)] and f.calls[0][3] == torch.float32
    # guidance: doubled batch inside the window only; d = d_uncond + w (d_cond - d_uncond)
    f = _Field()
    out = euler_sampler(f, x0, y, num_steps=2, cfg_scale=2.0, g_min=0.0, g_max=0.75)
    x = x0.double()
    x = x + (0.5 - 1.0) * (x + 1.0 - 1.0)                                    # t = 1 is outside the window: plain step
    d_c, d_u = x + 0.5, 3 * x + 0.5
    x = x + (0.0 - 0.5) * (d_u + 2.0 * (d_c - d_u))
    assert torch.allclose(out, x, atol=1e-6) and [c[0] for c in f.calls] == [3, 6]
    # the model is called in the dtype of the latents, the state is carried in fp64
    f = _Field()
    euler_sampler(f, x0.bfloat16(), y, num_steps=1)
    assert f.calls[0][3] == torch.bfloat16


@pytest.mark.gpu
def test_euler_sampler_bf16_model_fused_vs_base():
    """generate.py's setting: the model cast to bf16 (parameters included), 4 steps
    with classifier-free guidance; 'hip' attention + fused block glue against the
    naive attention and the reference's expressions on the same weights, and the
    model call replayed from a HIP graph against the eager call."""
    from dmf_amd.samplers import euler_sampler
    dev = "cuda:0"
    kw = dict(input_size=32, hidden_size=288, depth=4, num_heads=4, dmf_depth=3, qk_norm=True, use_logvar=False)
    m_ref = _dmft("base", **kw)
    m = _dmft("hip", block_ops="hip", **kw)
    m.load_state_dict(m_ref.state_dict())
    m_ref, m = m_ref.to(dev, torch.bfloat16).eval(), m.to(dev, torch.bfloat16).eval()
    g = torch.Generator().manual_seed(11)
    z = torch.randn(8, 4, 32, 32, generator=g).to(dev, torch.bfloat16)
    y = torch.randint(0, 1000, (8,), generator=g).to(dev)
    args = dict(num_steps=4, cfg_scale=1.5, g_min=0.0, g_max=0.8, shift=1.5)
    ref = euler_sampler(m_ref, z, y, **args)
    out = euler_sampler(m, z, y, **args)
    assert out.dtype == torch.float64 and ao.rel_l2(out, ref) <= 3e-2
    graphs = {}

    def call(x, t, r, yy):
        n = x.shape[0]
        if n not in graphs:
            with torch.no_grad():
                graphs[n] = harness.GraphedStep(lambda *a: m(*a), x, t, r, yy)
        return graphs[n](x, t, r, yy)

    out_g = euler_sampler(m, z, y, model_call=call, **args)
    assert sorted(graphs) == [8, 16] and ao.rel_l2(out_g, out) <= 1e-6


@pytest.mark.gpu
def test_graphed_dmf_step_follows_parameter_updates():
    """A captured step must read the parameters as they are at replay time -- the
    bf16 weight copies that the fused Linear layers share within a step are made
    inside the graph -- so a few SGD updates give the same losses replayed as
    eager, and the losses move."""
    dev = "cuda:0"
    kw = dict(input_size=16, hidden_size=128, depth=3, num_heads=2, dmf_depth=2)
    m_e = _dmft("hip", block_ops="hip", **kw).to(dev)
    m_g = _dmft("hip", block_ops="hip", **kw).to(dev)
    m_g.load_state_dict(m_e.state_dict())
    batch = harness.synthetic_loss_batch(8, dev, input_size=16)
    guidance = dict(g_type="mg", omega=0.5)

    def sgd(m, lr=0.5):
        with torch.no_grad():
            for p in m.parameters():
                if p.grad is not None:
                    p.add_(p.grad, alpha=-lr)

    def step_g(*b):
        m_g.zero_grad(set_to_none=True)
        return harness.dmf_train_step(m_g, b, functorch=False, **guidance).detach()

    graphed = harness.GraphedStep(step_g, *batch)
    m_g.load_state_dict(m_e.state_dict())        # the warm-up calls did not update anything, but start from equal weights for sure
    eager, replayed = [], []
    for _ in range(4):
        m_e.zero_grad(set_to_none=True)
        eager.append(float(harness.dmf_train_step(m_e, batch, functorch=False, **guidance)))
        sgd(m_e)
        replayed.append(float(graphed(*batch)))
        sgd(m_g)
    assert abs(eager[-1] - eager[0]) > 1e-3 * abs(eager[0]), eager            # the updates matter
    for a, b in zip(eager, replayed):
        assert abs(a - b) <= 2e-3 * abs(a) + 1e-5, (eager, replayed)
