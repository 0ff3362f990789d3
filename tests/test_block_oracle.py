"""Pins oracle/block_oracle.py by checks that do not restate its formulas:
library routines, numpy fp64 closed forms written independently, central finite
differences, invariants and the adjoint identity <JVP t, w> = <t, VJP w>."""
import numpy as np
import torch

from oracle import block_oracle as bo

torch.manual_seed(0)
D64 = torch.float64


def _inputs(B=2, L=5, C=16, seed=3):
    return bo.make_block_inputs(B, L, C, seed, D64)


def _fd(fn, args, tangents, h=1e-6):
    plus = fn(*[a + h * t for a, t in zip(args, tangents)])
    minus = fn(*[a - h * t for a, t in zip(args, tangents)])
    return (plus - minus) / (2 * h)


def test_layer_norm_matches_library_and_invariants():
    x = torch.randn(3, 7, 24, dtype=D64) * 3 + 1.5
    y = bo.layer_norm(x, 1e-6)
    ref = torch.nn.functional.layer_norm(x, (24,), eps=1e-6)
    assert torch.allclose(y, ref, atol=1e-12)
    assert y.mean(-1).abs().max() < 1e-12
    var = ((x - x.mean(-1, keepdim=True)) ** 2).mean(-1)
    assert torch.allclose((y ** 2).mean(-1), var / (var + 1e-6), atol=1e-12)


def test_modulate_special_cases():
    x = torch.randn(2, 3, 8, dtype=D64)
    z = torch.zeros(2, 1, 8, dtype=D64)
    assert torch.equal(bo.modulate(x, z, z), x)
    assert torch.allclose(bo.modulate(x, z + 2, z + 1), 2 * x + 2)


def test_ln_modulate_jvp_and_grads_against_closed_form_and_fd():
    d = _inputs()
    args = (d["x"], d["shift"], d["scale"])
    tans = (d["tx"], d["tshift"], d["tscale"])
    y, ty = bo.jvp(bo.ln_modulate, args, tans)
    cf = bo.ln_modulate_closed_fp64(*args, *tans, gy=d["gy"])
    assert np.allclose(y.numpy(), cf["y"], atol=1e-12)
    assert np.allclose(ty.numpy(), cf["ty"], atol=1e-11)
    assert torch.allclose(ty, _fd(bo.ln_modulate, args, tans), atol=1e-6)
    gx, gshift, gscale = bo.grads(bo.ln_modulate, args, d["gy"])
    assert np.allclose(gx.numpy(), cf["gx"], atol=1e-11)
    assert np.allclose(gshift.numpy(), cf["gshift"], atol=1e-11)
    assert np.allclose(gscale.numpy(), cf["gscale"], atol=1e-11)
    # adjoint identity ties the gradients to the (finite-difference-checked) tangent
    lhs = (ty * d["gy"]).sum()
    rhs = (gx * d["tx"]).sum() + (gshift * d["tshift"]).sum() + (gscale * d["tscale"]).sum()
    assert abs(lhs - rhs) < 1e-9 * max(1.0, abs(lhs))


def test_ln_modulate_tangent_special_cases():
    d = _inputs()
    z = torch.zeros_like(d["shift"])
    # a tangent along x itself or along a per-row constant is annihilated by the normalisation (up to eps)
    _, t1 = bo.jvp(bo.ln_modulate, (d["x"], d["shift"], d["scale"]), (torch.ones_like(d["x"]), z, z))
    assert t1.abs().max() < 1e-9
    # only the shift moves: ty = tshift broadcast
    _, t2 = bo.jvp(bo.ln_modulate, (d["x"], d["shift"], d["scale"]), (torch.zeros_like(d["x"]), d["tshift"], z))
    assert torch.allclose(t2, d["tshift"].expand_as(t2))


def test_gate_residual_closed_forms():
    d = _inputs()
    args, tans = (d["x"], d["gate"], d["h"]), (d["tx"], d["tgate"], d["th"])
    y, ty = bo.jvp(bo.gate_residual, args, tans)
    assert torch.allclose(y, d["x"] + d["gate"] * d["h"])
    assert torch.allclose(ty, d["tx"] + d["tgate"] * d["h"] + d["gate"] * d["th"], atol=1e-12)
    gx, gg, gh = bo.grads(bo.gate_residual, args, d["gy"])
    assert torch.equal(gx, d["gy"])
    assert torch.allclose(gh, d["gate"] * d["gy"])
    assert torch.allclose(gg, (d["gy"] * d["h"]).sum(1, keepdim=True), atol=1e-12)


def test_gelu_tanh_matches_library_and_derivative():
    x = torch.linspace(-6, 6, 241, dtype=D64)
    assert torch.allclose(bo.gelu_tanh(x), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-12)
    t = torch.randn(241, dtype=D64)
    _, ty = bo.jvp(bo.gelu_tanh, (x,), (t,))
    assert np.allclose(ty.numpy(), bo.gelu_tanh_grad_fp64(x) * t.numpy(), atol=1e-12)
    assert torch.allclose(ty, _fd(bo.gelu_tanh, (x,), (t,)), atol=1e-7)
    (gx,) = bo.grads(bo.gelu_tanh, (x,), t)
    assert np.allclose(gx.numpy(), bo.gelu_tanh_grad_fp64(x) * t.numpy(), atol=1e-12)
    # limits: identity for large x, zero for very negative x, value at 0
    assert abs(float(bo.gelu_tanh(torch.tensor(10.0, dtype=D64))) - 10.0) < 1e-9
    assert abs(float(bo.gelu_tanh(torch.tensor(-10.0, dtype=D64)))) < 1e-9
    assert float(bo.gelu_tanh(torch.tensor(0.0, dtype=D64))) == 0.0


def test_rms_norm_closed_form_jvp_grads():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 4, 3, 24, generator=g, dtype=D64)
    tx = torch.randn(2, 4, 3, 24, generator=g, dtype=D64)
    gy = torch.randn(2, 4, 3, 24, generator=g, dtype=D64)
    gain = 1 + 0.2 * torch.randn(24, generator=g, dtype=D64)
    cf = bo.rms_norm_closed_fp64(x, gain, tx, gy)
    fn = lambda a: bo.rms_norm(a, gain)
    y, ty = bo.jvp(fn, (x,), (tx,))
    assert np.allclose(y.numpy(), cf["y"], atol=1e-12)
    assert np.allclose(ty.numpy(), cf["ty"], atol=1e-11)
    assert torch.allclose(ty, _fd(fn, (x,), (tx,)), atol=1e-6)
    gx, ggain = bo.grads(bo.rms_norm, (x, gain), gy)
    assert np.allclose(gx.numpy(), cf["gx"], atol=1e-11)
    assert np.allclose(ggain.numpy(), cf["ggain"], atol=1e-11)
    assert abs((ty * gy).sum() - (gx * tx).sum()) < 1e-9
    # unit gain: every row has RMS 1 (up to eps); a tangent along x itself is annihilated (scale invariance)
    y1 = bo.rms_norm(x, torch.ones(24, dtype=D64))
    assert torch.allclose((y1 ** 2).mean(-1), torch.ones(2, 4, 3, dtype=D64), atol=1e-5)
    _, t_self = bo.jvp(fn, (x,), (x,))
    assert t_self.abs().max() < 1e-5


def test_rms_norm_agrees_with_attention_oracle_helper():
    from oracle import attn_oracle as ao
    x = torch.randn(2, 3, 2, 16)
    assert torch.allclose(bo.rms_norm(x, torch.ones(16)), ao.rms_norm(x), atol=1e-6)


def test_silu_matches_library_and_derivative():
    x = torch.linspace(-8, 8, 161, dtype=D64)
    assert torch.allclose(bo.silu(x), torch.nn.functional.silu(x), atol=1e-14)
    t = torch.randn(161, dtype=D64)
    _, ty = bo.jvp(bo.silu, (x,), (t,))
    assert torch.allclose(ty, _fd(bo.silu, (x,), (t,)), atol=1e-7)
    s = 1 / (1 + np.exp(-x.numpy()))
    assert np.allclose(ty.numpy(), s * (1 + x.numpy() * (1 - s)) * t.numpy(), atol=1e-12)


def _golden():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "block_vectors.npz"))


def test_golden_vectors():
    """The committed known-answer vectors (tests/golden/block_vectors.npz, written once by
    tests/golden/make_block_vectors.py from the fp64 closed forms): the torch restatements,
    evaluated in fp64 on the stored fp32 inputs, must reproduce them."""
    z = _golden()
    t = lambda k: torch.from_numpy(z[k]).double()
    close = lambda got, key, tol=1e-12: np.allclose(got.numpy(), z[key], atol=tol, rtol=tol)
    y, ty = bo.jvp(bo.ln_modulate, (t("x"), t("shift"), t("scale")), (t("tx"), t("tshift"), t("tscale")))
    gx, gsh, gsc = bo.grads(bo.ln_modulate, (t("x"), t("shift"), t("scale")), t("gy"))
    assert close(y, "ln_modulate.y") and close(ty, "ln_modulate.ty", 1e-11) and close(gx, "ln_modulate.gx", 1e-11)
    assert close(gsh, "ln_modulate.gshift", 1e-11) and close(gsc, "ln_modulate.gscale", 1e-11)
    y, ty = bo.jvp(bo.gate_residual, (t("x"), t("gate"), t("h")), (t("tx"), t("tgate"), t("th")))
    assert close(y, "gate_residual.y") and close(ty, "gate_residual.ty")
    u = t("gelu.x")
    assert close(bo.gelu_tanh(u), "gelu.y") and close(bo.silu(u), "silu.y")
    assert close(bo.jvp(bo.gelu_tanh, (u,), (torch.ones_like(u),))[1], "gelu.dy")
    assert close(bo.jvp(bo.silu, (u,), (torch.ones_like(u),))[1], "silu.dy")
    y, ty = bo.jvp(lambda a: bo.rms_norm(a, t("rms.gain")), (t("rms.x"),), (t("rms.tx"),))
    gx, gg = bo.grads(bo.rms_norm, (t("rms.x"), t("rms.gain")), t("rms.gy"))
    assert close(y, "rms.y") and close(ty, "rms.ty", 1e-11) and close(gx, "rms.gx", 1e-11) and close(gg, "rms.ggain", 1e-11)
