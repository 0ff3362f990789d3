"""GPU parity of the fused block-glue kernels (C ABI include/dmf_block.h) against
the CPU oracle (oracle/block_oracle.py) on the same seeded inputs.

Tolerances (relative L2): 1e-5 when everything is fp32; 6e-3 when the result is
stored in bf16 (one rounding of an fp32 result, 2^-9 relative per element, so
about 2.3e-3 in L2).  The oracle is always evaluated in fp32 on the values the
kernel was given (bf16 inputs are rounded first, then widened)."""
import pytest
import torch

from dmf_amd import _lib, block_ops
from oracle import attn_oracle as ao
from oracle import block_oracle as bo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


def _tol(*dtypes):
    return 6e-3 if any(d == BF16 for d in dtypes) else 1e-5


def _close(got, ref, tol, what=""):
    err = ao.rel_l2(got.float().cpu(), ref.float())
    assert err <= tol, f"{what}: rel-L2 {err:.3e} > {tol:.1e}"


def _rounded(d, keys, dtype):
    """Round the named inputs to dtype (what the kernel sees) and return fp32 CPU copies + device copies."""
    cpu = {k: d[k].to(dtype).float() for k in keys}
    dev = {k: d[k].to(dtype).to(DEV) for k in keys}
    return cpu, dev


SHAPES = [(2, 37, 768), (3, 64, 1152), (1, 5, 8), (2, 33, 2048), (2, 16, 1024), (4, 1, 384)]
DTYPES = [(F32, F32, F32), (F32, BF16, BF16), (BF16, BF16, BF16)]   # (x, mods, out)


@pytest.mark.parametrize("B,L,C", SHAPES)
@pytest.mark.parametrize("xdt,mdt,ydt", DTYPES)
def test_ln_modulate_fwd_jvp_bwd(B, L, C, xdt, mdt, ydt):
    print(f"ln_modulate B{B} L{L} C{C} {xdt} {mdt} {ydt}", flush=True)
    d = bo.make_block_inputs(B, L, C, seed=11)
    cx, gx_ = _rounded(d, ("x", "tx"), xdt)
    cm, gm = _rounded(d, ("shift", "scale", "tshift", "tscale"), mdt)
    cg, gg = _rounded(d, ("gy",), ydt)
    y_ref, ty_ref = bo.jvp(bo.ln_modulate, (cx["x"], cm["shift"], cm["scale"]), (cx["tx"], cm["tshift"], cm["tscale"]))
    tol = _tol(xdt, mdt, ydt)
    y, ty = _lib.ln_modulate_fwd(gx_["x"], gm["shift"], gm["scale"], gx_["tx"], gm["tshift"], gm["tscale"], 1e-6, ydt, True)
    assert y.dtype == ydt and ty.dtype == ydt
    _close(y, y_ref, tol, "y")
    _close(ty, ty_ref, tol, "ty")
    y0, none = _lib.ln_modulate_fwd(gx_["x"], gm["shift"], gm["scale"], eps=1e-6, out_dtype=ydt)
    assert none is None and torch.equal(y0, y)
    # missing tangents read as zeros
    _, ty_x = _lib.ln_modulate_fwd(gx_["x"], gm["shift"], gm["scale"], gx_["tx"], None, None, 1e-6, ydt, True)
    z = torch.zeros_like(cm["shift"])
    _, ty_x_ref = bo.jvp(bo.ln_modulate, (cx["x"], cm["shift"], cm["scale"]), (cx["tx"], z, z))
    _close(ty_x, ty_x_ref, tol, "ty (x tangent only)")
    gx_ref, gsh_ref, gsc_ref = bo.grads(bo.ln_modulate, (cx["x"], cm["shift"], cm["scale"]), cg["gy"])
    gx, gsh, gsc = _lib.ln_modulate_bwd(gg["gy"], gx_["x"], gm["scale"], 1e-6)
    assert gx.dtype == xdt and gsh.dtype == mdt and gsh.shape == (B, C)
    _close(gx, gx_ref, _tol(xdt, ydt), "gx")
    _close(gsh.view(B, 1, C), gsh_ref, _tol(mdt), "gshift")
    _close(gsc.view(B, 1, C), gsc_ref, _tol(mdt), "gscale")
    # a gradient reaching x from elsewhere is folded into gx
    gx2, gsh2, _ = _lib.ln_modulate_bwd(gg["gy"], gx_["x"], gm["scale"], 1e-6, gres=gx_["tx"])
    _close(gx2, gx_ref + cx["tx"], _tol(xdt, ydt), "gx + gres")
    assert torch.equal(gsh2, gsh)


@pytest.mark.parametrize("B,L,C", SHAPES)
@pytest.mark.parametrize("xdt,mdt,hdt", DTYPES)
def test_gate_residual_fwd_jvp_bwd(B, L, C, xdt, mdt, hdt):
    print(f"gate_residual B{B} L{L} C{C} {xdt} {mdt} {hdt}", flush=True)
    d = bo.make_block_inputs(B, L, C, seed=12)
    cx, gx_ = _rounded(d, ("x", "tx", "gy"), xdt)
    cm, gm = _rounded(d, ("gate", "tgate"), mdt)
    ch, gh_ = _rounded(d, ("h", "th"), hdt)
    y_ref, ty_ref = bo.jvp(bo.gate_residual, (cx["x"], cm["gate"], ch["h"]), (cx["tx"], cm["tgate"], ch["th"]))
    y, ty = _lib.gate_residual_fwd(gx_["x"], gm["gate"], gh_["h"], gx_["tx"], gm["tgate"], gh_["th"], True)
    assert y.dtype == xdt
    _close(y, y_ref, _tol(xdt), "y")
    _close(ty, ty_ref, _tol(xdt), "ty")
    y0, none = _lib.gate_residual_fwd(gx_["x"], gm["gate"], gh_["h"])
    assert none is None and torch.equal(y0, y)
    _, gg_ref, gh_ref = bo.grads(bo.gate_residual, (cx["x"], cm["gate"], ch["h"]), cx["gy"])
    gh, gg = _lib.gate_residual_bwd(gx_["gy"], gm["gate"], gh_["h"])
    _close(gh, gh_ref, _tol(hdt), "gh")
    _close(gg.view(B, 1, C), gg_ref, _tol(mdt), "ggate")


@pytest.mark.parametrize("shape", [(2, 37, 3072), (1, 8), (3, 5, 4608)])
@pytest.mark.parametrize("dt", [F32, BF16])
def test_gelu_tanh_fwd_jvp_bwd(shape, dt):
    print(f"gelu {shape} {dt}", flush=True)
    g = torch.Generator().manual_seed(13)
    x, t = (2 * torch.randn(*shape, generator=g)).to(dt), torch.randn(*shape, generator=g).to(dt)
    y_ref, ty_ref = bo.jvp(bo.gelu_tanh, (x.float(),), (t.float(),))
    y, ty = _lib.gelu_tanh_fwd(x.to(DEV), t.to(DEV))
    _close(y, y_ref, _tol(dt), "y")
    _close(ty, ty_ref, _tol(dt), "ty")
    y0, none = _lib.gelu_tanh_fwd(x.to(DEV))
    assert none is None and torch.equal(y0, y)
    (gx_ref,) = bo.grads(bo.gelu_tanh, (x.float(),), t.float())
    _close(_lib.gelu_tanh_bwd(t.to(DEV), x.to(DEV)), gx_ref, _tol(dt), "gx")


@pytest.mark.parametrize("B,L,H,D", [(2, 37, 16, 72), (1, 5, 3, 64), (2, 9, 2, 128), (1, 300, 5, 8), (2, 64, 12, 96)])
@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("packed", [False, True])
def test_rmsnorm_fwd_jvp_bwd(B, L, H, D, dt, packed):
    print(f"rmsnorm B{B} L{L} H{H} D{D} {dt} packed={packed}", flush=True)
    g = torch.Generator().manual_seed(14)
    x, tx, gy = (torch.randn(B, L, H, D, generator=g).to(dt) for _ in range(3))
    gain = 1 + 0.2 * torch.randn(D, generator=g)

    def dev(t):
        if not packed:
            return t.to(DEV)
        buf = torch.zeros(B, L, 3, H, D, dtype=dt, device=DEV)   # q-slot view of a packed qkv buffer
        buf[:, :, 0] = t.to(DEV)
        return buf[:, :, 0]

    cf = bo.rms_norm_closed_fp64(x.float(), gain, tx.float(), gy.float())
    y, ty = _lib.rmsnorm_fwd(dev(x), gain.to(DEV), dev(tx), 1e-6, True)
    assert y.is_contiguous() and y.dtype == dt
    _close(y, torch.from_numpy(cf["y"]), _tol(dt), "y")
    _close(ty, torch.from_numpy(cf["ty"]), _tol(dt), "ty")
    if dt == F32:  # the reference's own rounding points only matter in bf16; in fp32 the restatement agrees too
        _close(y, bo.rms_norm(x, gain), 1e-5, "y vs restated RMSNorm.forward")
    y0, none = _lib.rmsnorm_fwd(dev(x), gain.to(DEV))
    assert none is None and torch.equal(y0, y)
    gx, ggain = _lib.rmsnorm_bwd(gy.to(DEV), dev(x), gain.to(DEV))
    _close(gx, torch.from_numpy(cf["gx"]), _tol(dt), "gx")
    _close(ggain, torch.from_numpy(cf["ggain"]), 1e-5, "ggain")
    # gradient written in place into one slot of a packed (B, L, 3, H, D) buffer
    packed_grad = torch.zeros(B, L, 3, H, D, dtype=dt, device=DEV)
    gx2, ggain2 = _lib.rmsnorm_bwd(gy.to(DEV), dev(x), gain.to(DEV), out=packed_grad[:, :, 1])
    assert torch.equal(packed_grad[:, :, 1], gx) and torch.equal(ggain2, ggain)
    assert float(packed_grad[:, :, 0].abs().max()) == 0 and float(packed_grad[:, :, 2].abs().max()) == 0


def test_wrappers_under_func_jvp_and_autograd():
    """The dual-aware wrappers under torch.func.jvp with autograd on top, as the training step uses them."""
    B, L, C = 2, 24, 384
    d = bo.make_block_inputs(B, L, C, seed=15)
    dev = {k: v.to(DEV) for k, v in d.items()}

    def fused(x, shift, scale, gate):
        return block_ops.gate_residual(x, gate, block_ops.gelu_tanh(block_ops.ln_modulate(x, shift, scale)))

    def plain(x, shift, scale, gate):
        return bo.gate_residual(x, gate, bo.gelu_tanh(bo.ln_modulate(x, shift, scale)))

    keys, tkeys = ("x", "shift", "scale", "gate"), ("tx", "tshift", "tscale", "tgate")
    prim = [dev[k].clone().requires_grad_(True) for k in keys]
    y, ty = torch.func.jvp(fused, tuple(prim), tuple(dev[k] for k in tkeys))
    y_ref, ty_ref = bo.jvp(plain, [d[k] for k in keys], [d[k] for k in tkeys])
    _close(y, y_ref, 1e-5, "y")
    _close(ty, ty_ref, 1e-5, "ty")
    (y * dev["gy"]).sum().backward()
    refs = bo.grads(plain, [d[k] for k in keys], d["gy"])
    for k, p, r in zip(keys, prim, refs):
        _close(p.grad, r, 2e-5, f"grad {k}")
    # plain (non-dual) call gives the same primal
    assert torch.allclose(fused(*[dev[k] for k in keys]), y.detach(), atol=0, rtol=0)


def test_rms_norm_wrapper_under_func_jvp():
    g = torch.Generator().manual_seed(16)
    x, tx = torch.randn(2, 20, 4, 72, generator=g), torch.randn(2, 20, 4, 72, generator=g)
    gain = (1 + 0.2 * torch.randn(72, generator=g))
    y, ty = torch.func.jvp(lambda a: block_ops.rms_norm(a, gain.to(DEV)), (x.to(DEV),), (tx.to(DEV),))
    cf = bo.rms_norm_closed_fp64(x, gain, tx)
    _close(y, torch.from_numpy(cf["y"]), 1e-5)
    _close(ty, torch.from_numpy(cf["ty"]), 1e-5)


def test_block_abi_rejects_bad_arguments():
    x = torch.zeros(2, 4, 20, device=DEV)        # C = 20 is not a multiple of 8
    m = torch.zeros(2, 20, device=DEV)
    with pytest.raises(RuntimeError, match="bad shape"):
        _lib.ln_modulate_fwd(x, m, m)
    big = torch.zeros(1, 2, 4096, device=DEV)    # C above the supported maximum
    with pytest.raises(RuntimeError, match="bad shape"):
        _lib.gate_residual_fwd(big, torch.zeros(1, 4096, device=DEV), big)
    with pytest.raises(RuntimeError, match="head dim"):
        _lib.rmsnorm_fwd(torch.zeros(1, 2, 2, 20, device=DEV), torch.ones(20, device=DEV))


@pytest.mark.parametrize("rows,C", [(1000, 2304), (1, 8), (16384, 768), (77, 4608)])
@pytest.mark.parametrize("dt", [F32, BF16])
def test_colsum(rows, C, dt):
    print(f"colsum {rows}x{C} {dt}", flush=True)
    x = torch.randn(rows, C, generator=torch.Generator().manual_seed(17)).to(dt)
    got = _lib.colsum(x.to(DEV), torch.float32)
    _close(got, x.double().sum(0), 1e-5, "colsum")
    assert torch.equal(got, _lib.colsum(x.to(DEV), torch.float32))   # fixed summation order


def test_dual_linear_under_func_jvp_and_autograd():
    from torch.nn.functional import linear
    g = torch.Generator().manual_seed(18)
    x, tx, gy = torch.randn(2, 24, 64, generator=g), torch.randn(2, 24, 64, generator=g), torch.randn(2, 24, 48, generator=g)
    w, b = torch.randn(48, 64, generator=g) * 0.1, torch.randn(48, generator=g)
    xd, wd, bd = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_(), b.to(DEV).requires_grad_()
    y, ty = torch.func.jvp(lambda a: block_ops.dual_linear(a, wd, bd), (xd,), (tx.to(DEV),))
    _close(y, linear(x, w, b), 1e-5, "y")
    _close(ty, linear(tx, w), 1e-5, "ty")
    (y * gy.to(DEV)).sum().backward()
    gx, gw, gb = bo.grads(lambda a, ww, bb: linear(a, ww, bb), (x, w, b), gy)
    _close(xd.grad, gx, 1e-5, "gx")
    _close(wd.grad, gw, 1e-5, "gw")
    _close(bd.grad, gb, 1e-5, "gb")


@pytest.mark.parametrize("shape", [(64, 1, 768), (3, 8)])
@pytest.mark.parametrize("xdt,ydt", [(F32, F32), (F32, BF16), (BF16, BF16)])
def test_silu_fwd_jvp_bwd(shape, xdt, ydt):
    print(f"silu {shape} {xdt} {ydt}", flush=True)
    g = torch.Generator().manual_seed(19)
    x, t = (2 * torch.randn(*shape, generator=g)).to(xdt), torch.randn(*shape, generator=g).to(xdt)
    gy = torch.randn(*shape, generator=g).to(ydt)
    y_ref, ty_ref = bo.jvp(bo.silu, (x.float(),), (t.float(),))
    y, ty = _lib.silu_fwd(x.to(DEV), t.to(DEV), ydt)
    assert y.dtype == ydt
    _close(y, y_ref, _tol(xdt, ydt), "y")
    _close(ty, ty_ref, _tol(xdt, ydt), "ty")
    y0, none = _lib.silu_fwd(x.to(DEV), None, ydt)
    assert none is None and torch.equal(y0, y)
    (gx_ref,) = bo.grads(bo.silu, (x.float(),), gy.float())
    gx = _lib.silu_bwd(gy.to(DEV), x.to(DEV))
    assert gx.dtype == xdt
    _close(gx, gx_ref, _tol(xdt), "gx")


@pytest.mark.parametrize("B,L,C", SHAPES)
@pytest.mark.parametrize("xdt,mdt,zdt", DTYPES)
def test_residual_ln_modulate_fwd_jvp_bwd(B, L, C, xdt, mdt, zdt):
    """Fused gated residual + LayerNorm + modulate against the composition of the two oracle expressions."""
    print(f"residual_ln_modulate B{B} L{L} C{C} {xdt} {mdt} {zdt}", flush=True)
    d = bo.make_block_inputs(B, L, C, seed=20)
    g = torch.Generator().manual_seed(21)
    d["gz"] = torch.randn(B, L, C, generator=g)
    cx, gx_ = _rounded(d, ("x", "tx", "gy"), xdt)
    cm, gm = _rounded(d, ("gate", "tgate", "shift", "scale", "tshift", "tscale"), mdt)
    ch, gh_ = _rounded(d, ("h", "th"), mdt)
    cz, gz_ = _rounded(d, ("gz",), zdt)

    def comp(x, gate, h, shift, scale):
        y = bo.gate_residual(x, gate, h)
        return y, bo.ln_modulate(y, shift, scale)

    prim = (cx["x"], cm["gate"], ch["h"], cm["shift"], cm["scale"])
    tans = (cx["tx"], cm["tgate"], ch["th"], cm["tshift"], cm["tscale"])
    (y_ref, z_ref), (ty_ref, tz_ref) = bo.jvp(comp, prim, tans)
    y, z, ty, tz = _lib.residual_ln_modulate_fwd(gx_["x"], gm["gate"], gh_["h"], gm["shift"], gm["scale"], gx_["tx"], gm["tgate"],
                                                 gh_["th"], gm["tshift"], gm["tscale"], 1e-6, zdt, True)
    assert y.dtype == xdt and z.dtype == zdt
    _close(y, y_ref, _tol(xdt), "y")
    _close(ty, ty_ref, _tol(xdt), "ty")
    # z is normalised from the *stored* y when y is bf16 in the two-kernel path; here from the fp32 value: allow bf16 tolerance
    _close(z, z_ref, _tol(xdt, mdt, zdt), "z")
    _close(tz, tz_ref, _tol(xdt, mdt, zdt), "tz")
    y0, z0, n1, n2 = _lib.residual_ln_modulate_fwd(gx_["x"], gm["gate"], gh_["h"], gm["shift"], gm["scale"], eps=1e-6, out_dtype=zdt)
    assert n1 is None and n2 is None and torch.equal(y0, y) and torch.equal(z0, z)
    # backward: gradient reaching y from elsewhere (gy) plus the gradient of z
    inputs = [t.detach().clone().requires_grad_(True) for t in prim]
    yy, zz = comp(*inputs)
    refs = torch.autograd.grad([yy, zz], inputs, [cx["gy"], cz["gz"]])
    gx, gh, ggate, gshift, gscale = _lib.residual_ln_modulate_bwd(gx_["gy"], gz_["gz"], y, gh_["h"], gm["gate"], gm["scale"], 1e-6)
    tol = _tol(xdt, mdt, zdt)
    _close(gx, refs[0], tol, "gx")
    _close(ggate.view(B, 1, C), refs[1], tol, "ggate")
    _close(gh, refs[2], tol, "gh")
    _close(gshift.view(B, 1, C), refs[3], _tol(mdt), "gshift")
    _close(gscale.view(B, 1, C), refs[4], tol, "gscale")
    # without an outside gradient for y
    refs0 = torch.autograd.grad([comp(*inputs)[1]], inputs, [cz["gz"]])
    gx0, gh0, *_ = _lib.residual_ln_modulate_bwd(None, gz_["gz"], y, gh_["h"], gm["gate"], gm["scale"], 1e-6)
    _close(gx0, refs0[0], tol, "gx (no gy)")
    _close(gh0, refs0[2], tol, "gh (no gy)")


def test_residual_ln_modulate_wrapper_under_func_jvp_and_autograd():
    B, L, C = 2, 24, 384
    d = bo.make_block_inputs(B, L, C, seed=22)
    dev = {k: v.to(DEV) for k, v in d.items()}
    keys, tkeys = ("x", "gate", "h", "shift", "scale"), ("tx", "tgate", "th", "tshift", "tscale")

    def fused(*a):
        y, z = block_ops.residual_ln_modulate(*a)
        return y + 2 * z

    def plain(x, gate, h, shift, scale):
        y = bo.gate_residual(x, gate, h)
        return y + 2 * bo.ln_modulate(y, shift, scale)

    prim = [dev[k].clone().requires_grad_(True) for k in keys]
    out, tout = torch.func.jvp(fused, tuple(prim), tuple(dev[k] for k in tkeys))
    out_ref, tout_ref = bo.jvp(plain, [d[k] for k in keys], [d[k] for k in tkeys])
    _close(out, out_ref, 1e-5, "out")
    _close(tout, tout_ref, 1e-5, "tangent")
    (out * dev["gy"]).sum().backward()
    for k, p, r in zip(keys, prim, bo.grads(plain, [d[k] for k in keys], d["gy"])):
        _close(p.grad, r, 2e-5, f"grad {k}")


def test_golden_vectors():
    """fp32 kernels through the C ABI against the committed known-answer vectors
    (tests/golden/block_vectors.npz: fp64 closed forms on seeded inputs)."""
    import os
    import numpy as np
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "block_vectors.npz"))
    g = lambda k: torch.from_numpy(z[k]).to(DEV)
    ref = lambda k: torch.from_numpy(z[k])
    y, ty = _lib.ln_modulate_fwd(g("x"), g("shift"), g("scale"), g("tx"), g("tshift"), g("tscale"), 1e-6, F32, True)
    gx, gsh, gsc = _lib.ln_modulate_bwd(g("gy"), g("x"), g("scale"), 1e-6)
    B, L, C = z["x"].shape
    for got, key in ((y, "ln_modulate.y"), (ty, "ln_modulate.ty"), (gx, "ln_modulate.gx"),
                     (gsh.view(B, 1, C), "ln_modulate.gshift"), (gsc.view(B, 1, C), "ln_modulate.gscale")):
        _close(got, ref(key), 1e-5, key)
    y, ty = _lib.gate_residual_fwd(g("x"), g("gate"), g("h"), g("tx"), g("tgate"), g("th"), True)
    gh, gg = _lib.gate_residual_bwd(g("gy"), g("gate"), g("h"))
    for got, key in ((y, "gate_residual.y"), (ty, "gate_residual.ty"), (gh, "gate_residual.gh"), (gg.view(B, 1, C), "gate_residual.ggate")):
        _close(got, ref(key), 1e-5, key)
    u = g("gelu.x")
    y, dy = _lib.gelu_tanh_fwd(u, torch.ones_like(u))
    _close(y, ref("gelu.y"), 1e-5, "gelu.y")
    _close(dy, ref("gelu.dy"), 1e-5, "gelu.dy")
    y, dy = _lib.silu_fwd(u, torch.ones_like(u))
    _close(y, ref("silu.y"), 1e-5, "silu.y")
    _close(dy, ref("silu.dy"), 1e-5, "silu.dy")
    y, ty = _lib.rmsnorm_fwd(g("rms.x"), g("rms.gain"), g("rms.tx"), 1e-6, True)
    gx, gg = _lib.rmsnorm_bwd(g("rms.gy"), g("rms.x"), g("rms.gain"))
    for got, key in ((y, "rms.y"), (ty, "rms.ty"), (gx, "rms.gx"), (gg, "rms.ggain")):
        _close(got, ref(key), 1e-5, key)


@pytest.mark.parametrize("mode", ["bf16", "autocast", "fp32"])
def test_linear_gelu_tanh_epilogue_path(mode):
    """``linear_gelu_tanh`` without gradients (GELU in the GEMM epilogue) against the
    oracle's tanh-GELU of an fp32 linear, and against the two-kernel path that is
    taken as soon as a gradient or a tangent is involved."""
    g = torch.Generator().manual_seed(41)
    x = torch.randn(3, 50, 96, generator=g).to(DEV)
    w = (0.1 * torch.randn(384, 96, generator=g)).to(DEV)
    b = (0.5 * torch.randn(384, generator=g)).to(DEV)
    if mode == "bf16":
        x, w, b = x.bfloat16(), w.bfloat16(), b.bfloat16()
    ref = bo.gelu_tanh(torch.nn.functional.linear(x.float().cpu(), w.float().cpu(), b.float().cpu()))
    tol = 1e-5 if mode == "fp32" else 8e-3
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=mode == "autocast"):
        with torch.no_grad():
            y = block_ops.linear_gelu_tanh(x, w, b)
            y_lp = block_ops.linear_gelu_tanh(x, w, b, w.bfloat16(), b.bfloat16())      # pre-cast copies
        y2 = block_ops.linear_gelu_tanh(x, w.requires_grad_(), b)                          # grad mode: two kernels
        t = torch.randn(x.shape, generator=g).to(x)
        yd, tyd = torch.func.jvp(lambda a: block_ops.linear_gelu_tanh(a, w.detach(), b), (x,), (t,))
    assert y.shape == (3, 50, 384) and y.dtype == (torch.float32 if mode == "fp32" else torch.bfloat16)
    for got in (y, y_lp, y2, yd):
        assert ao.rel_l2(got.float().cpu(), ref) <= tol
    _, t_ref = bo.jvp(lambda a: bo.gelu_tanh(torch.nn.functional.linear(a, w.detach().float().cpu(), b.float().cpu())),
                      (x.float().cpu(),), (t.float().cpu(),))
    assert ao.rel_l2(tyd.float().cpu(), t_ref) <= tol
    y2.float().sum().backward()
    assert w.grad is not None and float(w.grad.abs().max()) > 0
