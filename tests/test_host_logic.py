"""CPU-only tests: the C-ABI library loads and exports what include/dmf_attn.h
and include/dmf_block.h declare, argument validation returns the documented codes (no kernel is
launched on those paths), and the autograd / forward-AD protocol of the Python
operator behaves like the reference's (models/flash_attention_2_jvp.py:177-319)
when the three kernel calls are replaced by stand-ins defined in this file."""
import ctypes
import os
import re

import pytest
import torch

import dmf_amd
from dmf_amd import _lib, flash_attention_hip_jvp as fa
from dmf_amd.layers import attn_op, Attention, RMSNorm, get_2d_sincos_pos_embed
from oracle import attn_oracle as ao

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = []
    for header in ("dmf_attn.h", "dmf_block.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        names += re.findall(r"DMF_ATTN_API\s+[\w\s\*]+?\b(dmf_\w+)\s*\(", text)
    return names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) == 22 and set(names) == set(_lib.SIGNATURES), names
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.dmf_attn_version() >= 1
    assert lib.dmf_attn_strerror(0) == b"ok"
    for code in range(-9, 0):
        assert b"unknown" not in lib.dmf_attn_strerror(code)
    assert b"unknown" in lib.dmf_attn_strerror(-99)


def test_plan_names_the_kernels_without_launching():
    """dmf_attn_plan is host-only: it answers on a machine without a GPU too (a device whose compute-unit count cannot
    be asked counts as 256 units, the MI355X's)."""
    bf, f32 = torch.bfloat16, torch.float32
    assert _lib.plan("fwd_jvp", 64, 16, 1024, 1024, 72, bf) == "dmf::attn_fwd_bf16_kernel<72, true, 8, false, false>"
    assert _lib.plan("fwd", 256, 16, 256, 256, 72, bf) == "dmf::attn_fwd_bf16_kernel<72, false, 8, false, false>"
    assert _lib.plan("bwd", 256, 16, 256, 256, 72, bf) == "dmf::attn_bwd_fused_bf16_kernel<72>"
    assert _lib.plan("bwd", 64, 16, 1024, 1024, 72, bf) == "dmf::attn_bwd_dq_bf16_kernel<72, 2> + dmf::attn_bwd_dkv_bf16_kernel<72, 4>"
    assert _lib.plan("bwd", 2, 2, 128, 128, 72, bf).startswith("dmf::attn_bwd_dq_bf16_kernel")     # too short for the single pass
    assert _lib.plan("fwd_jvp", 2, 12, 256, 256, 64, f32) == "dmf::attn_fwd_kernel<float, 64, true>"
    assert _lib.plan("fwd", 1, 1, 7, 9, 32, bf) == "dmf::attn_fwd_kernel<__bf16, 32, false>"            # no tuned kernel at head dim 32
    assert _lib.plan("fwd_qknorm_jvp", 16, 16, 1024, 1024, 72, bf) == "dmf::attn_fwd_bf16_kernel<72, true, 8, true, true>"
    with pytest.raises(RuntimeError, match="no kernel"):
        _lib.plan("fwd_qnorm_jvp", 1, 1, 64, 64, 72, f32)
    lib = _lib.load()
    small = ctypes.create_string_buffer(8)
    assert lib.dmf_attn_plan(1, 1, 1, 64, 64, 72, 1, small, 8) == 0 and small.value == b"dmf::at"   # truncated, NUL-terminated
    assert lib.dmf_attn_plan(1, 1, 1, 64, 64, 40, 1, small, 8) == -2
    assert lib.dmf_attn_plan(9, 1, 1, 64, 64, 72, 1, small, 8) == -3
    assert lib.dmf_attn_plan(1, 1, 1, 64, 64, 72, 1, None, 8) == -5


def test_validation_codes_without_launch():
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) // 16 * 16
    st4 = (ctypes.c_int64 * 16)(*([64 * 4 * 2, 64 * 2, 64, 1] * 4))
    call = lambda **kw: lib.dmf_attn_fwd(
        kw.get("q", p), p, p, p, None, kw.get("st", st4), kw.get("B", 1), 2, 4, 4, kw.get("D", 64), 0.125, kw.get("dtype", 0), None)
    assert call(D=40) == -2          # head dim
    assert call(dtype=7) == -1       # dtype
    assert call(B=0) == -3           # shape
    assert call(q=None) == -5        # null
    assert call(q=p + 4) == -6       # alignment
    bad = (ctypes.c_int64 * 16)(*([64 * 4 * 2, 64 * 2, 64, 2] * 4))
    assert call(st=bad) == -4        # last-dim stride
    bad2 = (ctypes.c_int64 * 16)(*([64 * 4 * 2, 64 * 2 + 1, 64, 1] * 4))
    assert call(st=bad2) == -4       # row alignment
    # fwd_jvp requires lse
    st8 = (ctypes.c_int64 * 32)(*([64 * 4 * 2, 64 * 2, 64, 1] * 8))
    assert lib.dmf_attn_fwd_jvp(p, p, p, p, p, p, p, p, None, None, st8, 1, 2, 4, 4, 64, 0.125, 0, None) == -5
    assert lib.dmf_attn_bwd(p, p, p, p, p, None, p, p, p, None, st8, 1, 2, 4, 4, 64, 0.125, 0, None) == -5


def test_cpu_tensors_fail_loudly():
    q = torch.randn(1, 4, 2, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        dmf_amd.flash_attn_func(q, q, q)
    with pytest.raises(ValueError):
        attn_op(q, q, q, op="nope")


@pytest.fixture
def fake_kernels(monkeypatch):
    """Replace the three C-ABI calls by plain-torch stand-ins and count calls."""
    calls = {"fwd": 0, "fwd_jvp": 0, "bwd": 0}

    def scaled(scale, d):   # the naive operator with the softmax scale the wrapper asks for instead of d ** -0.5
        return lambda q, k, v: ao.base_attn(q * (scale * d ** 0.5), k, v)

    def fwd(q, k, v, scale, need_lse=True):
        calls["fwd"] += 1
        return scaled(scale, q.shape[-1])(q, k, v).contiguous(), ao.lse_ref(q, k, scale).float()

    def fwd_jvp(q, k, v, tq, tk, tv, scale, need_dlse=False):
        calls["fwd_jvp"] += 1
        # plain torch ops only: this runs inside forward-AD / functorch levels
        o, to, lse, mu = ao.streaming_fwd_jvp(q, k, v, tq, tk, tv, scale=scale, block_kv=8, dtype=q.dtype)
        out = (o.contiguous(), to.contiguous(), lse.float())
        return out + (mu.float(),) if need_dlse else out

    def bwd(dout, q, k, v, o, lse, scale):
        calls["bwd"] += 1
        with torch.enable_grad():   # autograd runs backward() with grad mode off
            return ao.base_attn_grads(q, k, v, dout, fn=scaled(scale, q.shape[-1]))

    monkeypatch.setattr(_lib, "fwd", fwd)
    monkeypatch.setattr(_lib, "fwd_jvp", fwd_jvp)
    monkeypatch.setattr(_lib, "bwd", bwd)
    return calls


def test_func_jvp_then_backward_protocol(fake_kernels):
    """Structure of the reference self-test (flash_attention_2_jvp.py:344-376):
    jvp of the op, then backward on the primal output."""
    q, k, v, tq, tk, tv, do = [t.double() for t in ao.make_inputs(2, 16, 2, 8, seed=3, std=0.5)]
    q, k, v = (t.requires_grad_() for t in (q, k, v))
    u_ref, du_ref = torch.func.jvp(ao.raw_attn, (q, k, v), (tq, tk, tv))
    u, du = torch.func.jvp(fa.flash_attn_func, (q, k, v), (tq, tk, tv))
    assert fake_kernels == {"fwd": 0, "fwd_jvp": 1, "bwd": 0}     # one fused pass, no separate primal pass
    assert ao.rel_l2(u, u_ref) < 1e-12 and ao.rel_l2(du, du_ref) < 1e-12
    ref = torch.autograd.grad(u_ref, (q, k, v), do)
    got = torch.autograd.grad(u, (q, k, v), do)
    assert fake_kernels["bwd"] == 1
    for a, b in zip(got, ref):
        assert ao.rel_l2(a, b) < 1e-12


def test_partial_tangents_are_zero_filled(fake_kernels):
    """Only q is dual: k, v tangents become zeros (flash_attention_2_jvp.py:303-304)."""
    import torch.autograd.forward_ad as fwAD
    q, k, v, tq, *_ = [t.double() for t in ao.make_inputs(1, 12, 2, 8, seed=4)]
    with fwAD.dual_level():
        out = fa.flash_attn_func(fwAD.make_dual(q, tq), k, v)
        o, to = fwAD.unpack_dual(out)
    _, to_ref = ao.base_attn_jvp(q, k, v, tq, torch.zeros_like(k), torch.zeros_like(v))
    assert ao.rel_l2(to, to_ref) < 1e-12
    assert fake_kernels["fwd_jvp"] == 1


def test_plain_inputs_take_primal_only_path(fake_kernels):
    q, k, v, *_ = [t.double() for t in ao.make_inputs(1, 12, 2, 8, seed=5)]
    with torch.no_grad():
        o = fa.flash_attn_func(q, k, v)
    assert fake_kernels == {"fwd": 1, "fwd_jvp": 0, "bwd": 0}
    assert ao.rel_l2(o, ao.base_attn(q, k, v)) < 1e-12
    q.requires_grad_()
    o = fa.flash_attn_func(q, k, v)
    o.sum().backward()
    assert fake_kernels["bwd"] == 1 and q.grad is not None


def test_function_jvp_staticmethod_is_functional(fake_kernels):
    """Dual tensors handed straight to FlashAttnFunc.apply: forward runs
    primal-only, then ``jvp`` produces the tangent with a second fused pass."""
    q, k, v, tq, tk, tv, _ = [t.double() for t in ao.make_inputs(1, 12, 2, 8, seed=6)]
    f = lambda q, k, v: fa.FlashAttnFunc.apply(q, k, v, None, None, None, None)[0]
    o, to = torch.func.jvp(f, (q, k, v), (tq, tk, tv))
    o_ref, to_ref = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    assert ao.rel_l2(o, o_ref) < 1e-12 and ao.rel_l2(to, to_ref) < 1e-12
    assert fake_kernels["fwd"] == 1 and fake_kernels["fwd_jvp"] == 1
    # the lse output carries its tangent too (rowsum(P*dS))
    g = lambda q, k, v: fa.FlashAttnFunc.apply(q, k, v, None, None, None, None)[1]
    lse, dlse = torch.func.jvp(g, (q, k, v), (tq, tk, tv))
    cf = ao.closed_form_fp64(q, k, v, tq, tk, tv)
    assert ao.rel_l2(lse, torch.from_numpy(cf["lse"])) < 1e-6 and ao.rel_l2(dlse, torch.from_numpy(cf["mu"])) < 1e-6


def test_attn_op_base_and_sdpa_branches():
    q, k, v, *_ = ao.make_inputs(2, 10, 3, 16, seed=7)
    assert ao.rel_l2(attn_op(q, k, v, "base"), ao.base_attn(q, k, v)) < 1e-7
    assert ao.rel_l2(attn_op(q, k, v, "torch_sdpa"), ao.base_attn(q, k, v)) < 2e-6


def test_attention_module_feeds_packed_qkv_views(fake_kernels, monkeypatch):
    """q, k, v reach the operator as (B, L, H, D) views with strides
    (3LHD, 3HD, D, 1) (reference models/layers.py:143-147); with qk-norm q and k
    become contiguous and v stays a view."""
    seen = []
    orig = _lib.fwd
    monkeypatch.setattr(_lib, "fwd", lambda q, k, v, s, need_lse=True: (seen.append((q.stride(), k.stride(), v.stride())), orig(q, k, v, s))[1])
    B, L, H, D = 2, 6, 3, 32        # a head dim the kernels take as it is (others are padded into copies)
    x = torch.randn(B, L, H * D)
    for qk_norm in (False, True):
        m = Attention(H * D, num_heads=H, qkv_bias=True, qk_norm=qk_norm, attn_func="hip")
        m_ref = Attention(H * D, num_heads=H, qkv_bias=True, qk_norm=qk_norm, attn_func="base")
        m_ref.load_state_dict(m.state_dict())
        with torch.no_grad():
            assert ao.rel_l2(m(x), m_ref(x)) < 1e-5
    packed = (3 * L * H * D, 3 * H * D, D, 1)
    assert seen[0] == (packed, packed, packed)
    assert seen[1][2] == packed and seen[1][0] == (L * H * D, H * D, D, 1)


def test_rmsnorm_and_pos_embed_match_oracle_formulas():
    x = torch.randn(2, 5, 3, 72)
    assert ao.rel_l2(RMSNorm(72)(x), ao.rms_norm(x)) < 1e-7
    pe = get_2d_sincos_pos_embed(16, 4)
    assert pe.shape == (16, 16)
    # token (row r, col c) -> first half encodes c, second half r; position 0 -> sin 0, cos 1
    assert abs(pe[0, :4]).max() == 0 and (pe[0, 4:8] == 1).all()
    assert pe[1, 0] == pytest.approx(float(torch.sin(torch.tensor(1.0))))   # token 1 = (row 0, col 1)
    assert pe[4, 8] == pytest.approx(float(torch.sin(torch.tensor(1.0))))   # token 4 = (row 1, col 0)


def test_block_abi_validation_codes_without_launch():
    """Argument checks of the block-glue entry points return before any launch."""
    lib = _lib.load()
    buf = ctypes.create_string_buffer(1 << 16)
    p = (ctypes.addressof(buf) + 15) // 16 * 16
    ms = (ctypes.c_int64 * 4)(64, 64, 64, 64)
    ln = lambda **kw: lib.dmf_ln_modulate_fwd(
        kw.get("x", p), None, p, kw.get("scale", p), None, None, p, None, kw.get("ms", ms), kw.get("B", 2), 4, kw.get("C", 64),
        1e-6, kw.get("dt", 0), 0, 0, None)
    assert ln(C=20) == -3 and ln(C=4096) == -3 and ln(B=0) == -3
    assert ln(dt=5) == -1
    assert ln(x=None) == -5 and ln(scale=None) == -5
    assert ln(x=p + 8) == -6
    assert ln(ms=(ctypes.c_int64 * 4)(64, 66, 64, 64)) == -4
    assert lib.dmf_gelu_tanh_fwd(p, None, p, None, 12, 0, None) == -3      # n not a multiple of 8
    assert lib.dmf_gelu_tanh_fwd(p, None, p, p, 16, 0, None) == -5         # tangent output without tangent input
    assert lib.dmf_gelu_tanh_bwd(None, p, p, 16, 0, None) == -5
    st = (ctypes.c_int64 * 8)(*([4 * 2 * 24, 2 * 24, 24, 1] * 2))
    assert lib.dmf_rmsnorm_fwd(p, None, p, p, None, st, 1, 4, 2, 20, 1e-6, 0, 0, None) == -2   # head dim
    bad = (ctypes.c_int64 * 8)(*([4 * 2 * 24, 2 * 24, 24, 2] * 2))
    assert lib.dmf_rmsnorm_fwd(p, None, p, p, None, bad, 1, 4, 2, 24, 1e-6, 0, 0, None) == -4
    assert lib.dmf_gate_residual_bwd(p, p, p, p, p, None, 64, 2, 4, 64, 0, 0, 0, None) == -5   # workspace missing
    assert lib.dmf_block_workspace_floats(0, 2, 33, 64) == 2 * 3 * 2 * 64
    assert lib.dmf_block_workspace_floats(1, 2, 33, 64) == 2 * 3 * 64
    assert lib.dmf_block_workspace_floats(2, 1, 1, 72) == 1024 * 72
    assert lib.dmf_block_workspace_floats(9, 1, 1, 72) == 0


def test_run_function_below_a_single_jvp_level_matches_functorch_dispatch(monkeypatch):
    """``_lib.run_function`` with a gradient needed inside one ``torch.func.jvp`` level:
    running the autograd node below the level gives the values and gradients of
    functorch's own custom-Function dispatch; other transforms keep using ``apply``."""
    import torch.autograd.forward_ad as fwAD

    class Scale(torch.autograd.Function):
        """(x, tx, w) -> (x w, tx w), gradient through the primal output only."""
        calls = []

        @staticmethod
        def forward(x, tx, w):
            return x * w, (None if tx is None else tx * w)

        @staticmethod
        def setup_context(ctx, inputs, outputs):
            ctx.save_for_backward(inputs[0], inputs[2])
            ctx.set_materialize_grads(False)
            Scale.calls.append(_lib._functorch.is_functorch_wrapped_tensor(inputs[0]))

        @staticmethod
        def backward(ctx, gy, gty):
            x, w = ctx.saved_tensors
            return gy * w, None, (gy * x).sum(0)

    def op(x, w):
        p, t = fwAD.unpack_dual(x)
        y, ty = _lib.run_function(Scale, p, t, w)
        return y if t is None else fwAD.make_dual(y, ty)

    g = torch.Generator().manual_seed(9)
    w = torch.randn(8, generator=g).requires_grad_()
    x, v = torch.randn(4, 8, generator=g), torch.randn(4, 8, generator=g)
    f = lambda a: op(torch.tanh(op(a, w)), w)
    results = []
    for flag in (True, False):
        monkeypatch.setattr(_lib, "BASE_LEVEL_UNDER_JVP", flag)
        Scale.calls.clear()
        w.grad = None
        y, ty = torch.func.jvp(f, (x,), (v,))
        ((y - (0.5 * ty).detach()) ** 2).mean().backward()
        results.append((y.detach(), ty.detach(), w.grad.clone()))
        # below the level the node sees raw tensors, once per call; functorch's dispatch hands it wrapped ones as well
        assert Scale.calls == [False, False] if flag else any(Scale.calls)
    for a, b in zip(*results):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-7)
    # tangent against central differences, gradient against plain autograd of the same expression
    h = 1e-3
    fd = (f(x + h * v) - f(x - h * v)) / (2 * h)
    assert torch.allclose(results[0][1], fd.detach(), atol=1e-3)
    w.grad = None
    yy = f(x)
    ((yy - (0.5 * results[0][1])) ** 2).mean().backward()
    assert torch.allclose(results[0][2], w.grad, rtol=1e-5, atol=1e-6)
    # no gradient needed: forward is called directly (no autograd node at all)
    monkeypatch.setattr(_lib, "BASE_LEVEL_UNDER_JVP", True)
    Scale.calls.clear()
    torch.func.jvp(lambda a: op(a, w.detach()), (x,), (v,))
    assert Scale.calls == []
    # a grad transform is not a jvp level: plain apply
    Scale.calls.clear()
    gx = torch.func.grad(lambda a: op(a, w.detach()).sum())(x)
    assert torch.allclose(gx, w.detach().expand_as(x)) and any(Scale.calls)


def test_frozen_low_precision_params_nest_and_restore():
    from dmf_amd.layers import Linear, frozen_low_precision_params
    m = torch.nn.Sequential(Linear(8, 8, block_ops="hip"), Linear(8, 4, bias=False, block_ops="hip"), torch.nn.Linear(4, 4))
    with frozen_low_precision_params(m):
        outer = m[0].lp_weight
        assert outer.dtype == torch.bfloat16 and torch.equal(outer, m[0].weight.detach().bfloat16())
        assert m[1].lp_bias is None and m[1].lp_weight is not None and not hasattr(m[2], "lp_weight")
        with frozen_low_precision_params(m, torch.float16):
            assert m[0].lp_weight.dtype == torch.float16
        assert m[0].lp_weight is outer              # the inner context put the outer copies back
    assert m[0].lp_weight is None and m[0].lp_bias is None and m[1].lp_weight is None


def test_fused_block_operators_refuse_a_gradient_at_their_tangent_output():
    """The fused block operators back-propagate through the primal output only (exact for the MeanFlow loss, whose JVP
    target is detached, loss.py:171-172).  A loss that keeps the JVP output attached must hear about it instead of
    getting gradients without the second-order terms that the reference's tensor expressions would supply."""
    from dmf_amd import block_ops
    g = torch.ones(2, 3)
    for fn, grads in ((block_ops.LNModulateFunc, (None, g)), (block_ops.GateResidualFunc, (g, g)),
                      (block_ops.ResidualLNModulateFunc, (g, None, None, g)), (block_ops.GeluTanhFunc, (None, g)),
                      (block_ops.SiluFunc, (g, g)), (block_ops.RMSNormFunc, (None, g)), (block_ops.DualLinearFunc, (g, g, None))):
        with pytest.raises(NotImplementedError, match="primal output only"):
            fn.backward(None, *grads)


def test_stale_gradient_accumulator_probe():
    """GraphedStep refuses to capture a backward pass while an autograd graph of an earlier step is alive; the probe
    behind that refusal, on the CPU."""
    from dmf_amd.harness import stale_grad_accumulator
    p = torch.nn.Parameter(torch.randn(3))
    assert not stale_grad_accumulator(p) and not stale_grad_accumulator(p)
    with torch.no_grad():                      # the probe must not depend on the caller's gradient mode
        assert not stale_grad_accumulator(p)
    assert not stale_grad_accumulator(torch.zeros(3))   # no gradient, no accumulator
    loss = (p * 2).sum()
    assert stale_grad_accumulator(p)
    loss.backward()
    assert stale_grad_accumulator(p)          # the graph's nodes live as long as `loss` does
    del loss
    assert not stale_grad_accumulator(p)
