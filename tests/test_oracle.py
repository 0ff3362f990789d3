"""Pins the CPU oracle (oracle/attn_oracle.py) with checks that do not retype
its formulas: a library routine (torch SDPA), finite differences, gradcheck,
closed-form special cases and algebraic invariants.  The reference holds no
golden vectors for this path (its only test is differential with unseeded
inputs, models/flash_attention_2_jvp.py:339-376), so these checks are what
fixes the oracle."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as ao

torch.manual_seed(0)


def _inputs(B=2, L=48, H=3, D=24, seed=11, Lkv=None, dtype=torch.float64):
    return [t.to(dtype) for t in ao.make_inputs(B, L, H, D, seed, Lkv=Lkv)]


def test_base_matches_sdpa_library_routine():
    q, k, v, *_ = _inputs(dtype=torch.float32)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert ao.rel_l2(ao.base_attn(q, k, v), ref) < 2e-6
    assert ao.rel_l2(ao.raw_attn(q, k, v), ref) < 2e-6


def test_base_brute_force_tiny():
    q, k, v, *_ = _inputs(B=1, L=5, H=2, D=3, Lkv=7)
    out = ao.base_attn(q, k, v)
    for h in range(2):
        for i in range(5):
            w = np.array([math.exp(sum(q[0, i, h, d].item() * k[0, j, h, d].item() for d in range(3)) / math.sqrt(3))
                          for j in range(7)])
            w /= w.sum()
            exp = sum(w[j] * v[0, j, h].numpy() for j in range(7))
            np.testing.assert_allclose(out[0, i, h].numpy(), exp, rtol=1e-12, atol=1e-14)


def test_closed_form_primal_and_lse():
    q, k, v, *_ = _inputs(Lkv=40)
    cf = ao.closed_form_fp64(q, k, v)
    assert ao.rel_l2(torch.from_numpy(cf["o"]), ao.base_attn(q, k, v)) < 1e-13
    assert ao.rel_l2(torch.from_numpy(cf["lse"]), ao.lse_ref(q, k)) < 1e-13


def test_jvp_finite_differences():
    q, k, v, tq, tk, tv, _ = _inputs()
    _, to = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    h = 1e-6
    fd = (ao.base_attn(q + h * tq, k + h * tk, v + h * tv) - ao.base_attn(q - h * tq, k - h * tk, v - h * tv)) / (2 * h)
    assert ao.rel_l2(to, fd) < 1e-8
    cf = ao.closed_form_fp64(q, k, v, tq, tk, tv)
    assert ao.rel_l2(torch.from_numpy(cf["to"]), fd) < 1e-8
    assert ao.rel_l2(torch.from_numpy(cf["to"]), to) < 1e-13
    # tangent of lse is mu = rowsum(P*dS)
    fd_lse = (ao.lse_ref(q + h * tq, k + h * tk) - ao.lse_ref(q - h * tq, k - h * tk)) / (2 * h)
    assert ao.rel_l2(torch.from_numpy(cf["mu"]), fd_lse) < 1e-8


def test_jvp_special_cases():
    q, k, v, tq, tk, tv, _ = _inputs()
    z = torch.zeros_like(q)
    # dQ = dK = 0  =>  dO = Attn(Q, K, dV)
    _, to = ao.base_attn_jvp(q, k, v, z, z, tv)
    assert ao.rel_l2(to, ao.base_attn(q, k, tv)) < 1e-13
    # all keys equal and all key tangents equal => P = 1/N, dP = 0
    k1, tk1 = k[:, :1].expand_as(k).contiguous(), tk[:, :1].expand_as(k).contiguous()
    o, to = ao.base_attn_jvp(q, k1, v, tq, tk1, tv)
    assert ao.rel_l2(o, v.mean(1, keepdim=True).expand_as(o)) < 1e-13
    assert ao.rel_l2(to, tv.mean(1, keepdim=True).expand_as(o)) < 1e-12
    # all values equal => dP V = 0
    v1 = v[:, :1].expand_as(v).contiguous()
    _, to = ao.base_attn_jvp(q, k, v1, tq, tk, z)
    assert to.abs().max() < 1e-13
    # N = 1 => O = V, dO = dV
    o, to = ao.base_attn_jvp(q[:, :1], k[:, :1], v[:, :1], tq[:, :1], tk[:, :1], tv[:, :1])
    assert torch.equal(o, v[:, :1]) and ao.rel_l2(to, tv[:, :1]) < 1e-15


def test_jvp_linearity_and_shift_invariance():
    q, k, v, tq, tk, tv, w = _inputs()
    _, a = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    _, b = ao.base_attn_jvp(q, k, v, w, tk.flip(1), tv.flip(1))
    _, c = ao.base_attn_jvp(q, k, v, 2 * tq - 3 * w, 2 * tk - 3 * tk.flip(1), 2 * tv - 3 * tv.flip(1))
    assert ao.rel_l2(c, 2 * a - 3 * b) < 1e-12
    # adding the same vector to every key shifts each score row by a constant: P and O unchanged
    o0 = ao.base_attn(q, k, v)
    shift = torch.randn(1, 1, k.shape[2], k.shape[3], dtype=k.dtype)
    # (q . (k + c)) = q.k + q.c  -> constant per query row
    assert ao.rel_l2(ao.base_attn(q, k + shift, v), o0) < 1e-12


def test_grads_gradcheck_and_adjoint():
    q, k, v, tq, tk, tv, dout = _inputs(B=1, L=6, H=2, D=4, Lkv=5)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    assert torch.autograd.gradcheck(ao.base_attn, (qg, kg, vg), eps=1e-6, atol=1e-7)
    q, k, v, tq, tk, tv, dout = _inputs()
    dq, dk, dv = ao.base_attn_grads(q, k, v, dout)
    _, to = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    lhs = (to * dout).sum()
    rhs = (tq * dq).sum() + (tk * dk).sum() + (tv * dv).sum()
    assert abs(lhs - rhs) / abs(lhs) < 1e-12
    cf = ao.closed_form_fp64(q, k, v, dout=dout)
    for name, g in zip(("dq", "dk", "dv"), (dq, dk, dv)):
        assert ao.rel_l2(torch.from_numpy(cf[name]), g) < 1e-13, name


@pytest.mark.parametrize("Lq,Lkv,blk", [(64, 64, 16), (40, 72, 32), (33, 50, 64)])
def test_streaming_specs_match_closed_form(Lq, Lkv, blk):
    q, k, v, tq, tk, tv, dout = _inputs(L=Lq, Lkv=Lkv)
    cf = ao.closed_form_fp64(q, k, v, tq, tk, tv, dout)
    for fn in (ao.streaming_fwd_jvp, ao.reference_streaming_fwd_jvp):
        o, to, lse, mu = fn(q, k, v, tq, tk, tv, block_kv=blk)
        assert ao.rel_l2(o, torch.from_numpy(cf["o"])) < 1e-13
        assert ao.rel_l2(to, torch.from_numpy(cf["to"])) < 1e-12
        assert ao.rel_l2(lse, torch.from_numpy(cf["lse"])) < 1e-13
        assert ao.rel_l2(mu, torch.from_numpy(cf["mu"])) < 1e-12
    dq, dk, dv = ao.streaming_bwd(q, k, v, torch.from_numpy(cf["o"]), torch.from_numpy(cf["lse"]), dout, block=blk)
    for name, g in zip(("dq", "dk", "dv"), (dq, dk, dv)):
        assert ao.rel_l2(g, torch.from_numpy(cf[name])) < 1e-12, name


def test_rms_norm_closed_form():
    x = torch.randn(2, 5, 3, 72)
    y = ao.rms_norm(x)
    exp = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    assert ao.rel_l2(y, exp) < 1e-6
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(2, 5, 3), atol=1e-4)
    g = torch.rand(72) + 0.5
    assert ao.rel_l2(ao.rms_norm(x, g), exp * g.double()) < 1e-6


def test_split_head_dim_table():
    # the docstring table of models/triton_utils.py:28-33 plus the cases FlashAttnFunc dispatches on
    assert ao.split_head_dim(72) == (64, 16)
    assert ao.split_head_dim(96) == (64, 32)
    assert ao.split_head_dim(80) == (64, 16)
    assert ao.split_head_dim(128) == (128, 0)
    assert ao.split_head_dim(64) == (64, 0)


def test_config1_fp32_oracle_is_self_consistent():
    """The CPU-runnable benchmark case (B2 H12 N256 D64 fp32): the fp32 jvp oracle is itself
    within 1e-6 of the fp64 closed form, so a 1e-5 kernel tolerance is meaningful."""
    q, k, v, tq, tk, tv, dout = ao.make_inputs(2, 256, 12, 64, seed=1)
    o, to = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    cf = ao.closed_form_fp64(q, k, v, tq, tk, tv, dout)
    assert ao.rel_l2(o, torch.from_numpy(cf["o"])) < 2e-6
    assert ao.rel_l2(to, torch.from_numpy(cf["to"])) < 2e-6
    for name, g in zip(("dq", "dk", "dv"), ao.base_attn_grads(q, k, v, dout)):
        assert ao.rel_l2(g, torch.from_numpy(cf[name])) < 2e-6


def test_golden_vectors():
    """The committed known-answer vectors (tests/golden/attn_vectors.npz, written once by
    tests/golden/make_attn_vectors.py from the fp64 closed forms): the fp32 oracle -- naive
    attention under torch.func.jvp and autograd -- must reproduce them."""
    import os
    import numpy as np
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attn_vectors.npz"))
    names = sorted({k.split(".")[0] for k in z.files})
    assert names == ["d64", "d72_cross"]
    for n in names:
        q, k, v, tq, tk, tv, do = (torch.from_numpy(z[f"{n}.{key}"]) for key in ("q", "k", "v", "tq", "tk", "tv", "dout"))
        o, to = ao.base_attn_jvp(q, k, v, tq, tk, tv)
        dq, dk, dv = ao.base_attn_grads(q, k, v, do)
        for key, got in (("o", o), ("to", to), ("dq", dq), ("dk", dk), ("dv", dv), ("lse", ao.lse_ref(q, k))):
            assert ao.rel_l2(got.double(), torch.from_numpy(z[f"{n}.{key}"])) < 2e-6, (n, key)
