"""GPU parity over a seeded sweep of odd shapes and memory layouts (small enough for
the CPU oracle): sequence lengths that are not multiples of any tile size, different
query / key lengths, every supported head dim, and the three layouts the operator
meets -- contiguous (B, L, H, D), views into a packed (B, L, 3, H, D) qkv buffer
(models/layers.py:143-147), and head-contiguous storage viewed as (B, L, H, D).
Tolerances as in test_attn_gpu.py: rel-L2 1e-5 (fp32), 2e-2 (bf16)."""
import random

import pytest
import torch

from dmf_amd import _lib
from oracle import attn_oracle as ao

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def _layout(t_cpu, layout, dtype):
    """Device tensor with the values of t_cpu (B, L, H, D) stored in the given layout."""
    t = t_cpu.to(dtype)
    if layout == "contiguous":
        return t.to(DEV)
    if layout == "packed":      # slot 1 of a (B, L, 3, H, D) buffer
        B, L, H, D = t.shape
        buf = torch.zeros(B, L, 3, H, D, dtype=dtype, device=DEV)
        buf[:, :, 1] = t.to(DEV)
        return buf[:, :, 1]
    if layout == "head_major":  # stored (B, H, L, D), viewed (B, L, H, D)
        return t.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    raise ValueError(layout)


def _cases():
    rng = random.Random(1234)
    out = []
    for i in range(36):
        D = rng.choice([32, 64, 72, 80, 96, 128])
        out.append((rng.randint(1, 3), rng.randint(1, 5), rng.randint(1, 300), rng.randint(1, 300), D,
                    rng.choice(["contiguous", "packed", "head_major"]), torch.bfloat16 if i % 3 else torch.float32, 1000 + i))
    return out


@pytest.mark.parametrize("B,H,Lq,Lkv,D,layout,dtype,seed", _cases())
def test_shape_sweep(B, H, Lq, Lkv, D, layout, dtype, seed):
    print(f"case B{B} H{H} Lq{Lq} Lkv{Lkv} D{D} {layout} {dtype} seed{seed}", flush=True)
    cpu = [t.to(dtype).float() for t in ao.make_inputs(B, Lq, H, D, seed, Lkv=Lkv)]
    q, k, v, tq, tk, tv, do = cpu
    gq, gk, gv, gtq, gtk, gtv, gdo = (_layout(t, layout, dtype) for t in cpu)
    scale = D ** -0.5
    tol = TOL[dtype]
    o_ref, to_ref = ao.base_attn_jvp(q, k, v, tq, tk, tv)
    o, to, lse = _lib.fwd_jvp(gq, gk, gv, gtq, gtk, gtv, scale)
    assert o.is_contiguous() and to.is_contiguous()
    assert ao.rel_l2(o.float().cpu(), o_ref) <= tol
    assert ao.rel_l2(to.float().cpu(), to_ref) <= tol
    assert ao.rel_l2(lse.cpu(), ao.lse_ref(q, k)) <= (1e-5 if dtype == torch.float32 else 1e-3)
    o2, lse2 = _lib.fwd(gq, gk, gv, scale)
    assert ao.rel_l2(o2.float().cpu(), o_ref) <= tol
    if Lkv > 1:   # with a single key dQ and dK are exactly zero (no relative error)
        refs = ao.base_attn_grads(q, k, v, do)
        got = _lib.bwd(gdo, gq, gk, gv, o2, lse2, scale)
        for name, a, b in zip(("dq", "dk", "dv"), got, refs):
            assert ao.rel_l2(a.float().cpu(), b) <= tol, name
