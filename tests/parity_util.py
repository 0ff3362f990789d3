"""Helpers shared by the end-to-end parity tests."""
from oracle import attn_oracle as ao


def grads(model):
    return {n: p.grad.float().cpu() for n, p in model.named_parameters() if p.grad is not None}


def no_worse_than_base(g_fused, g_base, g_fp32, slack=1.5, floor=2e-3):
    """Gradient agreement under bf16 autocast, with the yardstick measured instead of guessed: the same step on the same
    weights in fp32 through the naive attention and the reference's expressions is the truth; the reference path under
    bf16 autocast sits at some distance from it (its rounding error), and the fused path may sit at most ``slack`` times
    as far, parameter by parameter (``floor`` covers parameters whose bf16 error is itself at fp32 rounding level)."""
    assert g_fused.keys() == g_base.keys() == g_fp32.keys()
    rows = []
    for n, ref in g_fp32.items():
        if float(ref.abs().max()) == 0:
            continue
        e_f, e_b = ao.rel_l2(g_fused[n], ref), ao.rel_l2(g_base[n], ref)
        rows.append((e_f / max(e_b, floor / slack), e_f, e_b, n))
    worst = max(rows)
    print(f"worst fused/base error ratio {worst[0]:.2f} (fused {worst[1]:.3e}, base {worst[2]:.3e}) at {worst[3]}; "
          f"largest base-bf16 error {max(r[2] for r in rows):.3e}", flush=True)
    for ratio, e_f, e_b, n in rows:
        assert e_f <= slack * e_b + floor, (n, e_f, e_b)
