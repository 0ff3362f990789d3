"""CPU restatement of the reference's attention semantics.  TEST INFRASTRUCTURE ONLY.

Every function cites the reference lines it follows (paths relative to the
reference repository root).  Parity status of each function, i.e. which
independent checks in ``tests/test_oracle.py`` pin it:

* ``base_attn``            -- pinned: torch SDPA (library routine), numpy fp64
                              brute force, N=1 and uniform-score closed forms.
* ``base_attn_jvp``        -- pinned: fp64 closed form (``closed_form_fp64``),
                              central finite differences, special cases
                              (dQ=dK=0, equal keys, equal values, N=1),
                              linearity, rowsum(dP)=0.
* ``base_attn_grads``      -- pinned: ``torch.autograd.gradcheck`` in fp64,
                              adjoint identity <JVP t, w> = <t, VJP w>, and the
                              explicit flash-attention backward formulas.
* ``closed_form_fp64``     -- numpy fp64 statement of the textbook formulas; it
                              is itself checked by finite differences.
* ``streaming_fwd_jvp``    -- blockwise executable spec of the one-pass
                              algorithm; pinned against ``closed_form_fp64``.
* ``reference_streaming_fwd_jvp`` -- the reference kernel's own per-block
                              renormalising recurrence; pinned against
                              ``closed_form_fp64`` (shows both recurrences agree).
* ``streaming_bwd``        -- blockwise spec of the backward; pinned against
                              autograd of ``base_attn``.
* ``rms_norm``             -- pinned: closed form x/sqrt(mean x^2+eps).
* ``split_head_dim``       -- pinned: the docstring table at
                              models/triton_utils.py:28-33.
* ``raw_attn``             -- pinned: equals ``base_attn`` up to rounding.
"""
from __future__ import annotations

import math

import numpy as np
import torch


# --------------------------------------------------------------------------
# Naive operator ('base' branch)
# --------------------------------------------------------------------------
def base_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Naive attention on (B, L, H, D) tensors, returns (B, L, H, D).

    Follows models/layers.py:101,108-114: transpose to (B, H, L, D), scale q
    by D**-0.5 *before* the score matmul, softmax over keys, multiply by v,
    transpose back.
    """
    q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    scale = q.shape[-1] ** -0.5
    q = q * scale
    attn = q @ k.transpose(-2, -1)
    attn = attn.softmax(dim=-1)
    x = attn @ v
    return x.transpose(1, 2)


def raw_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Naive attention that divides the scores by sqrt(D) *after* the matmul.

    Follows models/flash_attention_2_jvp.py:322-336 (the reference self-test's
    comparison function).
    """
    q, k, v = (t.permute(0, 2, 1, 3) for t in (q, k, v))
    scores = torch.matmul(q, k.transpose(-2, -1)) / (q.shape[-1] ** 0.5)
    out = torch.matmul(torch.softmax(scores, dim=-1), v)
    return out.permute(0, 2, 1, 3)


def base_attn_jvp(q, k, v, tq, tk, tv, fn=base_attn):
    """(O, dO) of the naive operator under ``torch.func.jvp``.

    This is the contract's oracle: the 'base' branch (models/layers.py:108-113)
    pushed through forward-mode AD the way loss.py:165-170 does it.
    """
    return torch.func.jvp(fn, (q, k, v), (tq, tk, tv))


def base_attn_grads(q, k, v, dout, fn=base_attn):
    """(dQ, dK, dV) of the naive operator by reverse-mode autograd, as in the
    reference self-test (models/flash_attention_2_jvp.py:361-369)."""
    q, k, v = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    out = fn(q, k, v)
    return torch.autograd.grad(out, (q, k, v), dout)


def lse_ref(q: torch.Tensor, k: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """Natural-log logsumexp of the *scaled* scores, shape (B, H, Lq), the
    convention of models/triton_utils.py:347 (``m_i + log(l_i)``)."""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    s = torch.einsum("bqhd,bkhd->bhqk", q.double(), k.double()) * scale
    return torch.logsumexp(s, dim=-1)


# --------------------------------------------------------------------------
# Textbook closed forms in fp64 (numpy)
# --------------------------------------------------------------------------
def closed_form_fp64(q, k, v, tq=None, tk=None, tv=None, dout=None, scale=None):
    """All quantities of the path from the explicit formulas, in numpy fp64.

    Inputs are array-likes of shape (B, L, H, D).  Returns a dict with
    ``o`` and ``lse`` always; ``to`` and ``mu`` when tangents are given
    (dS = s (dQ K^T + Q dK^T);  mu = rowsum(P*dS);  dP = P*(dS - mu);
    dO = dP V + P dV -- the quantities of models/triton_utils.py:92-118);
    ``dq, dk, dv`` when ``dout`` is given (delta = rowsum(dout*o);
    dV = P^T dout; dP = dout V^T; dS = P*(dP - delta); dQ = s dS K;
    dK = s dS^T Q -- the standard flash-attention backward that
    models/flash_attention_2_jvp.py:260-276 delegates to).
    """
    f = lambda t: None if t is None else np.asarray(
        t.detach().double().cpu().numpy() if isinstance(t, torch.Tensor) else t, dtype=np.float64
    ).transpose(0, 2, 1, 3)  # -> (B, H, L, D)
    Q, K, V, TQ, TK, TV, DO = map(f, (q, k, v, tq, tk, tv, dout))
    D = Q.shape[-1]
    s = D ** -0.5 if scale is None else float(scale)
    S = s * np.einsum("bhqd,bhkd->bhqk", Q, K)
    m = S.max(-1, keepdims=True)
    E = np.exp(S - m)
    l = E.sum(-1, keepdims=True)
    P = E / l
    O = np.einsum("bhqk,bhkd->bhqd", P, V)
    back = lambda t: np.ascontiguousarray(t.transpose(0, 2, 1, 3))
    out = {"o": back(O), "lse": (m + np.log(l))[..., 0]}
    if TQ is not None:
        dS = s * (np.einsum("bhqd,bhkd->bhqk", TQ, K) + np.einsum("bhqd,bhkd->bhqk", Q, TK))
        G = P * dS
        mu = G.sum(-1, keepdims=True)
        dP = G - P * mu
        TO = np.einsum("bhqk,bhkd->bhqd", dP, V) + np.einsum("bhqk,bhkd->bhqd", P, TV)
        out["to"] = back(TO)
        out["mu"] = mu[..., 0]
    if DO is not None:
        delta = (DO * O).sum(-1, keepdims=True)
        dV = np.einsum("bhqk,bhqd->bhkd", P, DO)
        dP = np.einsum("bhqd,bhkd->bhqk", DO, V)
        dS = P * (dP - delta)
        out["dq"] = back(s * np.einsum("bhqk,bhkd->bhqd", dS, K))
        out["dk"] = back(s * np.einsum("bhqk,bhqd->bhkd", dS, Q))
        out["dv"] = back(dV)
        out["delta"] = delta[..., 0]
    return out


# --------------------------------------------------------------------------
# Executable specs of the streaming algorithms (blockwise, CPU)
# --------------------------------------------------------------------------
def streaming_fwd_jvp(q, k, v, tq, tk, tv, scale=None, block_kv=64, dtype=torch.float64):
    """One-pass online-softmax forward + JVP with *unnormalised* accumulators.

    Per KV block with E = exp(S - m):  l += rowsum(E);  acc_o += E V;
    acc_t += (E*dS) V + E dV;  acc_mu += rowsum(E*dS), every accumulator being
    multiplied by exp(m_old - m_new) when the running maximum moves.  Epilogue:
    O = acc_o / l;  mu = acc_mu / l;  dO = acc_t / l - mu O;  lse = m + log l.
    Algebraically identical to the per-block renormalising update of
    models/triton_utils.py:92-118 (see ``reference_streaming_fwd_jvp``).
    Returns (o, to, lse, mu) with o/to shaped (B, L, H, D), lse/mu (B, H, Lq).
    """
    Q, K, V, TQ, TK, TV = (t.to(dtype).transpose(1, 2) for t in (q, k, v, tq, tk, tv))
    B, H, Lq, D = Q.shape
    Lk = K.shape[2]
    s = D ** -0.5 if scale is None else float(scale)
    m = torch.full((B, H, Lq, 1), -math.inf, dtype=dtype)
    l = torch.zeros((B, H, Lq, 1), dtype=dtype)
    mu = torch.zeros_like(l)
    acc_o = torch.zeros((B, H, Lq, D), dtype=dtype)
    acc_t = torch.zeros_like(acc_o)
    for j in range(0, Lk, block_kv):
        Kj, Vj, TKj, TVj = (t[:, :, j:j + block_kv] for t in (K, V, TK, TV))
        S = s * (Q @ Kj.transpose(-1, -2))
        dS = s * (TQ @ Kj.transpose(-1, -2) + Q @ TKj.transpose(-1, -2))
        m_new = torch.maximum(m, S.amax(-1, keepdim=True))
        alpha = torch.exp(m - m_new)
        E = torch.exp(S - m_new)
        G = E * dS
        l = l * alpha + E.sum(-1, keepdim=True)
        mu = mu * alpha + G.sum(-1, keepdim=True)
        acc_o = acc_o * alpha + E @ Vj
        acc_t = acc_t * alpha + G @ Vj + E @ TVj
        m = m_new
    o = acc_o / l
    mu = mu / l
    to = acc_t / l - mu * o
    lse = (m + torch.log(l))[..., 0]
    return o.transpose(1, 2), to.transpose(1, 2), lse, mu[..., 0]


def reference_streaming_fwd_jvp(q, k, v, tq, tk, tv, scale=None, block_kv=128, dtype=torch.float64):
    """The reference kernel's own recurrence, restated on CPU tensors: the
    running O, dO and mu are kept *normalised* after every KV block
    (models/triton_utils.py:92-118; epilogue lse at :347)."""
    Q, K, V, TQ, TK, TV = (t.to(dtype).transpose(1, 2) for t in (q, k, v, tq, tk, tv))
    B, H, Lq, D = Q.shape
    s = D ** -0.5 if scale is None else float(scale)
    m_i = torch.full((B, H, Lq), -math.inf, dtype=dtype)
    l_i = torch.zeros((B, H, Lq), dtype=dtype)   # the kernel starts l at 1 with o=0; 0 is equivalent
    mu_i = torch.zeros_like(l_i)
    o = torch.zeros((B, H, Lq, D), dtype=dtype)
    to = torch.zeros_like(o)
    for j in range(0, K.shape[2], block_kv):
        Kj, Vj, TKj, TVj = (t[:, :, j:j + block_kv] for t in (K, V, TK, TV))
        qk = s * (Q @ Kj.transpose(-1, -2))
        m_ij = torch.maximum(m_i, qk.amax(-1))
        p = torch.exp(qk - m_ij[..., None])
        l_ij = p.sum(-1)
        alpha = torch.exp(m_i - m_ij)
        tqk = s * (TQ @ Kj.transpose(-1, -2) + Q @ TKj.transpose(-1, -2))
        p_tqk = p * tqk
        l_new = l_i * alpha + l_ij
        inv = 1.0 / l_new
        scale_prev = alpha * l_i * inv
        o_new = scale_prev[..., None] * o + (p @ Vj) * inv[..., None]
        s_mu = p_tqk.sum(-1)
        mu_new = scale_prev * mu_i + s_mu * inv
        to = (scale_prev[..., None] * to
              + (scale_prev * mu_i)[..., None] * (o - o_new)
              + (p_tqk @ Vj + p @ TVj - s_mu[..., None] * o_new) * inv[..., None])
        mu_i, l_i, m_i, o = mu_new, l_new, m_ij, o_new
    lse = m_i + torch.log(l_i)
    return o.transpose(1, 2), to.transpose(1, 2), lse, mu_i


def streaming_bwd(q, k, v, o, lse, dout, scale=None, block=64, dtype=torch.float64):
    """Blockwise backward on the primal output from saved (o, lse):
    delta = rowsum(dout*o);  P = exp(s Q K^T - lse);  dV = P^T dout;
    dP = dout V^T;  dS = P*(dP - delta);  dQ = s dS K;  dK = s dS^T Q.
    This is the computation models/flash_attention_2_jvp.py:260-276 hands to
    the third-party flash-attention backward.  Returns (dq, dk, dv)."""
    Q, K, V, O, DO = (t.to(dtype).transpose(1, 2) for t in (q, k, v, o, dout))
    s = Q.shape[-1] ** -0.5 if scale is None else float(scale)
    L = lse.to(dtype)[..., None]
    delta = (DO * O).sum(-1, keepdim=True)
    dQ, dK, dV = torch.zeros_like(Q), torch.zeros_like(K), torch.zeros_like(V)
    for j in range(0, K.shape[2], block):
        Kj, Vj = K[:, :, j:j + block], V[:, :, j:j + block]
        for i in range(0, Q.shape[2], block):
            Qi, DOi = Q[:, :, i:i + block], DO[:, :, i:i + block]
            P = torch.exp(s * (Qi @ Kj.transpose(-1, -2)) - L[:, :, i:i + block])
            dS = P * (DOi @ Vj.transpose(-1, -2) - delta[:, :, i:i + block])
            dV[:, :, j:j + block] += P.transpose(-1, -2) @ DOi
            dK[:, :, j:j + block] += s * (dS.transpose(-1, -2) @ Qi)
            dQ[:, :, i:i + block] += s * (dS @ Kj)
    return dQ.transpose(1, 2), dK.transpose(1, 2), dV.transpose(1, 2)


# --------------------------------------------------------------------------
# Caller-side pieces
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, gain: torch.Tensor | None = None, eps: float = 1e-6) -> torch.Tensor:
    """Per-head RMS normalisation over the last dim, models/layers.py:39-42:
    x * rsqrt(mean_fp32(x^2) + eps).to(x.dtype) * gain.to(x.dtype)."""
    n = torch.rsqrt(x.pow(2).mean(-1, keepdim=True, dtype=torch.float32) + eps)
    y = x * n.to(x.dtype)
    return y if gain is None else y * gain.to(x.dtype)


def split_head_dim(head_dim: int):
    """(main, tail) tile widths the reference uses for a head dim,
    models/triton_utils.py:22-47 (72 -> (64, 16), 96 -> (64, 32), 128 -> (128, 0))."""
    main = min(1 << (head_dim.bit_length() - 1), 64)
    rem = head_dim - main
    if rem <= 0:
        return main, 0
    if rem <= 16:
        return main, 16
    if rem <= 32:
        return main, 32
    return 128, 0


# --------------------------------------------------------------------------
# Seeded synthetic inputs and the error metric
# --------------------------------------------------------------------------
def make_inputs(B, L, H, D, seed, std=1.0, n=7, Lkv=None):
    """Draw q,k,v,dq,dk,dv,dout (in that order) as fp32 (B, L, H, D) on the CPU
    from ``torch.Generator().manual_seed(seed)``; std 1.0 for the benchmark
    configurations, 0.5 for the reference self-test family
    (models/flash_attention_2_jvp.py:348-353)."""
    g = torch.Generator().manual_seed(seed)
    Lkv = L if Lkv is None else Lkv
    lens = [L, Lkv, Lkv, L, Lkv, Lkv, L]
    return [torch.randn(B, lens[i], H, D, generator=g, dtype=torch.float32) * std for i in range(n)]


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    """||a - b||_2 / ||b||_2 over all elements, in fp64."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))
