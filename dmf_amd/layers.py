"""Caller-side layers around the attention operator.

Host-side mirror of the parts of the reference's models/layers.py that sit on
the attention path: the ``attn_op`` switch (reference :86-115) extended with
``op="hip"``, ``RMSNorm`` (:33-42), ``Attention`` (:119-154) and the DiT block
pieces (:28-29, :59-82, :158-220) that the DMFT harness needs.
"""
from __future__ import annotations

import contextlib
import math
from functools import partial

import numpy as np
import torch
import torch.nn as nn
from torch import Tensor

from . import block_ops as fused
from ._lib import SUPPORTED_HEAD_DIMS
from .flash_attention_hip_jvp import flash_attn_func as hip_func
from .flash_attention_hip_jvp import flash_attn_qknorm_qkvpacked_func as hip_qknorm_qkvpacked_func
from .flash_attention_hip_jvp import flash_attn_qkvpacked_func as hip_qkvpacked_func

# values accepted by --attn-func; "hip" is the one this package adds
ATTN_FUNCS = ("base", "torch_sdpa", "hip")
# how the elementwise / normalisation glue of a block runs: "torch" = the reference's
# tensor expressions (one ATen kernel per primal and per tangent op), "hip" = the fused
# single-pass kernels of dmf_amd.block_ops
BLOCK_OPS = ("torch", "hip")


def _check_block_ops(block_ops: str) -> bool:
    if block_ops not in BLOCK_OPS:
        raise ValueError(f"unknown block_ops {block_ops!r}; expected one of {BLOCK_OPS}")
    return block_ops == "hip"


def attn_op(q: Tensor, k: Tensor, v: Tensor, op: str = "base") -> Tensor:
    """Attention on (B, L, H, D) tensors, returns (B, L, H, D).

    op: "hip"        -- fused gfx950 kernels with forward-mode (JVP) support,
        "base"       -- naive softmax(q k^T) v, the semantics of reference
                        models/layers.py:108-113 (JVP through ATen formulas),
        "torch_sdpa" -- torch SDPA (no JVP support), reference :103-107.
    Unlike the reference (which leaves the result unbound, :114) an unknown
    ``op`` raises ValueError.
    """
    if op == "hip":
        return hip_func(q, k, v)
    if op not in ("base", "torch_sdpa"):
        raise ValueError(f"unknown attention op {op!r}; expected one of {ATTN_FUNCS}")
    q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)  # (B, H, L, D)
    if op == "torch_sdpa":
        x = torch.nn.functional.scaled_dot_product_attention(q, k, v, dropout_p=0.0, is_causal=False)
    else:
        scale = q.shape[-1] ** -0.5
        attn = (q * scale) @ k.transpose(-2, -1)
        x = attn.softmax(dim=-1) @ v
    return x.transpose(1, 2)


class SiLU(nn.SiLU):
    """``nn.SiLU`` (no parameters); one fused primal + tangent kernel when ``block_ops="hip"``."""

    def __init__(self, block_ops: str = "torch"):
        super().__init__()
        self.fused = _check_block_ops(block_ops)

    def forward(self, x: Tensor) -> Tensor:
        return fused.silu(x) if self.fused else super().forward(x)


class Linear(nn.Linear):
    """``nn.Linear`` whose forward-mode pass costs one extra GEMM instead of two
    (``block_ops.dual_linear``) when ``block_ops="hip"``; parameters, state-dict
    keys and results are those of ``nn.Linear``.  ``lp_weight`` / ``lp_bias`` are
    set by ``frozen_low_precision_params`` while the parameters are known not to
    change."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, block_ops: str = "torch"):
        super().__init__(in_features, out_features, bias=bias)
        self.fused = _check_block_ops(block_ops)
        self.lp_weight = self.lp_bias = None

    def forward(self, x: Tensor) -> Tensor:
        if self.fused:
            return fused.dual_linear(x, self.weight, self.bias, self.lp_weight, self.lp_bias)
        return super().forward(x)


@contextlib.contextmanager
def frozen_low_precision_params(model: nn.Module, dtype: torch.dtype = torch.bfloat16):
    """While active, every fused ``Linear`` of ``model`` uses a copy of its parameters in
    ``dtype`` made once on entry, instead of the per-call casts of autocast -- for loops
    over frozen weights (sampling, evaluation, forward+JVP-only passes).  The caller must
    not modify the parameters inside the context; results are those of autocast.  Contexts
    nest: leaving an inner one puts back the copies of the outer one."""
    layers = [m for m in model.modules() if isinstance(m, Linear) and m.fused]
    saved = [(m.lp_weight, m.lp_bias) for m in layers]
    try:
        for m in layers:
            m.lp_weight = m.weight.detach().to(dtype)
            m.lp_bias = None if m.bias is None else m.bias.detach().to(dtype)
        yield model
    finally:
        for m, (w, b) in zip(layers, saved):
            m.lp_weight, m.lp_bias = w, b


def modulate(x: Tensor, shift: Tensor, scale: Tensor) -> Tensor:
    """adaLN modulation (reference models/layers.py:28-29)."""
    return x * (1 + scale) + shift


class RMSNorm(nn.Module):
    """Per-head RMS norm over the last dim (reference models/layers.py:33-42)."""

    def __init__(self, dim: int, eps: float = 1e-6, block_ops: str = "torch"):
        super().__init__()
        self.eps = eps
        self.scale = nn.Parameter(torch.ones(dim))
        self.fused = _check_block_ops(block_ops)

    def forward(self, x: Tensor) -> Tensor:
        if self.fused:
            return fused.rms_norm(x, self.scale, self.eps)
        norm_x = torch.rsqrt(x.pow(2).mean(-1, keepdim=True, dtype=torch.float32) + self.eps)
        return x * norm_x.to(dtype=x.dtype) * self.scale.to(dtype=x.dtype)


def timestep_embedding(t: Tensor, dim: int, max_period: int = 10000) -> Tensor:
    """Sinusoidal embedding (reference models/layers.py:46-55)."""
    half = dim // 2
    # built on t's device (the reference builds it on the host and copies, which a stream capture cannot record)
    freqs = torch.exp(-math.log(max_period) * torch.arange(0, half, dtype=torch.float32, device=t.device) / half)
    args = t[..., None].float() * freqs[None]
    emb = torch.cat([torch.cos(args), torch.sin(args)], dim=-1)
    if dim % 2:
        emb = torch.cat([emb, torch.zeros_like(emb[:, :1])], dim=-1)
    return emb


class TimestepEmbedder(nn.Module):
    """Reference models/layers.py:59-71."""

    def __init__(self, hidden_size: int, emb_size: int = 256):
        super().__init__()
        self.emb_size = emb_size
        self.mlp = nn.Sequential(nn.Linear(emb_size, hidden_size), nn.SiLU(), nn.Linear(hidden_size, hidden_size))

    def forward(self, t: Tensor) -> Tensor:
        return self.mlp(timestep_embedding(t, self.emb_size).to(t.dtype))


class LabelEmbedder(nn.Module):
    """Reference models/layers.py:75-82."""

    def __init__(self, num_classes: int = 1000, hidden_size: int = 768, use_cfg_embedding: bool = True):
        super().__init__()
        self.embedding_table = nn.Embedding(num_classes + use_cfg_embedding, hidden_size)

    def forward(self, labels: Tensor) -> Tensor:
        return self.embedding_table(labels)


class Attention(nn.Module):
    """qkv Linear -> (B, L, H, D) views -> optional per-head RMSNorm on q, k ->
    attention -> proj (reference models/layers.py:119-154).  q, k, v reach the
    operator as strided views into the packed qkv buffer; the "hip" op consumes
    them without a copy."""

    def __init__(self, dim: int, num_heads: int = 8, qkv_bias: bool = False, qk_norm: bool = False,
                 proj_bias: bool = True, attn_func: str = "torch_sdpa", block_ops: str = "torch") -> None:
        super().__init__()
        assert dim % num_heads == 0, "dim should be divisible by num_heads"
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.qkv = Linear(dim, dim * 3, bias=qkv_bias, block_ops=block_ops)
        self.q_norm = RMSNorm(self.head_dim, block_ops=block_ops) if qk_norm else nn.Identity()
        self.k_norm = RMSNorm(self.head_dim, block_ops=block_ops) if qk_norm else nn.Identity()
        self.proj = Linear(dim, dim, bias=proj_bias, block_ops=block_ops)
        self.attn = partial(attn_op, op=attn_func)
        # the 'hip' operator can take the projection output as it is (with or without qk-norm)
        # (head dims without a kernel of their own go through attn_op, which zero-pads them)
        self.packed = _check_block_ops(block_ops) and attn_func == "hip" and self.head_dim in SUPPORTED_HEAD_DIMS
        self.qk_norm = qk_norm

    def forward(self, x: Tensor) -> Tensor:
        B, L, C = x.shape
        if self.packed:
            qkv = self.qkv(x).reshape(B, L, 3, self.num_heads, self.head_dim)
            if self.qk_norm:
                x = hip_qknorm_qkvpacked_func(qkv, self.q_norm.scale, self.k_norm.scale, self.q_norm.eps)
            else:
                x = hip_qkvpacked_func(qkv)
            return self.proj(x.reshape(B, L, C))
        qkv = self.qkv(x).reshape(B, L, 3, self.num_heads, self.head_dim).permute(2, 0, 1, 3, 4)
        q, k, v = qkv.unbind(0)  # each (B, L, H, D), strides (3LHD, 3HD, D, 1)
        q, k = self.q_norm(q), self.k_norm(k)
        x = self.attn(q, k, v)
        return self.proj(x.reshape(B, L, C))


class Mlp(nn.Module):
    """Reference models/layers.py:158-166."""

    def __init__(self, in_features: int, hidden_features: int, block_ops: str = "torch"):
        super().__init__()
        self.fc1 = Linear(in_features, hidden_features, block_ops=block_ops)
        self.act = fused.gelu_tanh if _check_block_ops(block_ops) else nn.GELU(approximate="tanh")
        self.fc2 = Linear(hidden_features, in_features, block_ops=block_ops)

    def forward(self, x: Tensor) -> Tensor:
        if self.fc1.fused:
            return self.fc2(fused.linear_gelu_tanh(x, self.fc1.weight, self.fc1.bias, self.fc1.lp_weight, self.fc1.lp_bias))
        return self.fc2(self.act(self.fc1(x)))


class DiTBlock(nn.Module):
    """adaLN-Zero transformer block (reference models/layers.py:170-201)."""

    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float = 4.0, **block_kwargs):
        super().__init__()
        block_ops = block_kwargs.get("block_ops", "torch")
        self.fused = _check_block_ops(block_ops)
        self.norm1 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.attn = Attention(hidden_size, num_heads=num_heads, qkv_bias=True,
                              qk_norm=block_kwargs.get("qk_norm", False),
                              attn_func=block_kwargs.get("attn_func", "base"), block_ops=block_ops)
        self.norm2 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.mlp = Mlp(hidden_size, int(hidden_size * mlp_ratio), block_ops=block_ops)
        self.adaLN_modulation = nn.Sequential(SiLU(block_ops), Linear(hidden_size, 6 * hidden_size, block_ops=block_ops))

    def forward(self, x: Tensor, c: Tensor) -> Tensor:
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.adaLN_modulation(c).chunk(6, dim=-1)
        if self.fused:   # same expressions; the first residual is fused with the norm+modulate that follows it
            x, z = fused.residual_ln_modulate(x, gate_msa, self.attn(fused.ln_modulate(x, shift_msa, scale_msa, self.norm1.eps)),
                                              shift_mlp, scale_mlp, self.norm2.eps)
            return fused.gate_residual(x, gate_mlp, self.mlp(z))
        x = x + gate_msa * self.attn(modulate(self.norm1(x), shift_msa, scale_msa))
        x = x + gate_mlp * self.mlp(modulate(self.norm2(x), shift_mlp, scale_mlp))
        return x

    def forward_chained(self, x: Tensor, z: Tensor, mods, next_shift: Tensor, next_scale: Tensor, next_eps: float):
        """Fused-mode variant for a stack of blocks.  ``z`` is this block's already
        normalised and modulated input (``modulate(norm1(x), shift_msa, scale_msa)``,
        produced by the previous block's last kernel), ``mods`` the six chunks of
        ``self.adaLN_modulation(c)``; the block's second residual is fused with the
        *next* consumer's norm + modulate (``next_shift`` / ``next_scale``: the next
        block's msa pair, or the final layer's).  Returns ``(x_out, z_next)``; same
        values as ``forward``."""
        _, _, gate_msa, shift_mlp, scale_mlp, gate_mlp = mods
        x, z = fused.residual_ln_modulate(x, gate_msa, self.attn(z), shift_mlp, scale_mlp, self.norm2.eps)
        return fused.residual_ln_modulate(x, gate_mlp, self.mlp(z), next_shift, next_scale, next_eps)


class FinalLayer(nn.Module):
    """Reference models/layers.py:205-220."""

    def __init__(self, hidden_size: int, patch_size: int, out_channels: int, block_ops: str = "torch"):
        super().__init__()
        self.fused = _check_block_ops(block_ops)
        self.norm_final = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.linear = Linear(hidden_size, patch_size * patch_size * out_channels, block_ops=block_ops)
        self.adaLN_modulation = nn.Sequential(SiLU(block_ops), Linear(hidden_size, 2 * hidden_size, block_ops=block_ops))

    def forward(self, x: Tensor, c: Tensor) -> Tensor:
        shift, scale = self.adaLN_modulation(c).chunk(2, dim=-1)
        if self.fused:
            return self.linear(fused.ln_modulate(x, shift, scale, self.norm_final.eps))
        return self.linear(modulate(self.norm_final(x), shift, scale))


def get_2d_sincos_pos_embed(embed_dim: int, grid_size: int) -> np.ndarray:
    """Fixed 2-D sin-cos position table of shape (grid_size**2, embed_dim): half
    of the channels encode the column index, half the row index, each as
    [sin | cos] over frequencies 10000**(-i / (embed_dim/4))
    (reference models/layers.py:224-271)."""
    assert embed_dim % 4 == 0
    omega = 1.0 / 10000 ** (np.arange(embed_dim // 4, dtype=np.float64) / (embed_dim / 4.0))
    rows, cols = np.meshgrid(np.arange(grid_size, dtype=np.float64), np.arange(grid_size, dtype=np.float64), indexing="ij")

    def enc(pos):
        out = pos.reshape(-1)[:, None] * omega[None]
        return np.concatenate([np.sin(out), np.cos(out)], axis=1)

    return np.concatenate([enc(cols), enc(rows)], axis=1)
