"""DMFT harness model: the caller context of the attention operator.

Host-side mirror of the reference's Decoupled MeanFlow Transformer
(models/dmft.py:27-175): patch embedding + fixed sin-cos positions, ``dmf_depth``
encoder blocks conditioned on (t, y), the remaining decoder blocks and the final
layer conditioned on (r, y), optional log-variance head.  It exists so that the
attention kernels can be exercised and timed exactly as the MeanFlow loss calls
them (``torch.func.jvp`` through the whole model); ``attn_func`` selects the
operator, ``"hip"`` being this package's kernels, and ``block_ops="hip"`` swaps
the norm / modulate / gate / GELU glue of every block for the fused kernels of
``dmf_amd.block_ops``.
"""
from __future__ import annotations

from functools import partial

import torch
import torch.nn as nn
from torch import Tensor

from . import block_ops as block_ops_mod
from .layers import (DiTBlock, FinalLayer, LabelEmbedder, TimestepEmbedder, _check_block_ops, get_2d_sincos_pos_embed,
                     timestep_embedding)


class PatchEmbed(nn.Module):
    """Image -> patch tokens with a strided convolution; same parameters and
    output as the ``timm`` layer the reference uses (models/dmft.py:15,54-56):
    ``proj = Conv2d(C_in, C, kernel=stride=patch)``, tokens in row-major order."""

    def __init__(self, img_size: int, patch_size: int, in_chans: int, embed_dim: int, bias: bool = True,
                 block_ops: str = "torch"):
        super().__init__()
        self.patch_size = patch_size
        self.num_patches = (img_size // patch_size) ** 2
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=patch_size, stride=patch_size, bias=bias)
        self.fused = _check_block_ops(block_ops)

    def forward(self, x: Tensor) -> Tensor:
        if not self.fused:
            return self.proj(x).flatten(2).transpose(1, 2)
        # kernel == stride, so the convolution is a Linear over flattened (C_in, p, p) patches: one small GEMM
        # (and GEMM gradients) instead of the generic convolution path
        B, C, H, W = x.shape
        p = self.patch_size
        patches = x.reshape(B, C, H // p, p, W // p, p).permute(0, 2, 4, 1, 3, 5).reshape(B, (H // p) * (W // p), C * p * p)
        return block_ops_mod.dual_linear(patches, self.proj.weight.reshape(self.proj.out_channels, -1), self.proj.bias)


def chained_blocks(blocks, conds, final_layer, c_final, x, tap=None):
    """A stack of DiT blocks and the final layer in fused mode: same values as the
    plain loop ``for blk, c in zip(blocks, conds): x = blk(x, c)`` followed by
    ``final_layer(x, c_final)`` (before unpatchify), but every gated residual is
    computed by the kernel that also normalises and modulates the result for its
    consumer (the block's own MLP branch, the next block's attention branch, or the
    final layer), so the residual stream is read and written once per half block.
    ``tap(i, x)`` is called with the residual stream after block ``i``."""
    mods = [blk.adaLN_modulation(c).chunk(6, dim=-1) for blk, c in zip(blocks, conds)]
    f_shift, f_scale = final_layer.adaLN_modulation(c_final).chunk(2, dim=-1)
    z = block_ops_mod.ln_modulate(x, mods[0][0], mods[0][1], blocks[0].norm1.eps)
    for i, blk in enumerate(blocks):
        if i + 1 < len(blocks):
            nxt = (mods[i + 1][0], mods[i + 1][1], blocks[i + 1].norm1.eps)
        else:
            nxt = (f_shift, f_scale, final_layer.norm_final.eps)
        x, z = blk.forward_chained(x, z, mods[i], *nxt)
        if tap is not None:
            tap(i, x)
    return final_layer.linear(z)


def unpatchify(x: Tensor, channels: int, patch: int) -> Tensor:
    """(B, L, p*p*C) tokens -> (B, C, H, W) image (reference models/dmft.py:116-124, models/sit.py:122-129)."""
    h = w = int(x.shape[1] ** 0.5)
    assert h * w == x.shape[1]
    x = x.reshape(x.shape[0], h, w, patch, patch, channels)
    x = torch.einsum("nhwpqc->nchpwq", x)
    return x.reshape(x.shape[0], channels, h * patch, w * patch)


def reference_init_(model: nn.Module) -> nn.Module:
    """The reference's initialisation of a DMFT or SiT (models/dmft.py:79-121, models/sit.py:84-120): Xavier-uniform
    linears with zero biases (the patch projection counted as one), sin-cos positions, N(0, 0.02) label table and
    timestep MLP, and zeros for every adaLN modulation, the output layer and the log-variance head -- which makes
    every block an identity and the model output zero at step 0."""
    for m in model.modules():
        if isinstance(m, nn.Linear):
            nn.init.xavier_uniform_(m.weight)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
    grid = int(model.num_patches ** 0.5)
    model.pos_embed.data.copy_(torch.from_numpy(get_2d_sincos_pos_embed(model.pos_embed.shape[-1], grid)).float().unsqueeze(0))
    proj = model.x_embedder.proj
    nn.init.xavier_uniform_(proj.weight.data.view(proj.weight.shape[0], -1))
    nn.init.zeros_(proj.bias)
    for table in (model.y_embedder.embedding_table.weight, model.t_embedder.mlp[0].weight, model.t_embedder.mlp[2].weight):
        nn.init.normal_(table, std=0.02)
    zeroed = [blk.adaLN_modulation[-1] for blk in model.blocks] + [model.final_layer.adaLN_modulation[-1], model.final_layer.linear]
    if getattr(model, "use_logvar", False):
        zeroed.append(model.logvar_linear)
    for layer in zeroed:
        nn.init.zeros_(layer.weight)
        nn.init.zeros_(layer.bias)
    return model


def trunc_normal_init_(model: nn.Module, std: float = 0.02, seed: int = 0) -> nn.Module:
    """Benchmark initialisation: every weight matrix / embedding ~ truncated
    N(0, std) (cut at 2 std), biases zero.  With the reference's zero-gate
    initialisation attention contributes nothing to the output, so timing and
    parity runs use this instead.  Values are drawn on the device the parameters live
    on (a model built on the GPU is initialised there, in a fraction of the time), so
    the same seed gives different weights on different device types."""
    gens = {}
    for name, prm in model.named_parameters():
        if name == "pos_embed":
            continue
        if prm.dim() >= 2:
            g = gens.get(prm.device)
            if g is None:
                g = gens[prm.device] = torch.Generator(device=prm.device).manual_seed(seed)
            w = torch.empty(prm.shape, dtype=torch.float32, device=prm.device)
            nn.init.trunc_normal_(w, std=std, a=-2 * std, b=2 * std, generator=g)
            prm.data.copy_(w)
        elif name.endswith("bias"):
            prm.data.zero_()
    return model


class DMFT(nn.Module):
    """Reference models/dmft.py:27-151."""

    def __init__(self, input_size: int = 32, patch_size: int = 2, in_channels: int = 4, hidden_size: int = 1152,
                 depth: int = 28, num_heads: int = 16, mlp_ratio: float = 4.0, use_cfg_embedding: bool = True,
                 num_classes: int = 1000, dmf_depth: int = 8, use_logvar: bool = False, **block_kwargs):
        super().__init__()
        self.input_size, self.patch_size = input_size, patch_size
        self.in_channels = self.out_channels = in_channels
        self.num_heads, self.num_classes = num_heads, num_classes
        self.dmf_depth, self.use_logvar = dmf_depth, use_logvar
        self.fused = _check_block_ops(block_kwargs.get("block_ops", "torch"))

        self.x_embedder = PatchEmbed(input_size, patch_size, in_channels, hidden_size, bias=True,
                                     block_ops=block_kwargs.get("block_ops", "torch"))
        self.t_embedder = TimestepEmbedder(hidden_size)
        self.y_embedder = LabelEmbedder(num_classes, hidden_size, use_cfg_embedding)
        self.num_patches = self.x_embedder.num_patches
        self.pos_embed = nn.Parameter(torch.zeros(1, self.num_patches, hidden_size), requires_grad=False)
        self.blocks = nn.ModuleList(
            [DiTBlock(hidden_size, num_heads, mlp_ratio=mlp_ratio, **block_kwargs) for _ in range(depth)])
        self.final_layer = FinalLayer(hidden_size, patch_size, self.out_channels,
                                      block_ops=block_kwargs.get("block_ops", "torch"))
        if use_logvar:
            self.logvar_t_embedder = partial(timestep_embedding, dim=128)
            self.logvar_linear = nn.Linear(256, 1)
        self.initialize_weights()

    def initialize_weights(self) -> None:
        reference_init_(self)

    def init_trunc_normal_(self, std: float = 0.02, seed: int = 0) -> "DMFT":
        return trunc_normal_init_(self, std, seed)

    def unpatchify(self, x: Tensor) -> Tensor:
        return unpatchify(x, self.out_channels, self.patch_size)

    def _forward_chained(self, x, c_t, c_r):
        conds = [c_t] * self.dmf_depth + [c_r] * (len(self.blocks) - self.dmf_depth)
        return chained_blocks(self.blocks, conds, self.final_layer, c_r, x)

    def forward(self, x, t, r, y, return_logvar: bool = False):
        t, r = t.reshape(-1), r.reshape(-1)
        x = self.x_embedder(x) + self.pos_embed
        B, L, D = x.shape
        t_embed = self.t_embedder(t).reshape(B, -1, D)
        y_embed = self.y_embedder(y).reshape(B, -1, D)
        c_t = t_embed + y_embed
        if self.fused:
            x = self.unpatchify(self._forward_chained(x, c_t, self.t_embedder(r).reshape(B, -1, D) + y_embed))
        else:
            for block in self.blocks[:self.dmf_depth]:      # encoder: conditioned on t
                x = block(x, c_t)
            c_r = self.t_embedder(r).reshape(B, -1, D) + y_embed
            for block in self.blocks[self.dmf_depth:]:      # decoder: conditioned on r
                x = block(x, c_r)
            x = self.unpatchify(self.final_layer(x, c_r))
        if return_logvar:
            logvar = self.logvar_linear(torch.cat([self.logvar_t_embedder(t), self.logvar_t_embedder(r)], dim=1))
            return x, logvar.view(-1, *[1] * (x.ndim - 1))
        return x


# size registry (reference models/dmft.py:154-175)
_SIZES = {"XL": (28, 1152, 16), "L": (24, 1024, 16), "M": (16, 1024, 16), "B": (12, 768, 12), "S": (12, 384, 6)}
DMFT_models = {
    f"DMFT-{s}/{p}": partial(DMFT, depth=d, hidden_size=h, patch_size=p, num_heads=nh)
    for s, (d, h, nh) in _SIZES.items() for p in (2, 4, 8)
}
