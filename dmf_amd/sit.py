"""SiT harness model: the single-time caller of the same DiT blocks.

Host-side mirror of the reference's SiT (models/sit.py:27-175): patch embedding +
fixed sin-cos positions, ``depth`` blocks all conditioned on (t, y), the final
layer, and -- with ``repa_depth > 0`` -- projector MLPs on the residual stream
after block ``repa_depth`` (``return_feat=True``).  It is what ``train_fm.py``
trains (plain forward + backward, no JVP) and what ``train_dmf.py:176-188`` loads
as the frozen teacher of the ``"distill"`` guidance (loss.py:74-84: a no-grad call
on a 2B batch).  ``attn_func`` / ``block_ops`` select the operator and the block
glue exactly as for ``DMFT``.
"""
from __future__ import annotations

from functools import partial

import torch
import torch.nn as nn

from .dmft import PatchEmbed, chained_blocks, reference_init_, trunc_normal_init_, unpatchify
from .layers import DiTBlock, FinalLayer, LabelEmbedder, Linear, SiLU, TimestepEmbedder, _check_block_ops


def build_mlp(hidden_size: int, projector_dim: int, z_dim: int, block_ops: str = "torch") -> nn.Sequential:
    """Projector head (reference models/sit.py:27-34): Linear-SiLU-Linear-SiLU-Linear."""
    return nn.Sequential(
        Linear(hidden_size, projector_dim, block_ops=block_ops), SiLU(block_ops),
        Linear(projector_dim, projector_dim, block_ops=block_ops), SiLU(block_ops),
        Linear(projector_dim, z_dim, block_ops=block_ops))


class SiT(nn.Module):
    """Reference models/sit.py:38-146."""

    def __init__(self, input_size: int = 32, patch_size: int = 2, in_channels: int = 4, hidden_size: int = 1152,
                 depth: int = 28, num_heads: int = 16, mlp_ratio: float = 4.0, use_cfg_embedding: bool = True,
                 num_classes: int = 1000, repa_depth: int = 0, z_dims=(768,), projector_dim: int = 2048, **block_kwargs):
        super().__init__()
        block_ops = block_kwargs.get("block_ops", "torch")
        self.input_size, self.patch_size = input_size, patch_size
        self.in_channels = self.out_channels = in_channels
        self.num_heads, self.num_classes, self.repa_depth = num_heads, num_classes, repa_depth
        self.fused = _check_block_ops(block_ops)
        self.x_embedder = PatchEmbed(input_size, patch_size, in_channels, hidden_size, bias=True, block_ops=block_ops)
        self.num_patches = self.x_embedder.num_patches
        self.t_embedder = TimestepEmbedder(hidden_size)
        self.y_embedder = LabelEmbedder(num_classes, hidden_size, use_cfg_embedding)
        if repa_depth > 0:
            self.projectors = nn.ModuleList([build_mlp(hidden_size, projector_dim, z, block_ops) for z in z_dims])
        self.pos_embed = nn.Parameter(torch.zeros(1, self.num_patches, hidden_size), requires_grad=False)
        self.blocks = nn.ModuleList(
            [DiTBlock(hidden_size, num_heads, mlp_ratio=mlp_ratio, **block_kwargs) for _ in range(depth)])
        self.final_layer = FinalLayer(hidden_size, patch_size, self.out_channels, block_ops=block_ops)
        self.initialize_weights()

    def initialize_weights(self) -> None:
        reference_init_(self)

    def init_trunc_normal_(self, std: float = 0.02, seed: int = 0) -> "SiT":
        return trunc_normal_init_(self, std, seed)

    def unpatchify(self, x):
        return unpatchify(x, self.out_channels, self.patch_size)

    def forward(self, x, t, y, return_feat: bool = False):
        t = t.reshape(-1)
        x = self.x_embedder(x) + self.pos_embed
        B, L, D = x.shape
        c = self.t_embedder(t).reshape(B, -1, D) + self.y_embedder(y).reshape(B, -1, D)
        feats = []

        def project(i, h):   # residual stream after block i -> projector heads (models/sit.py:141-142)
            if self.repa_depth > 0 and i + 1 == self.repa_depth:
                feats.extend(p(h.reshape(-1, D)).reshape(B, L, -1) for p in self.projectors)

        if self.fused:
            x = chained_blocks(self.blocks, [c] * len(self.blocks), self.final_layer, c, x, tap=project)
        else:
            for i, block in enumerate(self.blocks):
                x = block(x, c)
                project(i, x)
            x = self.final_layer(x, c)
        x = self.unpatchify(x)
        if self.repa_depth > 0 and return_feat:
            return x, feats
        return x


# size registry (reference models/sit.py:149-175)
_SIZES = {"XL": (28, 1152, 16), "L": (24, 1024, 16), "M": (16, 1024, 16), "B": (12, 768, 12), "S": (12, 384, 6)}
SiT_models = {
    f"SiT-{s}/{p}": partial(SiT, depth=d, hidden_size=h, patch_size=p, num_heads=nh)
    for s, (d, h, nh) in _SIZES.items() for p in (2, 4, 8)
}
