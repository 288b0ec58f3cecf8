"""A plain-PyTorch ViT (patch embedding, pre-norm transformer blocks, class token, linear head)
used to measure and test the HOT layers inside a whole model: every nn.Linear / nn.Conv2d in it can
be swapped for HQ_Linear / HQ_Conv2d with ``hot_amd.utils.replace_layers``, as the reference does
with timm's ViT-B/16 (ViT_main.py:133-160).  Random initialisation only; not a model zoo.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class Attention(nn.Module):
    def __init__(self, dim: int, heads: int) -> None:
        super().__init__()
        self.heads = heads
        self.qkv = nn.Linear(dim, dim * 3)
        self.proj = nn.Linear(dim, dim)

    def forward(self, x):
        B, T, C = x.shape
        q, k, v = self.qkv(x).reshape(B, T, 3, self.heads, C // self.heads).permute(2, 0, 3, 1, 4).unbind(0)
        y = F.scaled_dot_product_attention(q, k, v)   # unbind: one gradient stack instead of three zero-filled ones
        return self.proj(y.transpose(1, 2).reshape(B, T, C))


class Block(nn.Module):
    def __init__(self, dim: int, heads: int, mlp: int) -> None:
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn = Attention(dim, heads)
        self.norm2 = nn.LayerNorm(dim)
        self.fc1 = nn.Linear(dim, mlp)
        self.fc2 = nn.Linear(mlp, dim)

    def forward(self, x):
        x = x + self.attn(self.norm1(x))
        return x + self.fc2(F.gelu(self.fc1(self.norm2(x))))


class ViT(nn.Module):
    """ViT-B/16 by default: 224 x 224 images, 16 x 16 patches, 12 blocks of width 768, 12 heads, MLP 3072."""

    def __init__(self, image=224, patch=16, dim=768, depth=12, heads=12, mlp=3072, classes=100, channels=3) -> None:
        super().__init__()
        self.patch_embed = nn.Conv2d(channels, dim, kernel_size=patch, stride=patch)
        tokens = (image // patch) ** 2
        self.cls = nn.Parameter(torch.zeros(1, 1, dim))
        self.pos = nn.Parameter(torch.randn(1, tokens + 1, dim) * 0.02)
        self.blocks = nn.ModuleList([Block(dim, heads, mlp) for _ in range(depth)])
        self.norm = nn.LayerNorm(dim)
        self.head = nn.Linear(dim, classes)

    def forward(self, img):
        x = self.patch_embed(img).flatten(2).transpose(1, 2)
        x = torch.cat([self.cls.expand(x.shape[0], -1, -1), x], dim=1) + self.pos
        for blk in self.blocks:
            x = blk(x)
        return self.head(self.norm(x)[:, 0])
