"""Vision Transformer (timm / HF ViT layout: pre-norm blocks, cls token, learned
positions, linear head), the model family of
bench_models/models/train_vit.py:150-169 and of the torchbench
`timm_vision_transformer[_large]` entries the reference's README benchmarks."""
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F


@dataclass
class ViTConfig:
    image_size: int = 224
    patch_size: int = 16
    channels: int = 3
    dim: int = 384
    depth: int = 12
    heads: int = 6
    mlp_dim: int = 1536
    num_classes: int = 1000
    eps: float = 1e-6

    @property
    def tokens(self):
        return (self.image_size // self.patch_size) ** 2 + 1


VIT_S16 = ViTConfig(dim=384, depth=12, heads=6, mlp_dim=1536)
VIT_L16 = ViTConfig(dim=1024, depth=24, heads=16, mlp_dim=4096)
VIT_G14_SHARE = ViTConfig(image_size=224, patch_size=14, dim=1408, depth=10, heads=16, mlp_dim=6144)


class Block(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        d = cfg.dim
        self.heads = cfg.heads
        self.norm1 = nn.LayerNorm(d, eps=cfg.eps)
        self.qkv = nn.Linear(d, 3 * d)
        self.proj = nn.Linear(d, d)
        self.norm2 = nn.LayerNorm(d, eps=cfg.eps)
        self.fc1 = nn.Linear(d, cfg.mlp_dim)
        self.fc2 = nn.Linear(cfg.mlp_dim, d)

    def forward(self, x):
        B, T, C = x.shape
        qkv = self.qkv(self.norm1(x)).reshape(B, T, 3, self.heads, C // self.heads).permute(2, 0, 3, 1, 4)
        q, k, v = qkv.unbind(0)
        a = F.scaled_dot_product_attention(q, k, v)
        x = x + self.proj(a.transpose(1, 2).reshape(B, T, C))
        x = x + self.fc2(F.gelu(self.fc1(self.norm2(x))))
        return x


class VisionTransformer(nn.Module):
    def __init__(self, cfg: ViTConfig):
        super().__init__()
        self.cfg = cfg
        self.patch_embed = nn.Conv2d(cfg.channels, cfg.dim, cfg.patch_size, cfg.patch_size)
        self.cls_token = nn.Parameter(torch.zeros(1, 1, cfg.dim))
        self.pos_embed = nn.Parameter(torch.randn(1, cfg.tokens, cfg.dim) * 0.02)
        self.blocks = nn.ModuleList([Block(cfg) for _ in range(cfg.depth)])
        self.norm = nn.LayerNorm(cfg.dim, eps=cfg.eps)
        self.head = nn.Linear(cfg.dim, cfg.num_classes)
        nn.init.normal_(self.cls_token, std=1e-6)

    def forward(self, pixel_values):
        x = self.patch_embed(pixel_values).flatten(2).transpose(1, 2)
        x = torch.cat([self.cls_token.expand(x.shape[0], -1, -1), x], dim=1) + self.pos_embed
        for blk in self.blocks:
            x = blk(x)
        x = self.norm(x)
        return self.head(x[:, 0])


class BlockStack(nn.Module):
    """A run of transformer blocks fed with activations: one GPU's share of a
    larger ViT (e.g. 10 of the 40 blocks of ViT-g/14)."""

    def __init__(self, cfg: ViTConfig):
        super().__init__()
        self.cfg = cfg
        self.blocks = nn.ModuleList([Block(cfg) for _ in range(cfg.depth)])

    def forward(self, x):
        for blk in self.blocks:
            x = blk(x)
        return x


class _FirstStage(nn.Module):
    def __init__(self, model, k):
        super().__init__()
        self.m, self.k = model, k

    def forward(self, pixel_values):
        m = self.m
        x = m.patch_embed(pixel_values).flatten(2).transpose(1, 2)
        x = torch.cat([m.cls_token.expand(x.shape[0], -1, -1), x], dim=1) + m.pos_embed
        for blk in m.blocks[:self.k]:
            x = blk(x)
        return x


class _LastStage(nn.Module):
    def __init__(self, model, k):
        super().__init__()
        self.m, self.k = model, k

    def forward(self, x):
        m = self.m
        for blk in m.blocks[self.k:]:
            x = blk(x)
        return m.head(m.norm(x)[:, 0])


def split_stages(model: VisionTransformer, k: int):
    """The two stage modules of `model` cut before block k (they share model's parameters)."""
    return [_FirstStage(model, k), _LastStage(model, k)]
