"""One pipeline stage of an SDXL-style UNet: `down_blocks[2]` (two ResNet blocks
640 -> 1280 -> 1280, each followed by a 10-layer spatial transformer, no
down-sampling) + `mid_block` (ResNet, 10-layer transformer, ResNet), written
in the structure of diffusers' ResnetBlock2D / Transformer2DModel /
BasicTransformerBlock, the model family of
bench_models/models/train_sdxl.py:805 (UNet2DConditionModel).

forward(hidden [B, C_in, H, W], temb [B, T_emb], context [B, 77, ctx_dim]) -> [B, C, H, W]
"""
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F


@dataclass
class UNetStageConfig:
    in_channels: int = 640
    channels: int = 1280
    temb_dim: int = 1280
    context_dim: int = 2048
    heads: int = 20
    layers: int = 10            # transformer blocks per spatial transformer
    groups: int = 32
    ff_mult: int = 4


SDXL_STAGE = UNetStageConfig()


class ResnetBlock(nn.Module):
    def __init__(self, cin, cout, temb_dim, groups):
        super().__init__()
        self.groups = groups
        self.norm1 = nn.GroupNorm(groups, cin, eps=1e-5)
        self.conv1 = nn.Conv2d(cin, cout, 3, padding=1)
        self.time_emb_proj = nn.Linear(temb_dim, cout)
        self.norm2 = nn.GroupNorm(groups, cout, eps=1e-5)
        self.conv2 = nn.Conv2d(cout, cout, 3, padding=1)
        self.shortcut = nn.Conv2d(cin, cout, 1) if cin != cout else None

    def forward(self, x, temb):
        h = self.conv1(F.silu(self.norm1(x)))
        h = h + self.time_emb_proj(F.silu(temb))[:, :, None, None]
        h = self.conv2(F.silu(self.norm2(h)))
        if self.shortcut is not None:
            x = self.shortcut(x)
        return x + h


class Attention(nn.Module):
    def __init__(self, dim, heads, kv_dim=None):
        super().__init__()
        self.heads = heads
        self.to_q = nn.Linear(dim, dim, bias=False)
        self.to_k = nn.Linear(kv_dim or dim, dim, bias=False)
        self.to_v = nn.Linear(kv_dim or dim, dim, bias=False)
        self.to_out = nn.Linear(dim, dim)

    def forward(self, x, context=None):
        B, T, C = x.shape
        ctx = x if context is None else context
        S = ctx.shape[1]
        hd = C // self.heads
        q = self.to_q(x).view(B, T, self.heads, hd).transpose(1, 2)
        k = self.to_k(ctx).view(B, S, self.heads, hd).transpose(1, 2)
        v = self.to_v(ctx).view(B, S, self.heads, hd).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v)
        return self.to_out(a.transpose(1, 2).reshape(B, T, C))


class GEGLUFeedForward(nn.Module):
    def __init__(self, dim, mult):
        super().__init__()
        self.proj = nn.Linear(dim, dim * mult * 2)
        self.out = nn.Linear(dim * mult, dim)

    def forward(self, x):
        hidden, gate = self.proj(x).chunk(2, dim=-1)
        return self.out(hidden * F.gelu(gate))


class BasicTransformerBlock(nn.Module):
    def __init__(self, dim, heads, context_dim, ff_mult):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn1 = Attention(dim, heads)
        self.norm2 = nn.LayerNorm(dim)
        self.attn2 = Attention(dim, heads, context_dim)
        self.norm3 = nn.LayerNorm(dim)
        self.ff = GEGLUFeedForward(dim, ff_mult)

    def forward(self, x, context):
        x = x + self.attn1(self.norm1(x))
        x = x + self.attn2(self.norm2(x), context)
        x = x + self.ff(self.norm3(x))
        return x


class SpatialTransformer(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        c = cfg.channels
        self.norm = nn.GroupNorm(cfg.groups, c, eps=1e-6)
        self.proj_in = nn.Linear(c, c)
        self.blocks = nn.ModuleList(
            [BasicTransformerBlock(c, cfg.heads, cfg.context_dim, cfg.ff_mult) for _ in range(cfg.layers)])
        self.proj_out = nn.Linear(c, c)

    def forward(self, x, context):
        B, C, H, W = x.shape
        h = self.norm(x).permute(0, 2, 3, 1).reshape(B, H * W, C)
        h = self.proj_in(h)
        for blk in self.blocks:
            h = blk(h, context)
        h = self.proj_out(h).reshape(B, H, W, C).permute(0, 3, 1, 2)
        return h + x


class UNetStage(nn.Module):
    def __init__(self, cfg: UNetStageConfig):
        super().__init__()
        self.cfg = cfg
        c = cfg.channels
        self.down_res = nn.ModuleList([ResnetBlock(cfg.in_channels, c, cfg.temb_dim, cfg.groups),
                                       ResnetBlock(c, c, cfg.temb_dim, cfg.groups)])
        self.down_attn = nn.ModuleList([SpatialTransformer(cfg), SpatialTransformer(cfg)])
        self.mid_res1 = ResnetBlock(c, c, cfg.temb_dim, cfg.groups)
        self.mid_attn = SpatialTransformer(cfg)
        self.mid_res2 = ResnetBlock(c, c, cfg.temb_dim, cfg.groups)

    def forward(self, hidden, temb, context):
        for res, attn in zip(self.down_res, self.down_attn):
            hidden = attn(res(hidden, temb), context)
        hidden = self.mid_res1(hidden, temb)
        hidden = self.mid_attn(hidden, context)
        return self.mid_res2(hidden, temb)
