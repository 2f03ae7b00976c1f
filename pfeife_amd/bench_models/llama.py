"""Llama-style decoder (RMSNorm, rotary embeddings, SwiGLU, untied lm_head,
next-token cross entropy inside the model), the family of
bench_models/models/train_llama.py:486-520 (HF LlamaConfig, eager attention).
The loss is part of the compiled graph, as in the reference's script where the
HF model returns `outputs.loss` (train_llama.py:782-786)."""
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F


@dataclass
class LlamaConfig:
    vocab: int = 32000
    dim: int = 2048
    layers: int = 16
    heads: int = 32
    ffn: int = 5632
    max_seq: int = 2048
    rope_theta: float = 10000.0
    eps: float = 1e-5


LLAMA_1B = LlamaConfig()


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary(x, cos, sin):
    # x: [B, H, T, D]; cos/sin: [T, D] (both halves equal)
    return x * cos + rotate_half(x) * sin


class DecoderLayer(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        d = cfg.dim
        self.heads = cfg.heads
        self.input_norm = nn.RMSNorm(d, eps=cfg.eps)
        self.q_proj = nn.Linear(d, d, bias=False)
        self.k_proj = nn.Linear(d, d, bias=False)
        self.v_proj = nn.Linear(d, d, bias=False)
        self.o_proj = nn.Linear(d, d, bias=False)
        self.post_norm = nn.RMSNorm(d, eps=cfg.eps)
        self.gate_proj = nn.Linear(d, cfg.ffn, bias=False)
        self.up_proj = nn.Linear(d, cfg.ffn, bias=False)
        self.down_proj = nn.Linear(cfg.ffn, d, bias=False)

    def forward(self, x, cos, sin):
        B, T, C = x.shape
        hd = C // self.heads
        h = self.input_norm(x)
        q = self.q_proj(h).view(B, T, self.heads, hd).transpose(1, 2)
        k = self.k_proj(h).view(B, T, self.heads, hd).transpose(1, 2)
        v = self.v_proj(h).view(B, T, self.heads, hd).transpose(1, 2)
        q, k = apply_rotary(q, cos, sin), apply_rotary(k, cos, sin)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.o_proj(a.transpose(1, 2).reshape(B, T, C))
        h = self.post_norm(x)
        x = x + self.down_proj(F.silu(self.gate_proj(h)) * self.up_proj(h))
        return x


class LlamaForCausalLM(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.dim)
        self.layers = nn.ModuleList([DecoderLayer(cfg) for _ in range(cfg.layers)])
        self.norm = nn.RMSNorm(cfg.dim, eps=cfg.eps)
        self.lm_head = nn.Linear(cfg.dim, cfg.vocab, bias=False)
        hd = cfg.dim // cfg.heads
        inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2).float() / hd))
        ang = torch.arange(cfg.max_seq).float()[:, None] * inv_freq[None, :]
        emb = torch.cat((ang, ang), dim=-1)
        self.register_buffer("rope_cos", emb.cos(), persistent=False)
        self.register_buffer("rope_sin", emb.sin(), persistent=False)

    def forward(self, input_ids, labels):
        T = input_ids.shape[1]
        x = self.embed(input_ids)
        cos, sin = self.rope_cos[:T], self.rope_sin[:T]
        for layer in self.layers:
            x = layer(x, cos, sin)
        logits = self.lm_head(self.norm(x))
        shift_logits = logits[:, :-1, :].reshape(-1, logits.shape[-1])
        shift_labels = labels[:, 1:].reshape(-1)
        return F.cross_entropy(shift_logits.float(), shift_labels)


class _LlamaStage(nn.Module):
    """Layers [lo, hi) of `model` (+ embedding first, + norm/lm_head/loss last)."""

    def __init__(self, model, lo, hi, first, last):
        super().__init__()
        self.m, self.lo, self.hi, self.first, self.last = model, lo, hi, first, last

    def forward(self, x, labels=None, input_len=None):
        m = self.m
        if self.first:
            x = m.embed(x)
        T = x.shape[1]
        cos, sin = m.rope_cos[:T], m.rope_sin[:T]
        for layer in m.layers[self.lo:self.hi]:
            x = layer(x, cos, sin)
        if not self.last:
            return x
        logits = m.lm_head(m.norm(x))
        return logits


def split_stages(model: LlamaForCausalLM, bounds):
    """Stage modules for layer boundaries `bounds` (e.g. [4, 8, 12] -> 4 stages).
    The last stage returns logits; the caller applies the shifted cross entropy."""
    edges = [0] + list(bounds) + [model.cfg.layers]
    n = len(edges) - 1
    return [_LlamaStage(model, edges[i], edges[i + 1], i == 0, i == n - 1) for i in range(n)]
