"""InternViT-shaped vision tower for the prefill side of the path: the module behind
`extract_feature`, which the reference's `custom_generate` calls in chunks of ten tiles
(patch_internvl.py:53-65) on the 448 x 448 tiles of infer.py:87-144.

The upstream model code (InternViT-300M / InternViT-6B and the InternVL chat wrapper) is
remote code that is not available offline, so this is an architecture-shaped, randomly
initialised re-statement from the published model configuration: its outputs are not pinned
against upstream weights (parity unpinned); what it gives the path is the real shape and
cost of the prefill - 1 025 tokens per tile through the encoder, 256 tokens of the language
model's width per tile out.

  tile (3, 448, 448) --patch 14--> 32 x 32 patches + class token, learned positions
  --> N pre-norm transformer layers (fused qkv with bias, layer scale on both branches)
  --> drop the class token --> pixel shuffle by 1/2 (32 x 32 x C -> 16 x 16 x 4C)
  --> LayerNorm(4C) -> Linear(4C, H) -> GELU -> Linear(H, H)  =  (256, H) per tile
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn


@dataclass
class InternViTConfig:
    hidden_size: int = 1024
    num_hidden_layers: int = 24
    num_attention_heads: int = 16
    intermediate_size: int = 4096
    image_size: int = 448
    patch_size: int = 14
    qkv_bias: bool = True
    rms_norm: bool = False            # InternViT-6B normalises with RMSNorm, the 300M model with LayerNorm
    qk_normalization: bool = False    # ... and normalises q and k across the heads
    layer_norm_eps: float = 1e-6
    layer_scale_init: float = 0.1
    downsample_ratio: float = 0.5

    @staticmethod
    def internvit_300m() -> "InternViTConfig":      # vision tower of InternVL2.5-8B
        return InternViTConfig()

    @staticmethod
    def internvit_6b() -> "InternViTConfig":        # vision tower of InternVL2.5-26B
        return InternViTConfig(hidden_size=3200, num_hidden_layers=45, num_attention_heads=25,
                               intermediate_size=12800, qkv_bias=False, rms_norm=True, qk_normalization=True)

    @staticmethod
    def tiny() -> "InternViTConfig":
        return InternViTConfig(hidden_size=64, num_hidden_layers=2, num_attention_heads=4, intermediate_size=128)


class _RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        dt = x.dtype
        x = x.float()
        return (self.weight * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps)).to(dt))


def _norm(cfg: InternViTConfig, dim: int) -> nn.Module:
    return _RMSNorm(dim, cfg.layer_norm_eps) if cfg.rms_norm else nn.LayerNorm(dim, eps=cfg.layer_norm_eps)


class InternVisionEmbeddings(nn.Module):
    def __init__(self, cfg: InternViTConfig):
        super().__init__()
        self.patch_embedding = nn.Conv2d(3, cfg.hidden_size, kernel_size=cfg.patch_size, stride=cfg.patch_size)
        self.num_patches = (cfg.image_size // cfg.patch_size) ** 2
        self.class_embedding = nn.Parameter(torch.randn(1, 1, cfg.hidden_size) * 0.02)
        self.position_embedding = nn.Parameter(torch.randn(1, self.num_patches + 1, cfg.hidden_size) * 0.02)

    def forward(self, pixel_values):
        x = self.patch_embedding(pixel_values.to(self.patch_embedding.weight.dtype))   # (n, C, 32, 32)
        x = x.flatten(2).transpose(1, 2)                                               # (n, 1024, C)
        cls = self.class_embedding.expand(x.shape[0], 1, -1).to(x.dtype)
        return torch.cat([cls, x], dim=1) + self.position_embedding.to(x.dtype)


class InternVisionAttention(nn.Module):
    def __init__(self, cfg: InternViTConfig):
        super().__init__()
        self.num_heads = cfg.num_attention_heads
        self.head_dim = cfg.hidden_size // cfg.num_attention_heads
        self.qkv = nn.Linear(cfg.hidden_size, 3 * cfg.hidden_size, bias=cfg.qkv_bias)
        self.proj = nn.Linear(cfg.hidden_size, cfg.hidden_size)
        self.qk_normalization = cfg.qk_normalization
        if cfg.qk_normalization:
            self.q_norm = _RMSNorm(cfg.hidden_size, cfg.layer_norm_eps)
            self.k_norm = _RMSNorm(cfg.hidden_size, cfg.layer_norm_eps)

    def forward(self, x):
        n, t, c = x.shape
        q, k, v = self.qkv(x).view(n, t, 3, self.num_heads, self.head_dim).unbind(2)     # (n, t, heads, d) each
        if self.qk_normalization:
            q = self.q_norm(q.reshape(n, t, c)).view(n, t, self.num_heads, self.head_dim)
            k = self.k_norm(k.reshape(n, t, c)).view(n, t, self.num_heads, self.head_dim)
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        return self.proj(o.transpose(1, 2).reshape(n, t, c))


class InternVisionEncoderLayer(nn.Module):
    def __init__(self, cfg: InternViTConfig):
        super().__init__()
        self.norm1 = _norm(cfg, cfg.hidden_size)
        self.attn = InternVisionAttention(cfg)
        self.norm2 = _norm(cfg, cfg.hidden_size)
        self.fc1 = nn.Linear(cfg.hidden_size, cfg.intermediate_size)
        self.fc2 = nn.Linear(cfg.intermediate_size, cfg.hidden_size)
        self.ls1 = nn.Parameter(cfg.layer_scale_init * torch.ones(cfg.hidden_size))
        self.ls2 = nn.Parameter(cfg.layer_scale_init * torch.ones(cfg.hidden_size))

    def forward(self, x):
        x = x + self.attn(self.norm1(x)) * self.ls1
        return x + self.fc2(F.gelu(self.fc1(self.norm2(x)))) * self.ls2


def pixel_shuffle(x: torch.Tensor, scale_factor: float = 0.5) -> torch.Tensor:
    """(n, w, h, c) -> (n, w*s, h*s, c/s^2): every 1/s x 1/s block of patches becomes one token whose
    channels are the block's patches side by side (the rearrangement 'n (w a) (h b) c -> n w h (a b c)')."""
    n, w, h, c = x.shape
    r = int(round(1 / scale_factor))
    x = x.view(n, w // r, r, h // r, r, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(n, w // r, h // r, r * r * c)


class InternViTTower(nn.Module):
    """448 x 448 tiles -> (tiles, 256, llm_hidden): encoder, class token dropped, pixel shuffle, projector."""

    def __init__(self, cfg: InternViTConfig, llm_hidden: int):
        super().__init__()
        self.config = cfg
        self.embeddings = InternVisionEmbeddings(cfg)
        self.layers = nn.ModuleList([InternVisionEncoderLayer(cfg) for _ in range(cfg.num_hidden_layers)])
        r = int(round(1 / cfg.downsample_ratio))
        self.side = cfg.image_size // cfg.patch_size
        self.num_image_token = (self.side // r) ** 2
        self.mlp1 = nn.Sequential(nn.LayerNorm(cfg.hidden_size * r * r), nn.Linear(cfg.hidden_size * r * r, llm_hidden),
                                  nn.GELU(), nn.Linear(llm_hidden, llm_hidden))

    def forward(self, pixel_values):
        x = self.embeddings(pixel_values)
        for layer in self.layers:
            x = layer(x)
        x = x[:, 1:, :]                                             # class token dropped
        n, _, c = x.shape
        x = pixel_shuffle(x.reshape(n, self.side, self.side, c), self.config.downsample_ratio)
        return self.mlp1(x.reshape(n, -1, x.shape[-1]))             # (tiles, 256, llm_hidden)
