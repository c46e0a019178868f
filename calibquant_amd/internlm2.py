"""InternLM2-shaped decoder (the language model of InternVL2.5) and a minimal
InternVL-chat-shaped wrapper, random-initialised, for running the patched
attention path without the upstream remote code or weights.

Only the attribute surface that the reference's patch touches is reproduced
(patch_internvl.py:141-484, 645-660): attention modules expose `wqkv`, `wo`,
`num_heads`, `num_key_value_heads`, `num_key_value_groups`, `head_dim`,
`hidden_size`, `rotary_emb(x, seq_len=)` and `_flash_attention_forward`; the
chat model exposes `language_model.model.layers[i].attention`,
`language_model.get_input_embeddings()`, `language_model.generate(...)`,
`extract_feature(pixel_values)` and `img_context_token_id`.  The fused wqkv
weight uses the `(h gs d)` interleave of the reference (patch_internvl.py:219-234):
per kv-head, `num_key_value_groups` query heads, then the key, then the value.
The vision tower is either the InternViT-shaped encoder of `internvit.py`
(`InternVLChatStandIn(cfg, vit=InternViTConfig...)`) or, by default, a one-layer
stand-in (patch projection to 256 tokens per tile) for tests that only need the
shapes: either way it only feeds the prefill."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from .kvbuffer import GrowingKV


@dataclass
class InternLM2Config:
    vocab_size: int = 92553
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    rms_norm_eps: float = 1e-5
    rope_theta: float = 1000000.0
    max_position_embeddings: int = 32768

    @staticmethod
    def internvl2_5_8b() -> "InternLM2Config":
        return InternLM2Config()

    @staticmethod
    def internvl2_5_26b() -> "InternLM2Config":
        return InternLM2Config(hidden_size=6144, intermediate_size=16384, num_hidden_layers=48,
                               num_attention_heads=48, num_key_value_heads=8)

    @staticmethod
    def tiny(layers: int = 2) -> "InternLM2Config":
        return InternLM2Config(vocab_size=512, hidden_size=512, intermediate_size=1024, num_hidden_layers=layers,
                               num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=8192)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        # one fused normalisation launch (fp32 statistics inside) instead of the six element-wise
        # launches of the textbook form: at decode the layer is bound by launches on the host.
        # (It rounds once, after the multiplication by the weight; the textbook form rounds the normalised
        # activations to the storage dtype before that multiplication.  The stand-in model's values shift by
        # that rounding - in its 1-bit and its full-precision runs alike; nothing on the quantised path
        # depends on it.)
        return F.rms_norm(x, self.weight.shape, self.weight, self.eps)


class RotaryEmbedding(nn.Module):
    """`rotary_emb(x, seq_len=n)` -> (cos, sin) tables of shape (n, head_dim), indexed by position id."""

    def __init__(self, dim: int, base: float, max_pos: int):
        super().__init__()
        self.dim, self.base = dim, base
        self.register_buffer("inv_freq", 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim)), persistent=False)
        self._cached = 0
        self._build(max(64, min(max_pos, 4096)))

    def _build(self, n: int):
        t = torch.arange(n, device=self.inv_freq.device, dtype=torch.float32)
        freqs = torch.outer(t, self.inv_freq.float())
        emb = torch.cat((freqs, freqs), dim=-1)
        self.register_buffer("cos_cached", emb.cos(), persistent=False)
        self.register_buffer("sin_cached", emb.sin(), persistent=False)
        self._cached = n

    def forward(self, x, seq_len: int):
        if seq_len > self._cached or self.cos_cached.device != x.device:
            self.inv_freq = self.inv_freq.to(x.device)
            self._build(max(seq_len, 2 * self._cached))
        return self.cos_cached[:seq_len].to(x.dtype), self.sin_cached[:seq_len].to(x.dtype)


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def _apply_rope(q, k, cos, sin, position_ids):
    cos = cos[position_ids].unsqueeze(1)
    sin = sin[position_ids].unsqueeze(1)
    return q * cos + _rotate_half(q) * sin, k * cos + _rotate_half(k) * sin


class InternLM2Attention(nn.Module):
    """Full-precision-KV attention; `patch_model` swaps the class `forward` for the quantised one."""

    def __init__(self, cfg: InternLM2Config):
        super().__init__()
        self.config = cfg
        self.hidden_size = cfg.hidden_size
        self.num_heads = cfg.num_attention_heads
        self.head_dim = cfg.hidden_size // cfg.num_attention_heads
        self.num_key_value_heads = cfg.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.is_causal = True
        self.wqkv = nn.Linear(cfg.hidden_size, (self.num_heads + 2 * self.num_key_value_heads) * self.head_dim,
                              bias=False)
        self.wo = nn.Linear(self.num_heads * self.head_dim, cfg.hidden_size, bias=False)
        self.rotary_emb = RotaryEmbedding(self.head_dim, cfg.rope_theta, cfg.max_position_embeddings)

    def _flash_attention_forward(self, query_states, key_states, value_states, attention_mask, query_length,
                                 dropout=0.0, softmax_scale=None):
        """(B, q, Hq, D) x (B, k, Hkv, D) causal attention, the last query row aligned
        with the last key row; returns (B, q, Hq, D).  `attention_mask` is an optional
        (B, k) 1/0 padding mask."""
        q = query_states.transpose(1, 2)
        k = key_states.transpose(1, 2)
        v = value_states.transpose(1, 2)
        ql, kl = q.shape[2], k.shape[2]
        if attention_mask is None and ql == kl:
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        elif attention_mask is None and ql == 1:
            o = F.scaled_dot_product_attention(q, k, v, enable_gqa=True)
        else:
            i = torch.arange(ql, device=q.device)[:, None] + (kl - ql)
            j = torch.arange(kl, device=q.device)[None, :]
            allow = (j <= i)[None, None]
            if attention_mask is not None:
                allow = allow & attention_mask[:, None, None, :kl].bool()
            o = F.scaled_dot_product_attention(q, k, v, attn_mask=allow, enable_gqa=True)
        return o.transpose(1, 2)

    def split_qkv(self, hidden_states):
        """The `(h gs d)` de-interleave of patch_internvl.py:219-234 (views, no copies)."""
        b, q_len, _ = hidden_states.shape
        qkv = self.wqkv(hidden_states).view(b, q_len, self.num_key_value_heads, 2 + self.num_key_value_groups,
                                            self.head_dim)
        q = qkv[..., : self.num_key_value_groups, :].reshape(b, q_len, self.num_heads, self.head_dim)
        return q, qkv[..., -2, :], qkv[..., -1, :]

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None,
                output_attentions=False, use_cache=False, **kwargs):
        bsz, q_len, _ = hidden_states.shape
        q, k, v = self.split_qkv(hidden_states)
        q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        kv_len = k.shape[-2] + (past_key_value[0].shape[-2] if past_key_value is not None else 0)
        cos, sin = self.rotary_emb(v, seq_len=kv_len)
        q, k = _apply_rope(q, k, cos, sin, position_ids)
        if use_cache:
            if not hasattr(self, "_kv"):
                self._kv = GrowingKV()
            k, v = self._kv.append(past_key_value, k, v)
        elif past_key_value is not None:
            k = torch.cat([past_key_value[0], k], dim=2)
            v = torch.cat([past_key_value[1], v], dim=2)
        past_key_value = (k, v) if use_cache else None
        pad = None
        if attention_mask is not None:
            pad = attention_mask if attention_mask.dim() == 2 else (attention_mask[:, 0, -1, :] == 0)
        o = self._flash_attention_forward(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), pad, q_len)
        o = o.reshape(bsz, q_len, self.hidden_size)
        return self.wo(o), None, past_key_value


class InternLM2MLP(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.w1 = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.w3 = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.w2 = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class InternLM2DecoderLayer(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.attention = InternLM2Attention(cfg)
        self.feed_forward = InternLM2MLP(cfg)
        self.attention_norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.ffn_norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)

    def forward(self, x, attention_mask, position_ids, past_key_value, use_cache):
        h, _, pkv = self.attention(self.attention_norm(x), attention_mask=attention_mask, position_ids=position_ids,
                                   past_key_value=past_key_value, use_cache=use_cache)
        x = x + h
        return x + self.feed_forward(self.ffn_norm(x)), pkv


class InternLM2Model(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.config = cfg
        self.tok_embeddings = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList([InternLM2DecoderLayer(cfg) for _ in range(cfg.num_hidden_layers)])
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)


class InternLM2ForCausalLM(nn.Module):
    def __init__(self, cfg: InternLM2Config):
        super().__init__()
        self.config = cfg
        self.model = InternLM2Model(cfg)
        self.output = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)

    def get_input_embeddings(self):
        return self.model.tok_embeddings

    def forward_step(self, inputs_embeds, position_ids, past, attention_mask=None):
        x = inputs_embeds
        new_past = []
        for i, layer in enumerate(self.model.layers):
            x, pkv = layer(x, attention_mask, position_ids, None if past is None else past[i], True)
            new_past.append(pkv)
        return self.output(self.model.norm(x[:, -1:, :])), new_past

    @torch.no_grad()
    def generate(self, inputs_embeds=None, attention_mask=None, generation_config=None, output_hidden_states=None,
                 use_cache=True, max_new_tokens: int = 16, on_step=None, **kwargs):
        """Greedy decoding from input embeddings; returns (B, max_new_tokens) token ids.
        `on_step(i)` is called after every generated token (used for timing)."""
        if generation_config is not None and getattr(generation_config, "max_new_tokens", None):
            max_new_tokens = generation_config.max_new_tokens
        B, N, _ = inputs_embeds.shape
        dev = inputs_embeds.device
        pos = torch.arange(N, device=dev)[None].expand(B, N)
        logits, past = self.forward_step(inputs_embeds, pos, None)
        out = []
        for i in range(max_new_tokens):
            tok = logits[:, -1].argmax(-1)
            out.append(tok)
            if on_step is not None:
                on_step(i)
            if i + 1 == max_new_tokens:
                break
            pos = torch.full((B, 1), N + i, device=dev, dtype=torch.long)
            logits, past = self.forward_step(self.get_input_embeddings()(tok)[:, None], pos, past)
        return torch.stack(out, dim=1)


class StandInVisionTower(nn.Module):
    """448x448 tile -> 256 tokens of `hidden` (28x28 patches of 16 px, 2x2 pooled to 14x14 ... here a
    single strided projection to a 16x16 grid): shape-compatible stand-in for InternViT + pixel shuffle + MLP."""

    def __init__(self, hidden: int):
        super().__init__()
        self.proj = nn.Conv2d(3, hidden, kernel_size=28, stride=28)

    def forward(self, pixel_values):
        x = self.proj(pixel_values)            # (tiles, hidden, 16, 16)
        return x.flatten(2).transpose(1, 2)    # (tiles, 256, hidden)


class InternVLChatStandIn(nn.Module):
    def __init__(self, cfg: InternLM2Config, img_context_token_id: Optional[int] = None, vit=None):
        """vit: an `internvit.InternViTConfig` for the InternViT-shaped tower (encoder, pixel shuffle,
        projector), or None for the one-layer stand-in."""
        super().__init__()
        self.config = cfg
        self.language_model = InternLM2ForCausalLM(cfg)
        if vit is None:
            self.vision = StandInVisionTower(cfg.hidden_size)
        else:
            from .internvit import InternViTTower
            self.vision = InternViTTower(vit, cfg.hidden_size)
        self.img_context_token_id = cfg.vocab_size - 1 if img_context_token_id is None else img_context_token_id
        self.num_image_token = 256

    def extract_feature(self, pixel_values):
        return self.vision(pixel_values)

    @torch.no_grad()
    def generate(self, pixel_values=None, input_ids=None, attention_mask=None, **kw):
        emb = self.language_model.get_input_embeddings()(input_ids)
        if pixel_values is not None:
            vit = self.extract_feature(pixel_values)
            sel = input_ids == self.img_context_token_id
            emb = emb.clone()
            emb[sel] = vit.reshape(-1, emb.shape[-1]).to(emb.dtype)
        return self.language_model.generate(inputs_embeds=emb, attention_mask=attention_mask, **kw)
