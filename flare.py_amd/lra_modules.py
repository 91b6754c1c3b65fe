"""Sequence-model FLARE block with a padding mask (lra/models/backends.py:541-672 of the
reference): same state_dict keys and constructor arguments; `forward(x, attention_mask)`.

Mask semantics: attention_mask [B,N], nonzero = real token.  Padded tokens are left out of
the gather softmax; their own output rows are written as 0 (torch's fused attention leaves
fully masked query rows backend dependent; 0 is the value that does not poison mean pooling).
Attention dropout inside the softmax is not implemented in the kernels: attn_drop > 0 in
training mode raises.
"""
from __future__ import annotations

import torch
from torch import nn
from torch.nn import functional as F

from .functional import flare_multihead_mixer
from .modules import ResidualMLP, _norm

__all__ = ["FLARE", "FLAREBlock"]


class FLARE(nn.Module):
    def __init__(self, channel_dim: int, num_heads: int = 8, num_latents: int = 32, act: str = None,
                 attn_scale: float = 1.0, num_layers_kv_proj: int = 3, kv_proj_hidden_dim: int = 1.0,
                 attn_drop: float = 0.0, proj_drop: float = 0.0, rope=None):
        super().__init__()
        assert attn_scale > 0.0, f"attn_scale must be greater than 0. Got {attn_scale}."
        self.attn_scale = attn_scale
        self.channel_dim = channel_dim
        self.num_latents = num_latents
        self.num_heads = channel_dim // 8 if num_heads is None else num_heads
        self.head_dim = channel_dim // self.num_heads
        self.rope = rope
        self.attn_drop_p = attn_drop
        self.proj_drop_p = proj_drop
        assert channel_dim % self.num_heads == 0, \
            f"channel_dim must be divisible by num_heads. Got {channel_dim} and {self.num_heads}."

        self.latent_q = nn.Parameter(torch.empty(channel_dim, num_latents))
        nn.init.normal_(self.latent_q, mean=0.0, std=0.1)
        self.k_proj = ResidualMLP(channel_dim, kv_proj_hidden_dim, channel_dim, num_layers=num_layers_kv_proj,
                                  act=act, input_residual=True, output_residual=True)
        self.v_proj = ResidualMLP(channel_dim, kv_proj_hidden_dim, channel_dim, num_layers=num_layers_kv_proj,
                                  act=act, input_residual=True, output_residual=True)
        self.out_proj = nn.Linear(channel_dim, channel_dim)

    def forward(self, x, attention_mask=None):
        B, N, C = x.shape
        if self.training and self.attn_drop_p > 0.0:
            raise NotImplementedError("attention dropout is not implemented in the FLARE HIP kernels")
        q = self.latent_q.view(self.num_heads, self.num_latents, self.head_dim)
        k = self.k_proj(x).view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        v = self.v_proj(x).view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        if self.rope is not None:
            k = self.rope(k)
        y = flare_multihead_mixer(q, k, v, scale=self.attn_scale, key_mask=attention_mask, token_major_out=True)
        y = self.out_proj(y.permute(0, 2, 1, 3).reshape(B, N, C))
        return F.dropout(y, p=self.proj_drop_p if self.training else 0.0)


class FLAREBlock(nn.Module):
    def __init__(self, channel_dim: int, num_heads: int = None, num_latents: int = None, act: str = None,
                 rmsnorm: bool = False, attn_scale: float = 1.0, num_layers_kv_proj: int = 3,
                 num_layers_ffn: int = 3, kv_proj_hidden_dim: int = 1.0, ffn_hidden_dim: int = 1.0,
                 attn_drop: float = 0.0, proj_drop: float = 0.0, rope=None):
        super().__init__()
        self.norm1 = _norm(rmsnorm, channel_dim)
        self.norm2 = _norm(rmsnorm, channel_dim)
        self.att = FLARE(channel_dim=channel_dim, num_heads=num_heads, num_latents=num_latents, act=act,
                         attn_scale=attn_scale, num_layers_kv_proj=num_layers_kv_proj,
                         kv_proj_hidden_dim=kv_proj_hidden_dim, attn_drop=attn_drop, proj_drop=proj_drop,
                         rope=rope)
        self.mlp = ResidualMLP(channel_dim, ffn_hidden_dim, channel_dim, num_layers=num_layers_ffn, act=act,
                               input_residual=True, output_residual=True)

    def forward(self, x, attention_mask=None):
        x = x + self.att(self.norm1(x), attention_mask=attention_mask)
        return x + self.mlp(self.norm2(x))
