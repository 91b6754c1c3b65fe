"""The ablation variant of the FLARE block (pdebench/models/flare_ablations.py:19-311 of the reference):
latent queries shared across heads, and self-attention blocks on the M latents between the gather and
the scatter.  Same constructor arguments and state_dict keys; the two halves of the mixer run on the HIP
kernels (`flare_gather`, `flare_scatter`), the latent blocks (lra/models/backends.py:17-136) are plain
torch layers on a [B, M, C] tensor.  Scale is 1 in both halves, as in the reference (:109-113).
"""
from __future__ import annotations

import torch
from torch import nn
from torch.nn import functional as F

from .functional import flare_gather, flare_multihead_mixer, flare_scatter
from .modules import FinalLayer, ResidualMLP

__all__ = ["BigFLAREModel", "BigFLAREBlock", "BigFLARE", "SelfAttentionBlock"]


class MLPBlock(nn.Module):
    """fc1 -> act -> dropout -> fc2 (backends.py:17-37); act is exact GELU unless 'silu' is asked for."""

    def __init__(self, in_dim: int, hidden_dim: int, out_dim: int, act: str = None, drop: float = 0.0):
        super().__init__()
        self.drop = nn.Dropout(drop)
        self.fc1 = nn.Linear(in_dim, hidden_dim)
        self.act = nn.GELU() if act in ["gelu", None] else nn.SiLU()
        self.fc2 = nn.Linear(hidden_dim, out_dim)

    def forward(self, x):
        return self.fc2(self.drop(self.act(self.fc1(x))))


class MultiHeadedSelfAttention(nn.Module):
    """Softmax self-attention with scale head_dim^-1/2 (backends.py:60-110)."""

    def __init__(self, channel_dim: int, num_heads: int = None, attn_drop: float = 0.0, proj_drop: float = 0.0, rope=None):
        super().__init__()
        self.channel_dim = channel_dim
        self.num_heads = channel_dim // 16 if num_heads is None else num_heads
        self.head_dim = channel_dim // self.num_heads
        self.scale = self.head_dim ** -0.5
        self.rope = rope
        assert channel_dim % self.num_heads == 0, \
            f"channel_dim must be divisible by num_heads. Got {channel_dim} and {self.num_heads}."
        self.qkv_proj = nn.Linear(channel_dim, 3 * channel_dim, bias=True)
        self.out_proj = nn.Linear(channel_dim, channel_dim)
        self.attn_drop_p = attn_drop
        self.proj_drop = nn.Dropout(proj_drop)

    def forward(self, x, attention_mask=None):
        B, N, C = x.shape
        q, k, v = (t.view(B, N, self.num_heads, self.head_dim).transpose(1, 2) for t in self.qkv_proj(x).chunk(3, dim=-1))
        if self.rope is not None:
            q, k = self.rope(q), self.rope(k)
        mask = None
        if attention_mask is not None:
            mask = attention_mask.view(B, 1, 1, N) * attention_mask.view(B, 1, N, 1)
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=self.scale,
                                           dropout_p=self.attn_drop_p if self.training else 0.0)
        return self.proj_drop(self.out_proj(y.transpose(1, 2).reshape(B, N, C)))


class SelfAttentionBlock(nn.Module):
    """Pre-norm transformer block (backends.py:112-136)."""

    def __init__(self, channel_dim: int, num_heads: int = None, mlp_ratio: float = 4.0, act: str = None,
                 rmsnorm: bool = False, attn_drop: float = 0.0, proj_drop: float = 0.0, rope=None):
        super().__init__()
        self.norm1 = nn.RMSNorm(channel_dim) if rmsnorm else nn.LayerNorm(channel_dim)
        self.norm2 = nn.RMSNorm(channel_dim) if rmsnorm else nn.LayerNorm(channel_dim)
        self.att = MultiHeadedSelfAttention(channel_dim, num_heads, attn_drop=attn_drop, proj_drop=proj_drop, rope=rope)
        self.mlp = MLPBlock(in_dim=channel_dim, hidden_dim=int(channel_dim * mlp_ratio), out_dim=channel_dim, act=act,
                            drop=proj_drop)

    def forward(self, x, attention_mask=None):
        x = x + self.att(self.norm1(x), attention_mask=attention_mask)
        return x + self.mlp(self.norm2(x))


class BigFLARE(nn.Module):
    def __init__(self, channel_dim: int, num_heads: int = 8, num_latents: int = 32, act: str = None,
                 num_layers_kv_proj: int = 3, kv_proj_hidden_dim: int = None, shared_latents: bool = False,
                 num_latent_blocks: int = 0):
        super().__init__()
        self.channel_dim = channel_dim
        self.num_latents = num_latents
        self.num_heads = channel_dim // 8 if num_heads is None else num_heads
        self.head_dim = channel_dim // self.num_heads
        self.shared_latents = shared_latents
        self.num_latent_blocks = num_latent_blocks
        assert channel_dim % self.num_heads == 0, \
            f"channel_dim must be divisible by num_heads. Got {channel_dim} and {self.num_heads}."
        if shared_latents:
            assert num_latent_blocks == 0, \
                f"num_latent_blocks must be 0 when shared_latents is True. Got {num_latent_blocks}."
            self.latent_q = nn.Parameter(torch.empty(self.head_dim, num_latents))
        else:
            self.latent_q = nn.Parameter(torch.empty(channel_dim, num_latents))
        nn.init.normal_(self.latent_q, mean=0.0, std=0.1)
        self.k_proj, self.v_proj = [
            ResidualMLP(in_dim=channel_dim, hidden_dim=kv_proj_hidden_dim, out_dim=channel_dim,
                        num_layers=num_layers_kv_proj, act=act, input_residual=True, output_residual=True)
            for _ in range(2)]
        self.out_proj = nn.Linear(channel_dim, channel_dim)
        if num_latent_blocks > 0:
            self.latent_blocks = nn.ModuleList(
                SelfAttentionBlock(channel_dim=channel_dim, num_heads=self.num_heads, mlp_ratio=4.0, act=act)
                for _ in range(num_latent_blocks))

    def apply_latent_blocks(self, z):
        if self.num_latent_blocks == 0:
            return z
        B, H, M, D = z.shape
        z = z.transpose(1, 2).reshape(B, M, H * D)
        for block in self.latent_blocks:
            z = block(z)
        return z.view(B, M, H, D).transpose(1, 2)

    def forward(self, x, return_scores: bool = False):
        B, N, C = x.shape
        if return_scores:
            assert self.num_latent_blocks == 0, \
                f"num_latent_blocks must be 0 when return_scores is True. Got {self.num_latent_blocks}."
        if self.shared_latents:
            q = self.latent_q.view(1, self.num_latents, self.head_dim).expand(self.num_heads, -1, -1)
        else:
            q = self.latent_q.view(self.num_heads, self.num_latents, self.head_dim)
        k = self.k_proj(x).view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        v = self.v_proj(x).view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        scores = None
        if self.num_latent_blocks == 0:
            y = flare_multihead_mixer(q, k, v, scale=1.0, token_major_out=True)
            if return_scores:       # the explicit restatement of :116-125; the output stays the kernels'
                scores = q.unsqueeze(0).to(k.dtype) @ k.transpose(-2, -1)
        else:
            z, _ = flare_gather(q, k, v, scale=1.0)
            z = self.apply_latent_blocks(z.to(x.dtype))
            y = flare_scatter(q, k, z, scale=1.0)
        y = y.permute(0, 2, 1, 3).reshape(B, N, C)
        return self.out_proj(y), scores


class BigFLAREBlock(nn.Module):
    def __init__(self, channel_dim: int, num_heads: int = None, num_latents: int = None, act: str = None,
                 num_layers_kv_proj: int = 3, num_layers_mlp: int = 3, kv_proj_hidden_dim: int = None,
                 mlp_hidden_dim: int = None, shared_latents: bool = False, num_latent_blocks: int = 0):
        super().__init__()
        self.ln1 = nn.LayerNorm(channel_dim)
        self.ln2 = nn.LayerNorm(channel_dim)
        self.att = BigFLARE(channel_dim=channel_dim, num_heads=num_heads, num_latents=num_latents, act=act,
                            num_layers_kv_proj=num_layers_kv_proj, kv_proj_hidden_dim=kv_proj_hidden_dim,
                            shared_latents=shared_latents, num_latent_blocks=num_latent_blocks)
        self.mlp = ResidualMLP(in_dim=channel_dim, hidden_dim=mlp_hidden_dim, out_dim=channel_dim,
                               num_layers=num_layers_mlp, act=act, input_residual=True, output_residual=True)

    def forward(self, x, return_scores: bool = False):
        h, scores = self.att(self.ln1(x), return_scores=return_scores)
        x = x + h
        return x + self.mlp(self.ln2(x)), scores


class BigFLAREModel(nn.Module):
    def __init__(self, in_dim: int, out_dim: int, channel_dim: int = 64, num_blocks: int = 8, num_latents: int = None,
                 num_heads: int = None, act: str = None, num_layers_kv_proj: int = 3, num_layers_mlp: int = 3,
                 num_layers_in_out_proj: int = 2, mlp_ratio: float = 1.0, kv_proj_ratio: float = 1.0,
                 in_out_proj_ratio: float = 1.0, out_proj_ln: bool = True, shared_latents: bool = False,
                 num_latent_blocks: int = 0):
        super().__init__()
        mlp_hidden_dim = int(channel_dim * mlp_ratio)
        kv_proj_hidden_dim = int(channel_dim * kv_proj_ratio)
        io_hidden_dim = int(channel_dim * in_out_proj_ratio)
        self.in_proj = ResidualMLP(in_dim=in_dim, hidden_dim=io_hidden_dim, out_dim=channel_dim,
                                   num_layers=num_layers_in_out_proj, act=act, output_residual=True)
        self.out_proj = FinalLayer(channel_dim=channel_dim, hidden_dim=io_hidden_dim, out_dim=out_dim, act=act,
                                   num_layers=num_layers_in_out_proj, ln=out_proj_ln)
        self.blocks = nn.ModuleList(
            BigFLAREBlock(channel_dim=channel_dim, num_latents=num_latents, num_heads=num_heads, act=act,
                          num_layers_kv_proj=num_layers_kv_proj, num_layers_mlp=num_layers_mlp,
                          kv_proj_hidden_dim=kv_proj_hidden_dim, mlp_hidden_dim=mlp_hidden_dim,
                          shared_latents=shared_latents, num_latent_blocks=num_latent_blocks)
            for _ in range(num_blocks))
        self.apply(self._init_weights)

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            if m.bias is not None:
                nn.init.constant_(m.bias, 0.)
        elif isinstance(m, nn.LayerNorm):
            nn.init.constant_(m.bias, 0.)
            nn.init.constant_(m.weight, 1.)

    def forward(self, x, return_scores: bool = False):
        scores = []
        x = self.in_proj(x)
        for block in self.blocks:
            x, score = block(x, return_scores=return_scores)
            scores.append(score)
        x = self.out_proj(x)
        return (x, scores) if return_scores else x
