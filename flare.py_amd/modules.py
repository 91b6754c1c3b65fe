"""FLARE encoder modules with the reference's constructor arguments and state_dict keys.

Drop-in counterparts of pdebench/models/flare.py of the reference (ResidualMLP :24-59, FLARE
:64-156, FLAREBlock :161-215, FinalLayer :220-246, FLAREModel :251-349): a checkpoint of
the reference loads with strict=True.  The projections, norms and MLPs are ordinary torch
layers (hipBLASLt GEMMs); the mixer is the HIP engine (`functional.flare_multihead_mixer`),
which reads k and v as strided [B,N,H*D] views, so no head-split copy is made.

Fast path: when the Linear layers may run in bf16/f16 (autocast, or 16-bit weights) and channel_dim
is 32, 64 or 128, FLAREBlock runs as four fused HIP launches around the mixer (norm1 + k_proj,
norm1 + v_proj, out_proj + residual, norm2 + FFN + residual; see fused.py) instead of ~70 torch
kernels; with gradients enabled the same launches are differentiable (fused._FusedMlpFn).  fp32
without autocast uses the torch layers.
"""
from __future__ import annotations

import torch
from torch import nn
from torch.nn import functional as F

from . import fused
from .functional import flare_multihead_mixer

__all__ = ["ResidualMLP", "FLARE", "FLAREBlock", "FinalLayer", "FLAREModel"]


def _activation(name):
    if name in (None, "gelu"):
        return nn.GELU(approximate="tanh")
    if name == "silu":
        return nn.SiLU()
    raise KeyError(name)


def _norm(rmsnorm: bool, dim: int):
    return nn.RMSNorm(dim) if rmsnorm else nn.LayerNorm(dim)


class _LinearLongRows(torch.autograd.Function):
    """F.linear whose weight gradient is formed as a batched product over slices of the rows.  dW = dY^T X is a small
    (out x in) matrix summed over all tokens; as one product the library runs it without splitting that long axis (measured on
    this GPU: 104 / 330 us for 32,768 / 131,072 rows of 128 channels in fp32, against 28 / 46 us as 16-64 slices summed afterwards),
    and a token-wise model spends half of its backward there."""

    @staticmethod
    def forward(ctx, x, w, b):
        ctx.save_for_backward(x, w)
        ctx.has_bias = b is not None
        return F.linear(x, w, b)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = dy @ w
        dy2, x2 = dy.reshape(-1, w.shape[0]), x.reshape(-1, w.shape[1])
        if ctx.needs_input_grad[1]:
            T = x2.shape[0]
            S = next(s for s in (64, 32, 16, 8, 4, 2, 1) if T % s == 0)
            if S > 1:
                dw = torch.bmm(dy2.view(S, T // S, -1).transpose(1, 2), x2.view(S, T // S, -1)).sum(0)
            else:
                dw = dy2.t() @ x2
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = dy2.sum(0)
        return dx, dw, db


_LONG_ROWS = 4096      # rows from which the sliced weight gradient pays (below, one product is as fast)


def _lin(layer: nn.Linear, x):
    """layer(x); in training, on a GPU, outside autocast and over many rows: through _LinearLongRows."""
    if (torch.is_grad_enabled() and layer.weight.requires_grad and x.is_cuda and x.dtype == layer.weight.dtype
            and not torch.is_autocast_enabled() and x.numel() // max(x.shape[-1], 1) >= _LONG_ROWS
            and max(layer.in_features, layer.out_features) <= 1024):
        return _LinearLongRows.apply(x, layer.weight, layer.bias)
    return layer(x)


class ResidualMLP(nn.Module):
    """fc1 -> act -> num_layers x (x + act(fc x)) -> fc2, with optional end residuals.
    num_layers == -1 degenerates to a single Linear named `fc`."""

    def __init__(self, in_dim: int, hidden_dim: int, out_dim: int, num_layers: int = 2,
                 act: str = None, input_residual: bool = False, output_residual: bool = False):
        super().__init__()
        assert num_layers >= -1, f"num_layers must be at least -1. Got {num_layers}."
        self.num_layers = num_layers
        if num_layers == -1:
            self.fc = nn.Linear(in_dim, out_dim)
            self.residual = input_residual and output_residual and in_dim == out_dim
            return
        self.act = _activation(act)
        self.fc1 = nn.Linear(in_dim, hidden_dim)
        self.fcs = nn.ModuleList(nn.Linear(hidden_dim, hidden_dim) for _ in range(num_layers))
        self.fc2 = nn.Linear(hidden_dim, out_dim)
        self.input_residual = input_residual and in_dim == hidden_dim
        self.output_residual = output_residual and hidden_dim == out_dim

    def forward(self, x):
        if self.num_layers == -1:
            return x + _lin(self.fc, x) if self.residual else _lin(self.fc, x)
        h = self.act(_lin(self.fc1, x))
        x = x + h if self.input_residual else h
        for fc in self.fcs:
            x = x + self.act(_lin(fc, x))
        h = _lin(self.fc2, x)
        return x + h if self.output_residual else h


class FLARE(nn.Module):
    """Latent gather-scatter attention layer: returns (y, scores)."""

    def __init__(self, channel_dim: int, num_heads: int = 8, num_latents: int = 32, attn_scale: float = 1.0,
                 act: str = None, num_layers_k_proj: int = 3, num_layers_v_proj: int = 3,
                 k_proj_mlp_ratio: float = 1.0, v_proj_mlp_ratio: float = 1.0, qk_norm: bool = False,
                 rmsnorm: bool = False):
        super().__init__()
        self.channel_dim = channel_dim
        self.num_latents = num_latents
        self.num_heads = channel_dim // 8 if num_heads is None else num_heads
        self.head_dim = channel_dim // self.num_heads
        assert channel_dim % self.num_heads == 0, \
            f"channel_dim must be divisible by num_heads. Got {channel_dim} and {self.num_heads}."
        assert attn_scale > 0.0, f"attn_scale must be greater than 0. Got {attn_scale}."
        self.attn_scale = attn_scale

        self.latent_q = nn.Parameter(torch.empty(channel_dim, num_latents))
        nn.init.normal_(self.latent_q, mean=0.0, std=0.1)

        self.qk_norm = qk_norm
        if qk_norm:
            self.q_norm = _norm(rmsnorm, self.head_dim)
            self.k_norm = _norm(rmsnorm, self.head_dim)

        def proj(layers, ratio):
            return ResidualMLP(channel_dim, int(channel_dim * ratio), channel_dim, num_layers=layers, act=act,
                               input_residual=True, output_residual=True)

        self.k_proj = proj(num_layers_k_proj, k_proj_mlp_ratio)
        self.v_proj = proj(num_layers_v_proj, v_proj_mlp_ratio)
        self.out_proj = nn.Linear(channel_dim, channel_dim)

    def _heads(self, t):
        B, N, _ = t.shape
        return t.view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)  # [B,H,N,D] view, no copy

    def _cached_q(self, cd, pad):
        """latent_q as [H, M, D + pad] in the compute dtype for the inference fast path, rebuilt when the parameter
        changes (saves a cast, a fill and a copy per call, which is most of a small launch-bound forward)."""
        key = (self.latent_q._version, self.latent_q.data_ptr(), cd, pad)
        c = getattr(self, "_q_cache", None)
        if c is None or c[0] != key:
            q = self.latent_q.detach().view(self.num_heads, self.num_latents, self.head_dim).to(cd)
            if pad:
                q = torch.nn.functional.pad(q, (0, pad))
            c = self._q_cache = (key, q.contiguous())
        return c[1]

    def _fusable(self, x, return_scores):
        """The 16-bit dtype for the fused projections, or None."""
        if return_scores:
            return None
        cds = {fused.compute_dtype(x, m) for m in (self.k_proj, self.v_proj, self.out_proj)}
        return cds.pop() if len(cds) == 1 else None

    def forward(self, x, return_scores: bool = False, _norm=None, _res=None):
        """(y, scores).  _norm / _res are FLAREBlock's pre-norm and residual, folded into the fused
        launches when the fast path applies: then y = _res + out_proj(mixer(.. _norm(x) ..))."""
        B, N, C = x.shape
        q = self.latent_q.view(self.num_heads, self.num_latents, self.head_dim)
        cd = self._fusable(x, return_scores)
        D = self.head_dim
        # (head-padded rows have no backward: with gradients enabled the generic fused branch pads inside the mixer)
        narrow = (cd is not None and not torch.is_grad_enabled() and D in (4, 8) and self.num_latents % 32 == 0 and not self.qk_norm
                  # head-padded rows exist for the chain of square layers only: an expanding two-layer k/v projection
                  # takes the generic fused branch below, where the mixer pads the heads itself
                  and not fused._expand_factor(self.k_proj, C) and not fused._expand_factor(self.v_proj, C))
        if narrow:
            # narrow heads: the projections write k, v head-padded to 16 columns, which is what the mixer's
            # matrix-core kernels take, and the output projection reads the mixer's padded rows: no copies between
            H = self.num_heads
            k = fused.fused_mlp(x, self.k_proj, cd, norm=_norm, out_dtype=cd, y_head=D).view(B, N, H, 16).permute(0, 2, 1, 3)
            v = fused.fused_mlp(x, self.v_proj, cd, norm=_norm, out_dtype=cd, y_head=D).view(B, N, H, 16).permute(0, 2, 1, 3)
            y = flare_multihead_mixer(self._cached_q(cd, 16 - D), k, v, scale=self.attn_scale, token_major_out=True)
            y = y.permute(0, 2, 1, 3).reshape(B, N, H * 16)          # a view: the kernel laid y out as [B,N,H,16]
            out_dtype = _res.dtype if _res is not None else x.dtype
            return fused.fused_mlp(y, self.out_proj, cd, res=_res, out_dtype=out_dtype, x_head=D), None
        if cd is not None:
            k, v = fused.fused_mlp_pair(x, self.k_proj, self.v_proj, cd, norm=_norm, out_dtype=cd)
            k, v = self._heads(k), self._heads(v)
            if self.qk_norm:
                q = self.q_norm(q)
                k = self.k_norm(k)
            elif not torch.is_grad_enabled():
                q = self._cached_q(cd, 0)
            # (with gradients enabled q stays the parameter's view: the mixer casts it itself and differentiates it)
            y = flare_multihead_mixer(q, k, v, scale=self.attn_scale, token_major_out=True)
            y = y.permute(0, 2, 1, 3).reshape(B, N, C)
            out_dtype = _res.dtype if _res is not None else x.dtype
            return fused.fused_mlp(y, self.out_proj, cd, res=_res, out_dtype=out_dtype), None
        if _norm is not None:
            x = _norm(x)
        k = self._heads(self.k_proj(x))
        v = self._heads(self.v_proj(x))
        if self.qk_norm:
            q = self.q_norm(q)
            k = self.k_norm(k)

        if not return_scores:
            y = flare_multihead_mixer(q, k, v, scale=self.attn_scale, token_major_out=True)
            scores = None
        else:
            # Diagnostic branch: materialises the [B,H,M,N] score matrix, exactly as the
            # reference's spelled-out branch does (and, like it, without attn_scale).
            scores = q @ k.transpose(-2, -1)
            z = F.softmax(scores, dim=-1) @ v
            y = F.softmax(scores.transpose(-2, -1), dim=-1) @ z

        y = y.permute(0, 2, 1, 3).reshape(B, N, C)
        y = _lin(self.out_proj, y)
        return (y if _res is None else _res + y), scores


class FLAREBlock(nn.Module):
    """x + att(norm1 x), then x + mlp(norm2 x); returns (x, scores)."""

    def __init__(self, channel_dim: int, num_heads: int = None, num_latents: int = None, attn_scale: float = 1.0,
                 act: str = None, rmsnorm: bool = False, num_layers_k_proj: int = 3, num_layers_v_proj: int = 3,
                 k_proj_mlp_ratio: float = 1.0, v_proj_mlp_ratio: float = 1.0, num_layers_ffn: int = 3,
                 ffn_mlp_ratio: float = 1.0, qk_norm: bool = False):
        super().__init__()
        self.norm1 = _norm(rmsnorm, channel_dim)
        self.norm2 = _norm(rmsnorm, channel_dim)
        self.att = FLARE(channel_dim=channel_dim, num_heads=num_heads, num_latents=num_latents,
                         attn_scale=attn_scale, act=act, num_layers_k_proj=num_layers_k_proj,
                         num_layers_v_proj=num_layers_v_proj, k_proj_mlp_ratio=k_proj_mlp_ratio,
                         v_proj_mlp_ratio=v_proj_mlp_ratio, qk_norm=qk_norm, rmsnorm=rmsnorm)
        self.mlp = ResidualMLP(channel_dim, int(channel_dim * ffn_mlp_ratio), channel_dim,
                               num_layers=num_layers_ffn, act=act, input_residual=True, output_residual=True)

    def forward(self, x, return_scores: bool = False):
        x, scores = self.att(x, return_scores=return_scores, _norm=self.norm1, _res=x)
        cd = fused.compute_dtype(x, self.mlp)
        if cd is not None:
            x = fused.fused_mlp(x, self.mlp, cd, norm=self.norm2, res=x)
        else:
            x = x + self.mlp(self.norm2(x))
        return x, scores


class FinalLayer(nn.Module):
    def __init__(self, channel_dim: int, out_dim: int, act: str = None, num_layers: int = 2,
                 hidden_dim: int = None, ln: bool = True):
        super().__init__()
        hidden_dim = channel_dim if hidden_dim is None else hidden_dim
        self.ln = nn.LayerNorm(channel_dim) if ln else nn.Identity()
        self.mlp = ResidualMLP(channel_dim, hidden_dim, out_dim, num_layers=num_layers, act=act,
                               input_residual=True, output_residual=False)

    def forward(self, x):
        cd = fused.compute_dtype(x, self.mlp)
        if cd is not None:
            return fused.fused_mlp(x, self.mlp, cd, norm=self.ln)
        return self.mlp(self.ln(x))


class FLAREModel(nn.Module):
    """in_proj -> num_blocks x FLAREBlock -> (norm, out MLP)."""

    def __init__(self, in_dim: int, out_dim: int, channel_dim: int = 64, num_blocks: int = 8,
                 num_heads: int = None, act: str = None, rmsnorm: bool = False, out_proj_norm: bool = True,
                 num_layers_in_out_proj: int = 2, attn_scale: float = 1.0, num_latents: int = None,
                 num_layers_k_proj: int = 3, num_layers_v_proj: int = 3, k_proj_mlp_ratio: float = 1.0,
                 v_proj_mlp_ratio: float = 1.0, num_layers_ffn: int = 3, ffn_mlp_ratio: float = 1.0,
                 qk_norm: bool = False):
        super().__init__()
        self.in_proj = ResidualMLP(in_dim, channel_dim, channel_dim, num_layers=num_layers_in_out_proj, act=act,
                                   input_residual=False, output_residual=True)
        self.out_proj = nn.Sequential(
            _norm(rmsnorm, channel_dim) if out_proj_norm else nn.Identity(),
            ResidualMLP(channel_dim, channel_dim, out_dim, num_layers=num_layers_in_out_proj, act=act,
                        input_residual=True, output_residual=False),
        )
        self.blocks = nn.ModuleList(
            FLAREBlock(channel_dim=channel_dim, num_heads=num_heads, act=act, rmsnorm=rmsnorm,
                       attn_scale=attn_scale, num_latents=num_latents, num_layers_k_proj=num_layers_k_proj,
                       num_layers_v_proj=num_layers_v_proj, k_proj_mlp_ratio=k_proj_mlp_ratio,
                       v_proj_mlp_ratio=v_proj_mlp_ratio, num_layers_ffn=num_layers_ffn,
                       ffn_mlp_ratio=ffn_mlp_ratio, qk_norm=qk_norm)
            for _ in range(num_blocks))
        self.initialize_weights()

    def initialize_weights(self):
        self.apply(self._init_weights)

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, (nn.LayerNorm, nn.RMSNorm)):
            if getattr(m, "weight", None) is not None:
                nn.init.ones_(m.weight)
            if getattr(m, "bias", None) is not None:
                nn.init.zeros_(m.bias)

    def forward(self, x, return_scores: bool = False):
        scores = []
        cd = fused.compute_dtype(x, self.in_proj)
        x = fused.fused_mlp(x, self.in_proj, cd) if cd is not None else self.in_proj(x)
        for block in self.blocks:
            x, s = block(x, return_scores=return_scores)
            if return_scores:
                scores.append(s)
        cd = fused.compute_dtype(x, self.out_proj[1])
        x = fused.fused_mlp(x, self.out_proj[1], cd, norm=self.out_proj[0]) if cd is not None else self.out_proj(x)
        return (x, scores) if return_scores else x
