"""Sequence-model FLARE block with a padding mask (lra/models/backends.py:541-672 of the
reference): same state_dict keys and constructor arguments; `forward(x, attention_mask)`.

Mask semantics: attention_mask [B,N], nonzero = real token.  Padded tokens are left out of
the gather softmax; their own output rows are written as 0 (torch's fused attention leaves
fully masked query rows backend dependent; 0 is the value that does not poison mean pooling).
Attention dropout (attn_drop > 0 in training mode) acts on both softmaxes' weights, as the
reference's two scaled_dot_product_attention calls do (backends.py:592,605-606); it runs on the
fp32-FMA kernels with a counter-based mask that the backward recomputes.

Also here: the third-order linear-attention block of the same file (`TripleAttention`,
`TripleBlock`, backends.py:1195-1331) and the feature maps it selects by name
(lra/models/kernels.py:16-61, 66-104, 206-246), with the HIP triple kernels in place of the
einsum / Triton pair.
"""
from __future__ import annotations

import torch
from torch import nn
from torch.nn import functional as F

from .functional import flare_multihead_mixer, triple_attention
from . import fused
from .modules import ResidualMLP, _lin, _norm

__all__ = ["FLARE", "FLAREBlock", "TripleAttention", "TripleBlock", "make_kernel", "RotaryPositionalEmbeddings"]


class RotaryPositionalEmbeddings(nn.Module):
    """The rotary embedding the sequence models hand to their blocks as `rope` (lra/models/embeddings.py:103-147;
    built at lra/models/wrapper.py:87-88 with D = head_dim), applied to k only (backends.py:600-601).

    Position p turns channel j by the angle p * base^(-(j // 2) / (D / 2)):  out = x * cos + r * sin, where the
    partner r is the reference's own arrangement: its first half holds the negated odd channels
    (-x[1], -x[3], ...) and its second half the even channels (x[0], x[2], ...) -- not the interleaved pairing
    of the usual rotary embedding.  Checkpoints trained with the reference depend on it, so it is kept.
    Buffers C, S [max_length, D] are not part of the state_dict (as in the reference)."""

    def __init__(self, D: int, max_length: int, base: int = 10_000):
        super().__init__()
        assert D % 2 == 0
        self.D, self.N, self.base = D, max_length, float(base)
        rate = self.base ** (-(torch.arange(D, dtype=torch.float32) // 2) / (D // 2))      # [D], equal in pairs
        angle = torch.arange(max_length, dtype=torch.float32)[:, None] * rate[None, :]     # [N, D]
        self.register_buffer("C", torch.cos(angle), persistent=False)
        self.register_buffer("S", torch.sin(angle), persistent=False)

    def forward(self, x: torch.Tensor):
        N, D = x.shape[-2], x.shape[-1]
        assert D == self.D and N <= self.N
        partner = torch.cat([-x[..., 1::2], x[..., 0::2]], dim=-1)
        return x * self.C[:N].to(x.dtype) + partner * self.S[:N].to(x.dtype)


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

    def _fusable(self, x):
        """The 16-bit dtype the fused token-wise launches may run the three projections in, or None (torch layers)."""
        cds = {fused.compute_dtype(x, m) for m in (self.k_proj, self.v_proj, self.out_proj)}
        return cds.pop() if len(cds) == 1 else None

    def forward(self, x, attention_mask=None, _norm=None, _res=None):
        """_norm / _res are FLAREBlock's pre-norm and residual: under autocast (or with 16-bit weights) they are folded
        into the fused launches of the projections, and the result is _res + att(_norm(x))."""
        B, N, C = x.shape
        drop = self.attn_drop_p if self.training else 0.0       # on both softmaxes, as backends.py:592,605-606
        pdrop = self.proj_drop_p if self.training else 0.0
        q = self.latent_q.view(self.num_heads, self.num_latents, self.head_dim)
        cd = self._fusable(x)
        if cd is not None:
            k, v = fused.fused_mlp_pair(x, self.k_proj, self.v_proj, cd, norm=_norm, out_dtype=cd)
        else:
            xn = x if _norm is None else _norm(x)
            k, v = self.k_proj(xn), self.v_proj(xn)
        k = k.view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        v = v.view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        if self.rope is not None:
            k = self.rope(k)
        y = flare_multihead_mixer(q, k, v, scale=self.attn_scale, key_mask=attention_mask, token_major_out=True,
                                  dropout_p=drop)
        y = y.permute(0, 2, 1, 3).reshape(B, N, C)
        if cd is not None and pdrop == 0.0:
            return fused.fused_mlp(y, self.out_proj, cd, res=_res, out_dtype=(x if _res is None else _res).dtype)
        y = F.dropout(_lin(self.out_proj, y), p=pdrop)
        return y if _res is None else _res + y


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
        x = self.att(x, attention_mask=attention_mask, _norm=self.norm1, _res=x)
        cd = fused.compute_dtype(x, self.mlp)
        if cd is not None:
            return fused.fused_mlp(x, self.mlp, cd, norm=self.norm2, res=x)
        return x + self.mlp(self.norm2(x))


# ---- feature maps ("kernels") applied to q1, q2, k1, k2 --------------------------------------
# Parameter-free maps keep the shape of x (lra/models/kernels.py:16-61 and the registry at :206-221).
_PLAIN_KERNELS = {
    "identity": lambda x: x,
    "relu": F.relu,
    "relu_squared": lambda x: F.relu(x).square(),
    "silu": lambda x: F.silu(x) + 0.5,
    "elu": lambda x: F.elu(x) + 1.0,
    "elu_norm": lambda x: F.elu(x / x.norm(dim=-1, keepdim=True).clamp_min(1e-6)) + 1.0,
    "gelu": F.gelu,
    "tanh": torch.tanh,
    "softplus": lambda x: F.softplus(x) + 1e-6,
    "softsign": F.softsign,
    "sigmoid": torch.sigmoid,
    "exp": lambda x: torch.exp(x.clamp(-30.0, 30.0)),
    "cos": torch.cos,
    "sin": torch.sin,
}


class HadamardFeatureMap(nn.Module):
    """Product of two linear maps head_dim -> qk_dim (kernels.py:66-74)."""

    def __init__(self, head_dim: int, qk_dim: int):
        super().__init__()
        self.layer1 = nn.Linear(head_dim, qk_dim)
        self.layer2 = nn.Linear(head_dim, qk_dim)

    def forward(self, x):
        return self.layer1(x) * self.layer2(x)


class SwiGLUFeatureMap(nn.Module):
    """Gated linear unit head_dim -> qk_dim (kernels.py:76-84)."""

    def __init__(self, head_dim: int, qk_dim: int):
        super().__init__()
        self.layer1 = nn.Linear(head_dim, 2 * qk_dim)
        self.layer3 = nn.Linear(qk_dim, qk_dim)

    def forward(self, x):
        a, gate = self.layer1(x).chunk(2, dim=-1)
        return self.layer3(a * F.silu(gate))


class HedgehogFeatureMap(nn.Module):
    """softmax([2 W x, -2 W x]) with W initialised to the identity (kernels.py:86-104).
    The reference registry constructs it with (head_dim, qk_dim) although it takes head_dim only
    (kernels.py:244 against :91), which raises there; here qk_dim is accepted and ignored."""

    def __init__(self, head_dim: int, qk_dim: int = None):
        super().__init__()
        self.layer = nn.Linear(head_dim, head_dim)
        with torch.no_grad():
            self.layer.weight.copy_(torch.eye(head_dim))
            self.layer.bias.zero_()

    def forward(self, x):
        x = self.layer(x)
        return torch.cat([2 * x, -2 * x], dim=-1).softmax(-1)


_LEARNED_KERNELS = {"swiglu": SwiGLUFeatureMap, "hadamard": HadamardFeatureMap, "hedgehog": HedgehogFeatureMap}


def make_kernel(kernel: str, head_dim: int, qk_dim: int = None):
    """Feature map by name (kernels.py:229-246): a function for the parameter-free ones, a module otherwise."""
    qk_dim = head_dim if qk_dim is None else qk_dim
    if kernel in _PLAIN_KERNELS:
        return _PLAIN_KERNELS[kernel]
    if kernel in _LEARNED_KERNELS:
        return _LEARNED_KERNELS[kernel](head_dim=head_dim, qk_dim=qk_dim)
    raise NotImplementedError(f"Kernel '{kernel}' not implemented. Available: "
                              f"{sorted(_PLAIN_KERNELS)} + {sorted(_LEARNED_KERNELS)}")


class TripleAttention(nn.Module):
    """Third-order linear attention layer (backends.py:1195-1292): five token-wise projections, the
    feature map on q1, q2, k1, k2, optional unit-norm rows, the padding mask as a multiplication,
    state[i,j,k] = sum_n k1[n,i] v[n,j] k2[n,k] / N and out[n,j] = sum_ik q1[n,i] state[i,j,k] q2[n,k]
    on the HIP kernels, then a norm over the merged heads and out_proj.

    `use_triton` is accepted for call compatibility: both of the reference's code paths compute the same
    contraction, and both land on the HIP kernels here.  With kernel='elu' and nothing between the
    feature map and the contraction (no norm_q / norm_k, no mask) and no gradient needed, the map is
    applied inside the kernels."""

    def __init__(self, channel_dim: int, num_heads: int, act: str = None, rmsnorm: bool = False,
                 num_layers_kv_proj: int = -1, kv_proj_mlp_ratio: float = 1.0, kernel: str = "identity",
                 norm_q: bool = False, norm_k: bool = False, qk_dim_ratio: float = 1.0, use_triton: bool = False,
                 attn_drop: float = 0.0, proj_drop: float = 0.0, rope=None):
        super().__init__()
        assert channel_dim % num_heads == 0
        self.channel_dim = channel_dim
        self.num_heads = num_heads
        self.head_dim = channel_dim // num_heads
        self.qk_dim = int(self.head_dim * qk_dim_ratio)
        self.rope = rope
        self.kernel_name = kernel
        self.use_triton = use_triton
        self.out_proj = nn.Linear(channel_dim, channel_dim)
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj_drop = nn.Dropout(proj_drop)
        kws = dict(in_dim=channel_dim, hidden_dim=channel_dim, out_dim=channel_dim, num_layers=num_layers_kv_proj,
                   act=act, input_residual=True, output_residual=True)
        self.q1_proj = ResidualMLP(**kws)
        self.q2_proj = ResidualMLP(**kws)
        self.k1_proj = ResidualMLP(**kws)
        self.k2_proj = ResidualMLP(**kws)
        self.v_proj = ResidualMLP(**kws)
        self.kernel = make_kernel(kernel, head_dim=self.head_dim, qk_dim=self.qk_dim)
        self.norm_q = norm_q
        self.norm_k = norm_k
        self.norm = _norm(rmsnorm, channel_dim)

    def forward(self, x, attention_mask=None):
        B, N, C = x.shape
        assert self.rope is None, f"Rope is not supported by {self.__class__.__name__}."
        heads = lambda t: t.view(B, N, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        q1, q2, k1, k2, v = (heads(p(x)) for p in (self.q1_proj, self.q2_proj, self.k1_proj, self.k2_proj, self.v_proj))
        needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (q1, q2, k1, k2, v))
        in_kernel_map = (self.kernel_name == "elu" and not self.norm_q and not self.norm_k
                         and attention_mask is None and not needs_grad)
        if not in_kernel_map:
            q1, q2, k1, k2 = (self.kernel(t) for t in (q1, q2, k1, k2))
            if self.norm_q:
                q1, q2 = (t / (t.norm(dim=-1, keepdim=True) + 1e-6) for t in (q1, q2))
            if self.norm_k:
                k1, k2 = (t / (t.norm(dim=-1, keepdim=True) + 1e-6) for t in (k1, k2))
            if attention_mask is not None:
                mask = attention_mask.view(B, 1, N, 1)
                q1, q2, k1, k2, v = (t * mask for t in (q1, q2, k1, k2, v))
        _, out = self.attn(q1, q2, k1, k2, v, feature_map="elu" if in_kernel_map else None)
        out = out.permute(0, 2, 1, 3).reshape(B, N, C)
        return self.proj_drop(_lin(self.out_proj, self.norm(out)))

    def attn(self, q1, q2, k1, k2, v, feature_map=None):
        """(state, out) of backends.py:1285-1292 on the HIP kernels."""
        return triple_attention(q1, q2, k1, k2, v, feature_map=feature_map)

    attn_einsum = attn


class TripleBlock(nn.Module):
    """Pre-norm residual block around TripleAttention (backends.py:1294-1331)."""

    def __init__(self, channel_dim: int, num_heads: int, act: str = None, rmsnorm: bool = False,
                 num_layers_kv_proj: int = -1, kv_proj_mlp_ratio: float = 1.0, num_layers_ffn: int = 0,
                 ffn_mlp_ratio: float = 4.0, kernel: str = "identity", norm_q: bool = False, norm_k: bool = False,
                 qk_dim_ratio: float = 1.0, use_triton: bool = False, attn_drop: float = 0.0,
                 proj_drop: float = 0.0, rope=None):
        super().__init__()
        self.norm1 = _norm(rmsnorm, channel_dim)
        self.norm2 = _norm(rmsnorm, channel_dim)
        self.att = TripleAttention(channel_dim, num_heads, act=act, rmsnorm=rmsnorm,
                                   num_layers_kv_proj=num_layers_kv_proj, kv_proj_mlp_ratio=kv_proj_mlp_ratio,
                                   kernel=kernel, norm_q=norm_q, norm_k=norm_k, qk_dim_ratio=qk_dim_ratio,
                                   use_triton=use_triton, attn_drop=attn_drop, proj_drop=proj_drop, rope=rope)
        self.mlp = ResidualMLP(in_dim=channel_dim, hidden_dim=int(channel_dim * ffn_mlp_ratio), out_dim=channel_dim,
                               num_layers=num_layers_ffn, act=act, input_residual=True, output_residual=True)

    def forward(self, x, attention_mask=None):
        x = x + self.att(self.norm1(x), attention_mask=attention_mask)
        return x + self.mlp(self.norm2(x))
