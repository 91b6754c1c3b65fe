"""Fused inference path for the token-wise layers around the mixer (HIP kernel flare_mlp_fwd).

`fused_mlp(x, mlp, norm=..., res=...)` evaluates, in ONE launch and without leaving the chip
between layers, what the reference runs as separate torch layers:

    res + ResidualMLP(norm(x))         pdebench/models/flare.py:45-59 and 204-215
    res + Linear(x)                    (out_proj, flare.py:156)

It is used by the modules only when no gradient is needed and the products may run in bf16/f16
(torch.autocast is on, or the weights already are bf16/f16) — the conditions under which torch
itself would run these Linear layers in that type.  Everything else stays with the torch layers.
The 16-bit copies of the weights are cached per module and rebuilt when a parameter changes.
"""
from __future__ import annotations

import ctypes as C

import torch
from torch import nn

from . import _lib
from .functional import _autocast_dtype, _dtype_code, _ptr, _stream_ptr

_SUPPORTED_C = (32, 64, 128)
_ACTS = {"gelu": 0, "silu": 1}


def _layers_of(mod):
    """(linear layers, act_mask, add_mask, act code) of a ResidualMLP or nn.Linear, or None."""
    if isinstance(mod, nn.Linear):
        return [mod], 0, 0, 0
    if getattr(mod, "num_layers", None) is None:
        return None
    if mod.num_layers == -1:
        return [mod.fc], 0, (1 if mod.residual else 0), 0
    layers = [mod.fc1, *mod.fcs, mod.fc2]
    L = len(layers)
    act_mask = (1 << (L - 1)) - 1
    add_mask = ((1 << (L - 1)) - 2) | (1 if mod.input_residual else 0) | ((1 << (L - 1)) if mod.output_residual else 0)
    if isinstance(mod.act, nn.GELU) and mod.act.approximate == "tanh":
        act = 0
    elif isinstance(mod.act, nn.SiLU):
        act = 1
    else:
        return None
    return layers, act_mask, add_mask, act


def compute_dtype(x, mod):
    """The 16-bit type the fused kernel may run this module in, or None (then torch runs it)."""
    if torch.is_grad_enabled() or x.device.type != "cuda":
        return None
    info = _layers_of(mod)
    if info is None:
        return None
    layers = info[0]
    Cdim = x.shape[-1]
    if Cdim not in _SUPPORTED_C or len(layers) > 16:
        return None
    if any(l.in_features != Cdim or l.out_features != Cdim for l in layers):
        return None
    if x.dtype not in (torch.float32, torch.bfloat16, torch.float16) or x.stride(-1) != 1:
        return None
    ac = _autocast_dtype(x)
    if ac in (torch.bfloat16, torch.float16):
        return ac
    wd = layers[0].weight.dtype
    if ac is None and wd in (torch.bfloat16, torch.float16) and all(l.weight.dtype == wd for l in layers):
        return wd
    return None


def _packed(mod, layers, cd):
    """[L,C,C] weights in the compute dtype and [L,C] fp32 biases, cached on the module."""
    key = (cd, tuple((l.weight.data_ptr(), l.weight._version, None if l.bias is None else l.bias._version) for l in layers))
    cache = getattr(mod, "_flare_packed", None)
    if cache is not None and cache[0] == key:
        return cache[1], cache[2]
    w = torch.stack([l.weight.detach() for l in layers]).to(cd).contiguous()
    Cdim = w.shape[-1]
    b = torch.stack([l.bias.detach().float() if l.bias is not None else w.new_zeros(Cdim, dtype=torch.float32) for l in layers]).contiguous()
    mod._flare_packed = (key, w, b)
    return w, b


def fused_mlp(x, mod, cd, norm=None, res=None, out_dtype=None):
    """y = res + mod(norm(x)) in one HIP launch.  x: [..., C]; mod: ResidualMLP or nn.Linear; cd: the
    dtype from compute_dtype(); norm: nn.LayerNorm / nn.RMSNorm / None; res: [..., C] or None."""
    lib = _lib.load()
    layers, act_mask, add_mask, act = _layers_of(mod)
    Cdim = x.shape[-1]
    w, b = _packed(mod, layers, cd)
    x2 = x.reshape(-1, Cdim)
    if x2.stride(-1) != 1 or x2.stride(0) % 4 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out_dtype = x.dtype if out_dtype is None else out_dtype
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L = x2.shape[0], Cdim, len(layers)
    d.w_dtype, d.x_dtype, d.y_dtype = _dtype_code(w), _dtype_code(x2), _dtype_code(y)
    d.act, d.act_mask, d.add_mask = act, act_mask, add_mask
    d.x_stride, d.y_stride = x2.stride(0), Cdim
    gamma = beta = None
    if norm is not None and not isinstance(norm, nn.Identity):
        if isinstance(norm, nn.LayerNorm):
            d.norm, d.eps = 1, float(norm.eps)
            beta = None if norm.bias is None else norm.bias.detach().float().contiguous()
        elif isinstance(norm, nn.RMSNorm):
            d.norm = 2
            d.eps = float(norm.eps) if norm.eps is not None else float(torch.finfo(x.dtype).eps)
        else:
            raise TypeError(f"unsupported norm {type(norm).__name__}")
        gamma = (norm.weight.detach().float().contiguous() if getattr(norm, "weight", None) is not None
                 else torch.ones(Cdim, dtype=torch.float32, device=x.device))
    r2 = None
    if res is not None:
        r2 = res.reshape(-1, Cdim)
        if r2.stride(-1) != 1 or r2.stride(0) % 4 or r2.data_ptr() % 16:
            r2 = r2.contiguous()
        d.res_dtype, d.res_stride = _dtype_code(r2), r2.stride(0)
    with torch.cuda.device(x.device):
        rc = lib.flare_mlp_fwd(C.byref(d), _ptr(x2), _ptr(w), _ptr(b), _ptr(gamma), _ptr(beta), _ptr(r2), _ptr(y),
                               C.c_void_p(_stream_ptr(x.device)))
    _lib.check(rc, "flare_mlp_fwd")
    return y
