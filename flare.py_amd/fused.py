"""Fused path for the token-wise layers around the mixer (HIP kernels flare_mlp_fwd / flare_mlp_bwd).

`fused_mlp(x, mlp, norm=..., res=...)` evaluates, in ONE launch and without leaving the chip
between layers, what the reference runs as separate torch layers:

    res + ResidualMLP(norm(x))         pdebench/models/flare.py:45-59 and 204-215
    res + Linear(x)                    (out_proj, flare.py:156)

    ResidualMLP(in_dim <= 4, C, C)     (the models' in_proj, flare.py:137-140: the narrow first layer runs on
    ResidualMLP(C, C, out_dim <= 4)     the vector ALU; of out_proj's last layer only the real rows are stored)

A ResidualMLP with num_layers == 0 and a hidden width of E*C (2 <= E <= 8; the "4x expansion" feed-forward
block) runs in the same launch as E pairs of C x C tiles, the hidden activations never leaving the registers.

It is used by the modules only when the products may run in bf16/f16 (torch.autocast is on, or the
weights already are bf16/f16) — the conditions under which torch itself would run these Linear layers
in that type.  Everything else stays with the torch layers.  The 16-bit copies of the weights are
cached per module and rebuilt when a parameter changes.

With gradients enabled the chain of C x C layers (the k/v projections, the feed-forward block and the output
projection of a FLAREBlock at the reference's default ratios) runs through `_FusedMlpFn`: the same forward
launch, and a backward that recomputes the chain per token tile in one launch (flare_mlp_bwd) and forms the
parameter gradients from the rows it leaves with one more launch (flare_mlp_wgrad); the expanding two-layer MLP has a
backward launch of its own (flare_mlp_expand_bwd).  A stack with a narrow first input or last output keeps that one
layer as a torch layer while gradients are enabled and sends the C x C layers between through the same path; the
head-padded variants have no backward.
"""
from __future__ import annotations

import ctypes as C

import torch
from torch import nn
from torch.autograd.function import once_differentiable

from . import _lib
from .functional import _autocast_dtype, _dtype_code, _on_device, _ptr, _stream_ptr

_SUPPORTED_C = (32, 64, 128)
_ACTS = {"gelu": 0, "silu": 1}


def _structure_key(mod):
    """Identity of everything the structural caches are built from: the layers, the activation module and the flags
    that set the masks.  Assigning a new submodule (a LoRA wrap, a re-initialisation by assignment) changes it.
    Read from the module's own tables: every fused call asks several times, and attribute access on a Module goes
    through its __getattr__ for submodules."""
    if isinstance(mod, _SubChain):
        return None
    d = mod.__dict__
    nl = d.get("num_layers")
    if isinstance(mod, nn.Linear) or nl is None:
        return (type(mod),)
    m = d["_modules"]
    if nl == -1:
        return (-1, id(m["fc"]), bool(d["residual"]))
    act = m["act"] if "act" in m else d.get("act")
    return (nl, id(m["fc1"]), tuple(map(id, m["fcs"]._modules.values())), id(m["fc2"]), id(act),
            getattr(act, "approximate", None), bool(d["input_residual"]), bool(d["output_residual"]))


def _layers_of(mod):
    """(linear layers, act_mask, add_mask, act code) of a ResidualMLP or nn.Linear, or None.  The answer is kept on
    the module together with the identities of the submodules it was read from, and rebuilt when one of them is
    replaced."""
    key = _structure_key(mod)
    cached = mod.__dict__.get("_flare_layers")
    if cached is not None and cached[1] == key:
        return cached[0]
    info = _layers_of_uncached(mod)
    mod.__dict__["_flare_layers"] = (info, key)
    return info


def _layers_of_uncached(mod):
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


def _expand_factor(mod, Cdim):
    """E when mod is the two-layer MLP C -> E*C -> C (ResidualMLP with num_layers == 0 and no residual that
    applies), else 0."""
    if getattr(mod, "num_layers", None) != 0 or mod.input_residual or mod.output_residual:
        return 0
    f1, f2 = mod.fc1, mod.fc2
    hid = f1.out_features
    if f1.in_features != Cdim or f2.out_features != Cdim or f2.in_features != hid or hid % Cdim or hid == Cdim:
        return 0
    E = hid // Cdim
    return E if 2 <= E <= 8 else 0


def _io_dims(mod, layers):
    """(C, in_dim, out_dim) of a stack that is C x C except for a narrow (<= 4) first input and/or last output
    (0 = that end is C wide), or None."""
    if len(layers) < 2:
        return None
    Cdim = layers[0].out_features
    if any(l.in_features != Cdim or l.out_features != Cdim for l in layers[1:-1]) or layers[-1].in_features != Cdim:
        return None
    i, o = layers[0].in_features, layers[-1].out_features
    if not ((i == Cdim or i <= 4) and (o == Cdim or o <= 4)):
        return None
    return Cdim, (0 if i == Cdim else i), (0 if o == Cdim else o)


_BWD_MAX_LAYERS = {32: 8, 64: 8, 128: 5}      # the backward keeps every layer's slopes in registers


class _SubChain:
    """The C x C layers of a stack whose first input and/or last output is narrow, as a stack of their own: what the
    fused launches and their backward see while gradients are enabled.  `first` / `last`: the narrow nn.Linear that
    stays a torch layer on that side (or None); the packed-weight caches live on this object."""

    num_layers = None

    def __init__(self, layers, act_mask, add_mask, act, C, first, first_act, last, act_module):
        self.__dict__["_flare_layers"] = ((layers, act_mask, add_mask, act), None)
        self.C, self.first, self.first_act, self.last, self.act_module = C, first, first_act, last, act_module


class _NarrowLinearFn(torch.autograd.Function):
    """t = x W^T + b for a Linear with a few input columns (the lift of the models' in_proj) under autocast.  Only the
    weight gradient differs from torch's own: dW = g^T x contracts over all tokens into a [C, in_dim] result, which the
    library runs as one long product with nothing to parallelise; here it is a batched product over chunks of 4096
    tokens whose partial results are summed in fp32."""

    @staticmethod
    def forward(ctx, x2, w, b, cd):
        ctx.save_for_backward(x2, w)
        ctx.has_bias = b is not None
        return torch.nn.functional.linear(x2.to(cd), w.to(cd), None if b is None else b.to(cd))

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        x2, w = ctx.saved_tensors
        T, chunk = g.shape[0], 4096
        n = T // chunk
        xc = x2.to(g.dtype)
        dw = torch.zeros(w.shape, dtype=torch.float32, device=g.device)
        if n > 0:
            dw += torch.bmm(g[:n * chunk].view(n, chunk, -1).transpose(1, 2), xc[:n * chunk].view(n, chunk, -1)).sum(0, dtype=torch.float32)
        if n * chunk < T:
            dw += (g[n * chunk:].t() @ xc[n * chunk:]).float()
        db = g.sum(0, dtype=torch.float32).to(w.dtype) if ctx.has_bias else None
        dx = (g @ w.to(g.dtype)).to(x2.dtype) if ctx.needs_input_grad[0] else None
        return dx, dw.to(w.dtype), db, None


def _train_subchain(mod):
    """_SubChain of a stack with a narrow end (None for every other module); kept on the module."""
    key = _structure_key(mod)
    cached = mod.__dict__.get("_flare_subchain")
    if cached is not None and cached[1] == key:
        return cached[0]
    sub = None
    info = _layers_of(mod)
    if info is not None:
        layers, act_mask, add_mask, act = info
        io = _io_dims(mod, layers)
        if io is not None and (io[1] or io[2]):
            Cdim, in_dim, out_dim = io
            lo, hi = (1 if in_dim else 0), (len(layers) - 1 if out_dim else len(layers))
            n = hi - lo
            if n >= 1:
                keep = (1 << n) - 1
                sub = _SubChain(layers[lo:hi], (act_mask >> lo) & keep, (add_mask >> lo) & keep, act, Cdim,
                                layers[0] if in_dim else None, bool(act_mask & 1), layers[-1] if out_dim else None, mod.act)
    mod.__dict__["_flare_subchain"] = (sub, key)
    return sub


def compute_dtype(x, mod):
    """The 16-bit type the fused kernels may run this module in, or None (then torch runs it).  With gradients
    enabled the chain of C x C layers and the expanding two-layer MLP qualify (the shapes flare_mlp_bwd and
    flare_mlp_expand_bwd differentiate), and a stack with a narrow end for the chain between its narrow layers."""
    if x.device.type != "cuda":
        return None
    # what depends on the module's structure and the row width only is decided once per (structure, width, grad mode)
    grad = torch.is_grad_enabled()
    key = (_structure_key(mod), x.shape[-1], grad)
    cached = mod.__dict__.get("_flare_shape_ok")
    if cached is None or cached[0] != key:
        cached = (key, _shape_ok(x.shape[-1], mod, grad))
        mod.__dict__["_flare_shape_ok"] = cached
    if not cached[1]:
        return None
    layers = _layers_of(mod)[0]
    if x.dtype not in (torch.float32, torch.bfloat16, torch.float16) or x.stride(-1) != 1:
        return None
    ac = _autocast_dtype(x)
    if ac in (torch.bfloat16, torch.float16):
        return ac
    wd = layers[0].weight.dtype
    if ac is None and wd in (torch.bfloat16, torch.float16) and all(l.weight.dtype == wd for l in layers):
        return wd
    return None


def _shape_ok(width, mod, grad):
    info = _layers_of(mod)
    if info is None:
        return False
    layers = info[0]
    if len(layers) > 16:
        return False
    if grad:
        sub = _train_subchain(mod)
        if sub is not None:                 # narrow first input / last output: the C x C layers between them
            n = len(_layers_of(sub)[0])
            if sub.C not in _SUPPORTED_C or n > _BWD_MAX_LAYERS[sub.C] or width != layers[0].in_features:
                return False
        else:
            if width not in _SUPPORTED_C:
                return False
            if not _expand_factor(mod, width):
                if len(layers) > _BWD_MAX_LAYERS[width] or any(l.in_features != width or l.out_features != width for l in layers):
                    return False
    io = _io_dims(mod, layers)
    if io is not None and (io[1] or io[2]):
        if io[0] not in _SUPPORTED_C or width != layers[0].in_features:
            return False
    else:
        if width not in _SUPPORTED_C:
            return False
        if not _expand_factor(mod, width) and any(l.in_features != width or l.out_features != width for l in layers):
            return False
    return True


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


def _packed_expand(mod, E, cd):
    """Tiles W1[0:C], W2[:,0:C], W1[C:2C], W2[:,C:2C], ... as [2E,C,C] and bias rows b1[0:C], b2, b1[C:2C], 0, ...
    (the layout FLARE_MLP_EXPAND asks for), cached on the module."""
    f1, f2 = mod.fc1, mod.fc2
    key = ("expand", cd, tuple((l.weight.data_ptr(), l.weight._version, None if l.bias is None else l.bias._version)
                               for l in (f1, f2)))
    cache = getattr(mod, "_flare_packed", None)
    if cache is not None and cache[0] == key:
        return cache[1], cache[2]
    Cdim = f1.in_features
    w1 = f1.weight.detach().to(cd).view(E, Cdim, Cdim)                       # [j][hidden row in chunk][in]
    w2 = f2.weight.detach().to(cd).view(Cdim, E, Cdim).permute(1, 0, 2)      # [j][out][hidden col in chunk]
    w = torch.stack([w1, w2], dim=1).reshape(2 * E, Cdim, Cdim).contiguous()
    b = torch.zeros(2 * E, Cdim, dtype=torch.float32, device=w.device)
    if f1.bias is not None:
        b[0::2] = f1.bias.detach().float().view(E, Cdim)
    if f2.bias is not None:
        b[1] = f2.bias.detach().float()
    mod._flare_packed = (key, w, b)
    return w, b


def _packed_io(mod, layers, cd, Cdim, in_dim, out_dim):
    """Tiles of a stack with a narrow first and/or last layer: (w [L,C,C], b [L,C], w_in [C,4] fp32, b_in [C]),
    the narrow last layer zero-padded to C rows; cached on the module."""
    key = ("io", cd, tuple((l.weight.data_ptr(), l.weight._version, None if l.bias is None else l.bias._version) for l in layers))
    cache = getattr(mod, "_flare_packed", None)
    if cache is not None and cache[0] == key:
        return cache[1:]
    dev = layers[0].weight.device
    tiles = layers[1:] if in_dim else layers
    w = torch.zeros(len(tiles), Cdim, Cdim, dtype=cd, device=dev)
    b = torch.zeros(len(tiles), Cdim, dtype=torch.float32, device=dev)
    for i, l in enumerate(tiles):
        w[i, :l.out_features] = l.weight.detach().to(cd)
        if l.bias is not None:
            b[i, :l.out_features] = l.bias.detach().float()
    w_in = b_in = None
    if in_dim:
        w_in = torch.zeros(Cdim, 4, dtype=torch.float32, device=dev)
        w_in[:, :in_dim] = layers[0].weight.detach().float()
        b_in = (layers[0].bias.detach().float().contiguous() if layers[0].bias is not None
                else torch.zeros(Cdim, dtype=torch.float32, device=dev))
    mod._flare_packed = (key, w, b, w_in, b_in)
    return w, b, w_in, b_in


def _fused_mlp_io(x, mod, cd, io, info, norm, out_dtype):
    lib = _lib.load()
    layers, act_mask, add_mask, act = info
    Cdim, in_dim, out_dim = io
    w, b, w_in, b_in = _packed_io(mod, layers, cd, Cdim, in_dim, out_dim)
    in_act = act_mask & 1
    if in_dim:                       # the first layer is not one of the tiles
        act_mask >>= 1
        add_mask >>= 1
    xw = x.shape[-1]
    x2 = x.reshape(-1, xw)
    if x2.stride(-1) != 1 or (not in_dim and (x2.stride(0) % 4 or x2.data_ptr() % 16)):
        x2 = x2.contiguous()
    out_dtype = x.dtype if out_dtype is None else out_dtype
    yw = out_dim if out_dim else Cdim
    y = torch.empty(*x.shape[:-1], yw, dtype=out_dtype, device=x.device)
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L = x2.shape[0], Cdim, w.shape[0]
    d.w_dtype, d.x_dtype, d.y_dtype = _dtype_code(w), _dtype_code(x2), _dtype_code(y)
    d.act, d.act_mask, d.add_mask = act, act_mask, add_mask
    d.x_stride, d.y_stride = x2.stride(0), yw
    gamma, beta = _norm_args(d, norm, x, Cdim)
    with _on_device(x.device):
        rc = lib.flare_mlp_io_fwd(C.byref(d), in_dim, in_act, _ptr(w_in), _ptr(b_in), out_dim, _ptr(x2), _ptr(w), _ptr(b),
                                  _ptr(gamma), _ptr(beta), None, _ptr(y), C.c_void_p(_stream_ptr(x.device)))
    _lib.check(rc, "flare_mlp_io_fwd")
    return y


def _norm_args(d, norm, x, Cdim):
    """Fill the descriptor's norm fields; returns (gamma, beta) fp32 tensors or None."""
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
    return gamma, beta


def fused_mlp(x, mod, cd, norm=None, res=None, out_dtype=None, x_head=0, y_head=0):
    """y = res + mod(norm(x)) in one HIP launch.  x: [..., C]; mod: ResidualMLP or nn.Linear; cd: the
    dtype from compute_dtype(); norm: nn.LayerNorm / nn.RMSNorm / None; res: [..., C] or None.
    x_head / y_head (4 or 8): x is / y comes back head-padded, [..., (C / head) * 16] with every head's channels
    followed by zeros up to 16 columns -- the layout the mixer reads and writes for head dims below 16.
    With gradients enabled the call is differentiable (chain of C x C layers only, see compute_dtype)."""
    if torch.is_grad_enabled():
        if x_head or y_head:
            raise ValueError("head-padded rows have no backward: call under torch.no_grad()")
        sub = _train_subchain(mod)
        if sub is not None:
            # narrow ends: those layers run as torch layers (under the caller's autocast), the chain between them fused
            out_dtype = x.dtype if out_dtype is None else out_dtype
            h, hn = x, norm
            if sub.first is not None:
                if hn is not None and not isinstance(hn, nn.Identity):
                    h, hn = hn(h), None
                h = _NarrowLinearFn.apply(h.reshape(-1, h.shape[-1]), sub.first.weight, sub.first.bias, cd).view(*h.shape[:-1], -1)
                if sub.first_act:
                    h = sub.act_module(h)
            y = _fused_mlp_train(h, sub, cd, hn, None, cd if sub.last is not None else out_dtype)
            if sub.last is not None:
                y = sub.last(y).to(out_dtype)
            return y if res is None else res + y
        return _fused_mlp_train(x, mod, cd, norm, res, out_dtype)
    return _fused_mlp_fwd(x, mod, cd, norm, res, out_dtype, x_head, y_head)


def fused_mlp_pair(x, mod_a, mod_b, cd, norm=None, out_dtype=None):
    """(mod_a(norm(x)), mod_b(norm(x))) as fused_mlp computes them, for two stacks that read the same rows through the
    same norm (a block's k and v projections).  With gradients enabled and both stacks plain chains of C x C layers the
    pair is one autograd node whose backward sums the two gradients of x inside the second launch."""
    if torch.is_grad_enabled() and all(_train_subchain(m) is None and not _expand_factor(m, x.shape[-1]) for m in (mod_a, mod_b)):
        has_norm = norm is not None and not isinstance(norm, nn.Identity)
        gamma = getattr(norm, "weight", None) if has_norm else None
        beta = getattr(norm, "bias", None) if has_norm else None
        wb = []
        for m in (mod_a, mod_b):
            layers = _layers_of(m)[0]
            wb += [l.weight for l in layers] + [l.bias for l in layers]
        return _FusedPairFn.apply(mod_a, mod_b, cd, norm if has_norm else None, out_dtype, x, gamma, beta, *wb)
    return fused_mlp(x, mod_a, cd, norm=norm, out_dtype=out_dtype), fused_mlp(x, mod_b, cd, norm=norm, out_dtype=out_dtype)


def _fused_mlp_fwd(x, mod, cd, norm=None, res=None, out_dtype=None, x_head=0, y_head=0):
    lib = _lib.load()
    info = _layers_of(mod)
    layers, act_mask, add_mask, act = info
    io = _io_dims(mod, layers)
    if io is not None and (io[1] or io[2]):
        y = _fused_mlp_io(x, mod, cd, io, info, norm, out_dtype)
        return y if res is None else res + y
    Cdim = layers[0].in_features
    if x.shape[-1] != (Cdim // x_head * 16 if x_head else Cdim):
        raise ValueError(f"x rows are {x.shape[-1]} wide, expected {Cdim // x_head * 16 if x_head else Cdim}")
    E = _expand_factor(mod, Cdim)
    if E:
        if x_head or y_head:
            raise ValueError("head-padded rows are not available for the expanding two-layer MLP")
        w, b = _packed_expand(mod, E, cd)
        act_mask, add_mask = 1, 0
    else:
        w, b = _packed(mod, layers, cd)
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or x2.stride(0) % 4 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out_dtype = x.dtype if out_dtype is None else out_dtype
    ywidth = Cdim // y_head * 16 if y_head else Cdim
    y = torch.empty(*x.shape[:-1], ywidth, dtype=out_dtype, device=x.device)
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L = x2.shape[0], Cdim, w.shape[0]
    d.flags = (_lib.MLP_EXPAND if E else 0) | ((x_head // 4) << 8) | ((y_head // 4) << 12)
    d.w_dtype, d.x_dtype, d.y_dtype = _dtype_code(w), _dtype_code(x2), _dtype_code(y)
    d.act, d.act_mask, d.add_mask = act, act_mask, add_mask
    d.x_stride, d.y_stride = x2.stride(0), ywidth
    gamma, beta = _norm_args(d, norm, x, Cdim)
    r2 = None
    if res is not None:
        r2 = res.reshape(-1, Cdim)
        if r2.stride(-1) != 1 or r2.stride(0) % 4 or r2.data_ptr() % 16:
            r2 = r2.contiguous()
        d.res_dtype, d.res_stride = _dtype_code(r2), r2.stride(0)
    with _on_device(x.device):
        rc = lib.flare_mlp_fwd(C.byref(d), _ptr(x2), _ptr(w), _ptr(b), _ptr(gamma), _ptr(beta), _ptr(r2), _ptr(y),
                               C.c_void_p(_stream_ptr(x.device)))
    _lib.check(rc, "flare_mlp_fwd")
    return y


# --------------------------------------------------------------------------------------
# training: forward launch + flare_mlp_bwd
# --------------------------------------------------------------------------------------
_IMG_INDEX = {}


def _image_index(Cdim, device):
    """For every 16-bit position of a weight tile's LDS image, the row-major element that sits there (the inverse of
    the formula in include/flare_hip.h): element (row, col) of the tile is the A operand of output row `row`, and
    the kernels read 8 consecutive k-slots per lane."""
    key = (Cdim, str(device))
    idx = _IMG_INDEX.get(key)
    if idx is None:
        sws = {128: 0, 64: 1, 32: 2}[Cdim]
        row = torch.arange(Cdim).view(-1, 1).expand(Cdim, Cdim)
        col = torch.arange(Cdim).view(1, -1).expand(Cdim, Cdim)
        ch, j = col // 8, col % 8
        chunk = 4 * (ch // 4) + 2 * (ch % 2) + j // 4
        pos = row * Cdim + 8 * (chunk ^ ((row % 16) >> sws)) + 4 * ((ch % 4) // 2) + j % 4
        idx = torch.empty(Cdim * Cdim, dtype=torch.long)
        idx[pos.reshape(-1)] = torch.arange(Cdim * Cdim)
        idx = _IMG_INDEX[key] = idx.to(device)
    return idx


def mlp_weight_image(w):
    """[L,C,C] weights ([out][in] per tile) -> the LDS images flare_mlp_bwd loads straight into its weight slots."""
    L, Cdim, _ = w.shape
    return w.reshape(L, Cdim * Cdim)[:, _image_index(Cdim, w.device)].contiguous()


_IMG_INDEX2 = {}


def mlp_weight_images(w):
    """(image of w, image of its transposes) as one gather: the transposed tile's element (row, col) is w[col][row], so
    its image reads w through the same index with row and column swapped.  A training step packs after every
    optimizer update, and on small meshes each saved launch counts."""
    L, Cdim, _ = w.shape
    key = (Cdim, L, str(w.device))
    ix = _IMG_INDEX2.get(key)
    if ix is None:
        idx = _image_index(Cdim, w.device)
        both = torch.stack([idx, (idx % Cdim) * Cdim + idx // Cdim])                     # [2, C*C]
        ix = _IMG_INDEX2[key] = (torch.arange(L, device=w.device).view(1, L, 1), both.view(2, 1, Cdim * Cdim))
    imgs = w.reshape(L, Cdim * Cdim)[ix[0], ix[1]]                                          # [2, L, C*C], contiguous
    return imgs[0], imgs[1]


def _packed_train(mod, layers, cd):
    """(w [L,C,C] for the forward launch, images of the weights and of their transposes for the backward, fp32 biases
    [L,C]), cached on the module until a parameter changes."""
    key = ("train", cd, tuple((l.weight.data_ptr(), l.weight._version, None if l.bias is None else l.bias._version) for l in layers))
    cache = mod.__dict__.get("_flare_packed_train")
    if cache is not None and cache[0] == key:
        return cache[1:]
    w, b = _packed(mod, layers, cd)
    w_img, wt_img = mlp_weight_images(w)
    mod.__dict__["_flare_packed_train"] = (key, w, b, w_img, wt_img)
    return w, b, w_img, wt_img


def _packed_train_expand(mod, E, cd):
    """The same for the expanding two-layer MLP: its 2 E tiles (see _packed_expand) and their transposes as images."""
    f1, f2 = mod.fc1, mod.fc2
    key = ("train-expand", cd, tuple((l.weight.data_ptr(), l.weight._version, None if l.bias is None else l.bias._version)
                                     for l in (f1, f2)))
    cache = mod.__dict__.get("_flare_packed_train")
    if cache is not None and cache[0] == key:
        return cache[1:]
    w, b = _packed_expand(mod, E, cd)
    w_img, wt_img = mlp_weight_images(w)
    mod.__dict__["_flare_packed_train"] = (key, w, b, w_img, wt_img)
    return w, b, w_img, wt_img


def _weight_grads(d, g_out, a_in, want_bias, L=None):
    """dW [L, C(out), C(in)] and db [L, C] (or None) in fp32 from the rows the backward launch left: one pass of
    flare_mlp_wgrad over both row arrays, partial results per token range summed in a fixed order.  g_out, a_in:
    [L,T,C], or [T,C] for an array all L layers share."""
    lib = _lib.load()
    T, Cdim = g_out.shape[-2:]
    L = (g_out.shape[0] if g_out.dim() == 3 else a_in.shape[0]) if L is None else L
    d2 = _lib.FlareMlpDesc()
    d2.T, d2.C, d2.L, d2.w_dtype = T, Cdim, L, d.w_dtype
    d = d2
    parts = C.c_int32(0)
    _lib.check(lib.flare_mlp_wgrad_partials(C.byref(d), C.byref(parts)), "flare_mlp_wgrad_partials")
    dev = g_out.device
    dwp = torch.empty(parts.value, L, Cdim, Cdim, dtype=torch.float32, device=dev)
    dbp = torch.empty(parts.value, L, Cdim, dtype=torch.float32, device=dev) if want_bias else None
    dw = torch.empty(L, Cdim, Cdim, dtype=torch.float32, device=dev)
    db = torch.empty(L, Cdim, dtype=torch.float32, device=dev) if want_bias else None
    with _on_device(dev):
        rc = lib.flare_mlp_wgrad(C.byref(d), _ptr(a_in), T * Cdim if a_in.dim() == 3 else 0,
                                 _ptr(g_out), T * Cdim if g_out.dim() == 3 else 0,
                                 _ptr(dwp), _ptr(dbp), _ptr(dw), _ptr(db), C.c_void_p(_stream_ptr(dev)))
    _lib.check(rc, "flare_mlp_wgrad")
    return dw, db


class _FusedMlpFn(torch.autograd.Function):
    """y = res + chain(norm(x)); parameters are passed as inputs so that autograd routes their gradients:
    (x, res, gamma, beta, w_0 .. w_{L-1}, b_0 .. b_{L-1}) with None where a tensor does not exist."""

    @staticmethod
    def forward(ctx, mod, cd, norm, out_dtype, x, res, gamma, beta, *wb):
        with torch.no_grad():
            y = _fused_mlp_fwd(x, mod, cd, norm=norm, res=res, out_dtype=out_dtype)
        ctx.mod, ctx.cd, ctx.norm = mod, cd, norm
        # res and x one tensor: dy is added to dx inside the kernel.  (Two tensors over the same memory are not
        # enough: one of them may be detached, and then its path carries no gradient.)
        ctx.res_is_x = res is x
        ctx.has_res = res is not None
        ctx.n_wb = len(wb)
        # the backward reads the parameters again (its packed copies are keyed by their versions) instead of saving
        # them: as with a saved tensor, changing one in place between forward and backward is an error
        ctx.versions = tuple(None if t is None else t._version for t in (gamma, beta, *wb))
        ctx.params = (gamma, beta, *wb)
        ctx.save_for_backward(x)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        if ctx.versions != tuple(None if t is None else t._version for t in ctx.params):
            raise RuntimeError("a parameter of the fused MLP was modified in place between its forward and its backward")
        mod, cd, norm = ctx.mod, ctx.cd, ctx.norm
        if _expand_factor(mod, x.shape[-1]):
            return _backward_expand(ctx, dy, x, _expand_factor(mod, x.shape[-1]))
        dx, gsum, dW, db, layers = _chain_backward(mod, cd, norm, x, dy, ctx.res_is_x)
        L = len(layers)
        need = ctx.needs_input_grad            # (mod, cd, norm, out_dtype, x, res, gamma, beta, *wb)
        grads = [None, None, None, None]
        grads.append(dx.view(x.shape) if need[4] else None)
        grads.append(None if (not ctx.has_res or ctx.res_is_x or not need[5]) else dy)
        grads += _norm_grads(norm, gsum, need[6], need[7])
        for i, l in enumerate(layers):
            grads.append(dW[i].to(l.weight.dtype) if need[8 + i] else None)
        for i, l in enumerate(layers):
            grads.append(db[i].to(l.bias.dtype) if (l.bias is not None and need[8 + L + i]) else None)
        return tuple(grads)


def _norm_grads(norm, gsum, need_gamma, need_beta):
    if gsum is None:
        return [None, None]
    return [gsum[0].to(norm.weight.dtype) if need_gamma else None,
            gsum[1].to(norm.bias.dtype) if (need_beta and getattr(norm, "bias", None) is not None) else None]


def _chain_backward(mod, cd, norm, x, dy, res_is_x, dx_acc=None):
    """Backward of y = [x +] chain(norm(x)) for the chain of C x C layers: (dx [T,C], the norm's [2,C] sums or None,
    dW [L,out,in], db [L,C] or None, the layers).  dx_acc: a [T,C] gradient of the same x that another chain left
    (x's dtype, contiguous); the kernel adds its result into it and it is returned as dx."""
    lib = _lib.load()
    layers, act_mask, add_mask, act = _layers_of(mod)
    L = len(layers)
    Cdim = x.shape[-1]
    _, b, w_img, wt_img = _packed_train(mod, layers, cd)
    x2 = x.reshape(-1, Cdim)
    if x2.stride(-1) != 1 or x2.stride(0) % 4 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    dy2 = _rows2d(dy, Cdim)
    T = x2.shape[0]
    dev = x.device
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L = T, Cdim, L
    d.w_dtype, d.x_dtype, d.y_dtype = _dtype_code(w_img), _dtype_code(x2), _dtype_code(dy2)
    d.act, d.act_mask, d.add_mask = act, act_mask, add_mask
    d.x_stride, d.y_stride = x2.stride(0), dy2.stride(0)
    gamma, beta = _norm_args(d, norm, x, Cdim)
    if dx_acc is not None and (dx_acc.shape != (T, Cdim) or dx_acc.dtype != x2.dtype or not dx_acc.is_contiguous()):
        raise ValueError("dx_acc must be a contiguous [T, C] tensor of x's dtype")
    dx = dx_acc if dx_acc is not None else torch.empty(T, Cdim, dtype=x2.dtype, device=dev)
    a_in = torch.empty(L, T, Cdim, dtype=cd, device=dev)
    g_out = torch.empty(L, T, Cdim, dtype=cd, device=dev)
    dn = stats = gb = gsum = None
    any_bias = any(l.bias is not None for l in layers)
    if d.norm:
        rows = C.c_int32(0)
        _lib.check(lib.flare_mlp_bwd_partial_rows(C.byref(d), C.byref(rows)), "flare_mlp_bwd_partial_rows")
        dn = torch.empty(T, Cdim, dtype=cd, device=dev)
        stats = torch.empty(T, 2, dtype=torch.float32, device=dev)
        gb = torch.empty(rows.value, 2, Cdim, dtype=torch.float32, device=dev)
        gsum = torch.empty(2, Cdim, dtype=torch.float32, device=dev)
    bits = (_lib.MLP_BWD_ADD_DY if res_is_x else 0) | (_lib.MLP_BWD_ACCUMULATE if dx_acc is not None else 0)
    with _on_device(dev):
        rc = lib.flare_mlp_bwd(C.byref(d), _ptr(x2), _ptr(dy2), _ptr(w_img), _ptr(wt_img), _ptr(b), _ptr(gamma), _ptr(beta),
                               bits, _ptr(dx), _ptr(a_in), _ptr(g_out), _ptr(dn), _ptr(stats), _ptr(gb),
                               _ptr(gsum), C.c_void_p(_stream_ptr(dev)))
    _lib.check(rc, "flare_mlp_bwd")
    # weight and bias gradients: one more launch over the rows the kernel left (16-bit products with fp32
    # accumulation, as torch runs a Linear's backward under autocast); norm gradients: partial rows, summed by the launch
    dW, db = _weight_grads(d, g_out, a_in, any_bias)                 # [L, out, in], [L, C] fp32
    return dx, gsum, dW, db, layers


class _FusedPairFn(torch.autograd.Function):
    """(ya, yb) = (chain_a(norm(x)), chain_b(norm(x))): two chains that read the same rows through the same norm (the k
    and v projections of a block).  Forward: the two launches of _FusedMlpFn.  Backward: the second chain's launch adds
    its gradient of x into the first one's, which autograd would otherwise do with a launch of its own over three
    [T, C] arrays.  Inputs: (x, gamma, beta, weights and biases of a, weights and biases of b)."""

    @staticmethod
    def forward(ctx, mod_a, mod_b, cd, norm, out_dtype, x, gamma, beta, *wb):
        with torch.no_grad():
            ya = _fused_mlp_fwd(x, mod_a, cd, norm=norm, out_dtype=out_dtype)
            yb = _fused_mlp_fwd(x, mod_b, cd, norm=norm, out_dtype=out_dtype)
        ctx.mods, ctx.cd, ctx.norm = (mod_a, mod_b), cd, norm
        ctx.versions = tuple(None if t is None else t._version for t in (gamma, beta, *wb))
        ctx.params = (gamma, beta, *wb)
        ctx.save_for_backward(x)
        return ya, yb

    @staticmethod
    @once_differentiable
    def backward(ctx, dya, dyb):
        (x,) = ctx.saved_tensors
        if ctx.versions != tuple(None if t is None else t._version for t in ctx.params):
            raise RuntimeError("a parameter of the fused MLP was modified in place between its forward and its backward")
        mod_a, mod_b = ctx.mods
        dx, gs_a, dWa, dba, la = _chain_backward(mod_a, ctx.cd, ctx.norm, x, dya, False)
        dx, gs_b, dWb, dbb, lb = _chain_backward(mod_b, ctx.cd, ctx.norm, x, dyb, False, dx_acc=dx)
        need = ctx.needs_input_grad            # (mod_a, mod_b, cd, norm, out_dtype, x, gamma, beta, *wb)
        grads = [None, None, None, None, None, dx.view(x.shape) if need[5] else None]
        grads += _norm_grads(ctx.norm, None if gs_a is None else gs_a + gs_b, need[6], need[7])
        at = 8
        for layers, dW, db in ((la, dWa, dba), (lb, dWb, dbb)):
            n = len(layers)
            for i, l in enumerate(layers):
                grads.append(dW[i].to(l.weight.dtype) if need[at + i] else None)
            for i, l in enumerate(layers):
                grads.append(db[i].to(l.bias.dtype) if (l.bias is not None and need[at + n + i]) else None)
            at += 2 * n
        return tuple(grads)


def _rows2d(t, Cdim):
    t2 = t.reshape(-1, Cdim)
    if t2.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        t2 = t2.float()
    if t2.stride(-1) != 1 or t2.stride(0) % 4 or t2.data_ptr() % 16:
        t2 = t2.contiguous()
    return t2


def _backward_expand(ctx, dy, x, E):
    """Backward of y = res + fc2(act(fc1(norm(x)))) with hidden width E C: flare_mlp_expand_bwd, then two passes of
    flare_mlp_wgrad (dW1, db1 from the rows dt against n; dW2, db2 from dy against the rows h)."""
    mod, cd, norm = ctx.mod, ctx.cd, ctx.norm
    lib = _lib.load()
    _, _, _, act = _layers_of(mod)
    f1, f2 = mod.fc1, mod.fc2
    Cdim = x.shape[-1]
    _, b, w_img, wt_img = _packed_train_expand(mod, E, cd)
    x2, dy2 = _rows2d(x, Cdim), _rows2d(dy, Cdim)
    T = x2.shape[0]
    dev = x.device
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L, d.flags = T, Cdim, 2 * E, _lib.MLP_EXPAND
    d.w_dtype, d.x_dtype, d.y_dtype = _dtype_code(w_img), _dtype_code(x2), _dtype_code(dy2)
    d.act, d.act_mask, d.add_mask = act, 1, 0
    d.x_stride, d.y_stride = x2.stride(0), dy2.stride(0)
    gamma, beta = _norm_args(d, norm, x, Cdim)
    dx = torch.empty(T, Cdim, dtype=x2.dtype, device=dev)
    n_row = torch.empty(T, Cdim, dtype=cd, device=dev)
    dy_row = torch.empty(T, Cdim, dtype=cd, device=dev)
    h = torch.empty(E, T, Cdim, dtype=cd, device=dev)
    dt = torch.empty(E, T, Cdim, dtype=cd, device=dev)
    dn = stats = gb = gsum = None
    if d.norm:
        rows = C.c_int32(0)
        _lib.check(lib.flare_mlp_bwd_partial_rows(C.byref(d), C.byref(rows)), "flare_mlp_bwd_partial_rows")
        dn = torch.empty(T, Cdim, dtype=cd, device=dev)
        stats = torch.empty(T, 2, dtype=torch.float32, device=dev)
        gb = torch.empty(rows.value, 2, Cdim, dtype=torch.float32, device=dev)
        gsum = torch.empty(2, Cdim, dtype=torch.float32, device=dev)
    with _on_device(dev):
        rc = lib.flare_mlp_expand_bwd(C.byref(d), _ptr(x2), _ptr(dy2), _ptr(w_img), _ptr(wt_img), _ptr(b), _ptr(gamma), _ptr(beta),
                                      1 if ctx.res_is_x else 0, _ptr(dx), _ptr(n_row), _ptr(dy_row), _ptr(h), _ptr(dt),
                                      _ptr(dn), _ptr(stats), _ptr(gb), _ptr(gsum), C.c_void_p(_stream_ptr(dev)))
    _lib.check(rc, "flare_mlp_expand_bwd")
    dW1, db1 = _weight_grads(d, dt, n_row, f1.bias is not None)          # [E, C(hidden chunk), C(in)], [E, C]
    dW2, db2 = _weight_grads(d, dy_row, h, f2.bias is not None, L=E)     # [E, C(out), C(hidden chunk)], [E, C] (E equal rows)
    need = ctx.needs_input_grad            # (mod, cd, norm, out_dtype, x, res, gamma, beta, w1, w2, b1, b2)
    grads = [None, None, None, None]
    grads.append(dx.view(x.shape) if need[4] else None)
    grads.append(None if (not ctx.has_res or ctx.res_is_x or not need[5]) else dy)
    if d.norm:
        grads.append(gsum[0].to(norm.weight.dtype) if need[6] else None)
        grads.append(gsum[1].to(norm.bias.dtype) if (need[7] and getattr(norm, "bias", None) is not None) else None)
    else:
        grads += [None, None]
    grads.append(dW1.reshape(E * Cdim, Cdim).to(f1.weight.dtype) if need[8] else None)
    grads.append(dW2.permute(1, 0, 2).reshape(Cdim, E * Cdim).to(f2.weight.dtype) if need[9] else None)
    grads.append(db1.reshape(E * Cdim).to(f1.bias.dtype) if (f1.bias is not None and need[10]) else None)
    grads.append(db2[0].to(f2.bias.dtype) if (f2.bias is not None and need[11]) else None)
    return tuple(grads)


def _fused_mlp_train(x, mod, cd, norm, res, out_dtype):
    layers = _layers_of(mod)[0]
    has_norm = norm is not None and not isinstance(norm, nn.Identity)
    gamma = getattr(norm, "weight", None) if has_norm else None
    beta = getattr(norm, "bias", None) if has_norm else None
    wb = [l.weight for l in layers] + [l.bias for l in layers]
    return _FusedMlpFn.apply(mod, cd, norm if has_norm else None, out_dtype, x, res, gamma, beta, *wb)
