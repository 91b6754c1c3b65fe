"""CPU oracle for the FLARE hot path — TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  Nothing under the product package imports it, and the product never falls back
to it: when the HIP library is missing the product raises.

Every function restates, in plain torch on the CPU, the arithmetic of one reference
function (paths relative to the reference tree):

  mixer_sdpa            README.md:39-52; pdebench/models/flare.py:136-138 (fused branch)
  mixer_explicit        pdebench/models/flare.py:142-150 (spelled-out branch; note that the
                        reference omits attn_scale there, this restatement applies it so
                        that it equals the fused branch for every scale)
  mixer_masked_explicit lra/models/backends.py:603-606,615-622 (key mask for the gather;
                        the scatter mask hits whole query rows, for which torch's result
                        is backend dependent — this oracle defines those rows as 0)
  triple_einsum         lra/models/backends.py:1285-1292 == lra/models/triton/triple.py:846-860
  elu_plus_one          lra/models/kernels.py:23-24
  causal_*              the reference has NO code for causal FLARE (README.md:60 links a blog
                        post).  The definition adopted is the causal restriction of the
                        mixer: z_t = softmax over tokens <= t, y_t = softmax_m(k_t q_m) z_t.
                        causal_recurrent follows the token recurrence shape of
                        lra/models/triton/causal_linear.py:317-336; causal_bruteforce applies
                        mixer_explicit to every prefix and keeps the last row.

  residual_mlp          pdebench/models/flare.py:45-59 (ResidualMLP.forward) with the pre-norm and
                        outer residual of FLAREBlock.forward :204-215
  causal_linear_*       lra/models/triton/causal_linear.py:317-336 (token recurrence, k and v
                        each scaled by N^-1/2) and :338-389 (chunked form)
  rope_reference        lra/models/embeddings.py:103-147 (rotary embedding applied to k, backends.py:600-601)
  flare_layer / flare_block / flare_model
                        pdebench/models/flare.py:122-156 (FLARE.forward), :204-215 (FLAREBlock.forward),
                        :337-349 (FLAREModel.forward) as functions of a state_dict with the reference's
                        key names; composed of mixer_explicit and residual_mlp only

Pinning status (what each function is checked against in tests/test_oracle.py):
  mixer_sdpa / mixer_explicit : each other (independent code paths: torch's SDPA kernel vs
      explicit softmax), the C restatement oracle/flare_oracle.c, closed forms (q=0 => mean,
      N=1 => y=v, M=1 => rows equal z_0, convex-hull bounds, shift invariance,
      permutation equivariance) and a pure-Python-float brute force.  The reference's own
      tests hold no golden values for this path, so none are used.
  causal_recurrent            : causal_bruteforce, last-row == non-causal mixer, chunk
      independence; C restatement.
  triple_einsum               : hand cases (N=1, D=1), pure-Python loops, linearity in v,
      (k1,q1)<->(k2,q2) symmetry; C restatement.
  residual_mlp                : torch's own nn.Linear / nn.GELU(approximate='tanh') / nn.SiLU /
      nn.LayerNorm / nn.RMSNorm modules carrying the same weights, and the erf-free closed form of
      tanh-GELU at a few points.
  flare_layer / flare_block / flare_model : compositions of the pinned functions above; the composition
      itself (norm and residual placement, head split 'b n (h d) -> b h n d', latent_q.view(H, M, D)) against
      torch.nn modules assembled in the test from nn.Linear / nn.LayerNorm and F.scaled_dot_product_attention.
  rope_reference              : position 0 is the identity; D = 2 is the plane rotation by p radians; a D = 4
      vector worked out by hand from the text of embeddings.py:136-147; linearity in x.
  causal_linear_recurrent     : the closed form tril(Q K^T) V / N, the chunked form for several
      chunk sizes, a pure-Python-float brute force, last row == non-causal linear attention.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# --------------------------------------------------------------------------------------
# mixer
# --------------------------------------------------------------------------------------
def mixer_sdpa(q, k, v, scale=1.0):
    """y = SDPA(k, q, SDPA(q, k, v)) on the torch MATH backend (README.md:49-50)."""
    from torch.nn.attention import SDPBackend, sdpa_kernel

    B = k.shape[0]
    qe = q.unsqueeze(0).expand(B, -1, -1, -1) if q.dim() == 3 else q
    with sdpa_kernel(SDPBackend.MATH):
        z = F.scaled_dot_product_attention(qe, k, v, scale=scale)
        y = F.scaled_dot_product_attention(k, qe, z, scale=scale)
    return y, z


def gather_explicit(q, k, v, scale=1.0, key_mask=None, dtype=torch.float64):
    """z = softmax_n(s q k^T) v, plus lse = log sum_n exp(s q k^T)."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    if q.dim() == 3:
        q = q.unsqueeze(0)
    scores = scale * (q @ k.transpose(-2, -1))  # [B,H,M,N]
    if key_mask is not None:
        keep = key_mask.to(torch.bool)[:, None, None, :]
        scores = scores.masked_fill(~keep, NEG_INF)
    lse = torch.logsumexp(scores, dim=-1)
    w = torch.exp(scores - lse.unsqueeze(-1))
    w = torch.nan_to_num(w, nan=0.0)  # latents whose every key is masked: z = 0
    z = w @ v
    return z, lse


def scatter_explicit(q, k, z, scale=1.0, key_mask=None, dtype=torch.float64):
    """y = softmax_m(s k q^T) z; rows of masked tokens are 0."""
    q, k, z = q.to(dtype), k.to(dtype), z.to(dtype)
    if q.dim() == 3:
        q = q.unsqueeze(0)
    scores = scale * (k @ q.transpose(-2, -1))  # [B,H,N,M]
    y = torch.softmax(scores, dim=-1) @ z
    if key_mask is not None:
        y = y * key_mask.to(dtype)[:, None, :, None]
    return y


def mixer_explicit(q, k, v, scale=1.0, key_mask=None, dtype=torch.float64):
    z, _ = gather_explicit(q, k, v, scale, key_mask, dtype)
    y = scatter_explicit(q, k, z, scale, key_mask, dtype)
    return y, z


def mixer_bruteforce_py(q, k, v, scale=1.0):
    """Pure-Python-float loops; tiny shapes only.  q [H,M,D], k,v [B,H,N,D] as nested lists
    or tensors.  Returns y as a nested list [B][H][N][D]."""
    q = q.tolist() if hasattr(q, "tolist") else q
    k = k.tolist() if hasattr(k, "tolist") else k
    v = v.tolist() if hasattr(v, "tolist") else v
    B, H, N, D, M = len(k), len(k[0]), len(k[0][0]), len(k[0][0][0]), len(q[0])
    out = []
    for b in range(B):
        ob = []
        for h in range(H):
            s = [[scale * sum(q[h][m][d] * k[b][h][n][d] for d in range(D)) for n in range(N)]
                 for m in range(M)]
            z = []
            for m in range(M):
                mx = max(s[m])
                e = [math.exp(x - mx) for x in s[m]]
                tot = sum(e)
                z.append([sum(e[n] * v[b][h][n][d] for n in range(N)) / tot for d in range(D)])
            rows = []
            for n in range(N):
                col = [s[m][n] for m in range(M)]
                mx = max(col)
                e = [math.exp(x - mx) for x in col]
                tot = sum(e)
                rows.append([sum(e[m] * z[m][d] for m in range(M)) / tot for d in range(D)])
            ob.append(rows)
        out.append(ob)
    return out


# --------------------------------------------------------------------------------------
# causal FLARE
# --------------------------------------------------------------------------------------
def causal_fresh_state(B, H, M, D, dtype=torch.float64):
    mu = torch.full((B, H, M), NEG_INF, dtype=dtype)
    den = torch.zeros((B, H, M), dtype=dtype)
    num = torch.zeros((B, H, M, D), dtype=dtype)
    return mu, den, num


def causal_recurrent(q, k, v, scale=1.0, state=None, dtype=torch.float64):
    """Token-by-token recurrence.  Returns (y [B,H,N,D], (mu, den, num))."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    B, H, N, D = k.shape
    M = q.shape[-2]
    if state is None:
        mu, den, num = causal_fresh_state(B, H, M, D, dtype)
    else:
        mu, den, num = (s.to(dtype).clone() for s in state)
        mu = torch.where(mu <= -1e30, torch.full_like(mu, NEG_INF), mu)
    y = torch.empty(B, H, N, D, dtype=dtype)
    for t in range(N):
        sigma = scale * torch.einsum("hmd,bhd->bhm", q, k[:, :, t])
        mu_new = torch.maximum(mu, sigma)
        a = torch.exp(mu - mu_new)
        a = torch.nan_to_num(a, nan=0.0)  # (-inf) - (-inf) on the first token
        p = torch.exp(sigma - mu_new)
        den = a * den + p
        num = a.unsqueeze(-1) * num + p.unsqueeze(-1) * v[:, :, t].unsqueeze(-2)
        mu = mu_new
        w = torch.softmax(sigma, dim=-1)
        y[:, :, t] = torch.einsum("bhm,bhmd->bhd", w, num / den.unsqueeze(-1))
    return y, (mu, den, num)


def causal_bruteforce(q, k, v, scale=1.0, dtype=torch.float64):
    """Row t of the non-causal mixer applied to the prefix [0..t]; O(N^2 M)."""
    B, H, N, D = k.shape
    y = torch.empty(B, H, N, D, dtype=dtype)
    for t in range(N):
        yt, _ = mixer_explicit(q, k[:, :, : t + 1], v[:, :, : t + 1], scale, dtype=dtype)
        y[:, :, t] = yt[:, :, t]
    return y


def causal_state_invariants(mu, den, num):
    """The shift-invariant content of a state: z = num/den and lse = mu + log den."""
    return num / den.unsqueeze(-1), mu + torch.log(den)


# --------------------------------------------------------------------------------------
# token-wise MLP stack (ResidualMLP, norm, residual)
# --------------------------------------------------------------------------------------
def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def residual_mlp(x, weights, biases, act="gelu", input_residual=True, output_residual=True,
                 norm=None, gamma=None, beta=None, eps=1e-5, res=None, dtype=torch.float64):
    """res + ResidualMLP(norm(x)) following pdebench/models/flare.py:45-59: fc1 -> act,
    (+ input if input_residual), n x (x + act(fc x)), fc2 (+ x if output_residual).  A single
    weight is the num_layers == -1 case (one Linear, residual iff both flags).
    norm: None | 'layer' | 'rms'."""
    f = gelu_tanh if act == "gelu" else (lambda t: t * torch.sigmoid(t))
    x = x.to(dtype)
    ws = [w.to(dtype) for w in weights]
    bs = [None if b is None else b.to(dtype) for b in biases]
    lin = lambda t, i: t @ ws[i].T + (0 if bs[i] is None else bs[i])
    if norm == "layer":
        mu = x.mean(-1, keepdim=True)
        var = ((x - mu) ** 2).mean(-1, keepdim=True)
        x = (x - mu) / torch.sqrt(var + eps)
    elif norm == "rms":
        x = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)
    if norm is not None:
        if gamma is not None:
            x = x * gamma.to(dtype)
        if beta is not None:
            x = x + beta.to(dtype)
    if len(ws) == 1:
        h = lin(x, 0)
        out = x + h if (input_residual and output_residual) else h
    else:
        h = f(lin(x, 0))
        x = x + h if input_residual else h
        for i in range(1, len(ws) - 1):
            x = x + f(lin(x, i))
        h = lin(x, len(ws) - 1)
        out = x + h if output_residual else h
    return out if res is None else res.to(dtype) + out


# --------------------------------------------------------------------------------------
# rotary embedding of the sequence models
# --------------------------------------------------------------------------------------
def rope_reference(x, base=10000.0):
    """lra/models/embeddings.py:103-147 element by element: for position p and channel j of x [..., N, D],
    out[p, j] = x[p, j] cos(p w_j) + r[p, j] sin(p w_j) with w_j = base^(-(j // 2) / (D / 2)) and the partner
    r[j] = -x[2 j + 1] for j < D/2, x[2 (j - D/2)] for j >= D/2 (the reference concatenates the negated odd
    channels and the even channels; it does not interleave them)."""
    x = x.double()
    N, D = x.shape[-2], x.shape[-1]
    out = torch.empty_like(x)
    for j in range(D):
        w = base ** (-(j // 2) / (D // 2))
        ang = torch.arange(N, dtype=torch.float64) * w
        r = -x[..., 2 * j + 1] if j < D // 2 else x[..., 2 * (j - D // 2)]
        out[..., j] = x[..., j] * torch.cos(ang) + r * torch.sin(ang)
    return out


# --------------------------------------------------------------------------------------
# FLARE layer, block and model as functions of a state_dict (reference key names)
# --------------------------------------------------------------------------------------
def _mlp_params(sd, prefix):
    """Weights and biases of the ResidualMLP stored under `prefix` (fc1, fcs.i, fc2; or the single fc)."""
    if prefix + "fc.weight" in sd:
        return [sd[prefix + "fc.weight"]], [sd.get(prefix + "fc.bias")]
    names = ["fc1"]
    i = 0
    while f"{prefix}fcs.{i}.weight" in sd:
        names.append(f"fcs.{i}")
        i += 1
    names.append("fc2")
    return [sd[prefix + n + ".weight"] for n in names], [sd.get(prefix + n + ".bias") for n in names]


def _mlp(sd, prefix, x, act, input_residual, output_residual):
    """ResidualMLP (flare.py:24-59): a residual flag only takes effect when the widths match."""
    ws, bs = _mlp_params(sd, prefix)
    if len(ws) > 1:
        input_residual = input_residual and ws[0].shape[1] == ws[0].shape[0]
        output_residual = output_residual and ws[-1].shape[1] == ws[-1].shape[0]
    else:
        input_residual = output_residual = input_residual and output_residual and ws[0].shape[0] == ws[0].shape[1]
    return residual_mlp(x, ws, bs, act, input_residual, output_residual)


def _norm(sd, prefix, x, rmsnorm, eps):
    """nn.LayerNorm (eps 1e-5) or nn.RMSNorm (eps=None: machine epsilon of the input type) over the last axis."""
    x = x.double()
    w = sd[prefix + "weight"].double()
    if rmsnorm:
        e = torch.finfo(torch.float32).eps if eps is None else eps
        return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + e) * w
    e = 1e-5 if eps is None else eps
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + e) * w + sd[prefix + "bias"].double()


def flare_layer(sd, prefix, x, num_heads, act="gelu", attn_scale=1.0, qk_norm=False, rmsnorm=False, key_mask=None,
                rope=None):
    """FLARE.forward (flare.py:122-156): k, v = MLPs of x split into heads, q = latent_q.view(H, M, D),
    y = out_proj(merge heads(mixer(q, k, v))).  key_mask [B,N] (True = real token) and rope (a function of k)
    give the sequence variant lra/models/backends.py:588-622: padded keys are left out of the gather, rope turns k only."""
    B, N, Cdim = x.shape
    H = num_heads
    D = Cdim // H
    q = sd[prefix + "latent_q"].double().reshape(H, -1, D)                       # view(H, M, D) of the [C, M] parameter
    k = _mlp(sd, prefix + "k_proj.", x, act, True, True).reshape(B, N, H, D).permute(0, 2, 1, 3)
    v = _mlp(sd, prefix + "v_proj.", x, act, True, True).reshape(B, N, H, D).permute(0, 2, 1, 3)
    if qk_norm:
        q = _norm(sd, prefix + "q_norm.", q, rmsnorm, None)
        k = _norm(sd, prefix + "k_norm.", k, rmsnorm, None)
    if rope is not None:
        k = rope(k)
    y, _ = mixer_explicit(q, k, v, attn_scale, key_mask, dtype=torch.float64)
    y = y.permute(0, 2, 1, 3).reshape(B, N, Cdim)
    return y @ sd[prefix + "out_proj.weight"].double().T + sd[prefix + "out_proj.bias"].double()


def flare_block(sd, prefix, x, num_heads, act="gelu", attn_scale=1.0, qk_norm=False, rmsnorm=False, key_mask=None,
                rope=None):
    """FLAREBlock.forward (flare.py:204-215; lra/models/backends.py:665-672 with attention_mask):
    x += att(norm1(x)); x += mlp(norm2(x))."""
    x = x.double()
    x = x + flare_layer(sd, prefix + "att.", _norm(sd, prefix + "norm1.", x, rmsnorm, None), num_heads, act,
                        attn_scale, qk_norm, rmsnorm, key_mask, rope)
    return x + _mlp(sd, prefix + "mlp.", _norm(sd, prefix + "norm2.", x, rmsnorm, None), act, True, True)


def flare_model(sd, x, num_heads, num_blocks, act="gelu", attn_scale=1.0, qk_norm=False, rmsnorm=False,
                out_proj_norm=True):
    """FLAREModel.forward (flare.py:337-349; layers built at :274-318): in_proj (output residual only), the blocks,
    then norm + out MLP (input residual only)."""
    x = _mlp(sd, "in_proj.", x.double(), act, False, True)
    for b in range(num_blocks):
        x = flare_block(sd, f"blocks.{b}.", x, num_heads, act, attn_scale, qk_norm, rmsnorm)
    if out_proj_norm:
        x = _norm(sd, "out_proj.0.", x, rmsnorm, None)
    return _mlp(sd, "out_proj.1.", x, act, True, False)


# --------------------------------------------------------------------------------------
# causal linear attention
# --------------------------------------------------------------------------------------
def causal_linear_recurrent(q, k, v, dtype=torch.float64):
    """Token recurrence of lra/models/triton/causal_linear.py:317-336:
    S += (v_t N^-1/2)(k_t N^-1/2)^T ;  y_t = S q_t."""
    B, H, N, Dk = k.shape
    Dv = v.shape[-1]
    scale = N ** -0.5
    q, k, v = q.to(dtype), k.to(dtype) * scale, v.to(dtype) * scale
    S = torch.zeros(B, H, Dv, Dk, dtype=dtype)
    y = torch.zeros(B, H, N, Dv, dtype=dtype)
    for t in range(N):
        S = S + v[:, :, t, :, None] * k[:, :, t, None, :]
        y[:, :, t] = (S @ q[:, :, t, :, None])[..., 0]
    return y


def causal_linear_closed_form(q, k, v, dtype=torch.float64):
    """y = tril(Q K^T) V / N  (the definition the recurrence unrolls to)."""
    N = k.shape[2]
    a = torch.tril(q.to(dtype) @ k.to(dtype).mT)
    return a @ v.to(dtype) / N


def causal_linear_chunked(q, k, v, chunk=128, dtype=torch.float64):
    """Chunked form of lra/models/triton/causal_linear.py:338-389: exclusive prefix of the
    per-chunk states for the inter-chunk term, masked Q K^T for the intra-chunk term."""
    B, H, N, Dk = k.shape
    scale = N ** -0.5
    q, k, v = q.to(dtype), k.to(dtype) * scale, v.to(dtype) * scale
    out = []
    S = torch.zeros(B, H, Dk, v.shape[-1], dtype=dtype)
    for n0 in range(0, N, chunk):
        qc, kc, vc = q[:, :, n0:n0 + chunk], k[:, :, n0:n0 + chunk], v[:, :, n0:n0 + chunk]
        out.append(qc @ S + torch.tril(qc @ kc.mT) @ vc)
        S = S + kc.mT @ vc
    return torch.cat(out, 2)


def causal_linear_bruteforce_py(q, k, v):
    """Pure-Python floats, one (b,h): q,k [N][Dk], v [N][Dv] nested lists."""
    N = len(k)
    y = []
    for t in range(N):
        row = [0.0] * len(v[0])
        for tau in range(t + 1):
            s = sum(a * b for a, b in zip(q[t], k[tau]))
            for j in range(len(row)):
                row[j] += s * v[tau][j] / N
        y.append(row)
    return y


# --------------------------------------------------------------------------------------
# triple attention
# --------------------------------------------------------------------------------------
def elu_plus_one(x):
    return F.elu(x) + 1.0


def triple_einsum(q1, q2, k1, k2, v, feature_map=False, normalize=False, dtype=torch.float32):
    """state = einsum(k1, v, k2)/N, out = einsum(q1, state, q2) (backends.py:1288-1291).

    The reference divides each of k1, k2, v by N**(1/3) in fp32; the product of the three
    factors is the 1/N used here (triple.py:368 applies 1/N in one piece as well)."""
    out_dtype = q1.dtype
    q1, q2, k1, k2, v = (t.to(dtype) for t in (q1, q2, k1, k2, v))
    if feature_map:
        q1, q2, k1, k2 = (elu_plus_one(t) for t in (q1, q2, k1, k2))
    N = q1.shape[-2]
    state = torch.einsum("bhni,bhnj,bhnk->bhijk", k1, v, k2) / N
    out = torch.einsum("bhni,bhijk,bhnk->bhnj", q1, state, q2)
    if normalize:
        kk = torch.einsum("bhni,bhnk->bhik", k1, k2) / N
        den = torch.einsum("bhni,bhik,bhnk->bhn", q1, kk, q2)
        out = out / den.unsqueeze(-1)
    return state, out.to(out_dtype) if dtype == torch.float32 else out


def triple_reference_scaling(q1, q2, k1, k2, v):
    """Literal restatement of backends.py:1288-1291 including the three N**(1/3) divisions
    (used to show that the single 1/N of triple_einsum is the same thing)."""
    N = q1.size(-2)
    k1, k2, v = [t.to(torch.float32) / (N ** (1 / 3)) for t in (k1, k2, v)]
    state = torch.einsum("bhni,bhnj,bhnk->bhijk", k1, v, k2)
    out = torch.einsum("bhni,bhijk,bhnk->bhnj", q1.to(torch.float32), state, q2.to(torch.float32))
    return state, out.to(q1.dtype)


# --------------------------------------------------------------------------------------
# helpers shared by tests and bench
# --------------------------------------------------------------------------------------
def rel_l2(a, b):
    a = a.detach().to(torch.float64).cpu()
    b = b.detach().to(torch.float64).cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))
