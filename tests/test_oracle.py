"""Pins the CPU oracle (oracle/flare_oracle.py and oracle/flare_oracle.c) WITHOUT the product.

The reference's tests hold no golden values for this path, so the oracle is pinned by
independent restatements against each other (torch SDPA kernel / explicit softmax / plain C /
pure-Python floats) and by what the mathematics fixes (closed forms and invariants chosen so
that a dropped scale, a softmax over the wrong axis, a transposed operand or a wrong index
fails at least one of them).
"""
import math

import pytest
import torch

from oracle import c_oracle
from oracle import flare_oracle as O


def _rand(B=2, H=3, N=37, M=5, D=4, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(H, M, D, generator=g, dtype=dtype) * D ** -0.5
    k = torch.randn(B, H, N, D, generator=g, dtype=dtype)
    v = torch.randn(B, H, N, D, generator=g, dtype=dtype)
    return q, k, v


# ---------------------------------------------------------------- mixer
@pytest.mark.parametrize("scale", [1.0, 0.37])
def test_mixer_sdpa_vs_explicit_vs_c(scale):
    q, k, v = _rand(dtype=torch.float32)
    y1, z1 = O.mixer_sdpa(q, k, v, scale)
    y2, z2 = O.mixer_explicit(q, k, v, scale)
    y3, z3 = c_oracle.mixer(q, k, v, scale)
    assert O.rel_l2(y1, y2) < 2e-6 and O.rel_l2(z1, z2) < 2e-6
    assert O.rel_l2(y3, y2) < 2e-7 and O.rel_l2(z3, z2) < 2e-7


def test_mixer_bruteforce_python_floats():
    q, k, v = _rand(B=1, H=2, N=6, M=3, D=2)
    y, _ = O.mixer_explicit(q, k, v, 0.8)
    yb = torch.tensor(O.mixer_bruteforce_py(q, k, v, 0.8), dtype=torch.float64)
    assert O.rel_l2(y, yb) < 1e-13


def test_mixer_cfg1_shape_sdpa_vs_explicit():
    # BASELINE config 1: q[8,64,16]~N(0,1/D), k,v[1,8,4096,16]~N(0,1), scale 1, fp32
    g = torch.Generator().manual_seed(0)
    q = torch.randn(8, 64, 16, generator=g) * 16 ** -0.5
    k = torch.randn(1, 8, 4096, 16, generator=g)
    v = torch.randn(1, 8, 4096, 16, generator=g)
    y1, _ = O.mixer_sdpa(q, k, v, 1.0)
    y2, _ = O.mixer_explicit(q, k, v, 1.0)
    assert O.rel_l2(y1, y2) < 1e-5


def test_mixer_zero_q_gives_mean():
    q, k, v = _rand()
    y, z = O.mixer_explicit(torch.zeros_like(q), k, v)
    mean = v.mean(dim=2, keepdim=True)
    assert torch.allclose(z, mean.expand_as(z), atol=1e-12)
    assert torch.allclose(y, mean.expand_as(y), atol=1e-12)


def test_mixer_single_token_and_single_latent():
    q, k, v = _rand(N=1)
    y, _ = O.mixer_explicit(q, k, v)
    assert torch.allclose(y, v, atol=1e-12)          # N=1: every softmax weight is 1
    q, k, v = _rand(M=1)
    y, z = O.mixer_explicit(q, k, v)
    assert torch.allclose(y, z.expand_as(y), atol=1e-12)  # M=1: every token receives z_0


def test_mixer_convex_hull_and_constant_v():
    q, k, v = _rand()
    y, z = O.mixer_explicit(q, k, v, 2.0)
    lo, hi = v.amin(dim=2, keepdim=True), v.amax(dim=2, keepdim=True)
    assert (y >= lo - 1e-12).all() and (y <= hi + 1e-12).all()
    c = torch.full_like(v, 3.25)
    y, _ = O.mixer_explicit(q, k, c, 2.0)
    assert torch.allclose(y, c, atol=1e-12)


def test_mixer_permutation_equivariance_and_axis():
    q, k, v = _rand()
    perm = torch.randperm(k.shape[2], generator=torch.Generator().manual_seed(1))
    y, z = O.mixer_explicit(q, k, v)
    yp, zp = O.mixer_explicit(q, k[:, :, perm], v[:, :, perm])
    assert torch.allclose(zp, z, atol=1e-12)               # gather is permutation invariant
    assert torch.allclose(yp, y[:, :, perm], atol=1e-12)   # scatter is equivariant
    # a softmax over the wrong axis would break this: duplicating every token leaves z, y unchanged
    y2, z2 = O.mixer_explicit(q, torch.cat([k, k], 2), torch.cat([v, v], 2))
    assert torch.allclose(z2, z, atol=1e-12) and torch.allclose(y2[:, :, : k.shape[2]], y, atol=1e-12)


def test_mixer_scale_is_applied_to_both_softmaxes():
    q, k, v = _rand()
    y1, z1 = O.mixer_explicit(q, k, v, 0.5)
    y2, z2 = O.mixer_explicit(0.5 * q, k, v, 1.0)
    assert torch.allclose(y1, y2, atol=1e-12) and torch.allclose(z1, z2, atol=1e-12)


def test_mixer_two_token_closed_form():
    # H=B=M=D=1, N=2: z = sigmoid(q(k0-k1)) v0 + (1-sigmoid) v1 ; y_n = z
    q = torch.tensor([[[0.7]]], dtype=torch.float64)
    k = torch.tensor([[[[1.0], [-2.0]]]], dtype=torch.float64)
    v = torch.tensor([[[[3.0], [5.0]]]], dtype=torch.float64)
    y, z = O.mixer_explicit(q, k, v)
    w0 = 1.0 / (1.0 + math.exp(-0.7 * 3.0))
    assert abs(float(z) - (w0 * 3.0 + (1 - w0) * 5.0)) < 1e-12
    assert torch.allclose(y, z.expand_as(y))


def test_masked_mixer_equals_dropping_tokens():
    q, k, v = _rand(B=2, N=11)
    mask = torch.ones(2, 11, dtype=torch.bool)
    mask[0, 7:] = False
    mask[1, 3:] = False
    y, z = O.mixer_explicit(q, k, v, key_mask=mask)
    yc, zc = c_oracle.mixer(q, k, v, key_mask=mask)
    assert O.rel_l2(yc, y) < 1e-6 and O.rel_l2(zc, z) < 1e-6
    for b, n in ((0, 7), (1, 3)):
        yb, zb = O.mixer_explicit(q, k[b : b + 1, :, :n], v[b : b + 1, :, :n])
        assert torch.allclose(z[b], zb[0], atol=1e-12)
        assert torch.allclose(y[b, :, :n], yb[0], atol=1e-12)
        assert (y[b, :, n:] == 0).all()


def test_gather_lse():
    q, k, v = _rand()
    _, lse = O.gather_explicit(q, k, v, 1.3)
    s = 1.3 * torch.einsum("hmd,bhnd->bhmn", q, k)
    assert torch.allclose(lse, torch.log(torch.exp(s).sum(-1)), atol=1e-12)


# ---------------------------------------------------------------- causal
def test_causal_recurrent_vs_bruteforce_vs_c():
    q, k, v = _rand(B=1, H=2, N=19, M=4, D=3)
    y, st = O.causal_recurrent(q, k, v, 0.9)
    yb = O.causal_bruteforce(q, k, v, 0.9)
    yc, stc = c_oracle.causal(q, k, v, 0.9)
    assert O.rel_l2(y, yb) < 1e-12
    assert O.rel_l2(yc, yb) < 1e-6
    z, lse = O.causal_state_invariants(*st)
    zc, lsec = O.causal_state_invariants(*stc)
    assert O.rel_l2(zc, z) < 1e-6 and O.rel_l2(lsec, lse) < 1e-6


def test_causal_last_row_is_noncausal_and_state_is_gather():
    q, k, v = _rand(B=1, H=2, N=23, M=4, D=3)
    y, st = O.causal_recurrent(q, k, v)
    yn, zn = O.mixer_explicit(q, k, v)
    assert torch.allclose(y[:, :, -1], yn[:, :, -1], atol=1e-12)
    z, lse = O.causal_state_invariants(*st)
    _, lse_n = O.gather_explicit(q, k, v)
    assert torch.allclose(z, zn, atol=1e-12) and torch.allclose(lse, lse_n, atol=1e-12)


def test_causal_continuation_and_first_token():
    q, k, v = _rand(B=2, H=2, N=17, M=3, D=2)
    y, st = O.causal_recurrent(q, k, v)
    y1, s1 = O.causal_recurrent(q, k[:, :, :9], v[:, :, :9])
    y2, s2 = O.causal_recurrent(q, k[:, :, 9:], v[:, :, 9:], state=s1)
    assert torch.allclose(torch.cat([y1, y2], 2), y, atol=1e-12)
    assert torch.allclose(y[:, :, 0], v[:, :, 0], atol=1e-12)   # first token sees only itself


# ---------------------------------------------------------------- triple
def _rand5(B=2, H=2, N=13, Dq=3, Dv=4, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    mk = lambda d: torch.randn(B, H, N, d, generator=g, dtype=dtype)
    return mk(Dq), mk(Dq), mk(Dq), mk(Dq), mk(Dv)


def test_triple_python_loops_and_c():
    q1, q2, k1, k2, v = _rand5(B=1, H=1, N=5, Dq=2, Dv=3)
    st, out = O.triple_einsum(q1, q2, k1, k2, v, dtype=torch.float64)
    N = 5
    for i in range(2):
        for j in range(3):
            for kk in range(2):
                ref = sum(float(k1[0, 0, n, i] * v[0, 0, n, j] * k2[0, 0, n, kk]) for n in range(N)) / N
                assert abs(float(st[0, 0, i, j, kk]) - ref) < 1e-12
    for n in range(N):
        for j in range(3):
            ref = sum(float(q1[0, 0, n, i] * st[0, 0, i, j, kk] * q2[0, 0, n, kk]) for i in range(2) for kk in range(2))
            assert abs(float(out[0, 0, n, j]) - ref) < 1e-12
    stc, outc = c_oracle.triple(q1, q2, k1, k2, v)
    assert O.rel_l2(stc, st) < 1e-6 and O.rel_l2(outc, out) < 1e-6


def test_triple_matches_reference_scaling_and_feature_map():
    q1, q2, k1, k2, v = _rand5(dtype=torch.float32)
    st, out = O.triple_einsum(q1, q2, k1, k2, v)
    st2, out2 = O.triple_reference_scaling(q1, q2, k1, k2, v)   # three N^(1/3) divisions
    assert O.rel_l2(st, st2) < 1e-6 and O.rel_l2(out, out2) < 1e-6
    stf, outf = O.triple_einsum(q1, q2, k1, k2, v, feature_map=True)
    f = O.elu_plus_one
    stg, outg = O.triple_einsum(f(q1), f(q2), f(k1), f(k2), v)
    assert O.rel_l2(stf, stg) < 1e-7 and O.rel_l2(outf, outg) < 1e-7
    stc, outc = c_oracle.triple(q1, q2, k1, k2, v, feature_map=True, normalize=True)
    stn, outn = O.triple_einsum(q1, q2, k1, k2, v, feature_map=True, normalize=True)
    assert O.rel_l2(stc, stn) < 1e-5 and O.rel_l2(outc, outn) < 1e-4
    x = torch.tensor([-2.0, -0.5, 0.0, 0.5, 3.0])
    assert torch.allclose(f(x), torch.where(x > 0, x + 1, torch.exp(x)))


def test_triple_invariants():
    q1, q2, k1, k2, v = _rand5()
    st, out = O.triple_einsum(q1, q2, k1, k2, v, dtype=torch.float64)
    # swapping (k1,q1) <-> (k2,q2) transposes the state in (i,k) and keeps the output
    st2, out2 = O.triple_einsum(q2, q1, k2, k1, v, dtype=torch.float64)
    assert torch.allclose(st2, st.transpose(2, 4), atol=1e-12) and torch.allclose(out2, out, atol=1e-12)
    # linear in v
    _, o3 = O.triple_einsum(q1, q2, k1, k2, 2.5 * v, dtype=torch.float64)
    assert torch.allclose(o3, 2.5 * out, atol=1e-12)
    # normalised, positive features, constant v  =>  constant output
    c = torch.full_like(v, 1.75)
    _, on = O.triple_einsum(q1, q2, k1, k2, c, feature_map=True, normalize=True, dtype=torch.float64)
    assert torch.allclose(on, c, atol=1e-12)
    # N = 1: state is the outer product, out = <q1,k1><q2,k2> v
    a = _rand5(N=1)
    st1, o1 = O.triple_einsum(*a, dtype=torch.float64)
    ref = (a[0] * a[2]).sum(-1, keepdim=True) * (a[1] * a[3]).sum(-1, keepdim=True) * a[4]
    assert torch.allclose(o1, ref, atol=1e-12)


# ---- causal linear attention ------------------------------------------------------------
def test_causal_linear_oracle_is_pinned():
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(2, 2, 70, 6, generator=g, dtype=torch.float64), torch.randn(2, 2, 70, 6, generator=g, dtype=torch.float64)
    v = torch.randn(2, 2, 70, 5, generator=g, dtype=torch.float64)
    yr = O.causal_linear_recurrent(q, k, v)
    assert O.rel_l2(yr, O.causal_linear_closed_form(q, k, v)) < 1e-12
    for c in (1, 7, 64, 70, 128):
        assert O.rel_l2(O.causal_linear_chunked(q, k, v, chunk=c), yr) < 1e-12
    # last token sees every key: equals non-causal linear attention  Q (K^T V) / N
    full = q[:, :, -1:] @ (k.mT @ v) / 70
    assert O.rel_l2(yr[:, :, -1:], full) < 1e-12
    # pure-Python floats on one (b,h)
    bp = O.causal_linear_bruteforce_py(q[0, 1, :9].tolist(), k[0, 1, :9].tolist(), v[0, 1, :9].tolist())
    y9 = O.causal_linear_recurrent(q[:1, 1:2, :9], k[:1, 1:2, :9], v[:1, 1:2, :9])
    assert O.rel_l2(torch.tensor(bp, dtype=torch.float64), y9[0, 0]) < 1e-12
    # a hand case: N=2, Dk=Dv=1: y0 = q0 k0 v0 / 2, y1 = q1 (k0 v0 + k1 v1) / 2
    q2 = torch.tensor([[[[2.0], [3.0]]]]); k2 = torch.tensor([[[[5.0], [7.0]]]]); v2 = torch.tensor([[[[11.0], [13.0]]]])
    y2 = O.causal_linear_recurrent(q2, k2, v2)
    assert torch.allclose(y2.flatten(), torch.tensor([2 * 5 * 11 / 2, 3 * (5 * 11 + 7 * 13) / 2], dtype=torch.float64))


# ---- token-wise MLP stack -----------------------------------------------------------------
def test_residual_mlp_oracle_matches_torch_layers():
    from torch import nn
    torch.manual_seed(0)
    C = 12
    for n, ir, orr, act, norm in [(3, True, True, "gelu", "layer"), (0, False, True, "silu", "rms"),
                                  (1, True, False, "gelu", None), (-1, True, True, "gelu", "layer")]:
        lins = [nn.Linear(C, C).double() for _ in range(n + 2 if n >= 0 else 1)]
        a = nn.GELU(approximate="tanh") if act == "gelu" else nn.SiLU()
        nm = {"layer": nn.LayerNorm(C).double(), "rms": nn.RMSNorm(C, eps=1e-6).double(), None: nn.Identity()}[norm]
        if norm is not None:
            nn.init.normal_(nm.weight, 1.0, 0.3)
            if norm == "layer":
                nn.init.normal_(nm.bias, 0.0, 0.3)
        x = torch.randn(5, 7, C, dtype=torch.float64)
        with torch.no_grad():
            s = nm(x)
            if n == -1:
                h = lins[0](s)
                ref = s + h if (ir and orr) else h
            else:
                h = a(lins[0](s))
                s = s + h if ir else h
                for l in lins[1:-1]:
                    s = s + a(l(s))
                h = lins[-1](s)
                ref = s + h if orr else h
            ref = x + ref
        got = O.residual_mlp(x, [l.weight.detach() for l in lins], [l.bias.detach() for l in lins], act, ir, orr,
                             norm, None if norm is None else nm.weight.detach(),
                             nm.bias.detach() if norm == "layer" else None, 1e-5 if norm == "layer" else 1e-6, res=x)
        assert O.rel_l2(got, ref) < 1e-12, (n, ir, orr, act, norm)
    # tanh-GELU known values: gelu(0) = 0, gelu(x) - gelu(-x) = x, gelu(1) = 0.841192 (tanh form)
    t = torch.tensor([0.0, 1.0, -1.0, 3.0, -3.0], dtype=torch.float64)
    gv = O.gelu_tanh(t)
    assert gv[0] == 0 and abs(float(gv[1]) - 0.8411919906082768) < 1e-12
    assert torch.allclose(gv[1] - gv[2], t[1]) and torch.allclose(gv[3] - gv[4], t[3])


# ---------------------------------------------------------------- frozen known answers
def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")) as f:
        return json.load(f)


def _t(x, dtype=torch.float64):
    return torch.tensor(x, dtype=dtype)


def test_golden_vectors_pin_both_oracles():
    """tests/golden/vectors.json holds outputs of pure-Python-float loops over the definitions
    (tests/golden/make_vectors.py).  The torch oracle (fp64) and the C oracle (fp32) must reproduce them."""
    g = _golden()
    m = g["mixer"]
    q, k, v = _t(m["q"]), _t(m["k"]).unsqueeze(0), _t(m["v"]).unsqueeze(0)
    assert O.rel_l2(O.mixer_explicit(q, k, v, m["scale"])[0][0], _t(m["y"])) < 1e-12
    assert O.rel_l2(O.mixer_sdpa(q.float(), k.float(), v.float(), m["scale"])[0][0], _t(m["y"])) < 2e-6
    assert O.rel_l2(c_oracle.mixer(q, k, v, m["scale"])[0][0], _t(m["y"])) < 2e-6
    c = g["causal"]
    q, k, v = _t(c["q"]), _t(c["k"]).unsqueeze(0), _t(c["v"]).unsqueeze(0)
    assert O.rel_l2(O.causal_recurrent(q, k, v, c["scale"])[0][0], _t(c["y"])) < 1e-12
    assert O.rel_l2(O.causal_bruteforce(q, k, v, c["scale"])[0], _t(c["y"])) < 1e-12
    assert O.rel_l2(c_oracle.causal(q, k, v, c["scale"])[0][0], _t(c["y"])) < 2e-6
    t = g["triple"]
    a = [_t(t[n]).unsqueeze(0) for n in ("q1", "q2", "k1", "k2", "v")]
    st, out = O.triple_einsum(*a, dtype=torch.float64)
    assert O.rel_l2(st[0], _t(t["state"])) < 1e-12 and O.rel_l2(out[0], _t(t["out"])) < 1e-12
    st, out = O.triple_reference_scaling(*[x.float() for x in a])
    assert O.rel_l2(st[0], _t(t["state"])) < 2e-6 and O.rel_l2(out[0], _t(t["out"])) < 2e-6
    st, out = c_oracle.triple(*a)
    assert O.rel_l2(st[0], _t(t["state"])) < 2e-6 and O.rel_l2(out[0], _t(t["out"])) < 2e-6
    cl = g["causal_linear"]
    q, k, v = _t(cl["q"]).unsqueeze(0), _t(cl["k"]).unsqueeze(0), _t(cl["v"]).unsqueeze(0)
    assert O.rel_l2(O.causal_linear_recurrent(q, k, v)[0], _t(cl["y"])) < 1e-12
    assert O.rel_l2(O.causal_linear_chunked(q, k, v, chunk=4)[0], _t(cl["y"])) < 1e-12
    ms = g["mlp_stack"]
    y = O.residual_mlp(_t(ms["x"]), [_t(w) for w in ms["w"]], [_t(b) for b in ms["b"]], "gelu", True, True, "layer",
                       _t(ms["gamma"]), _t(ms["beta"]), ms["eps"], _t(ms["res"]))
    assert O.rel_l2(y, _t(ms["y"])) < 1e-12
    rp = g["rope"]
    assert O.rel_l2(O.rope_reference(_t(rp["x"]), rp["base"]), _t(rp["y"])) < 1e-12
    from flare_py_amd.lra_modules import RotaryPositionalEmbeddings
    assert O.rel_l2(RotaryPositionalEmbeddings(8, 16, base=rp["base"])(_t(rp["x"], torch.float32)[None, None])[0, 0], _t(rp["y"])) < 1e-6


def test_golden_vectors_are_reproducible(tmp_path):
    """The committed fixture is what its generator writes (plain Python floats: platform independent up to libm's exp)."""
    import importlib.util
    import json
    import os
    here = os.path.join(os.path.dirname(__file__), "golden")
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(here, "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.HERE = str(tmp_path)
    mod.main()
    new = json.load(open(tmp_path / "vectors.json"))
    old = _golden()
    for key in old:
        for name, val in old[key].items():
            a, b = torch.tensor(val, dtype=torch.float64), torch.tensor(new[key][name], dtype=torch.float64)
            assert torch.allclose(a, b, rtol=1e-13, atol=1e-15), (key, name)


# ---- layer / block / model compositions ------------------------------------------------------------
class _TorchBlock(torch.nn.Module):
    """Pre-norm block assembled from torch's own layers and SDPA, for pinning flare_block's composition:
    x += out(merge(SDPA(k, q, SDPA(q, k, v)))) with k, v = MLP(norm1 x); x += MLP(norm2 x)."""

    def __init__(self, C, H, M, n):
        super().__init__()
        nn = torch.nn
        mk = lambda: nn.ModuleList(nn.Linear(C, C) for _ in range(n + 2))
        self.H, self.M, self.n1, self.n2 = H, M, nn.LayerNorm(C), nn.LayerNorm(C)
        self.kp, self.vp, self.ff, self.out = mk(), mk(), mk(), nn.Linear(C, C)
        self.lq = nn.Parameter(torch.randn(C, M) * 0.3)
        self.act = nn.GELU(approximate="tanh")

    def mlp(self, ls, x):
        x = x + self.act(ls[0](x))
        for l in ls[1:-1]:
            x = x + self.act(l(x))
        return x + ls[-1](x)

    def forward(self, x):
        B, N, C = x.shape
        h = self.n1(x)
        split = lambda t: t.view(B, N, self.H, C // self.H).transpose(1, 2)
        k, v = split(self.mlp(self.kp, h)), split(self.mlp(self.vp, h))
        q = self.lq.view(self.H, self.M, C // self.H).unsqueeze(0).expand(B, -1, -1, -1)
        sdpa = torch.nn.functional.scaled_dot_product_attention
        z = sdpa(q, k, v, scale=1.0)
        y = sdpa(k, q, z, scale=1.0)
        x = x + self.out(y.transpose(1, 2).reshape(B, N, C))
        return x + self.mlp(self.ff, self.n2(x))

    def reference_keys(self):
        """The same parameters under the state_dict names of pdebench/models/flare.py."""
        sd = {"norm1.weight": self.n1.weight, "norm1.bias": self.n1.bias, "norm2.weight": self.n2.weight,
              "norm2.bias": self.n2.bias, "att.latent_q": self.lq, "att.out_proj.weight": self.out.weight,
              "att.out_proj.bias": self.out.bias}
        for name, ls in (("att.k_proj.", self.kp), ("att.v_proj.", self.vp), ("mlp.", self.ff)):
            keys = ["fc1"] + [f"fcs.{i}" for i in range(len(ls) - 2)] + ["fc2"]
            for kname, l in zip(keys, ls):
                sd[name + kname + ".weight"], sd[name + kname + ".bias"] = l.weight, l.bias
        return {k: v.detach() for k, v in sd.items()}


@pytest.mark.parametrize("C,H,M,n", [(32, 4, 8, 1), (48, 3, 5, 0), (16, 2, 16, 3)])
def test_block_composition_against_torch_layers(C, H, M, n):
    torch.manual_seed(C + n)
    blk = _TorchBlock(C, H, M, n).double()
    for p_ in blk.parameters():
        if p_.dim() == 1:
            torch.nn.init.normal_(p_, 0.5, 0.3)
    x = torch.randn(2, 37, C, dtype=torch.float64)
    with torch.no_grad():
        ref = blk(x)
    got = O.flare_block(blk.reference_keys(), "", x, H)
    assert O.rel_l2(got, ref) <= 1e-12
    # a dropped residual, a swapped norm or a transposed head split must show
    sd = blk.reference_keys()
    sd["norm1.weight"], sd["norm2.weight"] = sd["norm2.weight"], sd["norm1.weight"]
    assert O.rel_l2(O.flare_block(sd, "", x, H), ref) > 1e-3


def test_product_modules_scores_branch_against_model_oracle():
    """The product's modules on the CPU (their spelled-out return_scores branch needs no HIP kernel) against the
    state_dict oracle: key names, flag handling and layer order of FLAREModel agree with flare.py:251-349."""
    import flare_py_amd as FA
    for kw in (dict(), dict(rmsnorm=True, qk_norm=True, act="silu"), dict(num_layers_ffn=0, ffn_mlp_ratio=2.0, num_layers_k_proj=-1),
               dict(out_proj_norm=False, num_layers_in_out_proj=0)):
        torch.manual_seed(1)
        m = FA.FLAREModel(in_dim=3, out_dim=2, channel_dim=32, num_blocks=2, num_heads=4, num_latents=8, **kw).eval()
        for p_ in m.parameters():
            torch.nn.init.normal_(p_, 0.0, 0.3) if p_.dim() > 1 else torch.nn.init.normal_(p_, 0.3, 0.3)
        x = torch.randn(2, 19, 3)
        with torch.no_grad():
            y, scores = m(x, return_scores=True)
        assert len(scores) == 2 and scores[0].shape == (2, 4, 8, 19)
        ref = O.flare_model(m.state_dict(), x, 4, 2, act=kw.get("act", "gelu") or "gelu", qk_norm=kw.get("qk_norm", False),
                            rmsnorm=kw.get("rmsnorm", False), out_proj_norm=kw.get("out_proj_norm", True))
        assert O.rel_l2(y, ref) <= 1e-5, kw


def test_rope_reference_hand_cases():
    # position 0: identity
    x = torch.randn(2, 3, 1, 8, dtype=torch.float64)
    assert torch.equal(O.rope_reference(x), x)
    # D = 2: the plane rotation by p radians
    x = torch.randn(5, 2, dtype=torch.float64)
    got = O.rope_reference(x)
    for p_ in range(5):
        c, s_ = math.cos(p_), math.sin(p_)
        assert abs(float(got[p_, 0]) - (float(x[p_, 0]) * c - float(x[p_, 1]) * s_)) < 1e-12
        assert abs(float(got[p_, 1]) - (float(x[p_, 1]) * c + float(x[p_, 0]) * s_)) < 1e-12
    # D = 4 by hand from lra/models/embeddings.py:136-147: rates (1, 1, b, b), b = base^-1/2; partner (-a1, -a3, a0, a2)
    a = [0.3, -1.1, 0.7, 2.0]
    x = torch.tensor([a, a, a], dtype=torch.float64)
    got = O.rope_reference(x, base=100.0)
    b = 100.0 ** -0.5
    for p_ in range(3):
        want = [a[0] * math.cos(p_) - a[1] * math.sin(p_), a[1] * math.cos(p_) - a[3] * math.sin(p_),
                a[2] * math.cos(p_ * b) + a[0] * math.sin(p_ * b), a[3] * math.cos(p_ * b) + a[2] * math.sin(p_ * b)]
        assert max(abs(float(got[p_, j]) - want[j]) for j in range(4)) < 1e-12
    # linear in x
    u, v = torch.randn(7, 6, dtype=torch.float64), torch.randn(7, 6, dtype=torch.float64)
    assert O.rel_l2(O.rope_reference(2.0 * u - v), 2.0 * O.rope_reference(u) - O.rope_reference(v)) < 1e-14
