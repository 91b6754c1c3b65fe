"""The HIP kernels (fp32, through the C-ABI) against the frozen known answers in tests/golden/vectors.json, which
come from pure-Python-float loops over the definitions (tests/golden/make_vectors.py).  Tolerance: the fp32 bar,
relative L2 <= 1e-5; the fused MLP launch computes in bf16 / f16 and is held to the 16-bit bar, 2e-2."""
import json
import os

import pytest
import torch

import flare_py_amd as F
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    with open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")) as f:
        return json.load(f)


def _t(x, dev):
    return torch.tensor(x, dtype=torch.float32, device=dev)


def test_mixer(dev, g):
    m = g["mixer"]
    y = F.flare_multihead_mixer(_t(m["q"], dev), _t(m["k"], dev).unsqueeze(0), _t(m["v"], dev).unsqueeze(0), scale=m["scale"])
    assert O.rel_l2(y[0], torch.tensor(m["y"], dtype=torch.float64)) <= 1e-5


def test_causal_prefill_and_decode(dev, g):
    c = g["causal"]
    q, k, v = _t(c["q"], dev), _t(c["k"], dev).unsqueeze(0), _t(c["v"], dev).unsqueeze(0)
    yr = torch.tensor(c["y"], dtype=torch.float64)
    y, _ = F.flare_causal_prefill(q, k, v, scale=c["scale"])
    assert O.rel_l2(y[0], yr) <= 1e-5
    y1, st = F.flare_causal_prefill(q, k[:, :, :4], v[:, :, :4], scale=c["scale"])
    y2, _ = F.flare_causal_decode(q, k[:, :, 4:], v[:, :, 4:], st, scale=c["scale"])
    assert O.rel_l2(torch.cat([y1, y2], 2)[0], yr) <= 1e-5


def test_triple(dev, g):
    t = g["triple"]
    a = [_t(t[n], dev).unsqueeze(0) for n in ("q1", "q2", "k1", "k2", "v")]
    st, out = F.triple_attention(*a)
    assert O.rel_l2(st[0], torch.tensor(t["state"], dtype=torch.float64)) <= 1e-5
    assert O.rel_l2(out[0], torch.tensor(t["out"], dtype=torch.float64)) <= 1e-5


def test_causal_linear(dev, g):
    c = g["causal_linear"]
    y = F.causal_linear_attention(_t(c["q"], dev).unsqueeze(0), _t(c["k"], dev).unsqueeze(0), _t(c["v"], dev).unsqueeze(0))
    assert O.rel_l2(y[0], torch.tensor(c["y"], dtype=torch.float64)) <= 1e-5


@pytest.mark.parametrize("cd", [torch.bfloat16, torch.float16])
def test_fused_mlp_stack(dev, g, cd):
    """res + ResidualMLP(LayerNorm(x)) in one launch (flare_mlp_fwd) against the plain-Python known answer."""
    from torch import nn
    from flare_py_amd import fused
    ms = g["mlp_stack"]
    Cdim = len(ms["gamma"])
    mlp = F.ResidualMLP(Cdim, Cdim, Cdim, num_layers=len(ms["w"]) - 2, input_residual=True, output_residual=True).to(dev)
    norm = nn.LayerNorm(Cdim, eps=ms["eps"]).to(dev)
    with torch.no_grad():
        for lin, w, b in zip([mlp.fc1, *mlp.fcs, mlp.fc2], ms["w"], ms["b"]):
            lin.weight.copy_(_t(w, dev))
            lin.bias.copy_(_t(b, dev))
        norm.weight.copy_(_t(ms["gamma"], dev))
        norm.bias.copy_(_t(ms["beta"], dev))
        x, res = _t(ms["x"], dev), _t(ms["res"], dev)
        ref = torch.tensor(ms["y"], dtype=torch.float64)
        assert O.rel_l2(res + mlp(norm(x)), ref) <= 1e-5                      # the module itself, fp32 torch layers
        with torch.autocast("cuda", dtype=cd):
            assert fused.compute_dtype(x, mlp) == cd
            y = fused.fused_mlp(x, mlp, cd, norm=norm, res=res)
    assert O.rel_l2(y, ref) <= 2e-2
