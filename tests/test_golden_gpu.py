"""The HIP kernels (fp32, through the C-ABI) against the frozen known answers in tests/golden/vectors.json, which
come from pure-Python-float loops over the definitions (tests/golden/make_vectors.py).  Tolerance: the fp32 bar,
relative L2 <= 1e-5."""
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
