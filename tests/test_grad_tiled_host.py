"""Host-side check (no GPU, no HIP) of the token-tiled gradient recomputation that backs the mixer where the HIP
backward does not apply (fp32 inputs, unusual shapes) and the two differentiable halves: against torch autograd
through the explicit softmax formulas of pdebench/models/flare.py:142-150 in fp64, with tiles far smaller than N
so that the online log-sum-exp, the carried dz and the accumulated dq are all exercised."""
import pytest
import torch

from flare_py_amd import functional as FN


def explicit(q, k, v, scale, mask):
    qe = q if q.dim() == 4 else q.unsqueeze(0)
    s = scale * (qe @ k.mT)
    se = s if mask is None else s.masked_fill(~mask[:, None, None, :], float("-inf"))
    z = torch.softmax(se, -1) @ v
    y = torch.softmax(s.mT, -1) @ z
    return (y if mask is None else y * mask[:, None, :, None]), z


@pytest.mark.parametrize("shared_q", [True, False])
@pytest.mark.parametrize("masked", [False, True])
def test_tiled_gradients_equal_autograd(shared_q, masked, monkeypatch):
    monkeypatch.setattr(FN, "GRAD_TILE_ELEMS", 4096)           # tiles of 256 tokens for N = 700
    torch.manual_seed(0)
    B, H, N, M, D = 2, 2, 700, 12, 8
    q = torch.randn(*(() if shared_q else (B,)), H, M, D, dtype=torch.double) * 0.5
    k, v, gy = (torch.randn(B, H, N, D, dtype=torch.double) for _ in range(3))
    gz = torch.randn(B, H, M, D, dtype=torch.double)
    mask = None
    if masked:
        mask = torch.ones(B, N, dtype=torch.bool)
        mask[0, 300:] = False
        mask[1, ::3] = False
    scale = 0.7

    def rel(a, b):
        return float((a.double() - b).norm() / b.norm())

    qr, kr, vr = (t.clone().requires_grad_(True) for t in (q, k, v))
    explicit(qr, kr, vr, scale, mask)[0].backward(gy)
    got = FN._mixer_torch_grad(q.float(), k.float(), v.float(), scale, mask, gy.float())
    assert all(rel(g, r.grad) < 5e-6 for g, r in zip(got, (qr, kr, vr)))

    qr, kr, vr = (t.clone().requires_grad_(True) for t in (q, k, v))
    explicit(qr, kr, vr, scale, mask)[1].backward(gz)
    got = FN._half_torch_grad("gather", q.float(), k.float(), v.float(), scale, mask, gz.float())
    assert all(rel(g, r.grad) < 5e-6 for g, r in zip(got, (qr, kr, vr)))

    zz = torch.randn(B, H, M, D, dtype=torch.double)
    qr, kr, zr = (t.clone().requires_grad_(True) for t in (q, k, zz))
    qe = qr if qr.dim() == 4 else qr.unsqueeze(0)
    y = torch.softmax(scale * (kr @ qe.mT), -1) @ zr
    (y if mask is None else y * mask[:, None, :, None]).backward(gy)
    got = FN._half_torch_grad("scatter", q.float(), k.float(), zz.float(), scale, mask, gy.float())
    assert all(rel(g, r.grad) < 5e-6 for g, r in zip(got, (qr, kr, zr)))


def test_batch_element_without_tokens_gets_zero_gradients():
    torch.manual_seed(1)
    B, H, N, M, D = 2, 1, 64, 8, 4
    q = torch.randn(H, M, D)
    k, v, gy = (torch.randn(B, H, N, D) for _ in range(3))
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[1] = False
    gq, gk, gv = FN._mixer_torch_grad(q, k, v, 1.0, mask, gy)
    assert torch.isfinite(gq).all() and torch.isfinite(gk).all() and torch.isfinite(gv).all()
    assert float(gk[1].abs().max()) == 0.0 and float(gv[1].abs().max()) == 0.0


def test_dropout_hash_restatement_matches_plain_python():
    """_dropout_keep (int64 tensors) against the same 32-bit hash written with Python integers."""
    def low(x):
        x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF; x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF; x ^= x >> 16
        return x
    seed, phase, p = 0x123456789ABCDEF, 1, 0.3
    B, H, M, n0, n1 = 2, 3, 5, 40, 47
    got = FN._dropout_keep(seed, phase, B, H, M, n0, n1, p, "cpu")
    thr = int(p * 16777216.0)
    for b in range(B):
        for h in range(H):
            for m in range(M):
                for n in range(n0, n1):
                    x = ((seed & 0xFFFFFFFF) + n * 0x9E3779B1 + m * 0x85EBCA77 + (b * H + h) * 0xC2B2AE3D + phase * 0x27D4EB2F) & 0xFFFFFFFF
                    keep = (low(low(x) ^ (seed >> 32)) >> 8) >= thr
                    assert bool(got[b, h, m, n - n0]) == keep
