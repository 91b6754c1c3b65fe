"""Attention dropout of the mixer (lra/models/backends.py:592,605-606: dropout_p on both scaled_dot_product_attention
calls in training).  torch defines it as: weights = softmax(scores); weights = weights * keep / (1 - p); out = weights @ v.
The kernels decide `keep` by a counter-based hash; the oracle below applies exactly that definition with the masks
rebuilt on the CPU by the host-side restatement of the hash, in fp64.
Tolerances: fp32 1e-5, bf16 2e-2 relative L2, gradients 1e-4 / 3e-2."""
import pytest
import torch

import flare_py_amd as F
from flare_py_amd import functional as FN
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu


def make(B, H, N, M, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).to(dtype)
    k = torch.randn(B, H, N, D, generator=g).to(dtype)
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    return q, k, v


def oracle(q, k, v, scale, mask, p, seed):
    """y, z with dropout on both softmaxes, fp64, masks from the hash."""
    B, H, N, D = k.shape
    M = q.shape[-2]
    qe = q.double().unsqueeze(0) if q.dim() == 3 else q.double()
    s = scale * (qe @ k.double().mT)
    se = s if mask is None else s.masked_fill(~mask[:, None, None, :], float("-inf"))
    K1 = FN._dropout_keep(seed, 0, B, H, M, 0, N, p, "cpu").double() / (1 - p)
    K2 = FN._dropout_keep(seed, 1, B, H, M, 0, N, p, "cpu").double() / (1 - p)
    z = (torch.softmax(se, -1) * K1) @ v.double()
    y = (torch.softmax(s, 2) * K2).mT @ z
    return (y if mask is None else y * mask[:, None, :, None]), z


def fwd_dropout_entry(q, k, v, scale, p, seed):
    """flare_mixer_fwd_dropout called through ctypes (the descriptor itself carries no dropout)."""
    import ctypes as C
    from flare_py_amd import _lib
    lib = _lib.load()
    B, H, N, D = k.shape
    q4 = FN._q4(q, B)
    y = torch.empty_like(k)
    z = torch.empty((B, H, q4.shape[2], D), dtype=torch.float32, device=k.device)
    d = FN._mixer_desc(q4, k, v, y, scale, 0, False)
    dd = FN._mixer_desc(q4, k, v, y, scale, 0, False, (p, seed))
    need = C.c_size_t(0)
    _lib.check(lib.flare_mixer_workspace_bytes(C.byref(dd), C.byref(need)), "flare_mixer_workspace_bytes")
    ws = torch.empty(max(int(need.value), 16), dtype=torch.uint8, device=k.device)
    rc = lib.flare_mixer_fwd_dropout(C.byref(d), q4.data_ptr(), k.data_ptr(), v.data_ptr(), None, C.c_float(p), C.c_uint64(seed),
                                     y.data_ptr(), z.data_ptr(), ws.data_ptr(), ws.numel(), C.c_void_p(FN._stream_ptr(k.device)))
    _lib.check(rc, "flare_mixer_fwd_dropout")
    return y, z


# (2, 2, 300, 16, 8) and (1, 2, 257, 20, 16): head dims / latent counts that end on the fp32-FMA kernels for fp32 (the first
# after padding D to 16 on the matrix cores); (1, 3, 1000, 64, 32), (2, 8, 1024, 128, 16) (the sequence benchmark's shape,
# out/lra/run.sh: 128 latents, 8 heads of 16) and (1, 2, 700, 96, 64): the fp32 16x16x4 and the 16-bit 16x16x32 kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 2, 300, 16, 8), (1, 3, 1000, 64, 32), (1, 2, 257, 20, 16), (2, 8, 1024, 128, 16),
                                   (1, 2, 700, 96, 64), (1, 1, 5000, 256, 32)])
def test_forward_with_dropout_equals_the_definition(dev, dtype, shape):
    q, k, v = make(*shape, dtype, seed=3)
    p, seed = 0.25, 123456789012345
    mask = torch.ones(shape[0], shape[2], dtype=torch.bool)
    mask[0, shape[2] // 2:] = False
    for km in (None, mask):
        y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, key_mask=None if km is None else km.to(dev),
                                       return_z=True, dropout_p=p, dropout_seed=seed)
        yr, zr = oracle(q, k, v, 0.8, km, p, seed)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert O.rel_l2(z, zr) <= tol and O.rel_l2(y, yr) <= tol, (O.rel_l2(z, zr), O.rel_l2(y, yr))
    # the same seed repeats the mask, another seed changes it
    y1 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, dropout_p=p, dropout_seed=seed)
    y2 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, dropout_p=p, dropout_seed=seed)
    y3 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, dropout_p=p, dropout_seed=seed + 1)
    assert torch.equal(y1, y2) and not torch.equal(y1, y3)


def test_threshold_follows_the_float32_p():
    import struct
    for p in (0.3, 0.1, 0.2, 0.25, 0.05):
        p32 = struct.unpack("f", struct.pack("f", p))[0]
        assert FN._dropout_threshold(p) == int(p32 * 16777216.0)
    assert FN._dropout_threshold(0.3) != int(0.3 * 16777216.0)      # the case that used to differ
    assert FN._dropout_threshold(1e-9) == 0


def test_keep_rate_and_mean_preservation(dev):
    """The hash keeps a fraction 1 - p of the weights (both phases, several seeds), and the mean over seeds of the
    dropped-out result approaches the result without dropout."""
    B, H, N, M, D = 1, 2, 2000, 32, 16
    q, k, v = make(B, H, N, M, D, torch.float32, seed=5)
    for p in (0.1, 0.5):
        for phase in (0, 1):
            rate = float(FN._dropout_keep(777 + phase, phase, B, H, M, 0, N, p, "cpu").float().mean())
            assert abs(rate - (1 - p)) < 5e-3
    y0 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev))
    acc = torch.zeros_like(y0)
    n_seeds = 64
    for s in range(n_seeds):
        acc += F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), dropout_p=0.3, dropout_seed=1000 + s)
    one = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), dropout_p=0.3, dropout_seed=1000)
    err_mean, err_one = O.rel_l2(acc / n_seeds, y0), O.rel_l2(one, y0)
    assert err_mean < 0.25 * err_one, (err_mean, err_one)       # 1/sqrt(64) = 0.125 of a single draw's deviation


def test_dropout_zero_is_the_plain_mixer(dev):
    q, k, v = make(1, 2, 500, 24, 16, torch.float32, seed=7)
    y0, z0 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), return_z=True)
    y1, z1 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), return_z=True, dropout_p=0.0)
    assert torch.equal(y0, y1) and torch.equal(z0, z1)
    # p = 0 (and a p below 2^-24, which keeps every weight and rescales nothing) through the dropout entry point of the
    # C ABI: the same numbers as flare_mixer_fwd
    for p in (0.0, 1e-9):
        y2, z2 = fwd_dropout_entry(q.to(dev), k.to(dev), v.to(dev), 1.0, p, 99)
        assert torch.equal(y2, y0) and torch.equal(z2, z0)
    # and a real p there gives what the descriptor's fields give
    y3, z3 = fwd_dropout_entry(q.to(dev), k.to(dev), v.to(dev), 1.0, 0.3, 99)
    y4, z4 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), return_z=True, dropout_p=0.3, dropout_seed=99)
    assert torch.equal(y3, y4) and torch.equal(z3, z4) and not torch.equal(y3, y0)


# p = 0.3 and 0.1 are not exact in float32: the threshold must come from the rounded value the kernels see
# (floor(p * 2^24) differs by one between the double and the float32 of 0.3)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,p", [((2, 2, 400, 16, 16), 0.2), ((2, 2, 400, 16, 16), 0.3), ((1, 4, 1024, 128, 16), 0.1),
                                     ((2, 2, 333, 48, 32), 0.3), ((1, 2, 500, 64, 64), 0.1), ((2, 1, 200, 24, 8), 0.3),
                                     ((2, 2, 700, 96, 32), 0.3), ((1, 2, 2000, 256, 32), 0.1), ((1, 1, 300, 256, 64), 0.3)])
def test_backward_uses_the_forward_mask(dev, dtype, shape, p):
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, dtype, seed=9)
    gy = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(10)).to(dtype)
    seed = 4242424242424242
    # the HIP backward takes these (it regenerates the masks); the others differentiate through the torch recomputation
    hip = D >= 16 and M % (16 if dtype == torch.float32 else 32) == 0
    assert FN._hip_backward_ok(q.to(dev), k.to(dev), v.to(dev), None, False, (p, seed)) == hip
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[B - 1, 100:] = False
    for km in (None, mask):
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        F.flare_multihead_mixer(qd, kd, vd, scale=0.9, key_mask=None if km is None else km.to(dev), dropout_p=p,
                                dropout_seed=seed).backward(gy.to(dev))
        qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
        oracle(qr, kr, vr, 0.9, km, p, seed)[0].backward(gy.double())
        tol = 1e-4 if dtype == torch.float32 else 3e-2 if dtype == torch.bfloat16 else 1e-2
        for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
            err = O.rel_l2(got, ref)
            assert err <= tol, f"{name} rel-L2 {err:.3e}"


def test_sequence_block_trains_with_attention_dropout(dev):
    """lra_modules.FLARE with attn_drop > 0: training mode drops (results differ between calls and from eval mode,
    gradients flow), eval mode does not."""
    from flare_py_amd import lra_modules
    torch.manual_seed(11)
    att = lra_modules.FLARE(channel_dim=32, num_heads=4, num_latents=8, kv_proj_hidden_dim=32, attn_drop=0.3).to(dev)
    x = torch.randn(2, 100, 32, device=dev)
    mask = torch.ones(2, 100, dtype=torch.bool, device=dev)
    mask[1, 60:] = False
    att.train()
    y1 = att(x, mask)
    y2 = att(x, mask)
    assert not torch.equal(y1, y2)
    y1.sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in att.parameters())
    att.eval()
    with torch.no_grad():
        e1, e2 = att(x, mask), att(x, mask)
    assert torch.equal(e1, e2)
