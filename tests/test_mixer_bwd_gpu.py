"""GPU parity of the HIP mixer backward (flare_mixer_bwd) vs autograd through the CPU oracle.

Oracle: torch autograd (fp64, CPU) through oracle.flare_oracle.mixer_explicit, the explicit
restatement of pdebench/models/flare.py:142-150 — i.e. exactly what the reference differentiates.
Tolerance: 3e-2 relative L2 per gradient for the 16-bit kernels (the gradients are assembled in
fp32 and rounded once to bf16 as matrix-core operands; dk, dv are returned in the element type).
"""
import pytest
import torch

import flare_py_amd as F
from flare_py_amd import functional as FN
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu


def make(B, H, N, M, D, dtype, seed=0, shared_q=True):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(*(() if shared_q else (B,)), H, M, D, generator=g) * D ** -0.5
    k = torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g)
    gy = torch.randn(B, H, N, D, generator=g)
    return q.to(dtype), k.to(dtype), v.to(dtype), gy.to(dtype)


def oracle_grads(q, k, v, gy, scale):
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    y, _ = O.mixer_explicit(qr, kr, vr, scale)
    y.backward(gy.double())
    return qr.grad, kr.grad, vr.grad


@pytest.mark.parametrize("shape", [(1, 2, 777, 64, 32), (2, 2, 1000, 128, 16), (1, 1, 300, 256, 32), (1, 2, 500, 128, 64),
                                   (2, 1, 2500, 256, 32), (1, 8, 4100, 64, 16), (1, 2, 900, 512, 16), (1, 1, 70001, 256, 32),
                                   (1, 2, 1300, 512, 32), (2, 1, 1111, 192, 32), (1, 3, 5000, 128, 32), (1, 1, 33, 64, 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_vs_autograd_oracle(dev, shape, dtype):
    q, k, v, gy = make(*shape, dtype)
    scale = 0.8
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert FN._hip_backward_ok(qd, kd, vd, None, False)
    y = F.flare_multihead_mixer(qd, kd, vd, scale=scale)
    y.backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, scale)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        assert got.dtype == dtype and got.shape == ref.shape
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


def test_backward_per_batch_q_strided_inputs_and_token_major(dev):
    B, H, N, M, D = 2, 4, 640, 128, 32
    q, k, v, gy = make(B, H, N, M, D, torch.bfloat16, seed=3, shared_q=False)
    x = torch.stack([k, v]).permute(0, 1, 3, 2, 4).reshape(2, B, N, H * D).contiguous().to(dev)   # [B,N,H*D] projections
    kd, vd = (t.view(B, N, H, D).permute(0, 2, 1, 3).detach().requires_grad_(True) for t in x)
    qd = q.to(dev).requires_grad_(True)
    y = F.flare_multihead_mixer(qd, kd, vd, token_major_out=True)
    (y * gy.to(dev)).sum().backward()
    gq, gk, gv = oracle_grads(q, k, v, gy, 1.0)
    assert O.rel_l2(qd.grad, gq) <= 3e-2 and O.rel_l2(kd.grad, gk) <= 3e-2 and O.rel_l2(vd.grad, gv) <= 3e-2


def test_backward_is_deterministic_and_matches_torch_recompute(dev):
    q, k, v, gy = make(1, 2, 3000, 128, 32, torch.bfloat16, seed=5)
    outs = []
    for _ in range(2):
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        F.flare_multihead_mixer(qd, kd, vd).backward(gy.to(dev))
        outs.append((qd.grad, kd.grad, vd.grad))
    assert all(torch.equal(a, b) for a, b in zip(*outs))                       # bit-stable
    ref = FN._mixer_torch_grad(q.to(dev), k.to(dev), v.to(dev), 1.0, None, gy.to(dev))
    for a, b in zip(outs[0], ref):
        assert O.rel_l2(a, b) <= 3e-2


def test_fallbacks_keep_working(dev):
    # shapes the kernels do not take (fp32 with a latent count that is not a multiple of 16) differentiate through the
    # torch recomputation
    q, k, v, gy = make(1, 2, 200, 40, 16, torch.float32, seed=7)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert not FN._hip_backward_ok(qd, kd, vd, None, False)
    big = [t.to(dev).bfloat16() for t in make(1, 1, 64, 2048, 64, torch.float32)[:3]]
    assert not FN._hip_backward_ok(*big, None, False)                      # more latents than four chunks of LDS hold
    F.flare_multihead_mixer(qd, kd, vd).backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 1.0)
    assert O.rel_l2(qd.grad, gq) <= 1e-4 and O.rel_l2(kd.grad, gk) <= 1e-4 and O.rel_l2(vd.grad, gv) <= 1e-4


# ---- fp32 inputs: backward kernels on the fp32 matrix instruction ----
@pytest.mark.parametrize("shape", [(1, 2, 777, 64, 32), (2, 2, 1000, 128, 16), (1, 1, 300, 256, 32), (1, 2, 500, 128, 64),
                                   (1, 1, 1, 16, 16), (1, 2, 15, 48, 32), (1, 3, 4100, 80, 16), (1, 1, 2100, 512, 32),
                                   (1, 1, 900, 272, 64), (1, 2, 70001, 256, 32), (1, 2, 333, 64, 8), (1, 2, 257, 32, 24)])
def test_fp32_backward_vs_autograd_oracle(dev, shape):
    """fp32 is the reference's default training precision (pdebench/__main__.py:1106): dq, dk, dv of the HIP kernels
    against fp64 autograd through the explicit-softmax oracle at 1e-4, incl. latent counts that need the token pass in
    chunks (512 x 32, 272 x 64), ragged token counts, a single token, and head dims that are zero-padded (8, 24)."""
    q, k, v, gy = make(*shape, torch.float32, seed=sum(shape))
    scale = 0.8
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    if shape[4] in (16, 32, 64):
        assert FN._hip_backward_ok(qd, kd, vd, None, False)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CUDA]) as prof:
        F.flare_multihead_mixer(qd, kd, vd, scale=scale).backward(gy.to(dev))
        torch.cuda.synchronize()
    kernels = " ".join(e.key for e in prof.key_averages())
    assert "bwd_f32_tok_kernel" in kernels and "bwd_f32_lat_kernel" in kernels, kernels
    gq, gk, gv = oracle_grads(q, k, v, gy, scale)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        assert got.dtype == torch.float32 and got.shape == ref.shape
        err = float((got.cpu().double() - ref).norm() / (ref.norm() + 1e-300))
        tol = 1e-4 if float(ref.norm()) > 1e-6 else float("inf")      # N = 1: dq, dk are exactly 0 up to rounding
        assert err <= tol, f"{name} rel-L2 {err:.3e}"
        if tol == float("inf"):
            assert float(got.abs().max()) <= 1e-5


def test_fp32_backward_masks_per_batch_q_strided_views_and_determinism(dev):
    B, H, N, M, D = 3, 2, 700, 64, 32
    g = torch.Generator().manual_seed(17)
    q = torch.randn(B, H, M, D, generator=g) * D ** -0.5                        # one latent set per batch element
    kk = torch.randn(B, N, H * D, generator=g)
    vv = torch.randn(B, N, H * D, generator=g)
    gy = torch.randn(B, H, N, D, generator=g)
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, 500:] = False
    mask[1, ::3] = False
    mask[2, :] = False                                                           # a batch element without a token
    kk[0, 600] = float("nan")                                                    # padding may hold anything
    outs = []
    for _ in range(2):
        qd = q.to(dev).requires_grad_(True)
        kd = kk.to(dev).requires_grad_(True)
        vd = vv.to(dev).requires_grad_(True)
        k4 = kd.view(B, N, H, D).permute(0, 2, 1, 3)
        v4 = vd.view(B, N, H, D).permute(0, 2, 1, 3)
        with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CUDA]) as prof:
            F.flare_multihead_mixer(qd, k4, v4, key_mask=mask.to(dev)).backward(gy.to(dev))
            torch.cuda.synchronize()
        assert "bwd_f32_tok_kernel" in " ".join(e.key for e in prof.key_averages())
        outs.append((qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()))
    assert all(torch.equal(a, b) for a, b in zip(*outs))                         # bit-stable
    kc = torch.nan_to_num(kk, nan=0.0)
    qr = q.double().requires_grad_(True)
    kr = kc.double().requires_grad_(True)
    vr = vv.double().requires_grad_(True)
    y, _ = O.mixer_explicit(qr, kr.view(B, N, H, D).permute(0, 2, 1, 3), vr.view(B, N, H, D).permute(0, 2, 1, 3), 1.0, mask)
    y.backward(gy.double())
    for name, got, ref in zip(("dq", "dk", "dv"), outs[0], (qr.grad, kr.grad, vr.grad)):
        assert torch.isfinite(got).all(), name
        err = float((got.double() - ref).norm() / ref.norm())
        assert err <= 1e-4, f"{name} rel-L2 {err:.3e}"
    assert (outs[0][1][0, 500:] == 0).all() and (outs[0][2][2] == 0).all()


@pytest.mark.parametrize("shape,masked", [((1, 2, 777, 64, 32), False), ((2, 2, 1000, 128, 16), True), ((1, 1, 300, 256, 64), False),
                                          ((2, 3, 97, 48, 32), True), ((1, 1, 1300, 512, 32), False)])
def test_fp32_halves_backward_vs_autograd_oracle(dev, shape, masked):
    """flare_gather and flare_scatter called separately with a layer between them (what the ablation models do,
    pdebench/models/flare_ablations.py): fp32 gradients of q, k, v from the HIP kernels of the two halves
    (flare_gather_bwd, flare_scatter_bwd) against fp64 autograd through the explicit formulas."""
    B, H, N, M, D = shape
    q, k, v, gy = make(*shape, torch.float32, seed=3 + N)
    w = torch.randn(D, D, generator=torch.Generator().manual_seed(1)) * D ** -0.5         # the layer between the halves
    mask = None
    if masked:
        mask = torch.ones(B, N, dtype=torch.bool)
        mask[0, N // 2:] = False
        mask[-1, ::4] = False
    qd, kd, vd, wd = (t.to(dev).requires_grad_(True) for t in (q, k, v, w))
    md = None if mask is None else mask.to(dev)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CUDA]) as prof:
        z, _ = F.flare_gather(qd, kd, vd, scale=0.9, key_mask=md)
        y = F.flare_scatter(qd, kd, torch.tanh(z @ wd), scale=0.9, key_mask=md)
        y.backward(gy.to(dev))
        torch.cuda.synchronize()
    kernels = " ".join(e.key for e in prof.key_averages())
    assert "bwd_f32_tok_kernel" in kernels and "bwd_f32_delta_kernel" in kernels, kernels
    qr, kr, vr, wr = (t.double().requires_grad_(True) for t in (q, k, v, w))
    zr = O.gather_explicit(qr, kr, vr, 0.9, mask)
    zr = zr[0] if isinstance(zr, tuple) else zr
    yr = O.scatter_explicit(qr, kr, torch.tanh(zr @ wr), 0.9, mask)
    yr.backward(gy.double())
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad), ("dw", wd.grad, wr.grad)):
        err = float((got.cpu().double() - ref).norm() / ref.norm())
        assert err <= 1e-4, f"{name} rel-L2 {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,masked", [((1, 2, 777, 64, 32), False), ((2, 2, 1000, 128, 16), True), ((1, 1, 300, 256, 64), False),
                                          ((2, 3, 97, 96, 32), True), ((1, 1, 1300, 512, 32), False), ((2, 2, 4000, 256, 32), False),
                                          ((3, 1, 2100, 128, 32), True)])
def test_16bit_halves_backward_vs_autograd_oracle(dev, dtype, shape, masked):
    """The two halves with a layer between them in bf16 / f16 (pdebench/models/flare_ablations.py under autocast): gradients
    from flare_gather_bwd / flare_scatter_bwd, which run the whole mixer's kernels with the other half's softmax weights
    switched off, against fp64 autograd through the explicit formulas on the same 16-bit inputs.  Bars: bf16 3e-2, f16 1e-2
    relative L2; z passes through the layer in fp32 here, so the only rounding is the kernels' own."""
    B, H, N, M, D = shape
    q, k, v, gy = make(*shape, dtype, seed=5 + N)
    w = torch.randn(D, D, generator=torch.Generator().manual_seed(1)) * D ** -0.5
    mask = None
    if masked:
        mask = torch.ones(B, N, dtype=torch.bool)
        mask[0, N // 2:] = False
        mask[-1, ::4] = False
        if B > 2:
            mask[1] = False          # a batch element without tokens
    qd, kd, vd, wd = (t.to(dev).requires_grad_(True) for t in (q, k, v, w))
    md = None if mask is None else mask.to(dev)
    assert FN._half_hip_ok(qd, kd, vd, md, False)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CUDA]) as prof:
        z, _ = F.flare_gather(qd, kd, vd, scale=0.9, key_mask=md)
        y = F.flare_scatter(qd, kd, torch.tanh(z @ wd), scale=0.9, key_mask=md)
        y.backward(gy.to(dev))
        torch.cuda.synchronize()
    kernels = " ".join(e.key for e in prof.key_averages())
    assert "bwd_half_prep_kernel" in kernels and "bwd_tok" in kernels, kernels
    qr, kr, vr, wr = (t.double().requires_grad_(True) for t in (q, k, v, w))
    zr = O.gather_explicit(qr, kr, vr, 0.9, mask)
    zr = zr[0] if isinstance(zr, tuple) else zr
    yr = O.scatter_explicit(qr, kr, torch.tanh(zr @ wr), 0.9, mask)
    yr.backward(gy.double())
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-2
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad), ("dw", wd.grad, wr.grad)):
        assert torch.isfinite(got).all(), name
        err = float((got.cpu().double() - ref).norm() / ref.norm())
        assert err <= tol, f"{name} rel-L2 {err:.3e}"
    if masked:
        assert (kd.grad[0, :, N // 2:] == 0).all() and (vd.grad[0, :, N // 2:] == 0).all()


def test_lse_outputs(dev):
    q, k, v, _ = make(1, 2, 500, 64, 32, torch.bfloat16, seed=9)
    y, z, lse_lat, lse_tok = FN._mixer_forward(q.to(dev), k.to(dev), v.to(dev), 0.7, None, 0, False, False, True)
    s = 0.7 * torch.einsum("hmd,bhnd->bhmn", q.double(), k.double())
    assert float((lse_lat.cpu().double() - torch.logsumexp(s, -1)).abs().max()) <= 2e-2
    assert float((lse_tok.cpu().double() - torch.logsumexp(s, -2)).abs().max()) <= 2e-2
    yg, zg, _, lt = FN._mixer_forward(q.to(dev), k.to(dev), v.to(dev), 0.7, None, 0, True, False, True)   # fp32-FMA kernels
    assert float((lt - lse_tok).abs().max()) <= 2e-2


@pytest.mark.parametrize("a", [3.0, 5.0, 6.75])
def test_backward_with_log_sum_exps_far_apart(dev, a):
    """The kernels form the token scatter's weights from the gather's (one exponential per score) only while the
    latents' largest log-sum-exp and the tokens' smallest are at most 2^64 apart, and take both exponentials
    otherwise.  Half of the tokens score +a^2 with every latent, the other half -a^2: a = 3 stays inside that span,
    a = 5 leaves it, and at a = 6.75 the gather's weights of the second half underflow in fp32 while their own
    softmax over the latents still decides their gradients."""
    B, H, N, M, D = 1, 2, 600, 64, 32
    q, k, v, gy = make(B, H, N, M, D, torch.bfloat16, seed=31)
    q[..., 0] = a
    k[..., 0] = a
    k[:, :, ::2, 0] = -a
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert FN._hip_backward_ok(qd, kd, vd, None, False)
    F.flare_multihead_mixer(qd, kd, vd).backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 1.0)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        assert torch.isfinite(got).all()
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"
    # The tokens of the low half on their own: their gradients are small next to the others' and must still be right.
    # They are differences <dy_n, z_m - y_n> of latent rows that are nearly equal here (every latent sees the same
    # dominant tokens) and enter the matrix cores rounded to bf16, hence the wider bar.
    err = O.rel_l2(kd.grad[:, :, ::2], gk[:, :, ::2])
    assert err <= 6e-2, f"dk of the low-scoring tokens rel-L2 {err:.3e}"


@pytest.mark.parametrize("a", [7.5, -7.5])
@pytest.mark.parametrize("M", [64, 256, 512])
def test_backward_with_large_log_sum_exps(dev, a, M):
    """The bf16 kernels on the 32x32x16 product take exp2(S) for the gather's weights and apply exp2(-L2_m) elsewhere
    while every latent log-sum-exp stays within +-60 (log2 units).  Every score near +56 or -56 puts all of them outside
    (the span between the two families of log-sum-exps stays small): these (b,h) take the general form, the dq pass in
    its plain passes and the token pass in the 16x16x32 kernel launched behind the 32x32x16 one; head 1 stays inside
    and takes the fast kernels in the same launch."""
    B, H, N, D = 1, 2, 700, 32
    q, k, v, gy = make(B, H, N, M, D, torch.bfloat16, seed=37)
    q[0, :, 0] = abs(a)
    k[:, 0, :, 0] = a
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    lse2 = torch.logsumexp(s, -1) * 1.4426950408889634
    assert float(lse2[0, 0].abs().min()) > 60 and float(lse2[0, 1].abs().max()) < 60
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert FN._hip_backward_ok(qd, kd, vd, None, False)
    F.flare_multihead_mixer(qd, kd, vd).backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 1.0)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        assert torch.isfinite(got).all()
        for hd in range(H):
            sl = (slice(None), hd) if name != "dq" else (hd,)
            err = O.rel_l2(got[sl], ref[sl])
            assert err <= 3e-2, f"{name} head {hd} rel-L2 {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_masked_backward_vs_autograd_oracle(dev, dtype):
    """Key mask (lra/models/backends.py:603-622) through the HIP backward: holes, a padded tail, a batch element with a
    single real token and one with none; padded rows hold NaN in k, v and dy and must not reach any gradient."""
    B, H, N, M, D = 4, 2, 1500, 128, 32
    q, k, v, gy = make(B, H, N, M, D, dtype, seed=13)
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, 900:] = False
    mask[0, 5:700:7] = False
    mask[1, 1:] = False
    mask[2] = False
    m4 = mask[:, None, :, None]
    nan = torch.full((), float("nan"), dtype=dtype)
    qd = q.to(dev).requires_grad_(True)
    kd, vd = (torch.where(m4, t, nan).to(dev).requires_grad_(True) for t in (k, v))
    assert FN._hip_backward_ok(qd, kd, vd, mask.to(dev), False)
    y = F.flare_multihead_mixer(qd, kd, vd, scale=0.9, key_mask=mask.to(dev))
    y.backward(torch.where(m4, gy, nan).to(dev))
    real = [0, 1, 3]                   # the oracle differentiates the batch elements that hold tokens; the empty one adds 0
    qr = q.double().requires_grad_(True)
    kr, vr = (t[real].double().requires_grad_(True) for t in (k, v))
    yr, _ = O.mixer_explicit(qr, kr, vr, 0.9, mask[real])
    yr.backward((gy.double() * m4)[real])
    assert torch.isfinite(qd.grad).all() and torch.isfinite(kd.grad).all() and torch.isfinite(vd.grad).all()
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad[real], kr.grad), ("dv", vd.grad[real], vr.grad)):
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"
    assert (kd.grad.cpu()[~m4.expand_as(k)] == 0).all() and (vd.grad.cpu()[~m4.expand_as(v)] == 0).all()


def test_narrow_head_backward(dev):
    """D = 8 (zero-padded to 16 around the kernels): gradients through the HIP backward against the fp64 oracle."""
    q, k, v, gy = make(2, 8, 2000, 64, 8, torch.bfloat16, seed=17)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    y = F.flare_multihead_mixer(qd, kd, vd, scale=1.1)
    assert y.shape == (2, 8, 2000, 8)
    y.backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 1.1)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        assert got.shape == ref.shape
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


@pytest.mark.parametrize("shape", [(1, 2, 1500, 256, 64), (1, 1, 1200, 512, 32), (1, 1, 900, 512, 64), (1, 1, 700, 1024, 32)])
def test_backward_with_latents_in_chunks(dev, shape):
    """M * D beyond one LDS-full of operand sets (160 KB = M * D of 16384): the token-side kernel runs once per chunk
    of latents and adds to dk, dv; at exactly 16384 everything is resident with the per-latent scalars read from global."""
    q, k, v, gy = make(*shape, torch.bfloat16, seed=19)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert FN._hip_backward_ok(qd, kd, vd, None, False)
    F.flare_multihead_mixer(qd, kd, vd, scale=0.8).backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 0.8)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


def test_z_handed_out_under_autograd_carries_gradients(dev):
    """flare_multihead_mixer(..., return_z=True) with gradients required: a loss that uses z as well as y must
    reach q, k, v through both (autograd of the explicit-softmax oracle in fp64 is the reference)."""
    q, k, v, gy = make(2, 2, 600, 64, 32, torch.bfloat16, seed=21)
    gz = torch.randn(2, 2, 64, 32, generator=torch.Generator().manual_seed(22))
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    y, z = F.flare_multihead_mixer(qd, kd, vd, scale=0.7, return_z=True)
    assert z.requires_grad
    ((y.float() * gy.to(dev).float()).sum() + (z * gz.to(dev)).sum()).backward()
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    yr, zr = O.mixer_explicit(qr, kr, vr, 0.7)
    ((yr * gy.double()).sum() + (zr * gz.double()).sum()).backward()
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


def test_backward_of_a_view_off_the_16_byte_grid(dev):
    """k, v views whose first element is not 16-byte aligned: the HIP backward does not take them, the gradients
    must come from the torch recomputation instead of an error."""
    q, k, v, gy = make(1, 2, 400, 64, 32, torch.bfloat16, seed=23)
    kb = torch.zeros(k.numel() + 4, dtype=k.dtype)
    vb = torch.zeros(v.numel() + 4, dtype=v.dtype)
    kb[4:] = k.reshape(-1)
    vb[4:] = v.reshape(-1)
    kd = kb.to(dev)[4:].view_as(k).requires_grad_(True)        # starts 8 bytes into the allocation
    vd = vb.to(dev)[4:].view_as(v).requires_grad_(True)
    assert kd.data_ptr() % 16 != 0
    assert not FN._hip_backward_ok(q.to(dev), kd, vd, None, False)
    qd = q.to(dev).requires_grad_(True)
    F.flare_multihead_mixer(qd, kd, vd, scale=0.9).backward(gy.to(dev))
    want = oracle_grads(q, k, v, gy, 0.9)
    for name, got, ref in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), want):
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


def test_fp32_backward_at_262144_tokens_stays_inside_a_memory_bound(dev):
    """fp32 inputs differentiate through the token-tiled recomputation: at N = 262,144, M = 256 it must never hold
    the [B,H,M,N] scores (268 MB per copy here; the old recomputation kept about eight of them) — peak extra
    memory is bounded by a few [B,H,M,T] tiles of 64 MiB — and match fp64 autograd of the explicit formulas,
    evaluated on the device, to 1e-4."""
    B, H, N, M, D = 1, 1, 262144, 256, 32
    g = torch.Generator().manual_seed(51)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).to(dev)
    k, v, gy = (torch.randn(B, H, N, D, generator=g).to(dev) for _ in range(3))
    qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    F.flare_multihead_mixer(qd, kd, vd, scale=0.9).backward(gy)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - base
    assert extra < 900 * 2 ** 20, f"{extra / 2 ** 20:.0f} MiB"        # y, grads, workspace (~140 MiB) + tiles (~450 MiB)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    s = 0.9 * (qr.unsqueeze(0) @ kr.mT)
    y = torch.softmax(s.mT, -1) @ (torch.softmax(s, -1) @ vr)
    y.backward(gy.double())
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        err = float((got.double() - ref).norm() / ref.norm())
        assert err <= 1e-4, f"{name} rel-L2 {err:.3e}"


def test_gradients_in_the_layout_of_token_major_inputs():
    """k and v that are views of [B,N,H,D] storage (a projection's output) get dk, dv in that layout
    (FLARE_FLAG_GRAD_LIKE_KV): same numbers as for head-major copies, and the [B,N,H*D] view of the gradient is
    contiguous."""
    torch.manual_seed(5)
    B, H, N, M, D = 2, 4, 1500, 64, 32
    dev = torch.device("cuda:0")
    q = (torch.randn(H, M, D, device=dev) * 0.3).bfloat16().requires_grad_(True)
    kt = torch.randn(B, N, H, D, device=dev).bfloat16().requires_grad_(True)
    vt = torch.randn(B, N, H, D, device=dev).bfloat16().requires_grad_(True)
    gy = torch.randn(B, H, N, D, device=dev).bfloat16()
    y = F.flare_multihead_mixer(q, kt.permute(0, 2, 1, 3), vt.permute(0, 2, 1, 3))
    y.backward(gy)
    got = (q.grad.clone(), kt.grad.clone(), vt.grad.clone())
    assert kt.grad.is_contiguous() and vt.grad.is_contiguous()
    q.grad = None
    kh = kt.detach().permute(0, 2, 1, 3).contiguous().requires_grad_(True)
    vh = vt.detach().permute(0, 2, 1, 3).contiguous().requires_grad_(True)
    F.flare_multihead_mixer(q, kh, vh).backward(gy)
    assert torch.equal(got[0], q.grad)
    assert torch.equal(got[1], kh.grad.permute(0, 2, 1, 3))
    assert torch.equal(got[2], vh.grad.permute(0, 2, 1, 3))


@pytest.mark.parametrize("shape", [(1, 2, 1, 40, 24), (1, 2, 7, 40, 16), (2, 1, 13, 24, 32), (1, 1, 300, 8, 16)])
def test_fp32_torch_recomputation_from_the_forwards_statistics_at_small_sizes(dev, shape):
    """fp32 latent counts that are not multiples of 16 differentiate through the tiled torch recomputation, which starts
    from the forward's own z, latent log-sum-exp and y.  One token, fewer tokens than a tile and odd latent counts; with
    a single token the true dq and dk are exactly 0 (the softmax over one token is constant), so those are held to an
    absolute bound instead of a relative one."""
    q, k, v, gy = make(*shape, torch.float32, seed=sum(shape))
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    assert not FN._hip_backward_ok(qd, kd, vd, None, False)
    F.flare_multihead_mixer(qd, kd, vd, scale=0.7).backward(gy.to(dev))
    gq, gk, gv = oracle_grads(q, k, v, gy, 0.7)
    for name, got, ref in (("dq", qd.grad, gq), ("dk", kd.grad, gk), ("dv", vd.grad, gv)):
        if float(ref.norm()) > 1e-6:
            err = float((got.cpu().double() - ref).norm() / ref.norm())
            assert err <= 1e-4, f"{name} rel-L2 {err:.3e}"
        else:
            assert float(got.abs().max()) <= 1e-5, name
