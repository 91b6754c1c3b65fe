"""GPU parity of causal linear attention (CausalLinear.apply) vs the CPU oracle.

The oracle is the token recurrence of lra/models/triton/causal_linear.py:317-336, pinned in
tests/test_oracle.py by the closed form tril(QK^T)V/N.  Tolerances: 1e-5 (fp32) and 2e-2 (bf16/f16)
relative L2 on the same rounded inputs (the reference's own self-test uses allclose 1e-5 / 1e-3,
causal_linear.py:455-457).
"""
import pytest
import torch

import flare_py_amd as F
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def make(B, H, N, Dk, Dv, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, H, N, Dk, generator=g).to(dtype), torch.randn(B, H, N, Dk, generator=g).to(dtype),
            torch.randn(B, H, N, Dv, generator=g).to(dtype))


@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (2, 3, 37, 5, 3), (1, 2, 64, 16, 16), (1, 2, 65, 16, 8),
                                   (2, 2, 300, 24, 40), (1, 2, 1000, 128, 128), (1, 1, 513, 100, 7)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_shapes_vs_recurrence(dev, shape, dtype):
    q, k, v = make(*shape, dtype)
    y = F.CausalLinear.apply(q.to(dev), k.to(dev), v.to(dev))
    yr = O.causal_linear_closed_form(q, k, v)
    assert y.dtype == dtype and y.shape == v.shape
    assert O.rel_l2(y, yr) <= TOL[dtype]


def test_reference_selftest_shape_fp32(dev):
    # the shape of the reference's own test: B=1, H=8, N=2048, Dk=128, Dv=32, fp32 (causal_linear.py:650)
    q, k, v = make(1, 8, 2048, 128, 32, torch.float32, seed=1)
    y = F.CausalLinear.apply(q.to(dev), k.to(dev), v.to(dev))
    yr = O.causal_linear_recurrent(q[:, :2], k[:, :2], v[:, :2])      # token loop on two heads
    assert O.rel_l2(y[:, :2], yr) <= 1e-5
    assert O.rel_l2(y, O.causal_linear_closed_form(q, k, v)) <= 1e-5
    assert torch.allclose(y.cpu().double(), O.causal_linear_closed_form(q, k, v), atol=1e-5, rtol=1e-5)


def test_segment_count_independence_and_determinism(dev):
    q, k, v = make(1, 2, 1500, 32, 32, torch.float32, seed=2)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    yr = O.causal_linear_closed_form(q, k, v)
    for s in (1, 2, 5, 24, 1000):
        y = F.causal_linear_attention(qd, kd, vd, n_segs=s)
        assert torch.equal(y, F.causal_linear_attention(qd, kd, vd, n_segs=s))
        assert O.rel_l2(y, yr) <= 1e-5, s


def test_last_row_is_noncausal_linear_attention_and_strided_views(dev):
    B, H, N, D = 2, 4, 200, 16
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, B, N, H * D, generator=g).to(dev)
    q, k, v = (t.view(B, N, H, D).permute(0, 2, 1, 3) for t in x)     # 'b n (h d) -> b h n d' views, no copy
    y = F.causal_linear_attention(q, k, v)
    full = q[:, :, -1:].double() @ (k.double().mT @ v.double()) / N
    assert O.rel_l2(y[:, :, -1:], full.cpu()) <= 1e-5
    assert O.rel_l2(y, O.causal_linear_closed_form(q.cpu(), k.cpu(), v.cpu())) <= 1e-5


def test_errors_and_autograd_plumbing(dev):
    q, k, v = make(1, 1, 32, 8, 8, torch.float32)
    with pytest.raises(ValueError):
        F.CausalLinear.apply(q.to(dev), k[:, :, :16].to(dev), v.to(dev))
    with pytest.raises(NotImplementedError):
        F.CausalLinear.apply(torch.zeros(1, 1, 8, 200, device=dev), torch.zeros(1, 1, 8, 200, device=dev),
                             torch.zeros(1, 1, 8, 4, device=dev))
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    y = F.CausalLinear.apply(qd, kd, vd)
    y.square().sum().backward()
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.causal_linear_closed_form(qr, kr, vr).square().sum().backward()
    for a, b in ((qd, qr), (kd, kr), (vd, vr)):
        assert O.rel_l2(a.grad, b.grad) <= 1e-4


# ---- matrix-core kernels (Dk in {64, 128}; bf16 / f16 with Dv in {32, 64, 128}, fp32 with Dv in {32, 64}) ------
@pytest.mark.parametrize("shape", [(1, 2, 64, 64, 32), (1, 2, 65, 64, 32), (2, 2, 300, 64, 64), (1, 1, 513, 128, 32),
                                   (1, 3, 1, 64, 128), (2, 1, 17, 128, 64), (1, 2, 4096, 64, 32), (1, 1, 2500, 128, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_matrix_core_shapes(dev, shape, dtype):
    """Every segment count gives the oracle's result (the state crosses tile and segment boundaries), twice the same
    bits, and close to the fp32-arithmetic kernel on the same inputs."""
    if dtype == torch.float32 and shape[4] > 64:
        shape = shape[:4] + (64,)             # the fp32 kernels (16x16x4 products) take Dv up to 64
    q, k, v = make(*shape, dtype, seed=shape[2])
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    yr = O.causal_linear_closed_form(q, k, v)
    for s in (0, 1, 3):
        y = F.causal_linear_attention(qd, kd, vd, n_segs=s)
        assert y.dtype == dtype and torch.equal(y, F.causal_linear_attention(qd, kd, vd, n_segs=s))
        assert O.rel_l2(y, yr) <= TOL[dtype], s
    yg = F.causal_linear_attention(qd, kd, vd, force_generic=True)
    assert O.rel_l2(y, yg.cpu()) <= TOL[dtype]


def test_matrix_core_kernel_runs_and_takes_token_major_views(dev):
    """The reference's own test shape in bf16, q, k, v as 'b n (h d) -> b h n d' views: the matrix-core kernels run
    (profiler), no copy is made, and rows that are not 16-byte aligned fall back to the fp32-arithmetic kernel."""
    from torch.profiler import ProfilerActivity, profile
    B, H, N, Dk, Dv = 1, 8, 2048, 128, 32
    g = torch.Generator().manual_seed(7)
    xq = torch.randn(2, B, N, H * Dk, generator=g).bfloat16().to(dev)
    xv = torch.randn(B, N, H * Dv, generator=g).bfloat16().to(dev)
    q, k = (t.view(B, N, H, Dk).permute(0, 2, 1, 3) for t in xq)
    v = xv.view(B, N, H, Dv).permute(0, 2, 1, 3)
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        y = F.causal_linear_attention(q, k, v)
        torch.cuda.synchronize()
    names = {e.key for e in prof.key_averages()}
    assert any("causal_linear_mfma_kernel" in n for n in names), names
    assert not any("copy" in n.lower() for n in names), names
    yr = O.causal_linear_closed_form(q.cpu(), k.cpu(), v.cpu())
    assert O.rel_l2(y, yr) <= 2e-2
    # a view that starts 8 bytes into a row: the same values through the other kernel
    pad = torch.zeros(B, H, N, Dk + 4, dtype=torch.bfloat16, device=dev)
    pad[..., 4:] = q
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        y2 = F.causal_linear_attention(pad[..., 4:], k, v)
        torch.cuda.synchronize()
    assert not any("causal_linear_mfma_kernel" in e.key for e in prof.key_averages())
    assert O.rel_l2(y2, yr) <= 2e-2


def test_fp32_matrix_core_kernel_runs_at_the_reference_shape(dev):
    """B=1, H=8, N=2048, Dk=128, Dv=32 in fp32 (causal_linear.py:650) goes through the 16x16x4 fp32 products."""
    from torch.profiler import ProfilerActivity, profile
    q, k, v = make(1, 8, 2048, 128, 32, torch.float32, seed=3)
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        y = F.causal_linear_attention(q.to(dev), k.to(dev), v.to(dev))
        torch.cuda.synchronize()
    assert any("causal_linear_f32_kernel" in e.key for e in prof.key_averages())
    yr = O.causal_linear_closed_form(q, k, v)
    assert O.rel_l2(y, yr) <= 1e-5
    assert torch.allclose(y.cpu().double(), yr, atol=1e-5, rtol=1e-5)
    yg = F.causal_linear_attention(q.to(dev), k.to(dev), v.to(dev), force_generic=True)
    assert O.rel_l2(yg, yr) <= 1e-5


@pytest.mark.parametrize("shape,dtype,tol", [((2, 2, 700, 64, 64), torch.bfloat16, 3e-2), ((1, 2, 1000, 128, 32), torch.float16, 3e-2),
                                             ((1, 3, 333, 64, 32), torch.float32, 1e-4), ((2, 1, 100, 24, 40), torch.float32, 1e-4)])
def test_gradients_through_the_same_kernels(dev, shape, dtype, tol):
    """dq, dk, dv are causal linear attentions themselves (dk, dv on the reversed token axis): against fp64 autograd of
    the closed form on the same rounded inputs."""
    q, k, v = make(*shape, dtype, seed=9)
    g = torch.Generator().manual_seed(10)
    gy = torch.randn(shape[0], shape[1], shape[2], shape[4], generator=g).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.CausalLinear.apply(qd, kd, vd).backward(gy.to(dev))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.causal_linear_closed_form(qr, kr, vr).backward(gy.double())
    for a, b in ((qd, qr), (kd, kr), (vd, vr)):
        assert a.grad.dtype == dtype and a.grad.shape == b.grad.shape
        assert O.rel_l2(a.grad, b.grad) <= tol
