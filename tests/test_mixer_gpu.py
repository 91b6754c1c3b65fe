"""GPU parity tests of the FLARE mixer: HIP kernels (through the C-ABI) vs the CPU oracle.

Tolerances are the ones the task states: relative L2 error <= 1e-5 for fp32 and <= 2e-2 for
bf16/f16, both measured against the fp32/fp64 oracle evaluated on the SAME (already rounded)
inputs upcast, so input rounding is not charged to the kernel.
"""
import pytest
import torch

import flare_py_amd as F
from oracle import c_oracle
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def make(B, H, N, M, D, dtype, seed=0, qstd=None, kstd=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(H, M, D, generator=g) * (D ** -0.5 if qstd is None else qstd)).to(dtype)
    k = (torch.randn(B, H, N, D, generator=g) * kstd).to(dtype)
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    return q, k, v


def check(dev, q, k, v, scale=1.0, key_mask=None, tol=None, **kw):
    y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=scale,
                                   key_mask=None if key_mask is None else key_mask.to(dev),
                                   return_z=True, **kw)
    torch.cuda.synchronize()
    yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), scale, key_mask)
    tol = TOL[k.dtype] if tol is None else tol
    ez, ey = O.rel_l2(z, zr), O.rel_l2(y, yr)
    assert torch.isfinite(y.float()).all()
    assert ez <= tol, f"z rel-L2 {ez:.3e} > {tol}"
    assert ey <= tol, f"y rel-L2 {ey:.3e} > {tol}"
    return y, z


def test_cfg1_fp32_vs_sdpa_oracle(dev):
    # BASELINE config 1: q[8,64,16]~N(0,1/D), k,v[1,8,4096,16]~N(0,1), scale 1, fp32, seed 0
    q, k, v = make(1, 8, 4096, 64, 16, torch.float32)
    assert F.mixer_kernel_name(q, k, v) == "generic"
    y = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev))
    ys, _ = O.mixer_sdpa(q, k, v, 1.0)      # torch SDPA, MATH backend, CPU (README.md:49-50)
    yc, _ = c_oracle.mixer(q, k, v, 1.0)    # plain-C restatement
    assert O.rel_l2(y, ys) <= 1e-5
    assert O.rel_l2(y, yc) <= 1e-5


@pytest.mark.parametrize("shape", [
    (1, 1, 1, 1, 1), (2, 3, 37, 5, 4), (1, 2, 300, 16, 8), (2, 2, 1000, 70, 24), (1, 1, 513, 130, 128),
    (1, 4, 2048, 64, 16),
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_generic_shapes(dev, shape, dtype):
    q, k, v = make(*shape, dtype)
    check(dev, q, k, v, scale=0.7, force_generic=True)


@pytest.mark.parametrize("shape", [
    (1, 2, 64, 64, 32), (1, 2, 200, 64, 32), (2, 2, 1000, 128, 32), (1, 3, 4096, 256, 32),
    (1, 2, 777, 64, 16), (1, 2, 3000, 128, 16), (1, 1, 2500, 256, 64), (1, 1, 1111, 192, 64),
    (1, 1, 900, 512, 32), (1, 2, 5000, 320, 16),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mfma_shapes(dev, shape, dtype):
    q, k, v = make(*shape, dtype)
    assert F.mixer_kernel_name(q, k, v).startswith("mfma")
    check(dev, q, k, v)


@pytest.mark.parametrize("scale", [0.25, 1.0, 3.0])
def test_mfma_scale(dev, scale):
    q, k, v = make(1, 2, 1500, 128, 32, torch.bfloat16)
    check(dev, q, k, v, scale=scale)


def test_mfma_matches_generic_kernels(dev):
    q, k, v = make(2, 2, 3000, 256, 32, torch.bfloat16)
    y1, z1 = check(dev, q, k, v)
    y2, z2 = check(dev, q, k, v, force_generic=True)
    assert O.rel_l2(z1, z2) < 1e-2 and O.rel_l2(y1, y2) < 1.5e-2


def test_strided_views_no_copy(dev):
    # k, v as the 'b n (h d) -> b h n d' views the block modules produce; q expanded over batch
    B, H, N, M, D = 2, 4, 700, 64, 32
    g = torch.Generator().manual_seed(3)
    kx = torch.randn(B, N, H * D, generator=g).bfloat16().to(dev)
    vx = torch.randn(B, N, H * D, generator=g).bfloat16().to(dev)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).bfloat16().to(dev)
    k = kx.view(B, N, H, D).permute(0, 2, 1, 3)
    v = vx.view(B, N, H, D).permute(0, 2, 1, 3)
    assert not k.is_contiguous()
    for fg in (False, True):
        y = F.flare_multihead_mixer(q, k, v, force_generic=fg)
        yr, _ = O.mixer_explicit(q.float().cpu(), k.float().cpu(), v.float().cpu())
        assert O.rel_l2(y, yr) <= 2e-2
    # per-batch latent queries
    qb = (torch.randn(B, H, M, D, generator=g) * D ** -0.5).bfloat16().to(dev)
    y = F.flare_multihead_mixer(qb, k, v)
    yr, _ = O.mixer_explicit(qb.float().cpu(), k.float().cpu(), v.float().cpu())
    assert O.rel_l2(y, yr) <= 2e-2


@pytest.mark.parametrize("dtype,fg", [(torch.float32, True), (torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_key_mask(dev, dtype, fg):
    q, k, v = make(3, 2, 333, 64, 32, dtype, seed=5)
    mask = torch.ones(3, 333, dtype=torch.bool)
    mask[0, 100:] = False
    mask[1, 1:] = False          # a single real token
    mask[2, ::3] = False         # holes
    y, _ = check(dev, q, k, v, key_mask=mask, force_generic=fg)
    assert (y.cpu()[~mask[:, None, :, None].expand_as(y)] == 0).all()


@pytest.mark.parametrize("fg", [False, True])
@pytest.mark.parametrize("garbage", [0.0, 300.0, float("nan")])
def test_key_mask_over_many_splits_and_padding_garbage(dev, garbage, fg):
    """A long masked batch: whole split ranges without a real token (their zero denominators are legitimate), ranges
    that end in padding, and padded rows holding values that overflow the unshifted exponentials or are NaN
    (the kernel then repeats the range exactly; padding must never reach the result)."""
    q, k, v = make(3, 2, 8192, 128, 32, torch.bfloat16, seed=11)
    mask = torch.ones(3, 8192, dtype=torch.bool)
    mask[1, 100:] = False
    mask[2, 5000:] = False
    mask[2, 17:4000:5] = False
    kk, vv = k.clone(), v.clone()
    if garbage != 0.0:
        kk[~mask[:, None, :, None].expand_as(k)] = garbage
        vv[~mask[:, None, :, None].expand_as(v)] = garbage
    y, z = F.flare_multihead_mixer(q.to(dev), kk.to(dev), vv.to(dev), key_mask=mask.to(dev), return_z=True,
                                   force_generic=fg)
    yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 1.0, mask)
    keep = mask[:, None, :, None].expand_as(yr)
    assert torch.isfinite(z).all() and O.rel_l2(z, zr) <= 2e-2
    assert O.rel_l2(y.float().cpu()[keep], yr[keep]) <= 2e-2
    assert (y.cpu()[~keep] == 0).all()


def test_fully_masked_batch_gives_zero(dev):
    q, k, v = make(2, 1, 130, 64, 32, torch.bfloat16)
    mask = torch.ones(2, 130, dtype=torch.bool)
    mask[1] = False
    for fg in (False, True):
        y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), key_mask=mask.to(dev), return_z=True,
                                       force_generic=fg)
        assert (z[1] == 0).all() and (y[1] == 0).all() and torch.isfinite(y.float()).all()


@pytest.mark.parametrize("fg", [False, True])
def test_large_scores_exact_path(dev, fg):
    # Scores that grow along N and along M by far more than the lazy-shift window: the kernels
    # must take their exact rescaling path and stay finite and accurate.
    B, H, N, M, D = 1, 2, 2048, 128, 32
    g = torch.Generator().manual_seed(7)
    q = torch.randn(H, M, D, generator=g)
    k = torch.randn(B, H, N, D, generator=g)
    q = q * torch.linspace(0.2, 2.0, M)[None, :, None]          # later latents score higher
    k = k * torch.linspace(0.2, 3.0, N)[None, None, :, None]    # later tokens score higher
    v = torch.randn(B, H, N, D, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    assert float(s.max()) > 40.0
    check(dev, q, k, v, force_generic=fg, tol=3e-2)


def test_split_invariance_and_determinism(dev):
    q, k, v = make(1, 2, 5000, 128, 32, torch.bfloat16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    ref = None
    for s in (1, 2, 5, 16):
        y, z = F.flare_multihead_mixer(qd, kd, vd, return_z=True, n_splits=s)
        y2, z2 = F.flare_multihead_mixer(qd, kd, vd, return_z=True, n_splits=s)
        assert torch.equal(y, y2) and torch.equal(z, z2)       # bit-stable for a fixed split
        if ref is None:
            ref = z
        assert O.rel_l2(z, ref) < 5e-3                          # any split: same result up to rounding


def test_closed_forms_on_device(dev):
    q, k, v = make(1, 2, 1000, 64, 32, torch.bfloat16)
    c = torch.full_like(v, 1.5)
    y = F.flare_multihead_mixer(q.to(dev), k.to(dev), c.to(dev))
    assert torch.allclose(y.float().cpu(), c.float(), atol=1e-2)          # constant v -> constant y
    y, z = F.flare_multihead_mixer(torch.zeros_like(q).to(dev), k.to(dev), v.to(dev), return_z=True)
    mean = v.float().mean(dim=2, keepdim=True)
    assert torch.allclose(z.cpu(), mean.expand_as(z), atol=2e-3)          # q = 0 -> z = mean(v)
    assert torch.allclose(y.float().cpu(), mean.expand_as(y), atol=1e-2)


def test_gather_and_scatter_entry_points(dev):
    q, k, v = make(1, 2, 900, 64, 32, torch.bfloat16)
    z, lse = F.flare_gather(q.to(dev), k.to(dev), v.to(dev), scale=0.9)
    zr, lser = O.gather_explicit(q.float(), k.float(), v.float(), 0.9)
    assert O.rel_l2(z, zr) <= 2e-2
    assert float((lse.cpu().double() - lser).abs().max()) < 2e-2
    y = F.flare_scatter(q.to(dev), k.to(dev), zr.float().to(dev), scale=0.9)
    yr = O.scatter_explicit(q.float(), k.float(), zr, 0.9)
    assert O.rel_l2(y, yr) <= 2e-2


def test_headline_shape_properties_and_sampled_parity(dev):
    # BASELINE headline: B=1,H=8,N=1,048,576,M=256,D=32 bf16, q~N(0,1/D), k,v~N(0,1), scale 1.
    B, H, N, M, D = 1, 8, 1 << 20, 256, 32
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).bfloat16()
    k = torch.randn(B, H, N, D, generator=g).bfloat16()
    v = torch.randn(B, H, N, D, generator=g).bfloat16()
    y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), return_z=True)
    torch.cuda.synchronize()
    y, z = y.cpu(), z.cpu()
    assert torch.isfinite(y.float()).all()
    # size-independent properties: y in the convex hull of z rows, z in that of v rows
    assert (y.float() <= z.amax(2, keepdim=True) + 2e-2).all() and (y.float() >= z.amin(2, keepdim=True) - 2e-2).all()
    assert (z <= v.float().amax(2, keepdim=True)).all() and (z >= v.float().amin(2, keepdim=True)).all()
    # oracle on one head for z (full N) and on sampled tokens for y
    h = 5
    zr, _ = O.gather_explicit(q[h : h + 1].float(), k[:, h : h + 1].float(), v[:, h : h + 1].float(), 1.0,
                              dtype=torch.float32)
    assert O.rel_l2(z[:, h : h + 1], zr) <= 2e-2
    idx = torch.randint(0, N, (4096,), generator=g)
    yr = O.scatter_explicit(q[h : h + 1].float(), k[:, h : h + 1, idx].float(), zr.double(), 1.0)
    assert O.rel_l2(y[:, h : h + 1, idx], yr) <= 2e-2
    # determinism at full size
    y2 = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev)).cpu()
    assert torch.equal(y, y2)


def test_autograd_plumbing(dev):
    q, k, v = make(1, 2, 200, 64, 32, torch.float32)
    q, k, v = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    y = F.flare_multihead_mixer(q, k, v)
    y.square().sum().backward()
    qr, kr, vr = (t.detach().cpu().double().requires_grad_(True) for t in (q, k, v))
    yr, _ = O.mixer_explicit(qr, kr, vr)
    yr.square().sum().backward()
    for a, b in ((q, qr), (k, kr), (v, vr)):
        assert O.rel_l2(a.grad, b.grad) < 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("offset", [-16.0, 14.0])
def test_constant_score_offset(dev, dtype, offset):
    # One feature column makes every score carry the same constant (in natural-log units).  Both
    # softmaxes are invariant to it, so the oracle result is that of the remaining columns; the
    # kernels must not lose precision to it whatever the element type (f16 probabilities of
    # e^-16 would be subnormal, of e^14 infinite).
    q, k, v = make(1, 2, 3000, 128, 32, dtype)
    q[..., 0] = 4.0
    k[..., 0] = offset / 4.0
    assert F.mixer_kernel_name(q, k, v).startswith("mfma")
    check(dev, q, k, v)


def test_offsets_beyond_2_31_elements(dev):
    """k, v, y of exactly 2^31 elements each: the last (batch, head) slice sits beyond what 32-bit element
    offsets reach.  Heads are independent, so that slice computed alone (small offsets) must give the same rows."""
    B, H, N, M, D = 4, 8, 1 << 21, 64, 32
    g = torch.Generator(device=dev).manual_seed(3)
    q = (torch.randn(H, M, D, device=dev, generator=g) * D ** -0.5).bfloat16()
    k = torch.randn(B, H, N, D, device=dev, generator=g, dtype=torch.bfloat16)
    v = torch.randn(B, H, N, D, device=dev, generator=g, dtype=torch.bfloat16)
    assert k.numel() == 1 << 31
    y = F.flare_multihead_mixer(q, k, v)
    ks, vs = k[B - 1:, H - 1:].clone(), v[B - 1:, H - 1:].clone()
    ys = F.flare_multihead_mixer(q[H - 1:], ks, vs)
    assert O.rel_l2(y[B - 1:, H - 1:], ys) <= 2e-3        # same kernels, another split of N: rounding only
    # and against the oracle on the first tokens of that slice: y_n needs z of the whole slice, from the small call
    _, z = F.flare_multihead_mixer(q[H - 1:], ks, vs, return_z=True)
    n = 4096
    s = (ks[0, 0, :n].float() @ q[H - 1].float().T)
    yr = torch.softmax(s, dim=-1) @ z[0, 0]
    assert O.rel_l2(y[B - 1, H - 1, :n], yr) <= TOL[torch.bfloat16]
    assert y.amax() <= v.amax() and y.amin() >= v.amin()    # every output is a convex combination of rows of v


def test_graph_capture_and_replay(dev):
    """The mixer and the causal prefill (whose flags are cleared by a kernel, not a memset) captured in a HIP
    graph: every replay, with eager work in between, reproduces the eager result bit for bit."""
    q, k, v = (t.to(dev) for t in make(2, 4, 5000, 128, 32, torch.bfloat16, seed=9))
    y_eager = F.flare_multihead_mixer(q, k, v)
    qc = (torch.randn(4, 128, 32, device=dev) * 0.3).bfloat16()
    yc_eager, st_eager = F.flare_causal_prefill(qc, k, v)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):      # warm the allocator on the side stream
            F.flare_multihead_mixer(q, k, v)
            F.flare_causal_prefill(qc, k, v)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g = F.flare_multihead_mixer(q, k, v)
        yc_g, st_g = F.flare_causal_prefill(qc, k, v)
    for i in range(3):
        y_g.zero_(); yc_g.zero_()
        (k.float().sum() + i).item()          # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_eager), f"mixer replay {i}"
        assert torch.equal(yc_g, yc_eager), f"causal replay {i}"
        assert all(torch.equal(a, b) for a, b in zip(st_g, st_eager))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_localized_large_scores_mix_fast_and_exact_paths(dev, dtype):
    """A short burst of tokens with scores far outside the window in which the kernels may skip the running
    maximum: only the token splits / tiles that contain the burst take the exact path, the rest stays on the fast
    one, and the merge has to combine partials with and without a shift."""
    B, H, N, M, D = 1, 2, 40000, 128, 32
    q, k, v = make(B, H, N, M, D, dtype, seed=21, qstd=1.0)
    k[:, :, 17000:17100] *= 6.0
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    assert float(s[:, :, :, 17000:17100].abs().max()) > 130 and float(s[:, :, :, :17000].abs().max()) < 60
    y, _ = check(dev, q, k, v)
    # and the gradients on the same inputs (both exponentials of the backward are bounded by construction)
    gy = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(1)).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.flare_multihead_mixer(qd, kd, vd).backward(gy.to(dev))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.mixer_explicit(qr, kr, vr, 1.0)[0].backward(gy.double())
    assert O.rel_l2(qd.grad, qr.grad) <= 3e-2 and O.rel_l2(kd.grad, kr.grad) <= 3e-2 and O.rel_l2(vd.grad, vr.grad) <= 3e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 8, 3000, 64, 8), (1, 4, 1111, 256, 8), (1, 2, 500, 128, 4), (1, 2, 900, 64, 24), (1, 2, 700, 128, 40), (1, 3, 800, 32, 10)])
def test_narrow_heads_run_on_the_matrix_core_kernels(dev, shape, dtype):
    """Head dims other than 16, 32, 64 (the reference's default model has channel_dim 64 / 8 heads = 8,
    pdebench/__main__.py:1122-1123) are zero-padded to the next of them: same scores, same outputs, matrix-core kernels."""
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, dtype, seed=21)
    x = torch.stack([k, v]).permute(0, 1, 3, 2, 4).reshape(2, B, N, H * D).contiguous().to(dev)
    kd, vd = (t.view(B, N, H, D).permute(0, 2, 1, 3) for t in x)                # the views the modules hand over
    assert F.mixer_kernel_name(q.to(dev), kd, vd) == ("mfma_bf16" if dtype == torch.bfloat16 else "mfma_f16")
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, N // 2:] = False
    for km in (None, mask):
        y, z = F.flare_multihead_mixer(q.to(dev), kd, vd, scale=0.7, key_mask=None if km is None else km.to(dev), return_z=True)
        yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 0.7, km)
        assert y.shape == (B, H, N, D) and z.shape == (B, H, M, D)
        assert O.rel_l2(y, yr) <= 2e-2 and O.rel_l2(z, zr) <= 2e-2
    # the two halves separately, and the fp32 kernels on request
    zg, _ = F.flare_gather(q.to(dev), kd, vd, scale=0.7)
    yg = F.flare_scatter(q.to(dev), kd, zg, scale=0.7)
    yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 0.7)
    assert zg.shape == zr.shape and O.rel_l2(zg, zr) <= 2e-2 and O.rel_l2(yg, yr) <= 2e-2
    assert F.mixer_kernel_name(q.to(dev), kd, vd, force_generic=True) == "generic"
    assert O.rel_l2(F.flare_multihead_mixer(q.to(dev), kd, vd, scale=0.7, force_generic=True), yr) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 2, 3000, 32, 32), (1, 3, 1500, 96, 16), (1, 2, 700, 160, 64), (2, 4, 2000, 32, 8)])
def test_latent_counts_that_are_odd_multiples_of_32(dev, shape, dtype):
    """M = 32 is the FLARE layer's own default (pdebench/models/flare.py:68): the gather pads its last 64-latent block
    with waves that own no latent, the scatter walks the latents 32 at a time."""
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, dtype, seed=31)
    assert F.mixer_kernel_name(q.to(dev), k.to(dev), v.to(dev)).startswith("mfma")
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, N // 3:] = False
    for km in (None, mask):
        y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.9, key_mask=None if km is None else km.to(dev),
                                       return_z=True)
        yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 0.9, km)
        assert z.shape == zr.shape and O.rel_l2(z, zr) <= 2e-2 and O.rel_l2(y, yr) <= 2e-2
    # gradients through the HIP backward, against fp64 autograd through the oracle
    g = torch.Generator().manual_seed(32)
    gy = torch.randn(B, H, N, D, generator=g).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.flare_multihead_mixer(qd, kd, vd, scale=0.9).backward(gy.to(dev))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.mixer_explicit(qr, kr, vr, 0.9)[0].backward(gy.double())
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_against_torch_fused_attention_on_the_device(dev, dtype):
    """The reference computes y = SDPA(k, q, SDPA(q, k, v)) with torch's own fused attention (README.md:49-50); on a HIP
    device that is the kernel its users would get.  Both results round through 16 bits, hence the 16-bit bar."""
    import torch.nn.functional as TF
    B, H, N, M, D = 2, 4, 20000, 128, 32
    q, k, v = make(B, H, N, M, D, dtype, seed=41)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    qe = qd.unsqueeze(0).expand(B, -1, -1, -1)
    for scale in (1.0, 0.6):
        z = TF.scaled_dot_product_attention(qe, kd, vd, scale=scale)
        yt = TF.scaled_dot_product_attention(kd, qe, z, scale=scale)
        y = F.flare_multihead_mixer(qd, kd, vd, scale=scale)
        assert O.rel_l2(y, yt) <= 2e-2
        yr, _ = O.mixer_explicit(q.float(), k.float(), v.float(), scale)
        # and about as close to the fp64 oracle as torch is (for f16 inputs the HIP kernels still carry the
        # probabilities in bf16, whose exponent range the unshifted softmax needs: 3e-3 there)
        assert O.rel_l2(y, yr) <= max(O.rel_l2(yt, yr) * 1.5 + 1e-3, 3e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 2, 2000, 48, 16), (1, 3, 1500, 100, 32), (1, 2, 900, 20, 8), (1, 2, 700, 7, 24)])
def test_latent_counts_that_are_not_multiples_of_32(dev, shape, dtype):
    """Dead latents fill M up to a multiple of 32 (zero queries in the gather, a -16384 score offset in the scatter):
    forward against the oracle with and without a mask, gradients against fp64 autograd, strongly negative scores."""
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, dtype, seed=51)
    assert F.mixer_kernel_name(q.to(dev), k.to(dev), v.to(dev)).startswith("mfma")
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, N // 2:] = False
    for km in (None, mask):
        y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, key_mask=None if km is None else km.to(dev), return_z=True)
        yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 0.8, km)
        assert y.shape == yr.shape and z.shape == zr.shape
        assert O.rel_l2(z, zr) <= 2e-2 and O.rel_l2(y, yr) <= 2e-2
    # every real score far below the dead latents' gather score of 0: the dead ones must still get no weight
    k2 = (k.float() * 0.05).to(dtype)
    q2 = (q.float() - 3.0).to(dtype) if D >= 16 else q
    y2 = F.flare_multihead_mixer(q2.to(dev), (k2.float().abs()).to(dtype).to(dev), v.to(dev), scale=4.0)
    yr2, _ = O.mixer_explicit(q2.float(), k2.float().abs().to(dtype).float(), v.float(), 4.0)
    assert O.rel_l2(y2, yr2) <= 2e-2
    gy = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(52)).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.flare_multihead_mixer(qd, kd, vd, scale=0.8).backward(gy.to(dev))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.mixer_explicit(qr, kr, vr, 0.8)[0].backward(gy.double())
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        assert got.shape == ref.shape
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 2, 800, 16, 32), (1, 2, 600, 8, 64), (2, 1, 900, 48, 64), (1, 2, 500, 24, 8), (1, 1, 700, 80, 16)])
def test_latent_counts_that_are_multiples_of_8(dev, shape, dtype):
    """A latent count that is a multiple of 8 but not of 32 runs as 2 or 4 copies of every latent on the matrix-core
    kernels, forward and backward (the copies share each latent's softmax weight, autograd sums their gradients):
    y and z against the oracle with and without a mask, gradients against fp64 autograd."""
    from flare_py_amd import functional as fn
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, dtype, seed=61)
    assert F.mixer_kernel_name(q.to(dev), k.to(dev), v.to(dev)).startswith("mfma")
    r = fn._latent_copies(q.to(dev), k.to(dev), False)
    assert r in (2, 4) and (r * M) % 32 == 0
    assert fn._hip_backward_ok(q.to(dev).repeat(1, r, 1), k.to(dev), v.to(dev), None, False) or D < 16
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, N // 3:] = False
    for km in (None, mask):
        y, z = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), scale=0.8, key_mask=None if km is None else km.to(dev), return_z=True)
        yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 0.8, km)
        assert y.shape == yr.shape and z.shape == zr.shape
        assert O.rel_l2(z, zr) <= 2e-2 and O.rel_l2(y, yr) <= 2e-2
    gy = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(62)).to(dtype)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.flare_multihead_mixer(qd, kd, vd, scale=0.8).backward(gy.to(dev))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.mixer_explicit(qr, kr, vr, 0.8)[0].backward(gy.double())
    for name, got, ref in (("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        assert got.shape == ref.shape
        err = O.rel_l2(got, ref)
        assert err <= 3e-2, f"{name} rel-L2 {err:.3e}"


# ---- 32x32x16 kernels (bf16, D = 32, no key mask): scatter at M in {64, 128, 256, 512}, gather at M % 64 == 0 ----
@pytest.mark.parametrize("shape", [
    (1, 1, 1, 256, 32), (1, 2, 5, 256, 32), (1, 2, 31, 256, 32), (1, 2, 33, 256, 32), (2, 2, 127, 256, 32),
    (1, 2, 129, 256, 32), (1, 3, 1000, 256, 32), (2, 2, 4096 + 17, 256, 32), (1, 2, 3000, 512, 32),
    (1, 2, 20000, 256, 32), (1, 2, 777, 64, 32), (1, 2, 1999, 128, 32),
    (1, 2, 2500, 192, 32), (1, 1, 1300, 320, 32), (1, 2, 2100, 384, 32), (1, 1, 5000, 768, 32),   # 3, 5, 3, 3 latent blocks
])
def test_mfma32_shapes_and_ragged_ends(dev, shape):
    from flare_py_amd import _lib
    from flare_py_amd import functional as FN
    q, k, v = make(*shape, torch.bfloat16, seed=3)
    y, z = check(dev, q, k, v)                  # default: 32x32x16 gather and scatter
    with FN.mixer_flags(_lib.FLAG_MFMA16):      # the 16x16x32 kernels on the same problem
        y16, z16 = check(dev, q, k, v)
    assert O.rel_l2(z, z16) < 5e-3 and O.rel_l2(y, y16) < 1e-2


@pytest.mark.parametrize("n_splits", [1, 3, 7, 64])
def test_mfma32_split_invariance_and_determinism(dev, n_splits):
    from flare_py_amd import _lib
    from flare_py_amd import functional as FN
    q, k, v = make(1, 2, 9000, 256, 32, torch.bfloat16, seed=5)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y, z = F.flare_multihead_mixer(qd, kd, vd, return_z=True, n_splits=n_splits)
    y2, z2 = F.flare_multihead_mixer(qd, kd, vd, return_z=True, n_splits=n_splits)
    assert torch.equal(y, y2) and torch.equal(z, z2)
    yr, zr = O.mixer_explicit(q.float(), k.float(), v.float(), 1.0)
    assert O.rel_l2(z, zr) <= 2e-2 and O.rel_l2(y, yr) <= 2e-2


def test_mfma32_large_scores_take_the_exact_paths(dev):
    # scores far outside the unshifted window in both directions, along N and along M
    B, H, N, M, D = 1, 2, 3000, 256, 32
    g = torch.Generator().manual_seed(7)
    q = torch.randn(H, M, D, generator=g) * torch.linspace(0.2, 2.0, M)[None, :, None]
    k = torch.randn(B, H, N, D, generator=g) * torch.linspace(0.2, 3.0, N)[None, None, :, None]
    v = torch.randn(B, H, N, D, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    assert float(s.max()) > 100.0
    from flare_py_amd import _lib
    from flare_py_amd import functional as FN
    check(dev, q, k, v, tol=3e-2)
    check(dev, q, k, v, n_splits=4, tol=3e-2)
    with FN.mixer_flags(_lib.FLAG_MFMA16):
        check(dev, q, k, v, tol=3e-2)


@pytest.mark.parametrize("wave", [0, 2, 3])
def test_gather32_one_wave_repeats_exactly_the_others_do_not(dev, wave):
    # the gather's waves own the 32-token passes w, w + 4, ... of a range and decide each for itself whether its sums
    # left the unshifted window: huge scores on one wave's tokens only make that wave repeat with a running maximum,
    # and the workgroup then adds partial sums that carry different shifts
    B, H, N, M, D = 1, 2, 4096, 256, 32
    g = torch.Generator().manual_seed(21)
    q = torch.randn(H, M, D, generator=g) * D ** -0.5
    k = torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g)
    n = torch.arange(N)
    hot = ((n // 32) % 4 == wave) & (n >= 1024) & (n < 1536)
    k[:, :, hot] *= 60.0
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float()) * 1.4427
    assert float(s.max()) > 130.0
    for n_splits in (1, 2, 0):
        check(dev, q, k, v, n_splits=n_splits, tol=3e-2)


@pytest.mark.parametrize("offset", [-30.0, 60.0])
def test_mfma32_constant_score_offset_stays_on_the_fast_path(dev, offset):
    # a constant added to every score (one extra head-dim pair) moves all exponentials by e^offset and cancels in
    # both softmaxes: inside the unshifted window the result must not change
    q, k, v = make(1, 2, 2000, 256, 32, torch.bfloat16, seed=9)
    q2, k2 = q.clone(), k.clone()
    q2[..., 0] = 1.0
    k2[..., 0] = offset
    q0, k0 = q.clone(), k.clone()
    q0[..., 0] = 0.0
    k0[..., 0] = 0.0
    from flare_py_amd import _lib
    from flare_py_amd import functional as FN
    for flags in (0, _lib.FLAG_MFMA16):
        with FN.mixer_flags(flags):
            y0, _ = check(dev, q0, k0, v)
            y1, _ = check(dev, q2, k2, v)
        assert O.rel_l2(y1, y0) < 1e-2


def test_mfma32_strided_views_per_batch_q_mask_and_lse(dev):
    B, H, N, M, D = 2, 4, 1500, 256, 32
    g = torch.Generator().manual_seed(11)
    kk = torch.randn(B, N, H * D, generator=g).bfloat16()
    vv = torch.randn(B, N, H * D, generator=g).bfloat16()
    q = (torch.randn(B, H, M, D, generator=g) * D ** -0.5).bfloat16()      # one latent set per batch element
    k = kk.view(B, N, H, D).permute(0, 2, 1, 3)
    v = vv.view(B, N, H, D).permute(0, 2, 1, 3)
    y = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev))
    yr, _ = O.mixer_explicit(q.float(), k.float(), v.float(), 1.0)
    assert O.rel_l2(y, yr) <= 2e-2
    # key mask: both halves keep the 16x16x32 kernels, padded rows come out as zeros
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[0, 1000:] = False
    mask[1, ::3] = False
    ym = F.flare_multihead_mixer(q.to(dev), k.to(dev), v.to(dev), key_mask=mask.to(dev))
    yr, _ = O.mixer_explicit(q.float(), k.float(), v.float(), 1.0, mask)
    assert O.rel_l2(ym, yr) <= 2e-2
    assert (ym.cpu()[0, :, 1000:] == 0).all()
    # token log-sum-exp of the scatter (the backward needs it)
    z, lse = F.flare_gather(q.to(dev), k.to(dev), v.to(dev))
    sc = torch.einsum("bhnd,bhmd->bhnm", k.float(), q.float())
    want = torch.logsumexp(sc, dim=-1)
    from flare_py_amd import functional as FN
    out = FN._mixer_forward(q.to(dev), k.to(dev), v.to(dev), 1.0, None, 0, False, False, True)
    assert float((out[3].cpu() - want).abs().max()) < 3e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale", [1e-4, 3e-3, 1.0, 40.0])
def test_dead_latents_get_no_weight_at_any_scale(dev, dtype, scale):
    """M = 20 runs with 12 dead latents whose scores are scale * bias: the bias follows the scale, and where the
    element type cannot hold it (f16 with a tiny scale) the fp32-FMA kernels take the problem."""
    from flare_py_amd import functional as FN
    q, k, v = make(1, 2, 700, 20, 16, dtype, seed=31)
    bias = FN._dead_latent_bias(scale, dtype)
    assert bias is None or scale * bias <= -200.0
    if dtype == torch.float16 and scale == 1e-4:
        assert bias is None and F.mixer_kernel_name(q.to(dev), k.to(dev), v.to(dev), scale=scale) == "generic"
    check(dev, q, k, v, scale=scale)


# ---- fp32 inputs on the fp32 matrix instruction (taken by the generic launchers when the problem allows) -------------
@pytest.mark.parametrize("shape", [(1, 8, 4096, 64, 16), (2, 3, 1000, 16, 16), (1, 2, 777, 48, 32), (1, 2, 5000, 256, 32),
                                   (2, 1, 333, 80, 64), (1, 1, 1, 16, 16), (1, 2, 17, 128, 64), (3, 2, 2049, 32, 32)])
def test_fp32_matrix_core_mixer_shapes(dev, shape):
    """Parity at the fp32 bar, every split count the same result to rounding, two runs the same bits, the latents'
    log-sum-exp against the oracle's."""
    from torch.profiler import ProfilerActivity, profile
    q, k, v = make(*shape, torch.float32, seed=shape[2])
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        y, z = check(dev, q, k, v, scale=0.8)
    names = {e.key for e in prof.key_averages()}
    assert any("gather_f32_mfma_kernel" in n for n in names) and any("scatter_f32_mfma_kernel" in n for n in names), names
    y2, z2 = F.flare_multihead_mixer(qd, kd, vd, scale=0.8, return_z=True)
    assert torch.equal(y, y2) and torch.equal(z, z2)
    for s in (1, 3):
        ys, zs = check(dev, q, k, v, scale=0.8, n_splits=s)
    zg, lse = F.flare_gather(qd, kd, vd, scale=0.8)
    sc = 0.8 * torch.einsum("hmd,bhnd->bhmn", q.double(), k.double())
    assert float((lse.double().cpu() - torch.logsumexp(sc, -1)).abs().max()) <= 1e-4
    assert O.rel_l2(F.flare_scatter(qd, kd, zg, scale=0.8), y) <= 1e-5


def test_fp32_matrix_core_mixer_views_and_fallbacks(dev):
    """Token-major 'b n (h d) -> b h n d' views go through without a copy, a key mask too; a latent count that is not a
    multiple of 16 keeps the FMA kernels, and so does force_generic."""
    from torch.profiler import ProfilerActivity, profile
    B, H, N, M, D = 2, 4, 3000, 64, 32
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, B, N, H * D, generator=g)
    q = torch.randn(H, M, D, generator=g) * D ** -0.5
    k, v = (t.view(B, N, H, D).permute(0, 2, 1, 3) for t in x)
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        y = F.flare_multihead_mixer(q.to(dev), *(t.to(dev).view(B, N, H, D).permute(0, 2, 1, 3) for t in x))
        torch.cuda.synchronize()
    names = {e.key for e in prof.key_averages()}
    assert any("scatter_f32_mfma_kernel" in n for n in names) and not any("copy" in n.lower() for n in names), names
    yr, _ = O.mixer_explicit(q, k, v, 1.0, None)
    assert O.rel_l2(y, yr) <= 1e-5
    mask = torch.ones(B, N, dtype=torch.bool)
    mask[1, 2000:] = False
    # a key mask and a head dim of 24 (zero-padded to 32) take the matrix-core kernels; the other two do not
    for kw, qq, kk, vv, mfma in (({"key_mask": mask}, q, k, v, True), ({}, q[:, :, :24], k[..., :24], v[..., :24], True),
                                 ({}, q[:, :40], k, v, False), ({"force_generic": True}, q, k, v, False)):
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            check(dev, qq.contiguous(), kk.contiguous(), vv.contiguous(), **kw)
        assert any("f32_mfma" in e.key for e in prof.key_averages()) == mfma, kw


def test_fp32_narrow_heads_are_padded_to_the_matrix_core_kernels(dev):
    """D = 8 (the reference's default model: 64 channels, 8 heads) in fp32: q, k, v zero-padded to 16 columns run on
    the fp32 matrix-core kernels; values and gradients as the oracle's."""
    from torch.profiler import ProfilerActivity, profile
    q, k, v = make(2, 8, 3000, 64, 8, torch.float32, seed=4)
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        check(dev, q, k, v, scale=1.3)
    assert any("gather_f32_mfma_kernel" in e.key for e in prof.key_averages())
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    F.flare_multihead_mixer(qd, kd, vd, scale=1.3).square().sum().backward()
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    O.mixer_explicit(qr, kr, vr, 1.3, None)[0].square().sum().backward()
    for a, b in ((qd, qr), (kd, kr), (vd, vr)):
        assert a.grad.shape == b.grad.shape and O.rel_l2(a.grad, b.grad) <= 1e-4


@pytest.mark.parametrize("garbage", [0.0, 1.0e30, float("nan")])
def test_fp32_key_mask_over_many_splits_and_padding_garbage(dev, garbage):
    """The fp32 matrix-core kernels with a key mask: split ranges without a real token, a fully padded batch element,
    holes, and padded rows that hold huge values or NaN never reach a result."""
    q, k, v = make(4, 2, 8192, 128, 32, torch.float32, seed=12)
    mask = torch.ones(4, 8192, dtype=torch.bool)
    mask[1, 100:] = False
    mask[2, 5000:] = False
    mask[2, 17:4000:5] = False
    mask[3] = False
    kk, vv = k.clone(), v.clone()
    if garbage != 0.0:
        kk[~mask[:, None, :, None].expand_as(k)] = garbage
        vv[~mask[:, None, :, None].expand_as(v)] = garbage
    y, z = F.flare_multihead_mixer(q.to(dev), kk.to(dev), vv.to(dev), key_mask=mask.to(dev), return_z=True)
    yr, zr = O.mixer_explicit(q, k, v, 1.0, mask)
    keep = mask[:, None, :, None].expand_as(yr)
    assert torch.isfinite(z).all() and O.rel_l2(z, zr) <= 1e-5
    assert O.rel_l2(y.cpu()[keep], yr[keep]) <= 1e-5
    assert (y.cpu()[~keep] == 0).all() and (z[3] == 0).all()


def test_fp32_scatter_takes_a_misaligned_z(dev):
    """z handed to flare_scatter four bytes off a 16-byte boundary: the FMA kernel takes it (same values)."""
    q, k, v = make(1, 2, 500, 32, 16, torch.float32, seed=6)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    z, _ = F.flare_gather(qd, kd, vd)
    buf = torch.zeros(z.numel() + 1, device=dev)
    zo = buf[1:].view_as(z)
    zo.copy_(z)
    assert zo.data_ptr() % 16 != 0
    assert O.rel_l2(F.flare_scatter(qd, kd, zo), F.flare_scatter(qd, kd, z)) <= 1e-6
