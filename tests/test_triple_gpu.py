"""GPU parity of the triple (third-order) linear attention kernels vs the einsum oracle
(lra/models/backends.py:1285-1292 of the reference).  Tolerance: relative L2 <= 1e-5 for fp32,
<= 2e-2 for bf16/f16 (the reference's own check is allclose(rtol=atol=1e-3) on half inputs,
lra/models/triton/triple.py:1130), against the oracle on the same rounded inputs."""
import pytest
import torch

import flare_py_amd as F
from oracle import c_oracle
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def make(B, H, N, Dq, Dv, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda d: (torch.randn(B, H, N, d, generator=g) * Dq ** -0.5).to(dtype)
    return mk(Dq), mk(Dq), mk(Dq), mk(Dq), mk(Dv)


@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (2, 2, 13, 3, 4), (1, 2, 500, 16, 16), (1, 2, 300, 32, 32),
                                   (1, 1, 130, 64, 64), (2, 1, 1000, 16, 24), (1, 1, 77, 20, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_reference_exact_mode(dev, shape, dtype):
    a = make(*shape, dtype)
    st, out = F.triple_attention(*[t.to(dev) for t in a])
    sr, orf = O.triple_einsum(*[t.float() for t in a], dtype=torch.float64)
    # state: fp32 accumulation; the 16-bit kernels round each product k1[n,i] k2[n,k] to the element type once before
    # the matrix product (half an ulp, 2^-9 for bf16: with a single token nothing averages it out)
    assert O.rel_l2(st, sr) <= (1e-5 if dtype == torch.float32 else 4e-3)
    assert O.rel_l2(out, orf) <= TOL[dtype]
    assert st.dtype == torch.float32 and out.dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feature_map_and_normaliser(dev, dtype):
    a = make(2, 2, 700, 16, 16, dtype, seed=1)
    st, out = F.triple_attention(*[t.to(dev) for t in a], normalize=True, feature_map="elu")
    sr, orf = O.triple_einsum(*[t.float() for t in a], feature_map=True, normalize=True, dtype=torch.float64)
    # half types: features and the k1*k2 products are rounded to the element type before the MFMA
    assert O.rel_l2(st, sr) <= (1e-5 if dtype == torch.float32 else 1e-2) and O.rel_l2(out, orf) <= TOL[dtype]
    sc, oc = c_oracle.triple(*[t.float() for t in a], feature_map=True, normalize=True)
    assert O.rel_l2(out, oc) <= TOL[dtype]
    # positive features, constant v, normalised  =>  constant output
    c = torch.full_like(a[4], 0.75)
    _, oc = F.triple_attention(*[t.to(dev) for t in a[:4]], c.to(dev), normalize=True, feature_map="elu")
    assert torch.allclose(oc.float().cpu(), c.float(), atol=1e-2 if dtype != torch.float32 else 1e-5)


def test_function_apply_signature_and_split_stability(dev):
    a = [t.to(dev) for t in make(1, 2, 5000, 16, 16, torch.float32, seed=2)]
    st, out = F.TripleAttentionFunction.apply(*a)
    st2, out2 = F.TripleAttentionFunction.apply(*a)
    assert torch.equal(st, st2) and torch.equal(out, out2)      # no atomics: bit-stable
    for s in (1, 3, 16):
        sts, outs = F.triple_attention(*a, n_splits=s)
        assert O.rel_l2(sts, st) <= 2e-6 and O.rel_l2(outs, out) <= 2e-6


def test_strided_heads_view(dev):
    B, H, N, D = 2, 4, 300, 16
    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(B, N, H * D, generator=g).to(dev) * 0.25 for _ in range(5)]
    views = [x.view(B, N, H, D).permute(0, 2, 1, 3) for x in xs]
    st, out = F.triple_attention(*views)
    sr, orf = O.triple_einsum(*[t.cpu() for t in views], dtype=torch.float64)
    assert O.rel_l2(st, sr) <= 1e-5 and O.rel_l2(out, orf) <= 1e-5


def test_cfg5_shape(dev):
    # BASELINE config 5: B=4,H=8,N=16384,D=16, bf16 in / fp32 state, elu+1 features, normalised
    a = make(4, 8, 16384, 16, 16, torch.bfloat16)
    st, out = F.triple_attention(*[t.to(dev) for t in a], normalize=True, feature_map="elu")
    sr, orf = O.triple_einsum(*[t.float() for t in a], feature_map=True, normalize=True)
    assert O.rel_l2(st, sr) <= 1e-2 and O.rel_l2(out, orf) <= 2e-2


@pytest.mark.parametrize("dtype,D,Dv,tol", [(torch.float32, 16, 16, 1e-4), (torch.bfloat16, 16, 16, 3e-2), (torch.float32, 8, 12, 1e-4),
                                            (torch.bfloat16, 32, 32, 3e-2)])
def test_backward_matches_autograd_of_the_einsum_oracle(dev, dtype, D, Dv, tol):
    # gradients of lra/models/triton/triple.py:124-135, including a gradient flowing into STATE
    g = torch.Generator().manual_seed(11)
    B, H, N = 1, 2, 300
    ins = [(torch.randn(B, H, N, D, generator=g) * 0.5).to(dtype) for _ in range(4)] + [torch.randn(B, H, N, Dv, generator=g).to(dtype)]
    gs = torch.randn(B, H, D, Dv, D, generator=g)
    go = torch.randn(B, H, N, Dv, generator=g).to(dtype)
    dins = [t.to(dev).requires_grad_(True) for t in ins]
    st, out = F.TripleAttentionFunction.apply(*dins)
    (st * gs.to(dev)).sum().add((out.float() * go.to(dev).float()).sum()).backward()
    rins = [t.double().requires_grad_(True) for t in ins]
    sr, orf = O.triple_einsum(*rins, dtype=torch.float64)
    ((sr * gs.double()).sum() + (orf * go.double()).sum()).backward()
    for name, a, b in zip(("dq1", "dq2", "dk1", "dk2", "dv"), dins, rins):
        err = O.rel_l2(a.grad, b.grad)
        assert err <= tol, f"{name}: {err:.3e}"


@pytest.mark.parametrize("dtype,D,Dv,tol", [(torch.float32, 16, 16, 1e-4), (torch.bfloat16, 16, 16, 3e-2), (torch.float32, 8, 12, 1e-4)])
@pytest.mark.parametrize("fm,norm", [("elu", True), ("elu", False), (None, True)])
def test_backward_with_feature_map_and_normaliser(dev, dtype, D, Dv, tol, fm, norm):
    """Gradients with the elu + 1 feature map and / or the normaliser (the module's training mode, backends.py:1258,
    1285-1292): the map and the division differentiate through torch around the HIP contractions; checked against fp64
    autograd through the einsum definition."""
    g = torch.Generator().manual_seed(13)
    B, H, N = 1, 2, 260
    ins = [(torch.randn(B, H, N, D, generator=g) * 0.5).to(dtype) for _ in range(4)] + [torch.randn(B, H, N, Dv, generator=g).to(dtype)]
    if fm is None:
        ins[:4] = [t.abs() + 0.1 for t in ins[:4]]           # positive features, as a kernel map leaves them: the normaliser stays away from 0
    gs = torch.randn(B, H, D, Dv, D, generator=g)
    go = torch.randn(B, H, N, Dv, generator=g).to(dtype)
    dins = [t.to(dev).requires_grad_(True) for t in ins]
    st, out = F.triple_attention(*dins, normalize=norm, feature_map=fm)
    (st * gs.to(dev)).sum().add((out.float() * go.to(dev).float()).sum()).backward()
    rins = [t.double().requires_grad_(True) for t in ins]
    sr, orf = O.triple_einsum(*rins, feature_map=fm == "elu", normalize=norm, dtype=torch.float64)
    ((sr * gs.double()).sum() + (orf * go.double()).sum()).backward()
    assert O.rel_l2(out, orf) <= (1e-5 if dtype == torch.float32 else 2e-2)
    for name, a, b in zip(("dq1", "dq2", "dk1", "dk2", "dv"), dins, rins):
        err = O.rel_l2(a.grad, b.grad)
        assert err <= tol, f"{name}: {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Dq,Dv", [(32, 32), (16, 32), (32, 16), (64, 64), (48, 32), (8, 8), (20, 24), (4, 40)])
def test_head_dims_in_blocks_of_16(dev, Dq, Dv, dtype):
    """Head dims that are larger multiples of 16 run on the matrix-core kernels block by block inside one launch (state:
    one workgroup per 16 x 16 x 16 block and split; output: the (i, k) block pairs looped over LDS-resident operands);
    other head dims are zero-padded to a multiple of 16 first (the reference's Triton path takes any D >= 16 with
    D % 4 == 0, lra/models/triton/triple.py:69-70; its einsum path any D)."""
    a = make(2, 2, 900, Dq, Dv, dtype, seed=Dq + Dv)
    st, out = F.triple_attention(*[t.to(dev) for t in a], normalize=True, feature_map="elu")
    sr, orf = O.triple_einsum(*[t.float() for t in a], feature_map=True, normalize=True, dtype=torch.float64)
    assert st.shape == (2, 2, Dq, Dv, Dq) and out.shape == (2, 2, 900, Dv) and out.dtype == dtype
    assert O.rel_l2(st, sr) <= 1e-2 and O.rel_l2(out, orf) <= 2e-2
    c = torch.full_like(a[4], -0.5)                       # constant v, normalised => constant output
    _, oc = F.triple_attention(*[t.to(dev) for t in a[:4]], c.to(dev), normalize=True, feature_map="elu")
    assert torch.allclose(oc.float().cpu(), c.float(), atol=1e-2)


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 5e-3), (torch.float16, 1e-3)])
@pytest.mark.parametrize("D", [16, 32, 64])
def test_state_is_tight_for_any_number_of_tiles_per_wave(dev, dtype, tol, D):
    """The state kernel's waves walk 1, 2, 4 ... tiles depending on the split count; its per-tile factors are read
    through DPP row rotates, whose wait states the kernel provides itself.  The state must stay at rounding level
    (products rounded once to the element type: about 3e-3 in bf16, 4e-4 in f16) for every split count."""
    a = make(2, 2, 900, D, D, dtype, seed=3 * D)
    sr, orf = O.triple_einsum(*[t.float() for t in a], feature_map=True, normalize=True, dtype=torch.float64)
    for ns in (0, 1, 2, 4, 8):
        st, out = F.triple_attention(*[t.to(dev) for t in a], normalize=True, feature_map="elu", n_splits=ns)
        assert O.rel_l2(st, sr) <= tol, (ns, O.rel_l2(st, sr))
        assert O.rel_l2(out, orf) <= TOL[dtype]


@pytest.mark.parametrize("shape", [(1, 2, 500), (2, 3, 1), (1, 1, 17), (2, 2, 4097)])
@pytest.mark.parametrize("fm,nz", [(None, False), ("elu", True), ("elu", False)])
@pytest.mark.parametrize("D", [16, 32])
def test_fp32_head_dims_16_and_32_on_the_matrix_cores(dev, shape, fm, nz, D):
    """fp32 inputs with Dq = Dv = 16 or 32 run on the fp32 matrix instruction (profiler), at the fp32 bar, the same bits
    twice; rows that are not 16-byte aligned keep the FMA kernels."""
    from torch.profiler import ProfilerActivity, profile
    B, H, N = shape
    g = torch.Generator().manual_seed(N)
    a = [torch.randn(B, H, N, D, generator=g) * 0.25 for _ in range(5)]
    ad = [t.to(dev) for t in a]
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        st, out = F.triple_attention(*ad, normalize=nz, feature_map=fm)
        torch.cuda.synchronize()
    names = {e.key for e in prof.key_averages()}
    assert any("triple_state_f32_mfma" in n for n in names) and any("triple_out_f32_mfma" in n for n in names)
    sr, orf = O.triple_einsum(*a, feature_map=fm == "elu", normalize=nz)
    assert O.rel_l2(st, sr) <= 1e-5 and O.rel_l2(out, orf) <= 1e-5
    st2, out2 = F.triple_attention(*ad, normalize=nz, feature_map=fm)
    assert torch.equal(st, st2) and torch.equal(out, out2)
    pad = [torch.zeros(B, H, N, D + 1, device=dev) for _ in range(5)]
    for p, t in zip(pad, ad):
        p[..., 1:] = t
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        st3, out3 = F.triple_attention(*[p[..., 1:] for p in pad], normalize=nz, feature_map=fm)
        torch.cuda.synchronize()
    assert O.rel_l2(out3, orf) <= 1e-5


@pytest.mark.parametrize("dtype,eps", [(torch.bfloat16, 2.0 ** -8), (torch.float16, 2.0 ** -10)])
@pytest.mark.parametrize("N", [1, 2])
@pytest.mark.parametrize("Dq,Dv", [(32, 16), (16, 16), (32, 32), (64, 16)])
def test_16bit_kernels_with_one_or_two_tokens_against_the_conditioning_bound(dev, dtype, eps, N, Dq, Dv):
    """Signed features and one or two tokens: out[n,j] = sum_ik q1_i state_ijk q2_k is then (q1.k1)(q2.k2) v_j (a sum of
    two such products for N = 2), a sum of Dq^2 signed terms that mostly cancel, so its error relative to |out| says
    nothing about the kernel.  What the 16-bit kernels can promise is an error that is small against the sum of the
    terms' magnitudes: each term carries a few roundings to the element type (the products k1 k2 and q1 q2, the state
    as a matrix operand) and the output is rounded once.  Checked element by element."""
    for seed in range(4):
        a = make(1, 2, N, Dq, Dv, dtype, seed=100 * N + seed)
        st, out = F.triple_attention(*[t.to(dev) for t in a])
        q1, q2, k1, k2, v = (t.double() for t in a)
        sr, orf = O.triple_einsum(q1, q2, k1, k2, v, dtype=torch.float64)
        mag_state = torch.einsum("bhni,bhnj,bhnk->bhijk", k1.abs(), v.abs(), k2.abs()) / N
        mag = torch.einsum("bhni,bhijk,bhnk->bhnj", q1.abs(), mag_state, q2.abs())
        err = (out.double().cpu() - orf).abs()
        worst = float((err / mag).max())
        assert worst <= eps, (seed, worst, eps, float(mag.norm() / orf.norm()))
        # the state itself has no cancellation with one token (one term per entry) and little with two.  The kernel
        # rounds each product k1[n,i] k2[n,k] to the element type: in f16 a product below 2^-14 is subnormal and
        # carries an absolute error of up to 2^-25, which then meets |v[n,j]|
        sub = (2.0 ** -24 * v.abs().mean(2))[:, :, None, :, None] if dtype == torch.float16 else 0.0
        excess = (st.double().cpu() - sr).abs() - 2 * eps * mag_state - sub
        assert float(excess.max()) <= 0.0, float(excess.max())
