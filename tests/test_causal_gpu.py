"""GPU parity of causal FLARE (chunked prefill + recurrent decode) vs the CPU oracle.

The reference holds no causal-FLARE code; the oracle is the token recurrence, itself pinned by
the brute-force prefix definition in tests/test_oracle.py.  Tolerances: 1e-5 (fp32), 2e-2 (bf16/f16)
relative L2 against the fp64 oracle on the same rounded inputs.
"""
import pytest
import torch

import flare_py_amd as F
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def make(B, H, N, M, D, dtype, seed=0, std=None):
    g = torch.Generator().manual_seed(seed)
    std = D ** -0.25 if std is None else std
    q = (torch.randn(H, M, D, generator=g) * std).to(dtype)
    k = (torch.randn(B, H, N, D, generator=g) * std).to(dtype)
    v = (torch.randn(B, H, N, D, generator=g) * std).to(dtype)
    return q, k, v


def state_close(st, ref, tol):
    z, lse = O.causal_state_invariants(*(s.double().cpu() for s in st))
    zr, lser = O.causal_state_invariants(*ref)
    assert O.rel_l2(z, zr) <= tol
    assert float((lse - lser).abs().max()) <= max(tol, 1e-5) * 10


@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (2, 2, 37, 5, 4), (1, 2, 100, 16, 8), (2, 1, 70, 64, 32),
                                   (1, 2, 257, 128, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_prefill_vs_recurrence(dev, shape, dtype):
    q, k, v = make(*shape, dtype)
    y, st = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev), scale=0.8)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), 0.8)
    assert O.rel_l2(y, yr) <= TOL[dtype]
    state_close(st, str_, TOL[dtype] if dtype != torch.float32 else 1e-5)


def test_prefill_matches_bruteforce_definition(dev):
    q, k, v = make(1, 2, 40, 8, 4, torch.float32)
    y, _ = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev))
    assert O.rel_l2(y, O.causal_bruteforce(q, k, v)) <= 1e-5


def test_decode_steps_and_continuation(dev):
    # prefill(0..T) then decode steps == one long recurrence; decode-only from a fresh state too
    q, k, v = make(2, 2, 96, 32, 16, torch.float32, seed=1)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    yr, str_ = O.causal_recurrent(q, k, v)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :64], vd[:, :, :64])
    y2, st = F.flare_causal_decode(qd, kd[:, :, 64:], vd[:, :, 64:], st)
    assert O.rel_l2(torch.cat([y1, y2], 2), yr) <= 1e-5
    state_close(st, str_, 1e-5)
    # single-step API, token by token, from a fresh state
    st = None
    outs = []
    for t in range(8):
        if st is None:
            st = F.causal_fresh_state(2, 2, 32, 16, dev)
        yt, st = F.flare_causal_decode_step(qd, kd[:, :, t], vd[:, :, t], st)
        outs.append(yt)
    assert O.rel_l2(torch.stack(outs, 2), yr[:, :, :8]) <= 1e-5
    # last row of the causal output equals the non-causal mixer's last row
    yn, _ = O.mixer_explicit(q, k, v)
    assert O.rel_l2(y2[:, :, -1], yn[:, :, -1]) <= 1e-5


def test_chunk_and_split_independence(dev):
    q, k, v = make(1, 2, 150, 16, 8, torch.float32, seed=2)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y_full, st_full = F.flare_causal_prefill(qd, kd, vd)
    for cut in (1, 16, 17, 149):
        ya, st = F.flare_causal_prefill(qd, kd[:, :, :cut], vd[:, :, :cut])
        yb, st = F.flare_causal_prefill(qd, kd[:, :, cut:], vd[:, :, cut:], state=st)
        assert O.rel_l2(torch.cat([ya, yb], 2), y_full) <= 2e-6
        z1, l1 = O.causal_state_invariants(*(s.double().cpu() for s in st))
        z2, l2 = O.causal_state_invariants(*(s.double().cpu() for s in st_full))
        assert O.rel_l2(z1, z2) <= 2e-6 and float((l1 - l2).abs().max()) < 1e-5


def test_growing_scores_stay_finite(dev):
    # scores that grow steadily along the sequence: every block raises the running maximum
    q, k, v = make(1, 1, 200, 16, 8, torch.float32, seed=3, std=1.0)
    k = k * torch.linspace(0.1, 4.0, 200)[None, None, :, None]
    y, st = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev))
    yr, _ = O.causal_recurrent(q, k, v)
    assert torch.isfinite(y).all() and O.rel_l2(y, yr) <= 1e-5


def test_strided_inputs(dev):
    B, H, N, M, D = 2, 2, 50, 16, 16
    g = torch.Generator().manual_seed(4)
    kx = torch.randn(B, N, H * D, generator=g).to(dev)
    vx = torch.randn(B, N, H * D, generator=g).to(dev)
    q = (torch.randn(H, M, D, generator=g) * 0.3).to(dev)
    k = kx.view(B, N, H, D).permute(0, 2, 1, 3)
    v = vx.view(B, N, H, D).permute(0, 2, 1, 3)
    y, _ = F.flare_causal_prefill(q, k, v)
    yr, _ = O.causal_recurrent(q.cpu(), k.cpu(), v.cpu())
    assert O.rel_l2(y, yr) <= 1e-5


def test_cfg4_shape_reduced_length(dev):
    # BASELINE config 4 geometry (B=8,H=16,D=64,M=128, bf16, q,k,v ~ N(0, 1/sqrt(D))) at a length the
    # CPU recurrence finishes in seconds: prefill 512 tokens (chunk 256) + 32 decode steps.
    B, H, D, M, NP, ND = 8, 16, 64, 128, 512, 32
    q, k, v = make(B, H, NP + ND, M, D, torch.bfloat16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :NP], vd[:, :, :NP], chunk=256)
    y2, st = F.flare_causal_decode(qd, kd[:, :, NP:], vd[:, :, NP:], st)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(y1, yr[:, :, :NP]) <= 2e-2
    assert O.rel_l2(y2, yr[:, :, NP:]) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


# ---- matrix-core prefill kernel (bf16/f16, M in {128,256}, D in {32,64}) ------------------------
@pytest.mark.parametrize("shape", [(1, 2, 333, 128, 32), (1, 1, 100, 256, 32), (2, 1, 64, 128, 64), (1, 3, 1000, 128, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mfma_prefill_shapes(dev, shape, dtype):
    q, k, v = make(*shape, dtype)
    y, st = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev))
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(y, yr) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


def test_mfma_prefill_continuation_and_decode(dev):
    # state handed from one matrix-core prefill to the next and on to the recurrent decode
    q, k, v = make(1, 2, 700, 128, 64, torch.bfloat16, seed=6)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :300], vd[:, :, :300])
    y2, st = F.flare_causal_prefill(qd, kd[:, :, 300:650], vd[:, :, 300:650], state=st)
    y3, st = F.flare_causal_decode(qd, kd[:, :, 650:], vd[:, :, 650:], st)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(torch.cat([y1, y2, y3], 2), yr) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


def test_mfma_prefill_out_of_window_scores_fall_back(dev):
    # scores far outside the window in which the matrix-core kernel may skip the running maximum:
    # it must flag those (b,h) and the fp32 kernel must redo them; one head stays in the window.
    q, k, v = make(1, 2, 200, 128, 64, torch.bfloat16, seed=7, std=1.0)
    k[:, 0] *= 8.0                      # head 0: |score| up to several hundred
    k[:, 1] *= 0.05                     # head 1: tame
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    assert float(s[:, 0].abs().max()) > 150 and float(s[:, 1].abs().max()) < 20
    y, st = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev))
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    assert torch.isfinite(y.float()).all()
    assert O.rel_l2(y[:, 0], yr[:, 0]) <= 1e-5 * 1e3   # fp32 kernel on bf16 outputs: bf16 output rounding only
    assert O.rel_l2(y[:, 1], yr[:, 1]) <= 2e-2
    state_close(st, str_, 2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("offset", [-16.0, 14.0])
def test_mfma_prefill_constant_score_offset(dev, dtype, offset):
    # every score carries the same constant; all softmaxes of the recurrence are invariant to it
    q, k, v = make(1, 2, 300, 128, 32, dtype)
    q[..., 0] = 4.0
    k[..., 0] = offset / 4.0
    y, st = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev))
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), 1.0)
    assert O.rel_l2(y, yr) <= TOL[dtype]
    state_close(st, str_, TOL[dtype])


def test_mfma_prefill_segment_length_independence(dev):
    # the matrix-core prefill cuts the tokens into segments that run in parallel; any segment
    # length (one segment, ragged last segment, many short segments) gives the same result, with
    # and without an incoming state
    q, k, v = make(2, 2, 1000, 128, 64, torch.bfloat16, seed=9)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    _, st0 = F.flare_causal_prefill(qd, kd[:, :, :200], vd[:, :, :200], chunk=1000)
    for chunk in (0, 16, 48, 256, 400, 1000):
        y, st = F.flare_causal_prefill(qd, kd, vd, chunk=chunk)
        y2, st2 = F.flare_causal_prefill(qd, kd, vd, chunk=chunk)
        assert torch.equal(y, y2) and all(torch.equal(a, b) for a, b in zip(st, st2))   # bit-stable
        assert O.rel_l2(y, yr) <= 2e-2, chunk
        state_close(st, str_, 2e-2)
        yc, stc = F.flare_causal_prefill(qd, kd[:, :, 200:], vd[:, :, 200:], chunk=chunk, state=st0)
        assert O.rel_l2(yc, yr[:, :, 200:]) <= 2e-2, chunk
        state_close(stc, str_, 2e-2)


@pytest.mark.parametrize("shape", [(8, 16, 3000, 128, 64), (8, 16, 5000, 128, 32), (8, 16, 3000, 256, 32), (6, 16, 2611, 128, 64)])
def test_mfma_prefill_first_phase_pieces(dev, shape):
    """With as many (b,h) as config 4 the library's own plan has segments longer than 256 tokens, and its first phase
    runs as pieces that reach across segment boundaries (one local state on either side).  Same results as one
    segment, bit-stable, and the oracle's on the (b,h) checked."""
    B, H, N, M, D = shape
    q, k, v = make(B, H, N, M, D, torch.bfloat16, seed=21)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y, st = F.flare_causal_prefill(qd, kd, vd)
    y2, st2 = F.flare_causal_prefill(qd, kd, vd)
    assert torch.equal(y, y2) and all(torch.equal(a, b) for a, b in zip(st, st2))
    y1, st1 = F.flare_causal_prefill(qd, kd, vd, chunk=N)
    assert O.rel_l2(y, y1) <= 1e-2
    state_close(st, tuple(t.double().cpu() for t in st1), 1e-2)
    for b, h in ((0, 0), (B - 1, H - 1)):
        yr, _ = O.causal_recurrent(q[h:h + 1].float(), k[b:b + 1, h:h + 1].float(), v[b:b + 1, h:h + 1].float())
        assert O.rel_l2(y[b:b + 1, h:h + 1], yr) <= 2e-2


def test_mfma_prefill_fallback_from_a_middle_segment(dev):
    # only the tokens of one middle segment leave the window: the whole (b,h) must be redone by the
    # fp32 kernel FROM THE INCOMING STATE (which the matrix-core pass must not have touched)
    q, k, v = make(1, 2, 640, 128, 64, torch.bfloat16, seed=11, std=1.0)
    k[:, 1] *= 0.05
    k[:, 0, :256] *= 0.05
    k[:, 0, 256:384] *= 8.0
    k[:, 0, 384:] *= 0.05
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    _, st0 = F.flare_causal_prefill(qd, kd[:, :, :100], vd[:, :, :100])
    y, st = F.flare_causal_prefill(qd, kd[:, :, 100:], vd[:, :, 100:], chunk=128, state=st0)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    assert torch.isfinite(y.float()).all()
    assert O.rel_l2(y[:, 0], yr[:, 0, 100:]) <= 1e-2
    assert O.rel_l2(y[:, 1], yr[:, 1, 100:]) <= 2e-2
    state_close(st, str_, 2e-2)


@pytest.mark.parametrize("M,D", [(128, 64), (256, 32)])
def test_mfma_continues_a_state_with_per_latent_shifts(dev, M, D):
    """The fp32 kernel leaves a running maximum PER LATENT in the state (mu differs from latent to latent by
    several units here).  The matrix-core kernels keep those shifts for the state but must weigh the latents of
    one token against each other with ONE common shift: prefill (64-token chunks at M = 128, 16-token blocks at
    M = 256) and decode, continued from such a state, against one long pass of the oracle."""
    N1, N2, ND = 300, 200, 9
    q, k, v = make(1, 2, N1 + N2 + ND, M, D, torch.bfloat16, seed=11, std=0.8)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    _, st = F.flare_causal_prefill(q.float().to(dev), k[:, :, :N1].float().to(dev), v[:, :, :N1].float().to(dev))
    assert float((st[0].amax(-1) - st[0].amin(-1)).min()) > 2.0      # the shifts really differ
    y2, st2 = F.flare_causal_prefill(q.to(dev), k[:, :, N1:N1 + N2].to(dev), v[:, :, N1:N1 + N2].to(dev), state=st)
    assert O.rel_l2(y2, yr[:, :, N1:N1 + N2]) <= TOL[torch.bfloat16]
    y3, st3 = F.flare_causal_decode(q.to(dev), k[:, :, N1 + N2:].to(dev), v[:, :, N1 + N2:].to(dev), st2)
    assert O.rel_l2(y3, yr[:, :, N1 + N2:]) <= TOL[torch.bfloat16]
    state_close(st3, str_, TOL[torch.bfloat16])


def test_mfma_continues_after_a_fallback(dev):
    """A (b,h) the matrix-core kernel could not validate is redone by the fp32 kernel, which leaves per-latent
    shifts in its state; the next call starts from that state on the matrix cores again."""
    q, k, v = make(1, 2, 264, 128, 64, torch.bfloat16, seed=7, std=1.0)
    k[:, 0, :200] *= 8.0                # head 0 leaves the window during the first call only
    k[:, 0, 200:] *= 0.05
    k[:, 1] *= 0.05
    yr, _ = O.causal_recurrent(q.float(), k.float(), v.float())
    _, st = F.flare_causal_prefill(q.to(dev), k[:, :, :200].to(dev), v[:, :, :200].to(dev))
    y, _ = F.flare_causal_prefill(q.to(dev), k[:, :, 200:].to(dev), v[:, :, 200:].to(dev), state=st)
    assert torch.isfinite(y.float()).all()
    assert O.rel_l2(y, yr[:, :, 200:]) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("M,D", [(128, 64), (128, 32), (256, 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_kernel_shapes(dev, M, D, dtype):
    """Every instantiation of the one-launch decode kernel: 37 steps from a fresh state and 21 more from the state
    they leave, against the oracle's recurrence; the state at the end against the oracle's."""
    q, k, v = make(2, 3, 58, M, D, dtype, seed=5)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    st = F.causal_fresh_state(2, 3, M, D, dev)
    y1, st = F.flare_causal_decode(q.to(dev), k[:, :, :37].to(dev), v[:, :, :37].to(dev), st)
    y2, st = F.flare_causal_decode(q.to(dev), k[:, :, 37:].to(dev), v[:, :, 37:].to(dev), st)
    assert O.rel_l2(torch.cat([y1, y2], 2), yr) <= TOL[dtype]
    state_close(st, str_, TOL[dtype])


@pytest.mark.parametrize("chunk", [256, 0])
def test_cfg4_full_size_properties(dev, chunk):
    """BASELINE config 4 at its full size (B=8, H=16, D=64, M=128, bf16; 8192 prefill tokens in chunks of 256 as the
    config words it, and in the segments the library chooses itself (chunk=0: what bench.py times), then 256
    decode steps), through properties that need no full-size CPU run: decode after prefill = one longer prefill;
    the final state = the non-causal gather over all tokens; the last output row = the non-causal mixer's;
    and one (b, h) pair against the fp64 token recurrence over the whole length."""
    B, H, D, M, NP, ND = 8, 16, 64, 128, 8192, 256
    q, k, v = make(B, H, NP + ND, M, D, torch.bfloat16, seed=4)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :NP], vd[:, :, :NP], chunk=chunk)
    y2, st = F.flare_causal_decode(qd, kd[:, :, NP:], vd[:, :, NP:], st)
    yl, stl = F.flare_causal_prefill(qd, kd, vd, chunk=chunk)
    assert torch.isfinite(y1).all() and torch.isfinite(y2).all()
    # chunks of 256: same kernel, same segment boundaries; the library's own plan cuts the longer call elsewhere
    assert O.rel_l2(y1, yl[:, :, :NP]) <= (1e-6 if chunk else 2e-2)
    assert O.rel_l2(y2, yl[:, :, NP:]) <= 2e-2
    z, lse = O.causal_state_invariants(*(t.double() for t in st))
    zl, lsel = O.causal_state_invariants(*(t.double() for t in stl))
    assert O.rel_l2(z, zl) <= 2e-2 and float((lse - lsel).abs().max()) <= 0.2
    zg, lseg = F.flare_gather(qd, kd, vd)
    assert O.rel_l2(z, zg.double()) <= 2e-2 and float((lse - lseg.double()).abs().max()) <= 0.2
    yn = F.flare_multihead_mixer(qd, kd, vd)
    assert O.rel_l2(y2[:, :, -1], yn[:, :, -1]) <= 2e-2
    b, h = 5, 11
    yr, str_ = O.causal_recurrent(q[h:h + 1].float(), k[b:b + 1, h:h + 1].float(), v[b:b + 1, h:h + 1].float(), dtype=torch.float64)
    assert O.rel_l2(y1[b, h], yr[0, 0, :NP]) <= 2e-2
    assert O.rel_l2(y2[b, h], yr[0, 0, NP:]) <= 2e-2
    zr, lser = O.causal_state_invariants(*str_)
    assert O.rel_l2(z[b, h].cpu(), zr[0, 0]) <= 2e-2 and float((lse[b, h].cpu() - lser[0, 0]).abs().max()) <= 0.2


@pytest.mark.parametrize("M,D", [(128, 16), (256, 8), (128, 48)])
def test_narrow_heads_on_the_matrix_core_path(dev, M, D):
    """D below 32 is zero-padded to 32, D between 32 and 64 to 64 (128 latents: 256 x 64 does not fit the kernels' LDS), around the matrix-core kernels: prefill, a second prefill from the returned
    state, then decode, against the recurrence; the state comes back with its own D columns."""
    q, k, v = make(2, 2, 900, M, D, torch.bfloat16, seed=12)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :400], vd[:, :, :400])
    assert st[2].shape == (2, 2, M, D)
    y2, st = F.flare_causal_prefill(qd, kd[:, :, 400:850], vd[:, :, 400:850], state=st)
    y3, st = F.flare_causal_decode(qd, kd[:, :, 850:], vd[:, :, 850:], st)
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(torch.cat([y1, y2, y3], 2), yr) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


@pytest.mark.parametrize("M,D", [(64, 32), (64, 8), (32, 64), (16, 16), (64, 40)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_power_of_two_latent_counts_below_128(dev, M, D, dtype):
    """Fewer than 128 latents run on the matrix-core kernels as 128 // M copies of every latent (the copies share
    the softmax weight of the one they stand for): prefill, a continued prefill, a long decode (same route) and
    single steps (fp32 step kernel) against the recurrence; the state comes back with M latents, and matches
    what the fp32 kernels give for the same call."""
    q, k, v = make(2, 2, 700, M, D, dtype, seed=21)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :300], vd[:, :, :300])
    assert st[0].shape == (2, 2, M) and st[2].shape == (2, 2, M, D)
    y2, st = F.flare_causal_prefill(qd, kd[:, :, 300:640], vd[:, :, 300:640], state=st)
    y3, st = F.flare_causal_decode(qd, kd[:, :, 640:698], vd[:, :, 640:698], st)
    ys = []
    for t in (698, 699):
        yt, st = F.flare_causal_decode_step(qd, kd[:, :, t], vd[:, :, t], st)
        ys.append(yt.unsqueeze(2))
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(torch.cat([y1, y2, y3] + ys, 2), yr) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


@pytest.mark.parametrize("M,D", [(256, 64), (256, 48), (96, 32), (192, 64), (512, 32), (224, 16), (384, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_latent_counts_run_in_groups(dev, M, D, dtype):
    """Latent counts the matrix-core kernels do not take in one piece (256 with D above 32, 96, 192, 224, 384, 512)
    run as causal problems over groups of latents, joined per token by the groups' softmax weights: prefill,
    continued prefill, long decode and single steps against the recurrence, with the later latents' scores scaled
    so that the groups' weights differ by orders of magnitude on part of the tokens."""
    from flare_py_amd import functional as fn
    assert len(fn._causal_latent_groups(M, D)) > 1 and sum(fn._causal_latent_groups(M, D)) == M
    q, k, v = make(1, 2, 600, M, D, dtype, seed=31)
    q[:, M // 2:] = (q[:, M // 2:].float() * 1.5).to(dtype)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    y1, st = F.flare_causal_prefill(qd, kd[:, :, :250], vd[:, :, :250])
    assert st[0].shape == (1, 2, M) and st[2].shape == (1, 2, M, D)
    y2, st = F.flare_causal_prefill(qd, kd[:, :, 250:540], vd[:, :, 250:540], state=st)
    y3, st = F.flare_causal_decode(qd, kd[:, :, 540:598], vd[:, :, 540:598], st)
    ys = []
    for t in (598, 599):
        yt, st = F.flare_causal_decode_step(qd, kd[:, :, t], vd[:, :, t], st)
        ys.append(yt.unsqueeze(2))
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float(), dtype=torch.float32)
    assert O.rel_l2(torch.cat([y1, y2, y3] + ys, 2), yr) <= 2e-2
    state_close(st, tuple(s.double() for s in str_), 2e-2)


def test_latent_group_sizes():
    from flare_py_amd import functional as fn
    assert fn._causal_latent_groups(128, 64) == [128] and fn._causal_latent_groups(256, 32) == [256]
    assert fn._causal_latent_groups(64, 8) == [64] and fn._causal_latent_groups(48, 32) == []
    assert fn._causal_latent_groups(256, 33) == [128, 128] and fn._causal_latent_groups(224, 16) == [128, 64, 32]
    assert fn._causal_latent_groups(768, 32) == [256, 256, 256] and fn._causal_latent_groups(160, 64) == [128, 32]
    assert fn._causal_latent_groups(128, 65) == []


# ---- per-token log-sum-exp over the latents (what joins latent groups), from every kernel that writes y ----
@pytest.mark.parametrize("shape,dtype,chunk", [
    ((1, 2, 300, 128, 64), torch.bfloat16, 0),       # 64-token chunk kernel
    ((1, 2, 1200, 128, 32), torch.float16, 256),     # the same in several segments
    ((1, 1, 200, 256, 32), torch.bfloat16, 0),       # 16-token block kernel
    ((2, 1, 90, 24, 8), torch.float32, 0),           # fp32 kernel
    ((1, 2, 150, 64, 32), torch.bfloat16, 0),        # copies of every latent
    ((1, 2, 100, 128, 16), torch.bfloat16, 0),       # zero-padded head
])
def test_token_lse_of_prefill_and_decode(dev, shape, dtype, chunk):
    from flare_py_amd import functional as FN
    B, H, N, M, D = shape
    q, k, v = make(*shape, dtype, seed=41)
    scale = 0.9
    want = torch.logsumexp(scale * torch.einsum("bhnd,hmd->bhnm", k.double(), q.double()), dim=-1)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    y, st, lse = FN._causal_call("prefill", q.to(dev), k.to(dev), v.to(dev), scale, chunk, None, want_lse=True)
    assert lse.shape == (B, H, N) and float((lse.double().cpu() - want).abs().max()) <= tol
    y0, _ = F.flare_causal_prefill(q.to(dev), k.to(dev), v.to(dev), scale=scale, chunk=chunk)
    assert torch.equal(y, y0)                        # asking for the sums changes nothing else
    # decode: the last 40 tokens as steps after a prefill of the rest
    n0 = N - 40
    _, st = F.flare_causal_prefill(q.to(dev), k[:, :, :n0].contiguous().to(dev), v[:, :, :n0].contiguous().to(dev), scale=scale)
    _, _, lse_d = FN._causal_call("decode", q.to(dev), k[:, :, n0:].contiguous().to(dev), v[:, :, n0:].contiguous().to(dev),
                                  scale, 0, st, want_lse=True)
    assert float((lse_d.double().cpu() - want[:, :, n0:]).abs().max()) <= tol


def test_group_join_kernel(dev):
    from flare_py_amd import functional as FN
    g = torch.Generator().manual_seed(43)
    ys = [torch.randn(2, 3, 50, 32, generator=g).bfloat16() for _ in range(3)]
    lses = [torch.randn(2, 3, 50, generator=g) * 3 for _ in range(3)]
    got = FN._causal_join([t.to(dev) for t in ys], [t.to(dev) for t in lses])
    w = torch.softmax(torch.stack(lses).double(), dim=0).unsqueeze(-1)
    want = (w * torch.stack([t.double() for t in ys])).sum(0)
    assert got.dtype == torch.bfloat16 and O.rel_l2(got, want) <= 5e-3
    assert torch.equal(got, FN._causal_join([t.to(dev) for t in ys], [t.to(dev) for t in lses]))


# ---- decoding token by token: state advanced in place, buffers reused, nothing allocated per step ----
def test_single_step_calls_equal_one_launch_bit_for_bit(dev):
    B, H, M, D, NP, ND = 2, 4, 128, 64, 512, 256           # config 4's M, D and step count
    q, k, v = make(B, H, NP + ND, M, D, torch.bfloat16, seed=45)
    qd = q.to(dev)
    kp, vp = k[:, :, :NP].contiguous().to(dev), v[:, :, :NP].contiguous().to(dev)
    kd, vd = k[:, :, NP:].contiguous().to(dev), v[:, :, NP:].contiguous().to(dev)
    _, st0 = F.flare_causal_prefill(qd, kp, vp)
    y_all, st_all = F.flare_causal_decode(qd, kd, vd, st0)                 # 256 steps in one launch
    st = tuple(s.clone() for s in st0)
    ws = F.causal_workspace(qd, kd[:, :, :1])
    y_steps = torch.empty_like(y_all)
    ptrs = [s.data_ptr() for s in st]
    for t in range(ND):
        _, st_t = F.flare_causal_decode_step(qd, kd[:, :, t:t + 1], vd[:, :, t:t + 1], st, inplace=True, workspace=ws,
                                             out=y_steps[:, :, t:t + 1])
        assert [s.data_ptr() for s in st_t] == ptrs        # the same tensors, advanced
    assert torch.equal(y_steps, y_all)
    for a, b in zip(st, st_all):
        assert torch.equal(a, b)
    # the incoming state of a call without inplace is left as it was
    before = tuple(s.clone() for s in st0)
    F.flare_causal_decode(qd, kd[:, :, :3], vd[:, :, :3], st0)
    for a, b in zip(st0, before):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        q192 = torch.cat([qd, qd[:, :64]], dim=1)                  # 192 latents run as groups: no in-place form
        F.flare_causal_decode_step(q192, kd[:, :, :1], vd[:, :, :1], F.causal_fresh_state(B, H, 192, D, dev), inplace=True)


def test_decode_steps_replay_from_a_hip_graph(dev):
    """256 in-place single-token steps captured once in a HIP graph: every replay (with eager work in between) must
    reproduce the eager 256-step launch from the same starting state."""
    B, H, M, D, NP, ND = 2, 4, 128, 64, 256, 256
    q, k, v = make(B, H, NP + ND, M, D, torch.bfloat16, seed=47)
    qd = q.to(dev)
    kp, vp = k[:, :, :NP].contiguous().to(dev), v[:, :, :NP].contiguous().to(dev)
    kd, vd = k[:, :, NP:].contiguous().to(dev), v[:, :, NP:].contiguous().to(dev)
    _, st0 = F.flare_causal_prefill(qd, kp, vp)
    y_all, st_all = F.flare_causal_decode(qd, kd, vd, st0)
    st = tuple(s.clone() for s in st0)
    ws = F.causal_workspace(qd, kd[:, :, :1])
    y_steps = torch.empty_like(y_all)

    def steps():
        for t in range(ND):
            F.flare_causal_decode_step(qd, kd[:, :, t:t + 1], vd[:, :, t:t + 1], st, inplace=True, workspace=ws,
                                       out=y_steps[:, :, t:t + 1])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        steps()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        steps()
    for rep in range(3):
        for a, b in zip(st, st0):
            a.copy_(b)
        y_steps.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_steps, y_all), rep
        for a, b in zip(st, st_all):
            assert torch.equal(a, b)
        F.flare_causal_prefill(qd, kp, vp)               # eager work between replays


@pytest.mark.parametrize("M,D", [(128, 64), (256, 32)])
def test_decode_steps_outside_the_window_are_redone_in_the_same_launch(dev, M, D):
    """Decode steps whose scores leave the window in which the kernel may skip the running maximum: the workgroup of
    that (b,h) repeats the call's steps with a running maximum inside the same launch (fp32 scores, so what is left is
    the rounding of the 16-bit output); the other head stays on the fast path.  Then both continue from the states
    those calls left, back inside the window."""
    q, k, v = make(1, 2, 90, M, D, torch.bfloat16, seed=9, std=1.0)
    k[:, 0, :60] *= 8.0                   # head 0: |score| up to several hundred during the first call
    k[:, 0, 60:] *= 0.05
    k[:, 1] *= 0.05
    s = torch.einsum("hmd,bhnd->bhmn", q.float(), k.float())
    assert float(s[:, 0, :, :60].abs().max()) > 150 and float(s[:, 1].abs().max()) < 20
    yr, str_ = O.causal_recurrent(q.float(), k.float(), v.float())
    st = F.causal_fresh_state(1, 2, M, D, dev)
    y1, st = F.flare_causal_decode(q.to(dev), k[:, :, :60].to(dev), v[:, :, :60].to(dev), st)
    y2, st = F.flare_causal_decode(q.to(dev), k[:, :, 60:].to(dev), v[:, :, 60:].to(dev), st)
    y = torch.cat([y1, y2], 2)
    assert torch.isfinite(y.float()).all()
    assert O.rel_l2(y[:, 0, :60], yr[:, 0, :60]) <= 1e-2 and O.rel_l2(y[:, 1], yr[:, 1]) <= 2e-2
    assert O.rel_l2(y[:, 0, 60:], yr[:, 0, 60:]) <= 2e-2
    state_close(st, str_, 2e-2)
    # one step at a time through the same path gives the same rows to rounding
    st1 = F.causal_fresh_state(1, 2, M, D, dev)
    rows = []
    for t in range(8):
        yt, st1 = F.flare_causal_decode(q.to(dev), k[:, :, t:t + 1].to(dev), v[:, :, t:t + 1].to(dev), st1)
        rows.append(yt)
    assert O.rel_l2(torch.cat(rows, 2)[:, 0], yr[:, 0, :8]) <= 1e-2
