"""Host-side checks of the C-ABI that need no GPU: the library loads, exports every symbol
include/flare_hip.h declares, and rejects bad requests before anything is launched."""
import ctypes as C
import os
import re

import pytest
import torch

import flare_py_amd as F
from flare_py_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _mixer_desc(B=1, H=2, N=128, M=64, D=32, dtype=_lib.DT_BF16, scale=1.0):
    d = _lib.FlareMixerDesc()
    d.B, d.H, d.N, d.M, d.D, d.dtype, d.scale = B, H, N, M, D, dtype, scale
    d.q_stride = _lib.I3(0, M * D, D)
    d.k_stride = d.v_stride = d.y_stride = _lib.I3(H * N * D, N * D, D)
    return d


def test_header_symbols_all_exported():
    text = open(os.path.join(ROOT, "include", "flare_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(flare_[a-z_]+)\s*\(", text))
    assert declared, "no declarations parsed"
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in flare_hip.h but not exported"
    assert declared == set(_lib.SYMBOLS), "ctypes binding and header disagree"
    assert lib.flare_abi_version() == _lib.ABI_VERSION == 2


def test_struct_sizes_match_header_layout():
    assert C.sizeof(_lib.FlareMixerDesc) == 10 * 4 + 4 * 24 + 16       # + dropout_p, reserved2, dropout_seed
    assert C.sizeof(_lib.FlareCausalDesc) == 10 * 4 + 4 * 24
    assert C.sizeof(_lib.FlareTripleDesc) == 10 * 4 + 6 * 24


def test_workspace_query_and_kernel_choice():
    lib = _lib.load()
    n = C.c_size_t(0)
    d = _mixer_desc()
    assert lib.flare_mixer_workspace_bytes(C.byref(d), C.byref(n)) == 0 and n.value > 0
    assert lib.flare_mixer_kernel_name(C.byref(d)) == b"mfma_bf16"
    d.flags = _lib.FLAG_FORCE_GENERIC
    assert lib.flare_mixer_kernel_name(C.byref(d)) == b"generic"
    assert lib.flare_mixer_kernel_name(C.byref(_mixer_desc(dtype=_lib.DT_F32))) == b"generic"
    assert lib.flare_mixer_kernel_name(C.byref(_mixer_desc(M=16, D=8))) == b"generic"
    assert lib.flare_mixer_kernel_name(C.byref(_mixer_desc(dtype=_lib.DT_F16))) == b"mfma_f16"


@pytest.mark.parametrize("field,value,code", [
    ("N", 0, _lib.FLARE_EINVAL), ("M", -1, _lib.FLARE_EINVAL), ("D", 256, _lib.FLARE_EUNSUPPORTED),
    ("dtype", 7, _lib.FLARE_EINVAL), ("scale", 0.0, _lib.FLARE_EINVAL), ("n_splits", -2, _lib.FLARE_EINVAL),
])
def test_bad_descriptor_rejected(field, value, code):
    lib = _lib.load()
    d = _mixer_desc()
    setattr(d, field, value)
    n = C.c_size_t(0)
    assert lib.flare_mixer_workspace_bytes(C.byref(d), C.byref(n)) == code
    assert _lib.last_error() != ""


def test_null_pointers_and_workspace_rejected_before_launch():
    lib = _lib.load()
    d = _mixer_desc()
    one = C.c_void_p(16)  # never dereferenced: validation fails first
    assert lib.flare_mixer_fwd(C.byref(d), None, one, one, None, one, None, one, 1 << 30, None) == _lib.FLARE_EINVAL
    assert lib.flare_mixer_fwd(C.byref(d), one, one, one, None, one, None, None, 0, None) == _lib.FLARE_EWORKSPACE
    assert lib.flare_mixer_fwd(C.byref(d), one, one, one, None, one, None, one, 8, None) == _lib.FLARE_EWORKSPACE
    assert "needed" in _lib.last_error()
    assert lib.flare_gather_fwd(C.byref(d), one, one, one, None, None, None, one, 1 << 30, None) == _lib.FLARE_EINVAL
    assert lib.flare_scatter_fwd(C.byref(d), one, one, None, None, one, None) == _lib.FLARE_EINVAL
    d.k_stride = _lib.I3(0, 0, 3)  # row stride < D
    assert lib.flare_scatter_fwd(C.byref(d), one, one, one, None, one, None) == _lib.FLARE_EINVAL
    assert lib.flare_mixer_workspace_bytes(None, C.byref(C.c_size_t(0))) == _lib.FLARE_EINVAL


def test_causal_and_triple_validation():
    lib = _lib.load()
    one = C.c_void_p(16)
    c = _lib.FlareCausalDesc()
    c.B, c.H, c.N, c.M, c.D, c.dtype, c.scale = 1, 1, 8, 16, 16, 0, 1.0
    c.q_stride = _lib.I3(0, 256, 16)
    c.k_stride = c.v_stride = c.y_stride = _lib.I3(128, 128, 16)
    assert lib.flare_causal_prefill_fwd(C.byref(c), one, one, one, one, None, one, one, None, 0, None) == _lib.FLARE_EINVAL
    c.M, c.D = 4096, 128
    n = C.c_size_t(0)
    assert lib.flare_causal_workspace_bytes(C.byref(c), C.byref(n)) == _lib.FLARE_EUNSUPPORTED
    t = _lib.FlareTripleDesc()
    t.B, t.H, t.N, t.Dq, t.Dv, t.dtype = 1, 1, 64, 16, 16, 1
    assert lib.flare_triple_workspace_bytes(C.byref(t), C.byref(n)) == 0 and n.value > 0
    assert lib.flare_triple_fwd(C.byref(t), one, one, one, one, one, one, one, one, 4, None) == _lib.FLARE_EWORKSPACE
    t.Dq = 128
    assert lib.flare_triple_workspace_bytes(C.byref(t), C.byref(n)) == _lib.FLARE_EUNSUPPORTED
    t.Dq, t.feature_map = 16, 5
    assert lib.flare_triple_workspace_bytes(C.byref(t), C.byref(n)) == _lib.FLARE_EINVAL


def test_python_api_fails_loudly_on_cpu_tensors():
    q = torch.randn(2, 4, 8)
    k = torch.randn(1, 2, 16, 8)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        F.flare_multihead_mixer(q, k, k)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        F.triple_attention(k, k, k, k, k)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        F.flare_causal_prefill(q, k, k)


def test_status_to_exception_mapping():
    _lib.load().flare_mixer_workspace_bytes(None, None)
    with pytest.raises(ValueError):
        _lib.check(_lib.FLARE_EINVAL, "x")
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.FLARE_EUNSUPPORTED, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.FLARE_EHIP, "x")


def test_new_struct_sizes_and_entry_point_validation():
    assert C.sizeof(_lib.FlareCausalLinearDesc) == 8 * 4 + 4 * 24
    assert C.sizeof(_lib.FlareMlpDesc) == 8 + 12 * 4 + 3 * 8
    lib = _lib.load()
    # fused MLP: argument checks happen before anything is launched
    m = _lib.FlareMlpDesc()
    m.T, m.C, m.L, m.w_dtype = 16, 128, 2, _lib.DT_BF16
    m.x_stride = m.y_stride = 128
    assert lib.flare_mlp_fwd(m, None, None, None, None, None, None, None, None) == _lib.FLARE_EINVAL
    assert "must not be NULL" in _lib.last_error()
    m.C = 48
    assert lib.flare_mlp_fwd(m, None, None, None, None, None, None, None, None) == _lib.FLARE_EUNSUPPORTED
    m.C, m.L = 128, 0
    assert lib.flare_mlp_fwd(m, None, None, None, None, None, None, None, None) == _lib.FLARE_EINVAL
    m.L, m.w_dtype = 2, _lib.DT_F32
    assert lib.flare_mlp_fwd(m, None, None, None, None, None, None, None, None) == _lib.FLARE_EINVAL
    # narrow first / last layers: widths above 4, a norm in front of a lifting layer, expand mode and a
    # residual next to a narrow output are refused (fake non-NULL pointers: nothing is dereferenced before the checks)
    m.w_dtype = _lib.DT_BF16
    fake = C.c_void_p(4096)
    io = lambda i, o, res=None: lib.flare_mlp_io_fwd(m, i, 1, fake, fake, o, fake, fake, None, fake, None, res, fake, None)
    assert io(5, 0) == _lib.FLARE_EINVAL and "in_dim and out_dim" in _lib.last_error()
    assert io(0, 7) == _lib.FLARE_EINVAL
    m.norm = 1
    assert io(3, 0) == _lib.FLARE_EINVAL and "norm" in _lib.last_error()
    m.norm, m.flags = 0, _lib.MLP_EXPAND
    assert io(3, 0) == _lib.FLARE_EINVAL and "EXPAND" in _lib.last_error()
    m.flags = 0
    assert io(0, 2, fake) == _lib.FLARE_EINVAL and "res must be NULL" in _lib.last_error()
    m.x_stride = 2
    assert io(3, 0) == _lib.FLARE_EINVAL and "x_stride" in _lib.last_error()
    # head-padded rows: head dims 4 and 8 only, not next to in_dim / out_dim, and rows wide enough for the padding
    m.x_stride = 128
    m.flags = (12 // 4) << 8
    assert lib.flare_mlp_fwd(m, fake, fake, None, fake, None, None, fake, None) == _lib.FLARE_EINVAL and "head dim" in _lib.last_error()
    m.flags = (8 // 4) << 12
    assert io(3, 0) == _lib.FLARE_EINVAL and "head dim" in _lib.last_error()
    assert lib.flare_mlp_fwd(m, fake, fake, None, fake, None, None, fake, None) == _lib.FLARE_EINVAL and "row width" in _lib.last_error()
    m.flags = 0
    # causal linear attention
    c = _lib.FlareCausalLinearDesc()
    c.B, c.H, c.N, c.Dk, c.Dv, c.dtype = 1, 2, 100, 32, 16, _lib.DT_F32
    c.q_stride = c.k_stride = _lib.I3(6400, 3200, 32)
    c.v_stride = c.y_stride = _lib.I3(3200, 1600, 16)
    need = C.c_size_t(0)
    assert lib.flare_causal_linear_workspace_bytes(c, C.byref(need)) == _lib.FLARE_OK and need.value > 0
    assert lib.flare_causal_linear_fwd(c, None, None, None, None, None, 0, None) == _lib.FLARE_EINVAL
    c.Dk = 200
    assert lib.flare_causal_linear_workspace_bytes(c, C.byref(need)) == _lib.FLARE_EUNSUPPORTED
    # mixer backward: supported shapes only, workspace checked
    d = _mixer_desc(M=128, D=32)
    assert lib.flare_mixer_bwd_workspace_bytes(d, C.byref(need)) == _lib.FLARE_OK and need.value > 0
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(dtype=_lib.DT_F32), C.byref(need)) == _lib.FLARE_OK     # fp32 kernels
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(dtype=_lib.DT_F32, M=40), C.byref(need)) == _lib.FLARE_EUNSUPPORTED
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(dtype=_lib.DT_F32, D=24), C.byref(need)) == _lib.FLARE_EUNSUPPORTED
    # the halves' backward: every dtype (16-bit without dropout), arguments checked before anything is launched
    f = _mixer_desc(dtype=_lib.DT_F32)
    assert lib.flare_gather_bwd(d, *([None] * 9), None, 0, None) == _lib.FLARE_EWORKSPACE
    d.dropout_p = 0.25
    assert lib.flare_gather_bwd(d, *([None] * 9), None, 0, None) == _lib.FLARE_EUNSUPPORTED and "dropout" in _lib.last_error()
    d.dropout_p = 0.0
    assert lib.flare_gather_bwd(f, *([None] * 9), None, 0, None) == _lib.FLARE_EWORKSPACE
    assert lib.flare_scatter_bwd(f, *([None] * 6), None, None, None, None, None, 0, None) == _lib.FLARE_EWORKSPACE
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(M=256, D=64), C.byref(need)) == _lib.FLARE_OK      # one LDS-full exactly
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(M=1024, D=64), C.byref(need)) == _lib.FLARE_OK     # four chunks of latents
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(M=2048, D=64), C.byref(need)) == _lib.FLARE_EUNSUPPORTED
    assert lib.flare_mixer_bwd_workspace_bytes(_mixer_desc(M=48, D=32), C.byref(need)) == _lib.FLARE_EUNSUPPORTED
    assert lib.flare_mixer_bwd(d, *([None] * 8), None, None, None, None, None, 0, None) == _lib.FLARE_EINVAL
    assert lib.flare_scatter_fwd_lse(d, None, None, None, None, None, None, None) == _lib.FLARE_EINVAL


@pytest.mark.parametrize("Cdim,L", [(32, 1), (64, 3), (128, 8)])
def test_both_weight_images_from_one_gather_equal_the_two_single_ones(Cdim, L):
    """A training step builds the image of the weights and of their transposes in one indexed read; each has to be what
    mlp_weight_image (checked against the header's formula below) gives for the matrix and for its transpose."""
    from flare_py_amd import fused
    w = torch.randn(L, Cdim, Cdim, generator=torch.Generator().manual_seed(Cdim + L)).to(torch.bfloat16)
    img, img_t = fused.mlp_weight_images(w)
    assert img.is_contiguous() and img_t.is_contiguous() and img.shape == img_t.shape == (L, Cdim * Cdim)
    assert torch.equal(img, fused.mlp_weight_image(w))
    assert torch.equal(img_t, fused.mlp_weight_image(w.transpose(1, 2).contiguous()))


@pytest.mark.parametrize("Cdim", [32, 64, 128])
def test_mlp_weight_image_follows_the_header_formula(Cdim):
    """fused.mlp_weight_image against include/flare_hip.h's position formula, element by element in plain loops:
    the image is a permutation inside each row, and a 16-byte piece holds four columns of one 8-column block and the
    same four of the block two further on."""
    from flare_py_amd import fused
    shift = {128: 0, 64: 1, 32: 2}[Cdim]
    w = torch.arange(2 * Cdim * Cdim, dtype=torch.float32).view(2, Cdim, Cdim)
    img = fused.mlp_weight_image(w).view(2, Cdim * Cdim)
    seen = set()
    for row in range(Cdim):
        for col in range(Cdim):
            ch, j = col // 8, col % 8
            key = (row % 16) >> shift
            pos = row * Cdim + 8 * ((4 * (ch // 4) + 2 * (ch % 2) + j // 4) ^ key) + 4 * ((ch % 4) // 2) + j % 4
            assert pos // Cdim == row and pos not in seen
            seen.add(pos)
            for l in range(2):
                assert img[l, pos] == w[l, row, col]
    assert len(seen) == Cdim * Cdim
    piece = img[0].view(Cdim, Cdim // 8, 8)[5].long() - 5 * Cdim          # columns held by row 5's pieces
    for p in piece:
        lo, hi = p[:4].tolist(), p[4:].tolist()
        assert lo == list(range(lo[0], lo[0] + 4)) and lo[0] % 4 == 0
        assert hi == [c + 16 for c in lo]


def test_mlp_bwd_validation():
    lib = _lib.load()
    m = _lib.FlareMlpDesc()
    m.T, m.C, m.L = 64, 128, 2
    m.x_dtype = m.y_dtype = m.w_dtype = _lib.DT_BF16
    m.norm, m.act, m.eps = 1, 0, 1e-5      # layer norm, tanh gelu
    m.x_stride = m.y_stride = 128
    fake = C.c_void_p(4096)
    odd = C.c_void_p(4100)
    ff = fake
    rows = C.c_int32(0)
    assert lib.flare_mlp_bwd_partial_rows(m, C.byref(rows)) == _lib.FLARE_OK and rows.value == 1
    m.T = 1 << 20
    assert lib.flare_mlp_bwd_partial_rows(m, C.byref(rows)) == _lib.FLARE_OK and 1 <= rows.value <= 4096
    big = rows.value
    m.T = 1 << 22
    assert lib.flare_mlp_bwd_partial_rows(m, C.byref(rows)) == _lib.FLARE_OK and rows.value == big     # capped by the CU count
    assert lib.flare_mlp_bwd_partial_rows(m, None) == _lib.FLARE_EINVAL
    m.T = 64

    def call(x=fake, dy=fake, gamma=ff, dn=fake, stats=ff, gb=ff):
        return lib.flare_mlp_bwd(m, x, dy, fake, fake, ff, gamma, ff, 0, fake, fake, fake, dn, stats, gb, None, None)

    assert lib.flare_mlp_bwd(None, *([None] * 7), 0, *([None] * 8)) == _lib.FLARE_EINVAL
    # add_dy is a set of two bits (add dy, accumulate into dx); anything else is refused before a launch
    assert lib.flare_mlp_bwd(m, fake, fake, fake, fake, ff, ff, ff, 4, fake, fake, fake, fake, ff, ff, None, None) == _lib.FLARE_EINVAL
    assert "unknown bits" in _lib.last_error()
    assert call(x=None) == _lib.FLARE_EINVAL and "must not be NULL" in _lib.last_error()
    assert call(gamma=None) == _lib.FLARE_EINVAL and "norm" in _lib.last_error()
    assert call(gb=None) == _lib.FLARE_EINVAL and "norm" in _lib.last_error()
    assert call(x=odd) == _lib.FLARE_EINVAL and "16-byte" in _lib.last_error()
    assert call(dn=odd) == _lib.FLARE_EINVAL and "16-byte" in _lib.last_error()
    m.L = 6
    assert call() == _lib.FLARE_EUNSUPPORTED and "at most 5 layers" in _lib.last_error()
    m.C = 64
    m.x_stride = 62
    assert call() == _lib.FLARE_EINVAL and "row stride" in _lib.last_error()
    m.x_stride = 64
    m.y_stride = 66
    assert call() == _lib.FLARE_EINVAL and "y_stride" in _lib.last_error()
    m.y_stride = 64
    m.L = 9
    assert call() == _lib.FLARE_EUNSUPPORTED and "at most 8 layers" in _lib.last_error()
    m.L = 2
    m.C = 48
    assert call() == _lib.FLARE_EUNSUPPORTED and "32, 64 and 128" in _lib.last_error()
    m.C = 128
    m.x_stride = m.y_stride = 128
    m.flags = _lib.MLP_EXPAND
    assert call() == _lib.FLARE_EUNSUPPORTED and "flags must be 0" in _lib.last_error()
    m.flags = 0
    m.w_dtype = _lib.DT_F32
    assert call() == _lib.FLARE_EINVAL and "w_dtype" in _lib.last_error()
    m.w_dtype = _lib.DT_BF16
    m.act = 7
    assert call() == _lib.FLARE_EINVAL and "activation" in _lib.last_error()
    m.act, m.eps = 0, -1.0
    assert call() == _lib.FLARE_EINVAL and "eps" in _lib.last_error()


def test_mlp_wgrad_validation():
    lib = _lib.load()
    m = _lib.FlareMlpDesc()
    m.T, m.C, m.L = 262144, 128, 5
    m.w_dtype = _lib.DT_BF16
    fake, odd = C.c_void_p(4096), C.c_void_p(4100)
    parts = C.c_int32(0)
    assert lib.flare_mlp_wgrad_partials(m, C.byref(parts)) == _lib.FLARE_OK and 1 <= parts.value <= 1024
    big = parts.value
    m.T = 100
    assert lib.flare_mlp_wgrad_partials(m, C.byref(parts)) == _lib.FLARE_OK and parts.value == 1
    m.C = 32            # eight waves split a token tile: eight partials per token range
    assert lib.flare_mlp_wgrad_partials(m, C.byref(parts)) == _lib.FLARE_OK and parts.value == 8
    m.C, m.T = 128, 262144
    assert lib.flare_mlp_wgrad_partials(m, None) == _lib.FLARE_EINVAL
    assert lib.flare_mlp_wgrad(m, None, 0, fake, 0, fake, None, None, None, None) == _lib.FLARE_EINVAL and "must not be NULL" in _lib.last_error()
    assert lib.flare_mlp_wgrad(m, fake, 0, fake, 0, odd, None, None, None, None) == _lib.FLARE_EINVAL and "16-byte" in _lib.last_error()
    assert lib.flare_mlp_wgrad(m, fake, 0, fake, 0, fake, None, fake, fake, None) == _lib.FLARE_EINVAL and "db needs db_part" in _lib.last_error()
    m.C = 96
    assert lib.flare_mlp_wgrad(m, fake, 0, fake, 0, fake, None, None, None, None) == _lib.FLARE_EUNSUPPORTED
    m.C, m.w_dtype = 128, _lib.DT_F32
    assert lib.flare_mlp_wgrad(m, fake, 0, fake, 0, fake, None, None, None, None) == _lib.FLARE_EINVAL and "w_dtype" in _lib.last_error()
    m.w_dtype = _lib.DT_BF16
    assert lib.flare_mlp_wgrad(m, fake, 4, fake, 0, fake, None, None, None, None) == _lib.FLARE_EINVAL and "layer strides" in _lib.last_error()
    m.L = 0
    assert lib.flare_mlp_wgrad_partials(m, C.byref(parts)) == _lib.FLARE_EINVAL
    assert big >= 64


def test_mlp_expand_bwd_validation():
    lib = _lib.load()
    m = _lib.FlareMlpDesc()
    m.T, m.C, m.L, m.flags = 64, 128, 8, _lib.MLP_EXPAND
    m.x_dtype = m.y_dtype = m.w_dtype = _lib.DT_BF16
    m.norm, m.act, m.eps = 1, 0, 1e-5
    m.x_stride = m.y_stride = 128
    fake, odd = C.c_void_p(4096), C.c_void_p(4100)

    def call(x=fake, h=fake, gamma=fake, dn=fake):
        return lib.flare_mlp_expand_bwd(m, x, fake, fake, fake, fake, gamma, fake, 0, fake, fake, fake, h, fake, dn, fake, fake, None, None)

    assert call(x=None) == _lib.FLARE_EINVAL and "must not be NULL" in _lib.last_error()
    assert call(h=odd) == _lib.FLARE_EINVAL and "16-byte" in _lib.last_error()
    assert call(gamma=None) == _lib.FLARE_EINVAL and "norm" in _lib.last_error()
    m.L = 7
    assert call() == _lib.FLARE_EUNSUPPORTED and "2 E tiles" in _lib.last_error()
    m.L = 18
    assert call() == _lib.FLARE_EUNSUPPORTED
    m.L, m.flags = 8, 0
    assert call() == _lib.FLARE_EINVAL and "FLARE_MLP_EXPAND" in _lib.last_error()
    m.flags, m.C = _lib.MLP_EXPAND, 96
    assert call() == _lib.FLARE_EUNSUPPORTED
