"""The allocation-free mixer entry point (scratch inside the library's code object) against flare_mixer_fwd."""
import ctypes as C

import pytest
import torch

from flare_py_amd import _lib


def _desc(B, H, N, M, D, dtype=_lib.DT_BF16, scale=1.0):
    d = _lib.FlareMixerDesc()
    d.B, d.H, d.N, d.M, d.D, d.dtype, d.scale = B, H, N, M, D, dtype, scale
    d.q_stride = _lib.I3(0, M * D, D)
    d.k_stride = d.v_stride = d.y_stride = _lib.I3(H * N * D, N * D, D)
    return d


def test_static_scratch_rejects_oversized_problem_on_the_host():
    lib = _lib.load()
    d = _desc(64, 64, 1 << 16, 256, 32)
    n = C.c_size_t(0)
    assert lib.flare_mixer_workspace_bytes(C.byref(d), C.byref(n)) == 0 and n.value > _lib.STATIC_SCRATCH_BYTES
    one = C.c_void_p(16)        # never dereferenced: the size check comes first
    assert lib.flare_mixer_fwd_static(C.byref(d), one, one, one, None, one, None) == _lib.FLARE_EWORKSPACE
    assert "static buffer" in _lib.last_error()
    assert lib.flare_mixer_fwd_static(C.byref(d), None, one, one, None, one, None) == _lib.FLARE_EINVAL


def _both(lib, dev, B, H, N, M, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    tdt = {_lib.DT_BF16: torch.bfloat16, _lib.DT_F16: torch.float16, _lib.DT_F32: torch.float32}[dtype]
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).to(tdt).to(dev)
    k = torch.randn(B, H, N, D, generator=g).to(tdt).to(dev)
    v = torch.randn(B, H, N, D, generator=g).to(tdt).to(dev)
    d = _desc(B, H, N, M, D, dtype)
    n = C.c_size_t(0)
    assert lib.flare_mixer_workspace_bytes(C.byref(d), C.byref(n)) == 0
    assert n.value <= _lib.STATIC_SCRATCH_BYTES
    ws = torch.empty(n.value, dtype=torch.uint8, device=dev)
    y_ref = torch.empty_like(k)
    y_new = torch.full_like(k, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.flare_mixer_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), None, y_ref.data_ptr(), None,
                             ws.data_ptr(), n.value, st)
    assert rc == 0, _lib.last_error()
    rc = lib.flare_mixer_fwd_static(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), None, y_new.data_ptr(), st)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return y_ref, y_new, (q, k, v)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [_lib.DT_BF16, _lib.DT_F32])
def test_static_scratch_equals_workspace_entry_point_twice(dev, dtype):
    """Two calls in a row on the same scratch, the second with a smaller problem: both must equal the
    caller-workspace entry point bit for bit (same plan, same kernels), and the oracle at the dtype's bar."""
    from oracle import flare_oracle as O
    lib = _lib.load()
    shapes = [(2, 4, 4096 + 40, 128, 32), (1, 2, 700, 64, 32)] if dtype != _lib.DT_F32 else [(1, 2, 2048, 48, 16), (1, 1, 300, 16, 16)]
    for i, (B, H, N, M, D) in enumerate(shapes):
        print(f"static scratch case {i}: B={B} H={H} N={N} M={M} D={D} dtype={dtype}", flush=True)
        y_ref, y_new, (q, k, v) = _both(lib, dev, B, H, N, M, D, dtype, seed=11 + i)
        assert torch.equal(y_ref, y_new)
        want, _ = O.mixer_explicit(q.double().cpu(), k.double().cpu(), v.double().cpu(), 1.0)
        err = (y_new.double().cpu() - want).norm() / want.norm()
        assert err <= (1e-5 if dtype == _lib.DT_F32 else 2e-2), err


@pytest.mark.gpu
def test_static_scratch_with_key_mask_and_replayed_from_a_graph_on_dirty_scratch(dev):
    """A masked problem through the static scratch, first eagerly, then replayed from a captured graph after other
    problems have left their partials in the scratch: every replay equals the caller-workspace entry point."""
    lib = _lib.load()
    B, H, N, M, D = 2, 2, 3000, 64, 32
    g = torch.Generator().manual_seed(5)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).bfloat16().to(dev)
    k = torch.randn(B, H, N, D, generator=g).bfloat16().to(dev)
    v = torch.randn(B, H, N, D, generator=g).bfloat16().to(dev)
    mask = (torch.rand(B, N, generator=g) > 0.3).to(torch.uint8)
    mask[1, 1000:] = 0
    mask = mask.to(dev)
    d = _desc(B, H, N, M, D)
    n = C.c_size_t(0)
    assert lib.flare_mixer_workspace_bytes(C.byref(d), C.byref(n)) == 0 and n.value <= _lib.STATIC_SCRATCH_BYTES
    ws = torch.empty(n.value, dtype=torch.uint8, device=dev)
    y_ref = torch.empty_like(k)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.flare_mixer_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), y_ref.data_ptr(), None,
                               ws.data_ptr(), n.value, st) == 0, _lib.last_error()
    y = torch.full_like(k, float("nan"))
    # the first call on the device (it resolves the scratch address) happens before any capture
    assert lib.flare_mixer_fwd_static(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), y.data_ptr(), st) == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert torch.equal(y, y_ref)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.flare_mixer_fwd_static(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), y.data_ptr(),
                                            torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.current_stream().wait_stream(side)
    for i in range(3):
        print(f"static scratch graph replay {i}", flush=True)
        # another problem dirties the scratch between replays (eager work on the same scratch)
        _both(lib, dev, 1, 2 + i, 5000 + 100 * i, 128, 32, _lib.DT_BF16, seed=30 + i)
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_ref), i
