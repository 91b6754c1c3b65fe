"""GPU parity of the fused token-wise MLP launches (flare_mlp_fwd) and of the fused FLAREBlock path.

Oracle: oracle.flare_oracle.residual_mlp (restatement of pdebench/models/flare.py:45-59, 204-215),
evaluated in fp64 on the SAME weights rounded to the compute type, so weight rounding is not charged
to the kernel.  Tolerance 2e-2 relative L2 (the 16-bit bar): the stream is rounded to 16 bits once
per layer as a matrix-core operand, accumulation and the residual path are fp32.
"""
import pytest
import torch
from torch import nn

import flare_py_amd as F
from flare_py_amd import fused
from oracle import flare_oracle as O

pytestmark = pytest.mark.gpu


def make_mlp(C, n, ir, orr, act, dev, seed=0):
    torch.manual_seed(seed)
    m = F.ResidualMLP(C, C, C, num_layers=n, act=act, input_residual=ir, output_residual=orr)
    for l in m.modules():
        if isinstance(l, nn.Linear):
            nn.init.normal_(l.weight, 0.0, C ** -0.5)
            nn.init.normal_(l.bias, 0.0, 0.2)
    return m.to(dev)


def oracle_of(m, x, cd, norm=None, res=None):
    layers, _, _, act = fused._layers_of(m)
    ws = [l.weight.detach().to(cd).double().cpu() for l in layers]
    bs = [l.bias.detach().double().cpu() for l in layers]
    ir = getattr(m, "input_residual", getattr(m, "residual", False))
    orr = getattr(m, "output_residual", getattr(m, "residual", False))
    kind = gamma = beta = None
    eps = 1e-5
    if isinstance(norm, nn.LayerNorm):
        kind, gamma, beta, eps = "layer", norm.weight.detach().cpu(), norm.bias.detach().cpu(), norm.eps
    elif isinstance(norm, nn.RMSNorm):
        kind, gamma, eps = "rms", norm.weight.detach().cpu(), norm.eps
    return O.residual_mlp(x.double().cpu(), ws, bs, "gelu" if act == 0 else "silu", ir, orr, kind, gamma, beta, eps,
                          None if res is None else res.double().cpu())


@pytest.mark.parametrize("C", [32, 64, 128])
@pytest.mark.parametrize("n,ir,orr,act", [(3, True, True, "gelu"), (0, False, True, "silu"), (1, True, False, "gelu"),
                                          (-1, True, True, "gelu"), (6, True, True, "silu")])
def test_mlp_stack_vs_oracle(dev, C, n, ir, orr, act):
    m = make_mlp(C, n, ir, orr, act, dev)
    x = torch.randn(3, 333, C, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        cd = fused.compute_dtype(x, m)
        assert cd == torch.bfloat16
        y = fused.fused_mlp(x, m, cd)
    assert y.dtype == torch.float32 and y.shape == x.shape
    assert O.rel_l2(y, oracle_of(m, x, cd)) <= 2e-2


@pytest.mark.parametrize("norm_kind", ["layer", "rms"])
@pytest.mark.parametrize("xdt,odt,cd", [(torch.float32, torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                        (torch.float32, torch.float32, torch.float16), (torch.float16, torch.float16, torch.float16)])
def test_norm_residual_dtypes_and_ragged_rows(dev, norm_kind, xdt, odt, cd):
    C = 128
    m = make_mlp(C, 3, True, True, "gelu", dev, seed=1)
    norm = (nn.LayerNorm(C) if norm_kind == "layer" else nn.RMSNorm(C, eps=1e-6)).to(dev)
    nn.init.normal_(norm.weight, 1.0, 0.3)
    if norm_kind == "layer":
        nn.init.normal_(norm.bias, 0.0, 0.3)
    for T in (1, 17, 129, 1000):
        x = (torch.randn(T, C, device=dev) * 2 + 0.5).to(xdt)
        with torch.no_grad():
            y = fused.fused_mlp(x, m, cd, norm=norm, res=x, out_dtype=odt)
        assert y.dtype == odt
        assert O.rel_l2(y, oracle_of(m, x, cd, norm, x)) <= 2e-2, T


def test_single_linear_with_residual_and_strided_rows(dev):
    C = 64
    lin = nn.Linear(C, C).to(dev)
    big = torch.randn(500, 2 * C, device=dev)
    x = big[:, :C]                                   # row stride 2C: consumed without a copy
    res = torch.randn(500, C, device=dev)
    with torch.no_grad():
        y = fused.fused_mlp(x, lin, torch.bfloat16, res=res)
    ref = res.double().cpu() + x.double().cpu() @ lin.weight.detach().bfloat16().double().cpu().T + lin.bias.detach().double().cpu()
    assert O.rel_l2(y, ref) <= 2e-2


def test_fast_path_conditions(dev):
    m = make_mlp(128, 3, True, True, "gelu", dev)
    x = torch.randn(4, 128, device=dev)
    assert fused.compute_dtype(x, m) is None                                  # grad enabled
    with torch.no_grad():
        assert fused.compute_dtype(x, m) is None                              # fp32 weights, no autocast
        assert fused.compute_dtype(x.cpu(), m) is None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            assert fused.compute_dtype(x, m) == torch.bfloat16
            assert fused.compute_dtype(torch.randn(4, 48, device=dev), make_mlp(48, 1, True, True, "gelu", dev)) is None
        assert fused.compute_dtype(x.half(), m.half()) == torch.float16
    from flare_py_amd import _lib
    d = _lib.FlareMlpDesc()
    d.T, d.C, d.L, d.w_dtype = 4, 48, 1, 1
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.load().flare_mlp_fwd(d, None, None, None, None, None, None, None, None), "flare_mlp_fwd")


@pytest.mark.parametrize("C,H,M", [(128, 8, 128), (64, 4, 64)])
@pytest.mark.parametrize("rms", [False, True])
def test_block_fused_path_vs_torch_layers(dev, C, H, M, rms, monkeypatch):
    torch.manual_seed(3)
    blk = F.FLAREBlock(channel_dim=C, num_heads=H, num_latents=M, rmsnorm=rms).to(dev).eval()
    for l in blk.modules():
        if isinstance(l, nn.Linear):
            nn.init.xavier_uniform_(l.weight)
            nn.init.normal_(l.bias, 0.0, 0.1)
    x = torch.randn(2, 3000, C, device=dev)
    calls = []
    real = fused._fused_mlp_fwd                           # the forward launch behind every entry (plain, autograd node, pair)
    monkeypatch.setattr(fused, "_fused_mlp_fwd", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    with torch.no_grad():
        ref, _ = blk(x)                                   # fp32 torch layers + fp32 HIP mixer
        assert not calls
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y, _ = blk(x)                                 # four fused launches + bf16 HIP mixer
    assert len(calls) == 4
    assert y.dtype == torch.float32
    assert O.rel_l2(y, ref) <= 2e-2
    # with gradients enabled the same four launches run behind autograd (tests/test_fused_train_gpu.py holds their
    # backward to the torch layers)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        yt, _ = blk(x[:, :256])
    assert len(calls) == 8 and yt.requires_grad


def test_narrow_heads_with_expanding_kv_projection(dev):
    """D = 8 heads (the reference's default geometry) with the two-layer expanding k / v projections
    (num_layers_*_proj = 0, ratio 2): no head-padded rows exist for that MLP form, so the layer must take the
    generic fused branch (the mixer pads the heads) instead of raising, and match its own fp32 layers."""
    torch.manual_seed(13)
    att = F.FLARE(64, 8, 32, num_layers_k_proj=0, k_proj_mlp_ratio=2.0, num_layers_v_proj=0, v_proj_mlp_ratio=2.0).to(dev).eval()
    blk = F.FLAREBlock(64, 8, 32, num_layers_k_proj=0, k_proj_mlp_ratio=2.0).to(dev).eval()
    x = torch.randn(2, 1500, 64, device=dev)
    for mod in (att, blk):
        with torch.no_grad():
            ref = mod(x)[0]
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y = mod(x)[0]
        assert O.rel_l2(y, ref) <= 2e-2
    # against the state-dict restatement of the layer (fp64, same weights)
    sd = {k: v.detach().double().cpu() for k, v in att.state_dict().items()}
    want = O.flare_layer(sd, "", x.double().cpu(), num_heads=8)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        got = att(x)[0]
    assert O.rel_l2(got, want) <= 2e-2


def test_model_fused_path_vs_fp32(dev):
    torch.manual_seed(4)
    model = F.FLAREModel(in_dim=3, out_dim=2, channel_dim=64, num_blocks=2, num_heads=4, num_latents=64).to(dev).eval()
    for l in model.modules():
        if isinstance(l, nn.Linear):
            nn.init.xavier_uniform_(l.weight)
    x = torch.randn(2, 2000, 3, device=dev)
    with torch.no_grad():
        ref = model(x)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = model(x)
    assert O.rel_l2(y, ref) <= 3e-2


@pytest.mark.parametrize("C,E", [(32, 2), (64, 4), (128, 4), (128, 2)])
@pytest.mark.parametrize("act,cd", [("gelu", torch.bfloat16), ("silu", torch.float16)])
def test_expanding_two_layer_mlp(dev, C, E, act, cd):
    """The feed-forward block with a hidden width of E*C (ResidualMLP(C, E*C, C, num_layers=0)): one launch, E pairs of
    C x C tiles, against the oracle on the same rounded weights; with norm and outer residual, ragged row counts."""
    torch.manual_seed(4)
    m = F.ResidualMLP(C, E * C, C, num_layers=0, act=act, input_residual=True, output_residual=True)
    for l in (m.fc1, m.fc2):
        nn.init.normal_(l.weight, 0.0, l.in_features ** -0.5)
        nn.init.normal_(l.bias, 0.0, 0.2)
    m = m.to(dev)
    assert not m.input_residual and not m.output_residual
    norm = nn.LayerNorm(C).to(dev)
    nn.init.normal_(norm.weight, 1.0, 0.3)
    nn.init.normal_(norm.bias, 0.0, 0.3)
    for T in (5, 300, 2049):
        x = torch.randn(T, C, device=dev) * 1.5
        with torch.no_grad(), torch.autocast("cuda", dtype=cd):
            assert fused.compute_dtype(x, m) == cd
            y = fused.fused_mlp(x, m, cd, norm=norm, res=x)
            y0 = fused.fused_mlp(x, m, cd)
        assert O.rel_l2(y, oracle_of(m, x, cd, norm, x)) <= 2e-2, T
        assert O.rel_l2(y0, oracle_of(m, x, cd)) <= 2e-2, T


def test_block_with_4x_feed_forward(dev):
    """BASELINE config 2's block shape (pre-norm, H=8 heads of D=16, M=128 latents, feed-forward with 4x expansion) at
    reduced length: the fused path against the block's own torch layers in fp32."""
    torch.manual_seed(5)
    blk = F.FLAREBlock(channel_dim=128, num_heads=8, num_latents=128, ffn_mlp_ratio=4.0, num_layers_ffn=0).to(dev).eval()
    for mod in blk.modules():
        if isinstance(mod, nn.Linear):
            nn.init.xavier_uniform_(mod.weight)
    x = torch.randn(2, 3000, 128, device=dev)
    with torch.no_grad():
        ref = blk(x)[0]
        with torch.autocast("cuda", dtype=torch.bfloat16):
            assert fused.compute_dtype(x, blk.mlp) == torch.bfloat16
            y = blk(x)[0]
    assert O.rel_l2(y, ref) <= 2e-2


def _narrow_mlp(i, h, o, n, ir, orr, act, dev, seed):
    torch.manual_seed(seed)
    m = F.ResidualMLP(i, h, o, num_layers=n, act=act, input_residual=ir, output_residual=orr)
    for l in m.modules():
        if isinstance(l, nn.Linear):
            nn.init.normal_(l.weight, 0.0, l.in_features ** -0.5)
            nn.init.normal_(l.bias, 0.0, 0.2)
    return m.to(dev)


def _narrow_oracle(m, x, cd, norm=None):
    """fp64 oracle on the weights as the kernel holds them: the narrow first layer in fp32, the tiles in cd."""
    layers, _, _, act = fused._layers_of(m)
    C = layers[0].out_features
    ws = [(l.weight.detach() if l.in_features <= 4 and C > 4 else l.weight.detach().to(cd)).double().cpu() for l in layers]
    bs = [l.bias.detach().double().cpu() for l in layers]
    kind = gamma = beta = None
    eps = 1e-5
    if isinstance(norm, nn.LayerNorm):
        kind, gamma, beta, eps = "layer", norm.weight.detach().cpu(), norm.bias.detach().cpu(), norm.eps
    return O.residual_mlp(x.double().cpu(), ws, bs, "gelu" if act == 0 else "silu", m.input_residual, m.output_residual,
                          kind, gamma, beta, eps)


@pytest.mark.parametrize("C", [32, 64, 128])
@pytest.mark.parametrize("in_dim,n,act,xdt", [(3, 2, "gelu", torch.float32), (1, 0, "silu", torch.float32),
                                              (4, 3, "gelu", torch.bfloat16), (2, 1, "silu", torch.float16)])
def test_lifting_first_layer_vs_oracle(dev, C, in_dim, n, act, xdt):
    """ResidualMLP(in_dim <= 4, C, C): the model's in_proj (pdebench/models/flare.py:137-140) in one launch."""
    m = _narrow_mlp(in_dim, C, C, n, False, True, act, dev, seed=C + in_dim)
    x = torch.randn(2, 777, in_dim, device=dev).to(xdt)
    cdt = torch.float16 if xdt == torch.float16 else torch.bfloat16
    with torch.no_grad(), torch.autocast("cuda", dtype=cdt):
        cd = fused.compute_dtype(x, m)
        assert cd == cdt
        y = fused.fused_mlp(x, m, cd, out_dtype=torch.float32)
    assert y.shape == (2, 777, C) and y.dtype == torch.float32
    assert O.rel_l2(y, _narrow_oracle(m, x, cd)) <= 2e-2


@pytest.mark.parametrize("C", [32, 64, 128])
@pytest.mark.parametrize("out_dim,n,ln,odt", [(1, 2, True, torch.float32), (4, 0, False, torch.bfloat16), (3, 1, True, torch.float16)])
def test_projecting_last_layer_vs_oracle(dev, C, out_dim, n, ln, odt):
    """norm + ResidualMLP(C, C, out_dim <= 4): the model's out_proj (pdebench/models/flare.py:141-147)."""
    m = _narrow_mlp(C, C, out_dim, n, True, False, "gelu", dev, seed=C + out_dim)
    norm = nn.LayerNorm(C).to(dev) if ln else None
    if ln:
        nn.init.normal_(norm.weight, 1.0, 0.2)
        nn.init.normal_(norm.bias, 0.0, 0.2)
    x = torch.randn(3, 501, C, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        cd = fused.compute_dtype(x, m)
        assert cd == torch.bfloat16
        y = fused.fused_mlp(x, m, cd, norm=norm, out_dtype=odt)
    assert y.shape == (3, 501, out_dim) and y.dtype == odt
    assert O.rel_l2(y, _narrow_oracle(m, x, cd, norm)) <= 2e-2


def test_narrow_both_ends_and_torch_fallbacks(dev):
    """in_dim and out_dim narrow at once; widths the kernel does not take stay with the torch layers."""
    m = _narrow_mlp(2, 64, 3, 2, False, False, "gelu", dev, seed=9)
    x = torch.randn(1000, 2, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        cd = fused.compute_dtype(x, m)
        assert cd == torch.bfloat16
        y = fused.fused_mlp(x, m, cd)
        assert fused.compute_dtype(torch.randn(10, 5, device=dev), _narrow_mlp(5, 64, 64, 1, False, True, "gelu", dev, 1)) is None
        assert fused.compute_dtype(torch.randn(10, 3, device=dev), _narrow_mlp(3, 48, 48, 1, False, True, "gelu", dev, 1)) is None
        assert fused.compute_dtype(torch.randn(10, 64, device=dev), _narrow_mlp(64, 64, 8, 1, True, False, "gelu", dev, 1)) is None
    assert y.shape == (1000, 3)
    assert O.rel_l2(y, _narrow_oracle(m, x, cd)) <= 2e-2


def test_model_launch_count_with_fused_ends(dev):
    """The whole model forward under autocast is in_proj + per block (k, v, mixer x3, out, ffn) + out_proj launches:
    no torch Linear runs (each would show as an addmm / mm kernel in the profiler)."""
    torch.manual_seed(5)
    model = F.FLAREModel(in_dim=3, out_dim=1, channel_dim=64, num_blocks=2, num_heads=4, num_latents=64).to(dev).eval()
    x = torch.randn(2, 1500, 3, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        model(x)
        with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as prof:
            y = model(x)
    names = {e.name for e in prof.events()}
    assert not any(n in names for n in ("aten::linear", "aten::addmm", "aten::mm", "aten::layer_norm")), names
    assert y.shape == (2, 1500, 1)


def test_cfg2_full_size_fused_vs_fp32_layers(dev):
    """BASELINE config 2 at its full size (B=4 clouds of 65,536 points, 2 coordinates + 1 field; lift MLP to 128;
    block with H=8, D=16, M=128 and a 4x GELU MLP; Xavier weights): the fused bf16 path against the same modules run
    as fp32 torch layers around the fp32 HIP mixer, and 64 sampled tokens of the lift against the fp64 oracle."""
    torch.manual_seed(0)
    lift = F.ResidualMLP(3, 128, 128, num_layers=2, input_residual=False, output_residual=True).to(dev).eval()
    blk = F.FLAREBlock(channel_dim=128, num_heads=8, num_latents=128, num_layers_ffn=0, ffn_mlp_ratio=4.0).to(dev).eval()
    for l in [*lift.modules(), *blk.modules()]:
        if isinstance(l, nn.Linear):
            nn.init.xavier_uniform_(l.weight)
            nn.init.zeros_(l.bias)
    pts = torch.cat([torch.rand(4, 65536, 2, device=dev), torch.randn(4, 65536, 1, device=dev)], dim=-1)
    with torch.no_grad():
        ref = blk(lift(pts))[0]
        with torch.autocast("cuda", dtype=torch.bfloat16):
            cd = fused.compute_dtype(pts, lift)
            assert cd == torch.bfloat16 and fused.compute_dtype(ref, blk.mlp) == torch.bfloat16
            h = fused.fused_mlp(pts, lift, cd)
            y = blk(h)[0]
    assert y.shape == (4, 65536, 128) and torch.isfinite(y).all()
    assert O.rel_l2(y, ref) <= 2e-2
    idx = torch.randint(0, 65536, (64,), device=dev)
    assert O.rel_l2(h[2, idx], _narrow_oracle(lift, pts[2, idx], cd)) <= 2e-2


@pytest.mark.parametrize("C,hd", [(64, 8), (32, 4), (128, 8), (32, 8)])
def test_head_padded_rows(dev, C, hd):
    """Rows whose heads of hd < 16 channels are padded to 16 columns (the layout the mixer takes for narrow heads):
    written by one launch (pad columns are zeros), read back by another, against the oracle on plain rows."""
    H = C // hd
    m = make_mlp(C, 2, True, True, "gelu", dev, seed=C + hd)
    norm = nn.LayerNorm(C).to(dev)
    x = torch.randn(2, 301, C, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        cd = fused.compute_dtype(x, m)
        yp = fused.fused_mlp(x, m, cd, norm=norm, out_dtype=cd, y_head=hd)
        y = fused.fused_mlp(x, m, cd, norm=norm, out_dtype=cd)
    assert yp.shape == (2, 301, H * 16)
    yp4 = yp.view(2, 301, H, 16)
    assert torch.equal(yp4[..., :hd].reshape(2, 301, C), y) and (yp4[..., hd:] == 0).all()
    assert O.rel_l2(y, oracle_of(m, x, cd, norm)) <= 2e-2
    # reading padded rows: a single Linear with a residual, fed the padded tensor
    lin = nn.Linear(C, C).to(dev)
    res = torch.randn(2, 301, C, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        out_p = fused.fused_mlp(yp, lin, cd, res=res, out_dtype=torch.float32, x_head=hd)
        out = fused.fused_mlp(y, lin, cd, res=res, out_dtype=torch.float32)
    assert torch.equal(out_p, out)
    with pytest.raises(ValueError):
        fused.fused_mlp(y, lin, cd, x_head=hd)                    # plain rows where padded ones are announced


def test_block_forward_replays_from_a_hip_graph(dev):
    """A serving loop captures the fused block forward (7 launches, no host round trips) once and replays it: every
    replay, with new input written into the static buffer and eager work in between, must equal the eager result."""
    torch.manual_seed(8)
    blk = F.FLAREBlock(channel_dim=64, num_heads=8, num_latents=64).to(dev).eval()        # head dim 8: padded-row path
    blk2 = F.FLAREBlock(channel_dim=128, num_heads=8, num_latents=128, num_layers_ffn=0, ffn_mlp_ratio=4.0).to(dev).eval()
    for b, C in ((blk, 64), (blk2, 128)):
        static_x = torch.randn(2, 4096, C, device=dev)
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                for _ in range(3):
                    b(static_x)                                  # warm-up: weight packing, kernel attributes
            torch.cuda.current_stream().wait_stream(s)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = b(static_x)[0]
            for i in range(3):
                x = torch.randn(2, 4096, C, device=dev) * (1.0 + i)
                eager = b(x)[0]
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, eager), i


def test_graphed_forward_helper(dev):
    """serving.GraphedForward: one capture per input shape, replays equal the eager forward, reset() recaptures."""
    torch.manual_seed(9)
    model = F.FLAREModel(in_dim=3, out_dim=2, channel_dim=64, num_blocks=2, num_heads=8, num_latents=64).to(dev).eval()
    fwd = F.GraphedForward(model, autocast_dtype=torch.bfloat16)
    for shape in ((1, 2000, 3), (2, 777, 3), (1, 2000, 3)):
        for i in range(2):
            x = torch.randn(*shape, device=dev) * (1 + i)
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                eager = model(x)
            assert torch.equal(fwd(x), eager)
    assert len(fwd._graphs) == 2
    with torch.no_grad():
        model.out_proj[1].fc2.bias.add_(1.0)
    fwd.reset()
    x = torch.randn(1, 2000, 3, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(fwd(x), model(x))
    # a parameter update without reset(): the next call notices and captures again
    with torch.no_grad():
        for p in model.parameters():
            p.mul_(1.01)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(fwd(x), model(x))
    # an eager forward in another compute dtype rebuilds the modules' operand caches; the graph keeps the ones it
    # was captured with alive, so its replay still equals the bf16 eager result
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        want = model(x).clone()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        model(x)
    junk = [torch.full((1 << 20,), float("nan"), device=dev) for _ in range(8)]     # recycle whatever was freed
    assert torch.equal(fwd(x), want)
    del junk
    with pytest.raises(ValueError):
        fwd(torch.randn(1, 10, 3))
    model.train()
    with pytest.raises(RuntimeError):
        fwd(torch.randn(1, 11, 3, device=dev))


@pytest.mark.parametrize("C", [32, 64, 128])
def test_many_token_instances_of_every_mode(dev, C):
    """Launches of up to 32768 tokens take kernel instances with one 16-token tile per wave; this test feeds the
    many-token instances (4 tiles per wave, 2 at C = 128) of every mode: chain with both norms, expanding MLP,
    narrow ends, head-padded rows."""
    T = 40000
    x = torch.randn(T, C, device=dev) * 1.5 + 0.3
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        for kind in ("layer", "rms", None):
            m = make_mlp(C, 2, True, True, "gelu" if kind != "rms" else "silu", dev, seed=C)
            norm = None if kind is None else (nn.LayerNorm(C) if kind == "layer" else nn.RMSNorm(C, eps=1e-6)).to(dev)
            if norm is not None:
                nn.init.normal_(norm.weight, 1.0, 0.3)
            y = fused.fused_mlp(x, m, torch.bfloat16, norm=norm, res=x)
            assert O.rel_l2(y, oracle_of(m, x, torch.bfloat16, norm, x)) <= 2e-2, kind
        # expanding two-layer MLP
        torch.manual_seed(C)
        e = F.ResidualMLP(C, 4 * C, C, num_layers=0, act="gelu", input_residual=True, output_residual=True).to(dev)
        assert fused.compute_dtype(x, e) == torch.bfloat16
        ye = fused.fused_mlp(x, e, torch.bfloat16)
        w1, w2 = e.fc1.weight.bfloat16().double().cpu(), e.fc2.weight.bfloat16().double().cpu()
        h = O.gelu_tanh(x.double().cpu() @ w1.T + e.fc1.bias.double().cpu())
        assert O.rel_l2(ye, h @ w2.T + e.fc2.bias.double().cpu()) <= 2e-2
        # narrow ends
        lift = _narrow_mlp(3, C, C, 1, False, True, "gelu", dev, seed=C)
        pts = torch.randn(T, 3, device=dev)
        assert O.rel_l2(fused.fused_mlp(pts, lift, torch.bfloat16), _narrow_oracle(lift, pts, torch.bfloat16)) <= 2e-2
        proj = _narrow_mlp(C, C, 2, 1, True, False, "gelu", dev, seed=C + 1)
        assert O.rel_l2(fused.fused_mlp(x, proj, torch.bfloat16), _narrow_oracle(proj, x, torch.bfloat16)) <= 2e-2
        # head-padded rows out and back in
        m = make_mlp(C, 1, True, True, "gelu", dev, seed=C + 2)
        yp = fused.fused_mlp(x, m, torch.bfloat16, out_dtype=torch.bfloat16, y_head=8)
        y = fused.fused_mlp(x, m, torch.bfloat16, out_dtype=torch.bfloat16)
        assert torch.equal(yp.view(T, C // 8, 16)[..., :8].reshape(T, C), y) and (yp.view(T, C // 8, 16)[..., 8:] == 0).all()
        lin = nn.Linear(C, C).to(dev)
        assert torch.equal(fused.fused_mlp(yp, lin, torch.bfloat16, x_head=8), fused.fused_mlp(y, lin, torch.bfloat16))


@pytest.mark.parametrize("cd", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("C,n", [(128, -1), (128, 0), (128, 1), (128, 2), (128, 3), (64, 0), (64, 4), (64, 6), (64, 7), (32, 2)])
def test_bias_vectors_in_registers_over_several_passes(dev, C, n, cd):
    """The many-token chain keeps the bias of every layer in registers as a ring that turns by one per layer and has
    to be back at layer 0 when the workgroup's next pass begins, whatever the number of layers: enough tokens for
    three to four passes per workgroup, every chain length the ring takes at this width and one beyond it (C = 64,
    9 layers: bias from memory), a norm in front (its gamma and beta) and a residual behind."""
    T = 200000
    torch.manual_seed(C + n)
    x = torch.randn(T, C, device=dev) * 1.2 - 0.2
    m = make_mlp(C, n, True, True, "gelu", dev, seed=7 * C + n) if n >= 0 else nn.Linear(C, C).to(dev)
    if n < 0:
        nn.init.normal_(m.bias, 0.0, 0.5)
    norm = nn.LayerNorm(C).to(dev)
    nn.init.normal_(norm.weight, 1.0, 0.3)
    nn.init.normal_(norm.bias, 0.0, 0.3)
    with torch.no_grad(), torch.autocast("cuda", dtype=cd):
        y = fused.fused_mlp(x, m, cd, norm=norm, res=x)
        y2 = fused.fused_mlp(x, m, cd, norm=norm, res=x)
    assert torch.equal(y, y2)
    ref = oracle_of(m, x, cd, norm, x)
    assert O.rel_l2(y, ref) <= 2e-2
    # the last pass of the last workgroup as well as the first: a ring out of step shows as a wrong bias, i.e. an error of
    # the order of the bias itself in every row of the later passes
    for lo in (0, T - 4096):
        assert O.rel_l2(y[lo:lo + 4096], ref[lo:lo + 4096]) <= 2e-2


@pytest.mark.parametrize("C,H", [(64, 8), (64, 4)])
def test_cached_operands_follow_parameter_updates(dev, C, H):
    """The fast path caches 16-bit copies of the weights and of latent_q on the modules; an in-place update of a
    parameter (an optimiser step, load_state_dict) must show in the next forward."""
    import copy
    torch.manual_seed(10)
    blk = F.FLAREBlock(channel_dim=C, num_heads=H, num_latents=64).to(dev).eval()
    x = torch.randn(1, 1000, C, device=dev)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        y0 = blk(x)[0]
        blk.att.latent_q.mul_(3.0)
        blk.mlp.fc1.weight.add_(0.05)
        blk.att.out_proj.bias.add_(0.5)
        y1 = blk(x)[0]
        fresh = copy.deepcopy(blk)
        for mod in fresh.modules():
            for name in ("_q_cache", "_flare_packed"):
                if hasattr(mod, name):
                    delattr(mod, name)
        y2 = fresh(x)[0]
    assert not torch.equal(y0, y1) and torch.equal(y1, y2)
