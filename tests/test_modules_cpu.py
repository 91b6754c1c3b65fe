"""Module contract tests that run without a GPU, modelled on the reference's
tests/pdebench/test_pdebench_model_contracts.py:23-132 (smoke, determinism, state_dict round trip,
shape matrix).  On the CPU only the diagnostic return_scores=True branch (plain torch) can run;
the mixer branch must refuse, loudly.  The same four contracts run on the HIP path in
tests/test_modules_gpu.py."""
import pytest
import torch

from flare_py_amd import FLAREModel, FLAREBlock, ResidualMLP
from flare_py_amd import lra_modules

KW = dict(in_dim=4, out_dim=3, channel_dim=32, num_blocks=2, num_heads=4, num_latents=16)

# state_dict keys in registration order, read off the reference's __init__ bodies
# (pdebench/models/flare.py:91-118,179-202,277-317)
def _expected_keys(num_blocks=2, layers_io=2, layers_kv=3, layers_ffn=3):
    def mlp(prefix, n):
        ks = [f"{prefix}.fc1.weight", f"{prefix}.fc1.bias"]
        for i in range(n):
            ks += [f"{prefix}.fcs.{i}.weight", f"{prefix}.fcs.{i}.bias"]
        return ks + [f"{prefix}.fc2.weight", f"{prefix}.fc2.bias"]
    keys = mlp("in_proj", layers_io)
    keys += ["out_proj.0.weight", "out_proj.0.bias"] + mlp("out_proj.1", layers_io)
    for b in range(num_blocks):
        p = f"blocks.{b}"
        keys += [f"{p}.norm1.weight", f"{p}.norm1.bias", f"{p}.norm2.weight", f"{p}.norm2.bias",
                 f"{p}.att.latent_q"]
        keys += mlp(f"{p}.att.k_proj", layers_kv) + mlp(f"{p}.att.v_proj", layers_kv)
        keys += [f"{p}.att.out_proj.weight", f"{p}.att.out_proj.bias"] + mlp(f"{p}.mlp", layers_ffn)
    return keys


def test_state_dict_keys_and_shapes():
    m = FLAREModel(**KW)
    assert list(m.state_dict().keys()) == _expected_keys()
    assert m.blocks[0].att.latent_q.shape == (32, 16)


def test_init_statistics():
    torch.manual_seed(0)
    m = FLAREModel(in_dim=4, out_dim=3, channel_dim=128, num_blocks=1, num_heads=8, num_latents=64)
    w = m.blocks[0].att.k_proj.fc1.weight
    assert abs(float(w.std()) - 0.02) < 2e-3 and float(m.blocks[0].att.k_proj.fc1.bias.abs().max()) == 0
    assert abs(float(m.blocks[0].att.latent_q.std()) - 0.1) < 1e-2
    assert float(m.blocks[0].norm1.weight.min()) == 1.0


def test_mixer_branch_refuses_cpu():
    m = FLAREModel(**KW).eval()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        m(torch.randn(1, 16, 4))


@pytest.mark.parametrize("B,N", [(1, 16), (2, 32), (2, 64)])
def test_scores_branch_smoke_determinism_shapes(B, N):
    torch.manual_seed(0)
    m = FLAREModel(**KW).eval()
    x = torch.randn(B, N, 4)
    with torch.no_grad():
        y1, s1 = m(x, return_scores=True)
        y2, _ = m(x, return_scores=True)
    assert y1.shape == (B, N, 3) and torch.isfinite(y1).all()
    assert torch.allclose(y1, y2, atol=1e-6)
    assert len(s1) == 2 and s1[0].shape == (B, 4, 16, N)


def test_state_dict_roundtrip():
    torch.manual_seed(0)
    a, b = FLAREModel(**KW).eval(), FLAREModel(**KW).eval()
    b.load_state_dict(a.state_dict(), strict=True)
    x = torch.randn(2, 32, 4)
    with torch.no_grad():
        assert torch.allclose(a(x, return_scores=True)[0], b(x, return_scores=True)[0], atol=1e-6)


def test_residual_mlp_variants():
    x = torch.randn(3, 8)
    lin = ResidualMLP(8, 8, 8, num_layers=-1, input_residual=True, output_residual=True)
    assert torch.allclose(lin(x), x + lin.fc(x))
    assert list(lin.state_dict().keys()) == ["fc.weight", "fc.bias"]
    m = ResidualMLP(8, 16, 4, num_layers=1)
    assert not m.input_residual and not m.output_residual and m(x).shape == (3, 4)
    h = m.act(m.fc1(x)); h = h + m.act(m.fcs[0](h))
    assert torch.allclose(m(x), m.fc2(h))


def test_lra_block_keys():
    blk = lra_modules.FLAREBlock(channel_dim=64, num_heads=4, num_latents=16, kv_proj_hidden_dim=64,
                                 ffn_hidden_dim=64)
    keys = list(blk.state_dict().keys())
    assert keys[:5] == ["norm1.weight", "norm1.bias", "norm2.weight", "norm2.bias", "att.latent_q"]
    assert "att.k_proj.fcs.2.weight" in keys and "att.out_proj.bias" in keys and "mlp.fc2.bias" in keys
    blk2 = FLAREBlock(channel_dim=64, num_heads=4, num_latents=16)
    assert set(keys) == set(blk2.state_dict().keys())


def test_triple_block_keys_and_feature_maps():
    # construction order of backends.py:1222-1241, 1316-1328 fixes the state_dict key order
    blk = lra_modules.TripleBlock(64, 4, kernel="hadamard", qk_dim_ratio=0.5)
    keys = list(blk.state_dict().keys())
    assert keys[:6] == ["norm1.weight", "norm1.bias", "norm2.weight", "norm2.bias", "att.out_proj.weight", "att.out_proj.bias"]
    assert keys[6:16] == [f"att.{p}_proj.fc.{w}" for p in ("q1", "q2", "k1", "k2", "v") for w in ("weight", "bias")]
    assert keys[16:20] == ["att.kernel.layer1.weight", "att.kernel.layer1.bias", "att.kernel.layer2.weight", "att.kernel.layer2.bias"]
    assert keys[20:] == ["att.norm.weight", "att.norm.bias", "mlp.fc1.weight", "mlp.fc1.bias", "mlp.fc2.weight", "mlp.fc2.bias"]
    assert blk.att.kernel.layer1.weight.shape == (8, 16)
    x = torch.linspace(-3, 3, 24).view(2, 3, 4)
    k = lra_modules.make_kernel
    assert torch.allclose(k("elu", 4)(x), torch.where(x > 0, x + 1, x.exp()))
    assert torch.allclose(k("relu_squared", 4)(x), x.clamp_min(0) ** 2)
    assert torch.allclose(k("silu", 4)(x), x * torch.sigmoid(x) + 0.5)
    assert torch.allclose(k("exp", 4)(100 * x).max(), torch.tensor(30.0).exp())
    assert torch.allclose(k("elu_norm", 4)(x), k("elu", 4)(x / x.norm(dim=-1, keepdim=True)))
    assert k("identity", 4)(x) is x
    hh = k("hedgehog", 4)
    y = hh(x)
    assert y.shape == (2, 3, 8) and torch.allclose(y.sum(-1), torch.ones(2, 3))
    assert torch.allclose(y, torch.cat([2 * x, -2 * x], -1).softmax(-1))     # identity-initialised
    assert k("swiglu", 4, 6)(x).shape == (2, 3, 6)
    with pytest.raises(NotImplementedError):
        k("nope", 4)


def test_reference_trainer_snapshot_loads(tmp_path):
    """A snapshot in the layout of mlutils/trainer.py:382-432 (DDP-prefixed names, EMA shadow, optimiser state)
    loads with the non-executing loader; names and values arrive unchanged."""
    from flare_py_amd.checkpoint import load_reference_checkpoint, read_snapshot
    torch.manual_seed(0)
    src = FLAREModel(in_dim=3, out_dim=2, channel_dim=32, num_blocks=2, num_heads=4, num_latents=8)
    opt = torch.optim.AdamW(src.parameters(), lr=1e-3)
    for p_ in src.parameters():      # (no forward on the CPU: the mixer has no CPU path)
        p_.grad = torch.ones_like(p_)
    opt.step()
    ema = {k: v.detach() * 0.5 for k, v in src.named_parameters()}
    snap = {"model_state": {"module." + k: v for k, v in src.state_dict().items()},
            "ema_shadow": {"module." + k: v for k, v in ema.items()},
            "step": 7, "epoch": 1, "opt_state": opt.state_dict(), "schedule_state": None,
            "train_loss_per_batch": [0.5, 0.25], "memory_utilization": None}
    path = str(tmp_path / "model.pt")
    torch.save(snap, path)
    dst = FLAREModel(in_dim=3, out_dim=2, channel_dim=32, num_blocks=2, num_heads=4, num_latents=8)
    out = load_reference_checkpoint(dst, path)
    assert out["step"] == 7 and read_snapshot(path)["epoch"] == 1
    for (ka, a), (kb, b) in zip(src.state_dict().items(), dst.state_dict().items()):
        assert ka == kb and torch.equal(a, b)
    load_reference_checkpoint(dst, path, use_ema=True)
    assert torch.equal(dst.blocks[0].att.latent_q, src.blocks[0].att.latent_q * 0.5)
    torch.save({"weights": 1}, path)
    with pytest.raises(ValueError):
        read_snapshot(path)


def test_rotary_embedding_module_against_oracle():
    """RotaryPositionalEmbeddings (lra/models/embeddings.py:103-147): values, strided head views, and buffers that
    stay out of the state_dict."""
    from flare_py_amd.lra_modules import RotaryPositionalEmbeddings
    from oracle import flare_oracle as O
    rope = RotaryPositionalEmbeddings(16, 64)
    assert list(rope.state_dict().keys()) == [] and rope.C.shape == (64, 16)
    x = torch.randn(2, 50, 4 * 16)
    k = x.view(2, 50, 4, 16).permute(0, 2, 1, 3)                     # the view the block hands over
    assert O.rel_l2(rope(k), O.rope_reference(k)) <= 1e-6
    assert O.rel_l2(rope(k.bfloat16()).float(), O.rope_reference(k.bfloat16().float())) <= 2e-2
    with pytest.raises(AssertionError):
        rope(torch.randn(1, 1, 65, 16))


def test_fused_structure_cache_follows_replaced_submodules():
    """The layer list the fused path keeps on a module is rebuilt when a submodule or the activation is replaced
    after the first look (a LoRA wrap, a re-initialisation by assignment)."""
    from torch import nn
    from flare_py_amd import fused
    from flare_py_amd.modules import ResidualMLP
    mlp = ResidualMLP(3, 32, 32, num_layers=2, act="gelu")
    first = fused._layers_of(mlp)
    assert first is fused._layers_of(mlp)                      # cached while nothing changes
    sub = fused._train_subchain(mlp)
    assert sub is not None and sub.first is mlp.fc1 and sub is fused._train_subchain(mlp)
    mlp.fcs[0] = nn.Linear(32, 32)
    again = fused._layers_of(mlp)
    assert again is not first and again[0][1] is mlp.fcs[0]
    assert fused._layers_of(fused._train_subchain(mlp))[0][0] is mlp.fcs[0]
    mlp.fc1 = nn.Linear(3, 32)
    assert fused._train_subchain(mlp).first is mlp.fc1
    mlp.act = nn.ReLU()                                        # an activation the kernels do not have
    assert fused._layers_of(mlp) is None and fused._train_subchain(mlp) is None


def test_linear_with_sliced_weight_gradient_equals_linear():
    """modules._LinearLongRows (the Linear layers of a token-wise model in training: dW as a batched product over slices of
    the rows) against autograd through F.linear, for row counts with and without a power-of-two factor, with and without bias."""
    from flare_py_amd import modules
    torch.manual_seed(3)
    for rows, cin, cout, bias in ((4096, 24, 16, True), (4100, 8, 8, False), (777, 5, 7, True), (2, 3 * 640, 4, True)):
        x = torch.randn(2, rows // 2, cin, dtype=torch.float64, requires_grad=True)
        w = torch.randn(cout, cin, dtype=torch.float64, requires_grad=True)
        b = torch.randn(cout, dtype=torch.float64, requires_grad=True) if bias else None
        g = torch.randn(2, rows // 2, cout, dtype=torch.float64)
        y = modules._LinearLongRows.apply(x, w, b)
        y.backward(g)
        got = [t.grad.clone() for t in (x, w) + ((b,) if bias else ())]
        for t in (x, w) + ((b,) if bias else ()):
            t.grad = None
        yr = torch.nn.functional.linear(x, w, b)
        yr.backward(g)
        assert torch.equal(y, yr)
        for a_, t in zip(got, (x, w) + ((b,) if bias else ())):
            assert torch.allclose(a_, t.grad, rtol=1e-12, atol=1e-12)
    # the dispatcher only takes it in training, on a GPU, outside autocast, over many rows
    lin = torch.nn.Linear(8, 8)
    assert modules._lin(lin, torch.randn(5000, 8)).grad_fn.name() != "_LinearLongRowsBackward"
