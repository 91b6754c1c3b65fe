"""GraphedTrainStep: a training step (forward, loss, backward) of the FLARE blocks recorded in a HIP graph and replayed.

A replay must give bit for bit the loss and gradients of the eager step on the same inputs and parameters: the
launches are the same ones, the graph only removes the host's share.  Every case replays several times with an
in-place parameter update and eager work of the same module in between, since a graph that went wrong would do so on
later replays (stale packed weights, a cleared buffer that is not cleared again).
"""
import pytest
import torch

import flare_py_amd as F
from flare_py_amd import lra_modules, modules

pytestmark = pytest.mark.gpu


def _mse(out, target):
    y = out[0] if isinstance(out, tuple) else out
    return (y.float() - target).square().mean()


def _eager(blk, extra, x, t, ac):
    params = [p for p in blk.parameters()]
    for p in params:
        p.grad = None
    with torch.autocast("cuda", dtype=ac):
        out = blk(x, *extra)
    loss = _mse(out, t)
    loss.backward()
    return loss.detach().clone(), [p.grad.clone() for p in params]


def _lra_block(dev, attn_drop=0.0):
    return lra_modules.FLAREBlock(channel_dim=64, num_heads=4, num_latents=32, num_layers_kv_proj=3, num_layers_ffn=3,
                                  kv_proj_hidden_dim=64, ffn_hidden_dim=64, attn_drop=attn_drop).to(dev).train()


@pytest.mark.parametrize("kind,ac", [("lra", torch.bfloat16), ("lra_masked", torch.bfloat16), ("pde", torch.float16)])
def test_replays_equal_eager_steps_across_parameter_updates(dev, kind, ac):
    torch.manual_seed(11)
    B, N, C = 3, 640, 64
    if kind == "pde":
        blk, extra = modules.FLAREBlock(channel_dim=C, num_heads=4, num_latents=32).to(dev).train(), ()
    else:
        blk = _lra_block(dev)
        mask = None
        if kind == "lra_masked":
            lens = torch.tensor([N, N // 3, 17])
            mask = (torch.arange(N)[None, :] < lens[:, None]).to(dev)
        extra = (mask,)
    params = [p for p in blk.parameters()]
    opt = torch.optim.SGD(params, lr=5e-2)
    step = F.GraphedTrainStep(blk, _mse, autocast_dtype=ac)
    for it in range(4):
        x, t = torch.randn(B, N, C, device=dev), torch.randn(B, N, C, device=dev)
        loss_e, grads_e = _eager(blk, extra, x, t, ac)
        loss_g = step(x, *extra, t).clone()
        assert torch.equal(loss_g, loss_e), (kind, it)
        for p, ge in zip(params, grads_e):
            assert p.grad is not None and torch.equal(p.grad, ge), (kind, it)
        assert float(loss_e) > 0 and all(bool(torch.isfinite(g).all()) for g in grads_e)
        opt.zero_grad(set_to_none=True)            # the next call hands the gradients back
        step(x, *extra, t)
        opt.step()                                  # in place: the next replay has to pack the new weights itself
    assert len(step._graphs) == 1


def test_new_shapes_and_replaced_parameters_are_captured_again(dev):
    torch.manual_seed(12)
    blk = _lra_block(dev)
    step = F.GraphedTrainStep(blk, _mse, autocast_dtype=torch.bfloat16)
    for N in (256, 512, 256):
        x, t = torch.randn(2, N, 64, device=dev), torch.randn(2, N, 64, device=dev)
        loss_e, grads_e = _eager(blk, (None,), x, t, torch.bfloat16)
        assert torch.equal(step(x, None, t), loss_e)
        assert all(torch.equal(p.grad, g) for p, g in zip(blk.parameters(), grads_e))
    assert len(step._graphs) == 2
    first = step._graphs[next(iter(step._graphs))][0]
    lin = next(m for m in blk.modules() if isinstance(m, torch.nn.Linear))
    lin.weight = torch.nn.Parameter(lin.weight.detach().clone() * 0.5)      # a new tensor at a new address
    x, t = torch.randn(2, 256, 64, device=dev), torch.randn(2, 256, 64, device=dev)
    loss_e, grads_e = _eager(blk, (None,), x, t, torch.bfloat16)
    assert torch.equal(step(x, None, t), loss_e)
    assert all(torch.equal(p.grad, g) for p, g in zip(blk.parameters(), grads_e))
    assert step._graphs[next(iter(step._graphs))][0] is not first
    step.reset()
    assert not step._graphs


def test_input_gradient_is_handed_to_the_callers_tensor(dev):
    torch.manual_seed(13)
    blk = _lra_block(dev)
    step = F.GraphedTrainStep(blk, _mse, autocast_dtype=torch.bfloat16)
    for _ in range(3):
        x = torch.randn(2, 384, 64, device=dev, requires_grad=True)
        t = torch.randn(2, 384, 64, device=dev)
        loss_e, _ = _eager(blk, (None,), x, t, torch.bfloat16)
        gx_e, x.grad = x.grad.clone(), None
        assert torch.equal(step(x, None, t), loss_e)
        assert torch.equal(x.grad, gx_e)


def test_refuses_what_a_replay_would_get_wrong(dev):
    x, t = torch.randn(2, 128, 64, device=dev), torch.randn(2, 128, 64, device=dev)
    with pytest.raises(RuntimeError, match="attention dropout"):
        F.GraphedTrainStep(_lra_block(dev, attn_drop=0.1), _mse, autocast_dtype=torch.bfloat16)(x, None, t)
    with pytest.raises(RuntimeError, match="train"):
        F.GraphedTrainStep(_lra_block(dev).eval(), _mse, autocast_dtype=torch.bfloat16)(x, None, t)
    with pytest.raises(ValueError, match="HIP device"):
        F.GraphedTrainStep(_lra_block(dev), _mse)(x.cpu(), None, t.cpu())
    with pytest.raises(ValueError, match="target"):
        F.GraphedTrainStep(_lra_block(dev), _mse)(x)
