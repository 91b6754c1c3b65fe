"""Replay of a captured forward + backward for launch-bound training steps.

On short sequences and small meshes a training step of a FLARE block is a few dozen HIP launches whose kernels
take less time than the host needs to enqueue them (a sequence-benchmark block at B = 32, N = 1024 runs 0.6 ms of
kernels in a 1.2 ms step).  `GraphedTrainStep` records one step (forward, loss, backward) in a HIP graph per input
shape and replays it; there is no tracing compiler behind it and nothing is specialised beyond the shapes.

    step = GraphedTrainStep(model, loss_fn, autocast_dtype=torch.bfloat16)
    for x, target in loader:
        loss = step(x, target)          # first call with new shapes: warm-up + capture; later calls: copy in, replay
        optimizer.step()                # eager, reads p.grad

What the caller has to know:

* The gradients are the graph's own buffers: every call overwrites them (nothing accumulates over calls) and hands
  them to `p.grad` again, so `optimizer.zero_grad()` in either form between calls is harmless and not needed.  The
  returned loss is a static buffer too (clone it to keep it).  An input tensor with `requires_grad` set receives
  its gradient in `.grad` the same way.
* The 16-bit operand copies of the weights are packed inside the captured step from the parameters' own storage, so
  an optimizer that updates the parameters in place between calls is seen by the next replay.  Replacing a
  parameter tensor (`load_state_dict(assign=True)`, `.to()`, a new `nn.Parameter`) is detected by address and leads
  to a new capture.
* Attention dropout of the sequence-benchmark modules draws its seed on the host, where a replay would repeat it:
  modules with `attn_drop > 0` in training mode are refused.  torch's own dropout is capture-safe.
* Capture fails when an autograd graph of an earlier eager step on another stream is still alive (a kept loss tensor
  that was not detached holds the parameters' gradient accumulators on that stream): drop such references first.
* The module must not read values back to the host in its forward (no `.item()`, no data-dependent Python
  branches); the FLARE modules of this package do not.
"""
from __future__ import annotations

import contextlib

import torch

__all__ = ["GraphedTrainStep"]


class GraphedTrainStep:
    def __init__(self, module: torch.nn.Module, loss_fn, autocast_dtype=None, warmup: int = 3):
        self.module = module
        self.loss_fn = loss_fn
        self.autocast_dtype = autocast_dtype
        self.warmup = warmup
        self._graphs = {}

    def reset(self):
        """Drop every captured graph and its memory pool."""
        self._graphs.clear()

    def _context(self):
        if self.autocast_dtype is None:
            return contextlib.nullcontext()
        return torch.autocast("cuda", dtype=self.autocast_dtype)

    def _params(self):
        return [p for p in self.module.parameters() if p.requires_grad]

    def _check(self):
        if not self.module.training:
            raise RuntimeError("GraphedTrainStep captures training steps: call module.train() first")
        for m in self.module.modules():
            if float(getattr(m, "attn_drop_p", 0.0) or 0.0) > 0.0:
                raise RuntimeError("GraphedTrainStep: attention dropout draws its seed on the host, a replay would repeat "
                                   "the same keep mask every step; train this module eagerly or with attn_drop = 0")

    def _one_step(self, static_inputs, params):
        for p in params + [s for s in static_inputs if isinstance(s, torch.Tensor) and s.requires_grad]:
            p.grad = None
        with self._context():
            out = self.module(*static_inputs[:-1])
            loss = self.loss_fn(out, static_inputs[-1])
        loss.backward()
        return loss

    def _drop_operand_caches(self):
        """Forget the packed weights the warm-up left on the modules, so that the captured step packs them itself."""
        for m in self.module.modules():
            for name in ("_flare_packed", "_flare_packed_train", "_q_cache"):
                m.__dict__.pop(name, None)

    def _capture(self, inputs):
        self._check()
        params = self._params()
        dev = inputs[0].device
        static_inputs = [t.detach().clone().requires_grad_(t.requires_grad) if isinstance(t, torch.Tensor) else t for t in inputs]
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(self.warmup):          # kernel attributes, per-module structure caches, allocator warm-up
                self._one_step(static_inputs, params)
        torch.cuda.current_stream(dev).wait_stream(side)
        self._drop_operand_caches()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            loss = self._one_step(static_inputs, params).detach()   # no reference to the recorded autograd graph
        grads = [p.grad for p in params]
        self._drop_operand_caches()               # those of the capture live in the graph's pool: eager calls repack
        return graph, static_inputs, loss, grads, tuple(p.data_ptr() for p in params)

    def __call__(self, *inputs):
        """inputs = the module's positional arguments followed by the target handed to loss_fn(output, target)."""
        if len(inputs) < 2:
            raise ValueError("GraphedTrainStep: call with the module's inputs followed by the target")
        tensors = [t for t in inputs if isinstance(t, torch.Tensor)]
        if not tensors or any(t.device.type != "cuda" for t in tensors):
            raise ValueError("GraphedTrainStep replays HIP graphs: the tensors must live on a HIP device")
        key = tuple((tuple(t.shape), t.dtype, t.device.index) if isinstance(t, torch.Tensor) else ("const", t) for t in inputs)
        entry = self._graphs.get(key)
        params = self._params()
        if entry is not None and entry[4] != tuple(p.data_ptr() for p in params):
            entry = None                          # a parameter tensor was replaced: the graph reads the old one
        if entry is None:
            entry = self._graphs[key] = self._capture(inputs)
        else:
            self._check()
        graph, static_inputs, loss, grads, _ = entry
        with torch.no_grad():
            for s, t in zip(static_inputs, inputs):
                if isinstance(s, torch.Tensor):
                    s.copy_(t)
        graph.replay()
        for p, g in zip(params, grads):
            p.grad = g
        for s, t in zip(static_inputs, inputs):
            if isinstance(s, torch.Tensor) and s.requires_grad:
                t.grad = s.grad                   # an input that asked for its gradient gets the graph's buffer
        return loss
