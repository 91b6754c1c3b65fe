"""MI355X (gfx950) native FLARE attention engine.

Python host code on PyTorch-ROCm calling hand-written HIP kernels through the C-ABI of
libflare_hip.so (include/flare_hip.h).  The directory is named `flare.py_amd`; it is
importable as `flare_py_amd` (a symlink at the repository root).
"""
from . import _lib
from .functional import (
    CausalLinear,
    TripleAttentionFunction,
    causal_linear_attention,
    causal_fresh_state,
    causal_workspace,
    flare_causal_decode,
    flare_causal_decode_step,
    flare_causal_prefill,
    flare_gather,
    flare_multihead_mixer,
    flare_scatter,
    mixer_kernel_name,
    triple_attention,
)
from .modules import FLARE, FLAREBlock, FLAREModel, FinalLayer, ResidualMLP
from .serving import GraphedForward
from .train_graph import GraphedTrainStep

__all__ = [
    "CausalLinear", "causal_linear_attention", "FLARE", "FLAREBlock", "FLAREModel", "FinalLayer", "ResidualMLP", "TripleAttentionFunction",
    "causal_fresh_state", "causal_workspace", "flare_causal_decode", "flare_causal_decode_step", "flare_causal_prefill",
    "flare_gather", "flare_multihead_mixer", "flare_scatter", "mixer_kernel_name", "triple_attention", "GraphedForward", "GraphedTrainStep",
]
