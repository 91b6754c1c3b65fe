"""Loading the reference trainer's snapshots into the modules of this package.

mlutils/trainer.py:382-432 of the reference saves `torch.save(snapshot, path)` with
`snapshot['model_state']` = the model's state_dict (of `model.module` under DDP), optionally
`snapshot['ema_shadow']` = {parameter name: tensor}, plus optimiser, schedule and statistics entries
that are plain containers of tensors and numbers.  The modules here keep the reference's parameter
names, so the state loads as it is; this helper only opens the file without executing anything from
it (`weights_only=True`; the reference itself uses `weights_only=False`, trainer.py:443) and strips
the wrapper prefixes a training run may have left in the names.
"""
from __future__ import annotations

from typing import Dict, Iterable, Optional

import torch
from torch import nn

__all__ = ["read_snapshot", "load_reference_checkpoint"]

_WRAPPER_PREFIXES = ("module.", "_orig_mod.")


def read_snapshot(path: str) -> dict:
    """The snapshot dict of trainer.py:382-432, loaded on the CPU with the non-executing loader."""
    snap = torch.load(path, map_location="cpu", weights_only=True)
    if not isinstance(snap, dict) or "model_state" not in snap:
        raise ValueError(f"{path} is not a trainer snapshot: no 'model_state' entry")
    return snap


def _strip(name: str, prefixes: Iterable[str]) -> str:
    changed = True
    while changed:
        changed = False
        for p in prefixes:
            if p and name.startswith(p):
                name = name[len(p):]
                changed = True
    return name


def load_reference_checkpoint(model: nn.Module, path: str, use_ema: bool = False, strict: bool = True,
                              prefix: Optional[str] = None) -> dict:
    """Load `model_state` (or, with use_ema, the EMA shadow on top of it: trainer.py:451-455) into `model`.

    DDP's 'module.' and torch.compile's '_orig_mod.' prefixes are removed from the names, as is `prefix`
    when given (e.g. the attribute under which a wrapper holds the FLARE model).  Returns the snapshot
    so that the caller can read 'step', 'epoch' and the statistics."""
    snap = read_snapshot(path)
    prefixes = _WRAPPER_PREFIXES + ((prefix,) if prefix else ())
    state: Dict[str, torch.Tensor] = {_strip(k, prefixes): v for k, v in snap["model_state"].items()}
    if use_ema:
        shadow = snap.get("ema_shadow")
        if shadow is None:
            raise ValueError("EMA shadow not found in snapshot")
        for k, v in shadow.items():
            k = _strip(k, prefixes)
            if strict and k not in state:
                raise KeyError(f"EMA entry '{k}' has no counterpart in model_state")
            state[k] = v
    model.load_state_dict(state, strict=strict)
    return snap
