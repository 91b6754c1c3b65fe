"""ctypes wrapper of oracle/libflare_oracle.so — TEST INFRASTRUCTURE (see flare_oracle.c)."""
import ctypes as C
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libflare_oracle.so")
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            from . import build as _b
            _b.build(verbose=False)
        _lib = C.CDLL(LIB)
    return _lib


def _f32(t):
    return np.ascontiguousarray(t.detach().cpu().to(torch.float32).numpy())


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def mixer(q, k, v, scale=1.0, key_mask=None):
    """q [H,M,D], k,v [B,H,N,D] -> (y, z) float32 tensors."""
    qa, ka, va = _f32(q), _f32(k), _f32(v)
    B, H, N, D = ka.shape
    M = qa.shape[-2]
    y = np.empty((B, H, N, D), np.float32)
    z = np.empty((B, H, M, D), np.float32)
    mk = None if key_mask is None else np.ascontiguousarray(key_mask.cpu().numpy().astype(np.uint8))
    load().oracle_mixer(_p(qa), _p(ka), _p(va), None if mk is None else _p(mk), _p(y), _p(z),
                        B, H, N, M, D, C.c_float(scale))
    return torch.from_numpy(y), torch.from_numpy(z)


def causal(q, k, v, scale=1.0, state=None):
    """Token recurrence; returns (y float32, (mu, den, num) float64)."""
    qa, ka, va = _f32(q), _f32(k), _f32(v)
    B, H, N, D = ka.shape
    M = qa.shape[-2]
    if state is None:
        mu = np.full((B, H, M), -np.inf)
        den = np.zeros((B, H, M))
        num = np.zeros((B, H, M, D))
    else:
        mu, den, num = (np.ascontiguousarray(s.detach().cpu().to(torch.float64).numpy()).copy() for s in state)
    y = np.empty((B, H, N, D), np.float32)
    load().oracle_causal(_p(qa), _p(ka), _p(va), _p(y), _p(mu), _p(den), _p(num), B, H, N, M, D, C.c_float(scale))
    return torch.from_numpy(y), (torch.from_numpy(mu), torch.from_numpy(den), torch.from_numpy(num))


def triple(q1, q2, k1, k2, v, feature_map=False, normalize=False):
    a = [_f32(t) for t in (q1, q2, k1, k2, v)]
    B, H, N, Dq = a[0].shape
    Dv = a[4].shape[-1]
    state = np.empty((B, H, Dq, Dv, Dq), np.float32)
    out = np.empty((B, H, N, Dv), np.float32)
    load().oracle_triple(*[_p(x) for x in a], _p(state), _p(out), B, H, N, Dq, Dv, int(feature_map), int(normalize))
    return torch.from_numpy(state), torch.from_numpy(out)
