"""ctypes binding of libflare_hip.so (declared in include/flare_hip.h).

The library is loaded from this directory only.  There is no fallback: if it is missing the
loader raises, and every operator that needs it raises with it.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libflare_hip.so")

FLARE_OK, FLARE_EINVAL, FLARE_EUNSUPPORTED, FLARE_EWORKSPACE, FLARE_EHIP = 0, -1, -2, -3, -4
DT_F32, DT_BF16, DT_F16 = 0, 1, 2
FLAG_FORCE_GENERIC = 1
FLAG_MFMA16 = 2
FLAG_GRAD_LIKE_KV = 8
MLP_EXPAND = 1
MLP_BWD_ADD_DY = 1           # bits of flare_mlp_bwd's add_dy argument
MLP_BWD_ACCUMULATE = 2
ABI_VERSION = 2
STATIC_SCRATCH_BYTES = 64 << 20

I3 = C.c_int64 * 3


class FlareMixerDesc(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("M", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("scale", C.c_float), ("n_splits", C.c_int32), ("flags", C.c_int32),
        ("reserved", C.c_int32),
        ("q_stride", I3), ("k_stride", I3), ("v_stride", I3), ("y_stride", I3),
        ("dropout_p", C.c_float), ("reserved2", C.c_int32), ("dropout_seed", C.c_uint64),
    ]


class FlareCausalDesc(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("M", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("scale", C.c_float), ("chunk", C.c_int32), ("flags", C.c_int32),
        ("reserved", C.c_int32),
        ("q_stride", I3), ("k_stride", I3), ("v_stride", I3), ("y_stride", I3),
    ]


class FlareCausalLinearDesc(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("Dk", C.c_int32), ("Dv", C.c_int32),
        ("dtype", C.c_int32), ("n_segs", C.c_int32), ("flags", C.c_int32),
        ("q_stride", I3), ("k_stride", I3), ("v_stride", I3), ("y_stride", I3),
    ]


class FlareMlpDesc(C.Structure):
    _fields_ = [
        ("T", C.c_int64), ("C", C.c_int32), ("L", C.c_int32), ("w_dtype", C.c_int32),
        ("x_dtype", C.c_int32), ("res_dtype", C.c_int32), ("y_dtype", C.c_int32),
        ("norm", C.c_int32), ("eps", C.c_float), ("act", C.c_int32),
        ("act_mask", C.c_uint32), ("add_mask", C.c_uint32), ("flags", C.c_int32),
        ("x_stride", C.c_int64), ("res_stride", C.c_int64), ("y_stride", C.c_int64),
    ]


class FlareTripleDesc(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("Dq", C.c_int32), ("Dv", C.c_int32),
        ("dtype", C.c_int32), ("feature_map", C.c_int32), ("normalize", C.c_int32),
        ("n_splits", C.c_int32), ("flags", C.c_int32),
        ("q1_stride", I3), ("q2_stride", I3), ("k1_stride", I3), ("k2_stride", I3),
        ("v_stride", I3), ("o_stride", I3),
    ]


# every symbol include/flare_hip.h declares: name -> (restype, argtypes)
_P, _SZ = C.c_void_p, C.c_size_t
SYMBOLS = {
    "flare_abi_version": (C.c_int, []),
    "flare_last_error_string": (C.c_char_p, []),
    "flare_mixer_kernel_name": (C.c_char_p, [C.POINTER(FlareMixerDesc)]),
    "flare_mixer_workspace_bytes": (C.c_int, [C.POINTER(FlareMixerDesc), C.POINTER(_SZ)]),
    "flare_gather_fwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_scatter_fwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P]),
    "flare_scatter_fwd_lse": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, _P]),
    "flare_mixer_bwd_workspace_bytes": (C.c_int, [C.POINTER(FlareMixerDesc), C.POINTER(_SZ)]),
    "flare_mixer_bwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, _P, _P, C.POINTER(C.c_int64), _P, _P, _P, _P, _SZ, _P]),
    "flare_gather_bwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_scatter_bwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, C.POINTER(C.c_int64), _P, _P, _P, _P, _SZ, _P]),
    "flare_mixer_fwd": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_mixer_fwd_dropout": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, C.c_float, C.c_uint64, _P, _P, _P, _SZ, _P]),
    "flare_mixer_fwd_static": (C.c_int, [C.POINTER(FlareMixerDesc), _P, _P, _P, _P, _P, _P]),
    "flare_clock_probe": (C.c_int, [C.c_double, _P, _P]),
    "flare_causal_workspace_bytes": (C.c_int, [C.POINTER(FlareCausalDesc), C.POINTER(_SZ)]),
    "flare_causal_prefill_fwd": (C.c_int, [C.POINTER(FlareCausalDesc), _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_causal_decode_fwd": (C.c_int, [C.POINTER(FlareCausalDesc), _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_causal_prefill_fwd_lse": (C.c_int, [C.POINTER(FlareCausalDesc), _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_causal_decode_fwd_lse": (C.c_int, [C.POINTER(FlareCausalDesc), _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_causal_join": (C.c_int, [C.c_int32, C.c_int32, C.c_int64, C.c_int32, C.POINTER(_P), C.POINTER(_P), _P, _P]),
    "flare_causal_linear_workspace_bytes": (C.c_int, [C.POINTER(FlareCausalLinearDesc), C.POINTER(_SZ)]),
    "flare_causal_linear_fwd": (C.c_int, [C.POINTER(FlareCausalLinearDesc), _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_mlp_fwd": (C.c_int, [C.POINTER(FlareMlpDesc), _P, _P, _P, _P, _P, _P, _P, _P]),
    "flare_mlp_io_fwd": (C.c_int, [C.POINTER(FlareMlpDesc), C.c_int32, C.c_int32, _P, _P, C.c_int32,
                                   _P, _P, _P, _P, _P, _P, _P, _P]),
    "flare_mlp_bwd_partial_rows": (C.c_int, [C.POINTER(FlareMlpDesc), C.POINTER(C.c_int32)]),
    "flare_mlp_bwd": (C.c_int, [C.POINTER(FlareMlpDesc), _P, _P, _P, _P, _P, _P, _P, C.c_int32, _P, _P, _P, _P, _P, _P, _P, _P]),
    "flare_mlp_wgrad_partials": (C.c_int, [C.POINTER(FlareMlpDesc), C.POINTER(C.c_int32)]),
    "flare_mlp_wgrad": (C.c_int, [C.POINTER(FlareMlpDesc), _P, C.c_int64, _P, C.c_int64, _P, _P, _P, _P, _P]),
    "flare_mlp_expand_bwd": (C.c_int, [C.POINTER(FlareMlpDesc), _P, _P, _P, _P, _P, _P, _P, C.c_int32, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "flare_triple_workspace_bytes": (C.c_int, [C.POINTER(FlareTripleDesc), C.POINTER(_SZ)]),
    "flare_triple_state_fwd": (C.c_int, [C.POINTER(FlareTripleDesc), _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "flare_triple_out_fwd": (C.c_int, [C.POINTER(FlareTripleDesc), _P, _P, _P, _P, _P, _P]),
    "flare_triple_fwd": (C.c_int, [C.POINTER(FlareTripleDesc), _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
}

_lib = None
_lock = threading.Lock()


class FlareLibraryError(RuntimeError):
    pass


def load():
    """Load libflare_hip.so once; raise FlareLibraryError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise FlareLibraryError(
                f"{LIB_PATH} is missing: build it with `python flare.py_amd/build.py` "
                "(there is no CPU or PyTorch fallback for the FLARE kernels)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
        ver = lib.flare_abi_version()
        if ver != ABI_VERSION:
            raise FlareLibraryError(f"libflare_hip.so has ABI {ver}, the binding expects {ABI_VERSION}")
        _lib = lib
    return _lib


def last_error() -> str:
    s = load().flare_last_error_string()
    return s.decode() if s else ""


def check(status: int, what: str):
    """Map a status code to the exception class the reference's asserts would raise."""
    if status == FLARE_OK:
        return
    msg = f"{what}: {last_error()}"
    if status in (FLARE_EINVAL, FLARE_EWORKSPACE):
        raise ValueError(msg)
    if status == FLARE_EUNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
