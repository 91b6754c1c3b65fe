"""Build libflare_hip.so (gfx950) in-tree with hipcc.  Usage: python flare.py_amd/build.py"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libflare_hip.so")
SOURCES = ["capi.hip", "mixer_generic.hip", "mixer_f32_mfma.hip", "mixer_mfma.hip", "mixer_mfma32.hip", "mixer_bwd_mfma.hip", "mixer_bwd_mfma32.hip", "mixer_bwd_f32_mfma.hip", "causal.hip", "causal_mfma.hip", "causal_decode.hip", "causal_linear.hip", "causal_linear_mfma.hip", "mlp_mfma.hip", "mlp_bwd_mfma.hip", "mlp_wgrad_mfma.hip", "triple.hip", "triple_f32_mfma.hip", "triple_mfma.hip"]
# packed-fp32 instruction selection is switched off for every device translation unit
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-math-errno", "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libflare_hip.so")
    return exe


def build(verbose: bool = True, jobs: int = 7) -> str:
    cc = hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [cc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
