"""Compile the plain-C oracle into oracle/libflare_oracle.so (test infrastructure only)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libflare_oracle.so")


def build(verbose: bool = True) -> str:
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", LIB, os.path.join(HERE, "flare_oracle.c"), "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
