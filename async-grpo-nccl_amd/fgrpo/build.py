"""Builds ``csrc/libfgrpo.so`` for gfx950 with hipcc (one translation unit)."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIB_PATH = os.environ.get("FGRPO_LIB", os.path.join(CSRC, "libfgrpo.so"))

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, os.path.join(CSRC, "fgrpo_api.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
