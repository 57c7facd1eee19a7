"""Builds ``libtenmo_hip.so`` (hipcc, gfx950 only) next to this file.

    python -m tenmo_amd.build            # compile

The library is built in-tree so that the copy of the tree that runs on the GPU machine carries it.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "csrc", "tenmo_hip.hip")
LIB = os.path.join(HERE, "libtenmo_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 instructions stay off: the compiler must not form v_pk_{add,mul,fma}_f32
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-I", os.path.join(ROOT, "include"),
]


def build(verbose: bool = False) -> str:
    cmd = [HIPCC] + FLAGS + [SRC, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=os.path.join(HERE, "csrc"), capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
