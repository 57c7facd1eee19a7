"""Builds ``libtenmo_hip.so`` (hipcc, gfx950 only) next to this file.

    python -m tenmo_amd.build            # compile

The GEMM kernel is instantiated per workgroup tile in its own translation unit (``csrc/gemm_tiles.hip``
compiled once per tile); the units are compiled in parallel and linked with the host side
(``csrc/tenmo_hip.hip``).  The library is built in-tree so that the copy of the tree that runs on the
GPU machine carries it.
"""
from __future__ import annotations

import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
# TENMO_HIP_BUILD_OUT: another output path (a variant library to compare against; load it with TENMO_HIP_LIBRARY)
LIB = os.environ.get("TENMO_HIP_BUILD_OUT") or os.path.join(HERE, "libtenmo_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed fp32 instructions stay off: the compiler must not form v_pk_{add,mul,fma}_f32
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-I", os.path.join(ROOT, "include"),
] + os.environ.get("TENMO_HIP_BUILD_FLAGS", "").split()  # extra compiler flags, e.g. -D overrides of kernel constants

# (rows, cols, part) units of the GEMM: part 0 = one workgroup per tile, 1 = the stream-K kernels
TILES = [(256, 128, 0), (256, 128, 1), (128, 128, 0), (128, 128, 1), (64, 64, 0), (64, 64, 1), (128, 64, 0), (128, 64, 1), (64, 128, 0)]
NOISE = "is not a recognized feature for this target"


def _run(cmd):
    res = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + err)
    return err


def _headers_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")] + [os.path.join(ROOT, "include", "tenmo_hip.h")]
    return max(os.path.getmtime(p) for p in paths)


def build(verbose: bool = False) -> str:
    """Compiles every unit and links the library.  With TENMO_HIP_BUILD_DIR set, the objects are kept there and a unit
    is recompiled only when its source, a header or the flags changed (for iterating on one kernel); otherwise
    everything is compiled afresh in a temporary directory."""
    jobs = min(len(TILES) + 3, max(1, int(os.environ.get("MAX_JOBS", os.cpu_count() or 1))))
    keep = os.environ.get("TENMO_HIP_BUILD_DIR")
    tmp_ctx = None if keep else tempfile.TemporaryDirectory(prefix="tenmo_hip_build_")
    tmp = keep or tmp_ctx.name
    os.makedirs(tmp, exist_ok=True)
    try:
        units = [([os.path.join(CSRC, "tenmo_hip.hip")], os.path.join(tmp, "tenmo_hip.o"))]
        for bm, bn, sk in TILES:
            units.append(([f"-DTENMO_TILE_BM={bm}", f"-DTENMO_TILE_BN={bn}", f"-DTENMO_TILE_STREAMK={sk}",
                           os.path.join(CSRC, "gemm_tiles.hip")], os.path.join(tmp, f"gemm_{bm}x{bn}_{sk}.o")))
        units.append(([os.path.join(CSRC, "gemm_smallk.hip")], os.path.join(tmp, "gemm_smallk.o")))
        units.append(([os.path.join(CSRC, "gemm_panel.hip")], os.path.join(tmp, "gemm_panel.o")))
        units.append(([os.path.join(CSRC, "gemm_resident.hip")], os.path.join(tmp, "gemm_resident.o")))
        stamp = " ".join(FLAGS)
        stamp_file = os.path.join(tmp, "flags.txt")
        same_flags = keep and os.path.exists(stamp_file) and open(stamp_file).read() == stamp
        newest_header = _headers_mtime()

        def stale(src, obj):
            if not (same_flags and os.path.exists(obj)):
                return True
            return os.path.getmtime(obj) < max(newest_header, os.path.getmtime(src[-1]))

        cmds = [[HIPCC] + FLAGS + ["-c"] + src + ["-o", obj] for src, obj in units if stale(src, obj)]
        if verbose:
            for c in cmds:
                print(" ".join(c), flush=True)
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            errs = list(pool.map(_run, cmds))
        if keep:
            with open(stamp_file, "w") as f:
                f.write(stamp)
        link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + [obj for _, obj in units] + ["-o", LIB]
        if verbose:
            print(" ".join(link), flush=True)
        errs.append(_run(link))
    finally:
        if tmp_ctx:
            tmp_ctx.cleanup()
    if verbose:
        for e in errs:
            if e.strip():
                print(e)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
