"""Builds the CPU replay of the library (see hip/hip_runtime.h in this directory) with the host clang++ of the ROCm
installation: ``libtenmo_hip_replay.so`` (the C ABI of include/tenmo_hip.h over host memory, for ctypes) and
``replay_gemm_asan`` (replay_gemm_main.cpp with AddressSanitizer).  Objects and outputs live in ``_build/`` beside this
file and are rebuilt when a source, a header or the flags are newer.  Test infrastructure: nothing in the package uses it.

    python tests/replay/build.py            # both targets
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "tenmo_amd", "csrc")
OUT = os.path.join(HERE, "_build")
CXX = os.environ.get("REPLAY_CXX", "/opt/rocm/llvm/bin/clang++")

COMMON = ["-x", "c++", "-std=c++17", "-O1", "-fPIC", "-I", HERE, "-I", os.path.join(ROOT, "include"),
          "-Wno-unused-result", "-Wno-unknown-attributes", "-Wno-psabi"]
ASAN = ["-fsanitize=address", "-fno-omit-frame-pointer", "-gline-tables-only"]
TILES = [(256, 128, 0), (256, 128, 1), (128, 128, 0), (128, 128, 1), (64, 64, 0), (64, 64, 1), (128, 64, 0), (128, 64, 1), (64, 128, 0)]


def available() -> bool:
    return os.path.exists(CXX)


def _newest_dependency() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(ROOT, "include", "tenmo_hip.h")]
    for d, _, files in os.walk(HERE):
        if os.path.basename(d) == "_build":
            continue
        paths += [os.path.join(d, f) for f in files if f.endswith((".h", ".hpp", ".cpp", ".py"))]
    return max(os.path.getmtime(p) for p in paths)


def _units(extra_sources):
    units = [(["-c", os.path.join(HERE, "replay_runtime.cpp")], "runtime.o"),
             (["-c", os.path.join(CSRC, "tenmo_hip.hip")], "host.o"),
             (["-c", os.path.join(CSRC, "gemm_smallk.hip")], "smallk.o"),
             (["-c", os.path.join(CSRC, "gemm_panel.hip")], "panel.o"),
             (["-c", os.path.join(CSRC, "gemm_resident.hip")], "resident.o")]
    for bm, bn, sk in TILES:
        units.append(([f"-DTENMO_TILE_BM={bm}", f"-DTENMO_TILE_BN={bn}", f"-DTENMO_TILE_STREAMK={sk}", "-c", os.path.join(CSRC, "gemm_tiles.hip")],
                      f"tile_{bm}x{bn}_{sk}.o"))
    for src in extra_sources:
        units.append((["-c", os.path.join(HERE, src)], os.path.splitext(src)[0] + ".o"))
    return units


def _build(kind: str, flags, extra_sources, link_flags, target: str) -> str:
    out_dir = os.path.join(OUT, kind)
    os.makedirs(out_dir, exist_ok=True)
    target_path = os.path.join(OUT, target)
    newest = _newest_dependency()
    if os.path.exists(target_path) and os.path.getmtime(target_path) >= newest:
        return target_path
    units = _units(extra_sources)

    def compile_one(unit):
        args, obj = unit
        obj_path = os.path.join(out_dir, obj)
        if os.path.exists(obj_path) and os.path.getmtime(obj_path) >= newest:
            return
        res = subprocess.run([CXX] + COMMON + flags + args + ["-o", obj_path], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("replay build failed: " + " ".join(args) + "\n" + res.stderr[-4000:])

    jobs = max(1, min(len(units), int(os.environ.get("MAX_JOBS", os.cpu_count() or 1))))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, units))
    res = subprocess.run([CXX] + flags + link_flags + [os.path.join(out_dir, obj) for _, obj in units] + ["-o", target_path, "-lpthread"],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("replay link failed:\n" + res.stderr[-4000:])
    return target_path


def build_library() -> str:
    """The C ABI over host memory, for ctypes."""
    return _build("plain", [], [], ["-shared", "-fPIC"], "libtenmo_hip_replay.so")


def build_gemm_asan() -> str:
    """replay_gemm_main.cpp and the whole library under AddressSanitizer."""
    return _build("asan", ASAN, ["replay_gemm_main.cpp"], [], "replay_gemm_asan")


def build_gemm_plain() -> str:
    """replay_gemm_main.cpp without a sanitizer: the producer of launch dumps (REPLAY_DUMP_DIR) for tests/isa/."""
    return _build("plain", [], ["replay_gemm_main.cpp"], ["-ldl"], "replay_gemm_plain")


def build_selftest() -> str:
    """replay_selftest.cpp (deliberately wrong toy kernels) under AddressSanitizer."""
    os.makedirs(OUT, exist_ok=True)
    target = os.path.join(OUT, "replay_selftest_asan")
    if os.path.exists(target) and os.path.getmtime(target) >= _newest_dependency():
        return target
    cmd = [CXX] + COMMON + ASAN + [os.path.join(HERE, "replay_selftest.cpp"), os.path.join(HERE, "replay_runtime.cpp"), "-o", target, "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("replay self-test build failed:\n" + res.stderr[-4000:])
    return target


if __name__ == "__main__":
    print(build_selftest())
    print(build_library())
    print(build_gemm_asan())
