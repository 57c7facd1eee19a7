"""tests/c_abi_driver.c — a plain C11 program that binds the library the way a maintainer of the reference would:
include/tenmo_hip.h, nothing else.

Without a GPU: the header is valid C11 under -Wall -Wextra -Werror and every function it declares is referenced; the
program is then linked against the CPU replay of the library (tests/replay) and run, so the calls themselves — the
argument order of every kernel-level and view-level entry it uses, the CBLAS prototype, the error path — are executed,
not only compiled.  With a GPU (marked gpu): the same program linked against libtenmo_hip.so and the HIP runtime.
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi_driver.c")
OUT = os.path.join(ROOT, "tests", "_build")
CFLAGS = ["-std=c11", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include")]
sys.path.insert(0, os.path.join(ROOT, "tests", "replay"))
import build as replay_build  # noqa: E402


def build_gpu_driver() -> str:
    """The driver linked against the in-tree libtenmo_hip.so and the HIP runtime (links without a GPU)."""
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "c_abi_driver")
    lib_dir = os.path.join(ROOT, "tenmo_amd")
    # the run path is relative to the program ($ORIGIN = tests/_build), so the prebuilt program finds the library
    # wherever the tree is copied to
    subprocess.run(["gcc"] + CFLAGS + [SRC, "-L", lib_dir, "-ltenmo_hip", "-L", "/opt/rocm/lib", "-lamdhip64", "-lm",
                                       "-Wl,-rpath,$ORIGIN/../../tenmo_amd", "-Wl,-rpath,/opt/rocm/lib", "-o", exe],
                   check=True, capture_output=True, text=True)
    return exe


def test_prebuilt_driver_finds_the_library_in_a_relocated_tree(tmp_path):
    """The program is built in one place and run in a copy of the tree somewhere else: its run path must not name
    the place it was built in."""
    import shutil

    lib = os.path.join(ROOT, "tenmo_amd", "libtenmo_hip.so")
    if not os.path.exists(lib):
        pytest.skip("libtenmo_hip.so is not built")
    exe = build_gpu_driver()
    dyn = subprocess.run(["readelf", "-d", exe], capture_output=True, text=True).stdout
    assert ROOT not in dyn and "$ORIGIN/../../tenmo_amd" in dyn, dyn
    tree = tmp_path / "elsewhere" / "repo"
    os.makedirs(tree / "tests" / "_build")
    os.makedirs(tree / "tenmo_amd")
    shutil.copy(exe, tree / "tests" / "_build" / "c_abi_driver")
    shutil.copy(lib, tree / "tenmo_amd" / "libtenmo_hip.so")
    env = {k: v for k, v in os.environ.items() if k != "LD_LIBRARY_PATH"}
    out = subprocess.run(["ldd", str(tree / "tests" / "_build" / "c_abi_driver")], capture_output=True, text=True, env=env).stdout
    line = [ln for ln in out.splitlines() if "libtenmo_hip.so" in ln]
    assert line and str(tree / "tenmo_amd" / "libtenmo_hip.so") in os.path.normpath(line[0].split("=>")[1].split("(")[0].strip()), out


def test_header_is_c11_and_every_symbol_is_referenced(tmp_path):
    res = subprocess.run(["gcc"] + CFLAGS + ["-c", SRC, "-o", str(tmp_path / "driver.o")], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    # one table entry per prototype of the header
    import re

    header = open(os.path.join(ROOT, "include", "tenmo_hip.h")).read()
    declared = set(re.findall(r"\b(tenmo_hip_\w+|cblas_sgemm)\s*\(", header))
    source = open(SRC).read()
    table = source[source.index("every_symbol[] = {"):source.index("};", source.index("every_symbol[] = {"))]
    assert declared == set(re.findall(r"\(any_fn\)(\w+)", table))


@pytest.mark.skipif(not replay_build.available(), reason="no host clang++ at " + replay_build.CXX)
def test_driver_runs_against_the_cpu_replay(tmp_path):
    lib = replay_build.build_library()
    exe = str(tmp_path / "driver_replay")
    res = subprocess.run(["gcc"] + CFLAGS + [SRC, lib, "-lm", "-Wl,-rpath," + os.path.dirname(lib), "-o", exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and "c_abi_driver: ok" in run.stdout, run.stdout + run.stderr


@pytest.mark.gpu
def test_driver_runs_on_the_gpu():
    """The program was run by tests/conftest.py during collection, before this process touched the GPU (a process that has
    initialised the GPU does not start other programs on the GPU machines); here its outcome is checked."""
    import conftest

    res = conftest.C_DRIVER_RESULT
    assert "error" not in res, res
    assert res, "the C driver was not started (tests/conftest.py: early_c_driver_run)"
    assert res["returncode"] == 0 and "c_abi_driver: ok" in res["stdout"], res["stdout"] + res["stderr"]
