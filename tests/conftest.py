import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU machine)")


def _gpu_unavailable_reason():
    """None when the GPU tests can run here: a gfx950 device and the built HIP library."""
    lib = os.path.join(ROOT, "tenmo_amd", "libtenmo_hip.so")
    if not os.path.exists(os.environ.get("TENMO_HIP_LIBRARY") or lib):
        return "libtenmo_hip.so is not built (python -m tenmo_amd.build)"
    try:
        import torch
    except ImportError:
        return "torch is not importable"
    # (counting devices does not initialise the GPU in this process; torch.cuda.is_available() would, and a process that
    # has initialised the GPU should not start other programs any more — see early_c_driver_run below)
    if torch.cuda.device_count() < 1:
        return "no GPU visible to this process"
    return None


# The plain-C caller of the header (tests/c_abi_driver.c) is a program of its own.  It is started here, during collection,
# before anything in this process has touched the GPU, and tests/test_y_c_abi_driver.py asserts on what it printed: on the GPU
# machines a process that has initialised the GPU must not exec other programs, and whether a forked child of such a process
# may is not something a test should find out.
C_DRIVER_RESULT = {}


def early_c_driver_run():
    import subprocess

    exe = os.path.join(ROOT, "tests", "_build", "c_abi_driver")
    if not os.path.exists(exe):
        C_DRIVER_RESULT["error"] = exe + " is not built (python __graft_entry__.py)"
        return
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.path.join(ROOT, "tenmo_amd") + os.pathsep + env.get("LD_LIBRARY_PATH", "")  # the library of THIS tree first
    try:
        run = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
        C_DRIVER_RESULT.update(returncode=run.returncode, stdout=run.stdout, stderr=run.stderr)
    except (OSError, subprocess.SubprocessError) as e:
        C_DRIVER_RESULT["error"] = "%s: %s" % (type(e).__name__, e)


def pytest_collection_modifyitems(config, items):
    gpu_items = [it for it in items if it.get_closest_marker("gpu")]
    if not gpu_items:
        return
    # The GPU tests are parity evidence for the HIP library of this tree and nothing else: another library put in its
    # place through TENMO_HIP_LIBRARY is accepted only together with the host stand-in for torch's device (the CPU
    # replay of the kernels, tests/replay), which says what it is.
    override = os.environ.get("TENMO_HIP_LIBRARY")
    in_tree = os.path.join(ROOT, "tenmo_amd", "libtenmo_hip.so")
    if override and os.path.realpath(override) != os.path.realpath(in_tree) and not config.pluginmanager.has_plugin("torch_on_host"):
        raise pytest.UsageError("TENMO_HIP_LIBRARY=%s: the gpu tests run on %s only" % (override, in_tree))
    reason = _gpu_unavailable_reason()
    if reason:
        skip = pytest.mark.skip(reason="gpu test: " + reason)
        for it in gpu_items:
            it.add_marker(skip)
    elif any(it.name == "test_driver_runs_on_the_gpu" for it in gpu_items) and not config.pluginmanager.has_plugin("torch_on_host"):
        early_c_driver_run()


@pytest.fixture(scope="session")
def golden():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O

    O.build()
    return O
