"""The GPU parity tests, run on the CPU against the replay build of the library.

tests/test_gpu_parity.py, tests/test_zzz_gpu_first_run.py and tests/test_zz_no_alloc.py drive every entry point of the C ABI through the host mirror and
compare with the oracle and with float64.  Here the same test functions run in a child pytest process in which the
library is the CPU replay (tests/replay: the kernel sources compiled for the host, launches executed thread by thread)
and torch's "cuda" allocations are redirected to host memory (tests/replay/torch_on_host.py).  What this proves without
a GPU: the host side (dispatch, views, batching, workspace handling, error paths) and the kernels' arithmetic and
synchronisation as written in the source.  What it cannot: anything about the code the GPU compiler generates or timing.
The tests left out are the ones whose shapes would take minutes at CPU speed (TENMO_REPLAY_FULL=1 runs those too, about
a quarter of an hour; the kernels they cover are replayed on smaller shapes in tests/test_replay_addresses.py).
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "replay"))
import build as replay_build  # noqa: E402

pytestmark = pytest.mark.skipif(not replay_build.available(), reason="no host clang++ at " + replay_build.CXX)

# too large for any CPU replay (more than 2^31 elements), or about the GPU itself
LEFT_OUT = ["test_products_with_more_than_2_31_elements", "test_clock_probe"]
# minutes each at CPU speed
SLOW = ["test_stream_k", "test_kstream_kernel", "test_more_batches_than_a_grid_dimension", "test_conv2d_stream_k", "test_blocked_tile_order"]  # (test_kstream_kernel: every test whose name starts so)


def run_child(files, extra=()):
    lib = replay_build.build_library()
    small = {} if os.environ.get("TENMO_REPLAY_FULL") == "1" else {"TENMO_TEST_SMALL": "1"}  # a few tests shrink their largest cases at CPU speed
    env = dict(os.environ, **small, TENMO_HIP_LIBRARY=lib, REPLAY_STRICT="0", PYTHONPATH=os.path.join(ROOT, "tests", "replay") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    left_out = LEFT_OUT + ([] if os.environ.get("TENMO_REPLAY_FULL") == "1" else SLOW)
    deselect = " and ".join("not " + name for name in left_out)
    cmd = [sys.executable, "-m", "pytest", "-p", "torch_on_host", "-m", "gpu", "-x", "-q", "-k", deselect, "-p", "no:cacheprovider"] + list(extra) + files
    try:
        import xdist  # noqa: F401

        cmd += ["-n", str(min(8, os.cpu_count() or 1))]
    except ImportError:
        pass
    res = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=3000)
    tail = (res.stdout[-6000:] + "\n" + res.stderr[-3000:]).strip()
    assert res.returncode == 0, tail
    assert " passed" in res.stdout and "skipped" not in res.stdout.splitlines()[-1], tail
    return res.stdout


def test_gpu_parity_suite_on_the_replay():
    run_child([os.path.join("tests", "test_gpu_parity.py")])


def test_kernels_awaiting_their_first_gpu_run_on_the_replay():
    run_child([os.path.join("tests", "test_zzz_gpu_first_run.py")])


def test_allocation_free_entry_point_on_the_replay():
    run_child([os.path.join("tests", "test_zz_no_alloc.py")])


MLP_LAUNCH_COUNT_SCRIPT = r"""
import ctypes as C, json, sys
import numpy as np
lib = C.CDLL(sys.argv[1])
lib.replay_launch_count.restype = C.c_long
lib.tenmo_hip_mlp_create.restype = C.c_void_p
assert lib.tenmo_hip_init(0) == 0
dims = [784, 128, 32, 10]
rng = np.random.default_rng(3)
Ws = [(rng.standard_normal((dims[i], dims[i + 1])) * 0.05).astype(np.float32) for i in range(3)]
bs = [np.zeros(dims[i + 1], np.float32) for i in range(3)]
x = rng.standard_normal((64, 784)).astype(np.float32)
y = rng.integers(0, 10, 64).astype(np.int32)
loss = np.zeros(1, np.float32)
for arr in (x, y, loss):
    lib.replay_register(C.c_void_p(arr.ctypes.data), C.c_size_t(arr.nbytes))
fp = C.POINTER(C.c_float)
results = {}
for fused in (0, 1, 2, 3):
    W_ptrs = (fp * 3)(*[w.ctypes.data_as(fp) for w in Ws])
    b_ptrs = (fp * 3)(*[b.ctypes.data_as(fp) for b in bs])
    m = lib.tenmo_hip_mlp_create(3, (C.c_int64 * 4)(*dims), W_ptrs, b_ptrs, C.c_int64(64))
    assert m
    lib.tenmo_hip_set_tuning(b"mlp_fused_tail", fused)
    before = lib.replay_launch_count()
    rc = lib.tenmo_hip_mlp_step(C.c_void_p(m), x.ctypes.data_as(fp), y.ctypes.data_as(C.POINTER(C.c_int32)), C.c_int64(64), C.c_float(0.01),
                                loss.ctypes.data_as(fp), 1)
    assert rc == 0
    results[fused] = (lib.replay_launch_count() - before, float(loss[0]))
    lib.tenmo_hip_mlp_destroy(C.c_void_p(m))
print(json.dumps(results))
"""


def test_mlp_step_launch_count():
    """The MNIST-shaped training step (784 -> 128 -> 32 -> 10, batch 64) through the C ABI on the replay, counting kernel
    launches: op by op (nine); with the last two layers, the loss, their backward and their update fused into one launch
    (first-layer forward as K slices and their reduction, the fused tail, first-layer weight gradient, its update: five);
    with that gradient and update in one launch as well (four); and with the first-layer forward as one launch that cuts K
    inside its workgroups (three); same loss every way.  (In a child process: the replay
    ends the process when a kernel misbehaves.)"""
    import json

    res = subprocess.run([sys.executable, "-c", MLP_LAUNCH_COUNT_SCRIPT, replay_build.build_library()], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stdout + res.stderr
    results = {int(k): v for k, v in json.loads(res.stdout.strip().splitlines()[-1]).items()}
    assert results[3][0] <= 3 < results[2][0] <= 4 < results[1][0] <= 5 < results[0][0], results
    assert max(abs(results[0][1] - results[k][1]) for k in (1, 2, 3)) <= 1e-5, results
