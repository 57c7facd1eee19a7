"""tenmo_hip_vm_f32_noalloc — the allocation-free variant of tenmo_hip_vm_f32 — called through the C ABI and
checked against that entry point (same kernels: bit-identical) and against fp64, on two calls in a row, the
second with a smaller input, plus its refusal of a product whose partial sums exceed the static scratch."""
import ctypes as C
import os

import numpy as np
import pytest

from helpers import RTOL_FRO, rel_fro

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20  # TENMO_VM_NOALLOC_SCRATCH_BYTES of include/tenmo_hip.h
# set where the library under test is the CPU replay (tests/test_replay_parity.py): the largest products shrink, the cases stay
SMALL = os.environ.get("TENMO_TEST_SMALL") == "1"


@pytest.fixture(scope="module")
def lib():
    from tenmo_amd import _lib

    _lib.init(0)
    return _lib


def _vm_pair(lib, k, n, seed, accumulate=0, batch=None):
    """Runs vm through both entry points on the same seeded inputs; returns (with allocation, without, fp64)."""
    import torch

    L = lib.load()
    rng = np.random.default_rng(seed)
    bshape = () if batch is None else (batch,)
    W = rng.standard_normal(bshape + (k, n), dtype=np.float32)
    x = rng.standard_normal(bshape + (k,), dtype=np.float32)
    o0 = rng.standard_normal(bshape + (n,), dtype=np.float32)
    Wd, xd = torch.from_numpy(W).cuda(), torch.from_numpy(x).cuda()
    outs = []
    for fn in (L.tenmo_hip_vm_f32, L.tenmo_hip_vm_f32_noalloc):
        od = torch.from_numpy(o0).cuda()
        if batch is None:
            rc = fn(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, n, 1, od.data_ptr(), k, n, 0, None, None, None, accumulate, 1)
        else:
            rc = fn(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, n, 1, od.data_ptr(), k, n, 1, lib.i64([batch]), lib.i64([k]), lib.i64([k * n]), accumulate, 1)
        lib.check(rc)
        outs.append(od.cpu().numpy())
    ref = np.einsum("...k,...kn->...n", x.astype(np.float64), W.astype(np.float64))
    if accumulate:
        ref = ref + o0
    return outs[0], outs[1], ref


def test_no_alloc_vm_matches_vm_twice_in_a_row(lib):
    # K slices go through scratch in both calls; the second is smaller and lands in the first's leftovers
    big, wide = ((4096, 2048), (1024, 50257)) if SMALL else ((16384, 4096), (4096, 50257))
    for (k, n, acc, batch) in [big + (0, None), (3000, 1500, 0, None), wide + (1, None), (2048, 1027, 0, 3), (700, 260, 1, 2)]:
        with_alloc, without, ref = _vm_pair(lib, k, n, seed=k + n, accumulate=acc, batch=batch)
        assert np.array_equal(with_alloc, without), (k, n, acc, batch)
        assert rel_fro(without, ref) <= RTOL_FRO, (k, n, acc, batch)


def test_no_alloc_vm_column_major_matrix_needs_no_scratch(lib):
    import torch

    L = lib.load()
    rng = np.random.default_rng(5)
    k, n = 5000, 777
    Wt = rng.standard_normal((n, k), dtype=np.float32)  # the matrix as a transposed view of [n, k] storage
    x = rng.standard_normal(k, dtype=np.float32)
    Wd, xd = torch.from_numpy(Wt).cuda(), torch.from_numpy(x).cuda()
    od = torch.empty(n, device="cuda")
    lib.check(L.tenmo_hip_vm_f32_noalloc(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, 1, k, od.data_ptr(), k, n, 0, None, None, None, 0, 1))
    assert rel_fro(od.cpu().numpy(), Wt.astype(np.float64) @ x.astype(np.float64)) <= RTOL_FRO


def test_no_alloc_vm_refuses_what_exceeds_the_scratch(lib):
    import torch

    L = lib.load()
    k, n = 65536, 4096
    Wd = torch.zeros((k, n), device="cuda")
    xd = torch.zeros(k, device="cuda")
    od = torch.zeros(n, device="cuda")
    # 256 workgroups per CU wanted -> thousands of K slices of partial sums, far beyond 8 MiB
    lib.check(L.tenmo_hip_set_tuning(b"cols_wg_per_cu", 256))
    try:
        rc = L.tenmo_hip_vm_f32_noalloc(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, n, 1, od.data_ptr(), k, n, 0, None, None, None, 0, 1)
        assert rc == -5
        msg = L.tenmo_hip_last_error().decode()
        assert "static buffer" in msg and str(SCRATCH_BYTES) in msg
        # the allocating entry point takes the same product
        lib.check(L.tenmo_hip_vm_f32(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, n, 1, od.data_ptr(), k, n, 0, None, None, None, 0, 1))
    finally:
        lib.check(L.tenmo_hip_set_tuning(b"cols_wg_per_cu", 2))
    # and with the default knob the call goes through
    lib.check(L.tenmo_hip_vm_f32_noalloc(xd.data_ptr(), 0, 1, Wd.data_ptr(), 0, n, 1, od.data_ptr(), k, n, 0, None, None, None, 0, 1))
