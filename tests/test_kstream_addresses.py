"""CPU replay of whole launches of the persistent K-stream GEMM kernel (tenmo_amd/csrc/gemm_panel.hip).

tests/kstream_emulator.cpp walks every workgroup, wavefront and lane of a launch through the kernel's own index
arithmetic and control-flow templates (tenmo_amd/csrc/gemm_index.hpp) and checks that every global load lies inside
its operand's view, every LDS write inside the ring, that the loading and the multiplying wavefronts meet the same
number of barriers, that the ring hand-over is safe under any interleaving the barriers allow, that every MFMA operand
register holds the element the product needs, and that every element of C is stored exactly once.  No GPU involved:
this is the check that runs before such a kernel is ever launched on a shape.
"""
import ctypes as C
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MAX_BATCH_RANK = 6


class BatchDesc(C.Structure):
    _fields_ = [("rank", C.c_int32), ("shape", C.c_int64 * MAX_BATCH_RANK), ("a_str", C.c_int64 * MAX_BATCH_RANK), ("b_str", C.c_int64 * MAX_BATCH_RANK)]


class EmuProblem(C.Structure):
    _fields_ = [("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64), ("a_mn_major", C.c_int32), ("b_mn_major", C.c_int32),
                ("a_rs", C.c_int64), ("a_cs", C.c_int64), ("b_rs", C.c_int64), ("b_cs", C.c_int64), ("batch", BatchDesc),
                ("batch_count", C.c_int64), ("bm", C.c_int32), ("bn", C.c_int32), ("np", C.c_int32),
                ("cus", C.c_uint32), ("wgs_per_cu", C.c_uint32), ("group_by_xcd", C.c_int32)]


class EmuReport(C.Structure):
    _fields_ = [("loads", C.c_int64), ("lds_reads", C.c_int64), ("stores", C.c_int64), ("steps", C.c_int64), ("workgroups", C.c_int64),
                ("message", C.c_char * 512)]


@pytest.fixture(scope="module")
def emu(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("kstream") / "libkstream_emu.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", out, os.path.join(ROOT, "tests", "kstream_emulator.cpp")], check=True)
    lib = C.CDLL(out)
    lib.emulate_kstream.restype = C.c_int
    lib.emulate_kstream.argtypes = [C.POINTER(EmuProblem), C.POINTER(EmuReport)]
    return lib


def problem(M, N, K, a_layout, b_layout, batch=(), b_shared=False, a_pad=0, b_pad=0, tile=(128, 128), np_=5, cus=256, wpc=2, group=True):
    """a_layout / b_layout: 'k' (unit stride along the reduction: row-major A, transposed-view B) or 'mn'."""
    p = EmuProblem()
    p.M, p.N, p.K = M, N, K
    p.a_mn_major, p.b_mn_major = int(a_layout == "mn"), int(b_layout == "mn")
    if a_layout == "k":
        p.a_rs, p.a_cs, a_mat = K + a_pad, 1, M * (K + a_pad)
    else:
        p.a_rs, p.a_cs, a_mat = 1, M + a_pad, K * (M + a_pad)
    if b_layout == "k":   # B(k, n) = storage[n][k]
        p.b_rs, p.b_cs, b_mat = 1, K + b_pad, N * (K + b_pad)
    else:
        p.b_rs, p.b_cs, b_mat = N + b_pad, 1, K * (N + b_pad)
    p.batch.rank = len(batch)
    count, a_acc, b_acc = 1, a_mat, b_mat
    for d in range(MAX_BATCH_RANK):
        p.batch.shape[d] = 1
    for d in reversed(range(len(batch))):
        p.batch.shape[d] = batch[d]
        p.batch.a_str[d] = a_acc
        p.batch.b_str[d] = 0 if b_shared else b_acc
        a_acc *= batch[d]
        b_acc *= batch[d]
        count *= batch[d]
    p.batch_count = count
    p.bm, p.bn, p.np = tile[0], tile[1], np_
    p.cus, p.wgs_per_cu, p.group_by_xcd = cus, wpc, int(group)
    return p


def run(emu, p):
    rep = EmuReport()
    rc = emu.emulate_kstream(C.byref(p), C.byref(rep))
    assert rc == 0, rep.message.decode()
    assert rep.stores == p.batch_count * p.M * p.N
    return rep


LAYOUTS = [("k", "k"), ("k", "mn"), ("mn", "k"), ("mn", "mn")]


@pytest.mark.parametrize("la,lb", LAYOUTS)
def test_every_layout_ragged_tiles_and_k_tails(emu, la, lb):
    # extents of an MN-major operand must be multiples of 4, a K-major operand needs K % 4 == 0 when K % 16 != 0
    for (M, N, K) in [(128, 128, 16), (128, 128, 64), (300, 520, 100), (132, 260, 20), (4, 4, 4), (1000, 136, 8), (256, 384, 112), (128, 256, 36)]:
        for cus in (1, 3, 8, 256):
            rep = run(emu, problem(M, N, K, la, lb, cus=cus))
            assert rep.workgroups >= 1 and rep.steps >= (K + 15) // 16


def test_k_major_rows_that_are_no_multiple_of_four(emu):
    # a K-major operand may have any row count (rows are clamped one by one); K = 1..3 steps, padded pitches
    for (M, N, K) in [(1, 1, 16), (129, 131, 48), (77, 333, 32)]:
        run(emu, problem(M, N, K, "k", "k", a_pad=4, b_pad=8, cus=16))


@pytest.mark.parametrize("np_", [4, 5, 8])
def test_ring_depths(emu, np_):
    run(emu, problem(512, 512, 80, "k", "mn", np_=np_, cus=4))
    run(emu, problem(128, 128, 16, "mn", "k", np_=np_, cus=4))   # a single step in the whole stream
    run(emu, problem(128, 256, 32, "k", "k", np_=np_, cus=1))    # one workgroup walks everything


def test_batches_and_xcd_grouping(emu):
    # 8 and more batches: the workgroups of an XCD take whole batches; a shared (broadcast) B
    run(emu, problem(256, 256, 64, "k", "k", batch=(2, 6), cus=8))
    run(emu, problem(256, 384, 64, "k", "k", batch=(16,), cus=8))
    run(emu, problem(130, 260, 48, "k", "mn", batch=(9,), b_shared=True, cus=16))
    run(emu, problem(256, 256, 64, "k", "k", batch=(3,), cus=8, group=False))
    # few tile-rows, many tile-columns: whole column blocks per XCD
    run(emu, problem(256, 128 * 70, 32, "k", "mn", cus=8))
    run(emu, problem(100, 128 * 64 + 40, 256, "mn", "mn", cus=16))


def test_benchmark_shapes(emu):
    """The shapes the kernel is meant for, at their real sizes (one batch of the attention products: the walk of the
    full 96 batches is covered at reduced extents above)."""
    run(emu, problem(1024, 1024, 64, "k", "k", batch=(8,), cus=64))          # Q.K^T, dO.V^T
    run(emu, problem(256, 50000, 100, "k", "mn"))                            # CBOW logits
    run(emu, problem(100, 50000, 256, "mn", "mn"))                           # CBOW A^T.dC
    run(emu, problem(4096, 4096, 256, "k", "k"))
    run(emu, problem(1024, 1024, 128, "k", "mn", batch=(8,), cus=64, wpc=1))

@pytest.mark.parametrize("la,lb", LAYOUTS)
def test_64x64_tiles_with_a_ring_of_eight(emu, la, lb):
    for (M, N, K) in [(64, 64, 32), (300, 520, 100), (132, 260, 20), (1000, 136, 24), (1024, 1024, 1024), (64, 192, 36)]:
        for cus in (1, 3, 256):
            run(emu, problem(M, N, K, la, lb, tile=(64, 64), np_=8, cus=cus))
    run(emu, problem(256, 384, 64, la, lb, batch=(16,), tile=(64, 64), np_=8, cus=8))
    run(emu, problem(132, 260, 48, la, lb, batch=(9,), b_shared=True, tile=(64, 64), np_=8, cus=16))  # (an MN-major extent must be a multiple of 4)


def test_one_workgroup_per_cu(emu):
    run(emu, problem(300, 520, 100, "k", "mn", cus=8, wpc=1))
    run(emu, problem(256, 384, 64, "mn", "k", batch=(16,), cus=8, wpc=1))


def test_detects_a_broken_launch(emu):
    """The checks bite: an MN-major operand whose extent is no multiple of 4 (which the host refuses) is caught."""
    rep = EmuReport()
    p = problem(130, 128, 16, "mn", "k", cus=2)
    assert emu.emulate_kstream(C.byref(p), C.byref(rep)) == 1 and rep.message
