"""GPU parity: the HIP path, called through the C ABI (via the host mirror), against the CPU oracle
on the same seeded inputs, against the reference's literal vectors, and against fp64.

Tolerance (stated by the task): relative Frobenius error <= 1e-5 against the fp64-accumulated
reference; literal vectors with the reference's own all_close(rtol=1e-5, atol=1e-8)
(tenmo/ndbuffer.mojo:2263-2266)."""
import ctypes as C

import os

import numpy as np
import pytest

from helpers import GOLDEN_GRADIENT_KEYS, RTOL_FRO, ce_reference64, check_golden_extras, exact_product, generated_operand, numpy_view, ref_matmul64, rel_fro, scatter_to_storage, storage_of, strides_of

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import tenmo_amd.matmul as M
    import tenmo_amd.tensor as TT
    from tenmo_amd import _lib

    _lib.init(0)

    class NS:
        Tensor = TT.Tensor
        mm, mv, vm, dot = TT.mm, TT.mv, TT.vm, TT.dot
        Mm = M
        lib = _lib

    return NS


def fixture_tensor(T, t, requires_grad=False):
    base = T.Tensor.from_numpy(storage_of(t), requires_grad=False)
    return base.view(t["shape"], strides_of(t), t.get("offset", 0), requires_grad=requires_grad)


def oracle_view(O, t):
    return O.View(storage_of(t), t.get("offset", 0), t["shape"], strides_of(t))


def as_strided_tensor(T, arr, requires_grad=False):
    """Upload the storage behind a numpy view once and describe the same view on the device."""
    base = arr
    while base.base is not None:
        base = base.base
    base = np.ascontiguousarray(base)
    off = (arr.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // 4
    store = T.Tensor.from_numpy(base.reshape(-1))
    return store.view(arr.shape, tuple(s // 4 for s in arr.strides), off, requires_grad=requires_grad)


# ---- the reference's literal vectors ---------------------------------------------------------------

def test_golden_forward_and_backward(T, golden):
    mode = {"mm": T.mm, "mv": T.mv, "vm": T.vm, "dot": T.dot}
    for c in golden["cases"]:
        # (a one-element operand of dot is broadcast first, by the reference's Broadcast operator, whose backward is not part of
        # the matrix-product path: those cases are forward only)
        grads = not (c["op"] == "dot" and (c["A"]["shape"] == [] or c["B"]["shape"] == []))
        A = fixture_tensor(T, c["A"], requires_grad=grads)
        B = fixture_tensor(T, c["B"], requires_grad=grads)
        out = A.matmul(B, mode=mode[c["op"]])
        if "expect" in c:
            np.testing.assert_allclose(out.to_numpy(), np.asarray(c["expect"], np.float32), rtol=1e-5, atol=1e-8, err_msg=c["name"])
        if "expect_shape" in c:
            assert list(out.shape()) == c["expect_shape"], c["name"]
        check_golden_extras(c, out.to_numpy())
        if any(k in c for k in GOLDEN_GRADIENT_KEYS):
            out.backward(1.0)  # loss = out.sum(); loss.backward()
            check_golden_extras(c, out.to_numpy(), A.grad(), B.grad())
            if "grad_A" in c:
                np.testing.assert_allclose(A.grad(), np.asarray(c["grad_A"], np.float32), rtol=1e-5, err_msg=c["name"] + " grad_A")
            if "grad_B" in c:
                np.testing.assert_allclose(B.grad(), np.asarray(c["grad_B"], np.float32), rtol=1e-5, err_msg=c["name"] + " grad_B")
            # gradients asserted on the tensor behind a view: the view-shaped gradient scattered onto its storage
            if "base_grad_A" in c:
                np.testing.assert_allclose(scatter_to_storage(c["A"], A.grad()), c["base_grad_A"], rtol=1e-5, err_msg=c["name"] + " base_grad_A")
            if "base_grad_B" in c:
                np.testing.assert_allclose(scatter_to_storage(c["B"], B.grad()), c["base_grad_B"], rtol=1e-5, err_msg=c["name"] + " base_grad_B")


def test_reference_device_kernel_cases(T, golden, oracle):
    """The reference's tests of the launch functions this library replaces (tests/test_gpu.mojo:550-1575) compare the GPU result
    with the CPU result on these operands; here: the HIP result against the oracle (the restated CPU path), bit for bit where the
    sums are exact in fp32 (small integers: all of them), and against the values the tests state."""
    mode = {"mm": T.mm, "mv": T.mv, "vm": T.vm}
    for c in golden["device_kernel_cases"]["cases"]:
        a, b = generated_operand(c["A"]), generated_operand(c["B"])
        out = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), mode=mode[c["op"]], track_grad=False).to_numpy()
        cpu = {"mm": oracle.matmul, "mv": oracle.mv, "vm": oracle.vm}[c["op"]](a, b)
        assert out.shape == cpu.shape, c["name"]
        np.testing.assert_array_equal(out, cpu, err_msg=c["name"])
        np.testing.assert_array_equal(out, exact_product(c["op"], a, b).astype(np.float32), err_msg=c["name"])
        if "expect" in c:
            np.testing.assert_array_equal(out, np.asarray(c["expect"], np.float32), err_msg=c["name"])


def test_golden_result_shapes(T, golden):
    """The reference's shape-only tests (random operands there): the broadcast of the batch dimensions, from the library's own
    shape resolution (tenmo_hip_result_shape), and one of them computed."""
    import ctypes as C

    L, lib = T.lib.load(), T.lib
    for c in golden["shape_cases"]:
        va = lib.make_view(0, 0, c["A_shape"], [1] * len(c["A_shape"]))
        vb = lib.make_view(0, 0, c["B_shape"], [1] * len(c["B_shape"]))
        shape, rank = (C.c_int64 * 8)(), C.c_int32()
        n = L.tenmo_hip_result_shape(lib.OP_MM, C.byref(va), C.byref(vb), shape, C.byref(rank))
        assert list(shape[:rank.value]) == c["expect_shape"] and n == int(np.prod(c["expect_shape"])), c["name"]
    c = golden["shape_cases"][1]
    rng = np.random.default_rng(3)
    a, b = rng.standard_normal(c["A_shape"], dtype=np.float32), rng.standard_normal(c["B_shape"], dtype=np.float32)
    out = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False)
    assert list(out.shape()) == c["expect_shape"] and rel_fro(out.to_numpy(), ref_matmul64(a, b)) <= RTOL_FRO


def test_closed_forms(T, golden):
    for c in golden["closed_forms"]:
        A = T.Tensor.ones(*c["A_shape"], requires_grad=True)
        B = T.Tensor.ones(*c["B_shape"], requires_grad=True)
        out = A.matmul(B)
        got = out.to_numpy()
        assert np.all(got == c["expect_value"]), c["name"]
        if "grad_A_value" in c:
            out.backward(1.0)
            assert A.grad().shape == tuple(c["A_shape"]) and np.all(A.grad() == c["grad_A_value"])
            assert B.grad().shape == tuple(c["B_shape"]) and np.all(B.grad() == c["grad_B_value"])


# ---- 2-D GEMM against oracle and fp64 --------------------------------------------------------------

@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 4])
def test_verify_shapes(T, golden, oracle, tile):
    """Shape list of tests/test_matmul_2d_verify.mojo, each with A / B as row-major, transposed view
    and padded view, on every workgroup-tile configuration."""
    L = T.lib.load()
    L.tenmo_hip_set_tuning(b"gemm_tile", tile)
    try:
        rng = np.random.default_rng(17)
        for m, k, n in golden["verify_shapes"]["mkn"]:
            a = rng.standard_normal((m, k), dtype=np.float32)
            b = rng.standard_normal((k, n), dtype=np.float32)
            ref = ref_matmul64(a, b)
            a_views = [a, np.ascontiguousarray(a.T).T, np.pad(a, ((0, 0), (0, 3)))[:, :k]]
            b_views = [b, np.ascontiguousarray(b.T).T, np.pad(b, ((0, 0), (0, 5)))[:, :n]]
            for av in a_views:
                for bv in b_views:
                    got = as_strided_tensor(T, av).matmul(as_strided_tensor(T, bv), track_grad=False).to_numpy()
                    assert got.shape == (m, n)
                    assert rel_fro(got, ref) <= RTOL_FRO, (m, k, n, av.strides, bv.strides)
                    # and against the CPU restatement on identical inputs
                    assert rel_fro(got, oracle.mm2d(av, bv)) <= 2 * RTOL_FRO
    finally:
        L.tenmo_hip_set_tuning(b"gemm_tile", -1)


@pytest.mark.parametrize("tile", [-1, 0, 1, 3, 4])
def test_ragged_tiles_and_k_slices(T, oracle, tile):
    """Extents that leave partial tiles in M, N and K at once, in every operand layout: exercises the
    direct-to-LDS path with clamped rows (extent divisible by 4 or not), the checked tail, and
    explicit K slicing with its reduction."""
    L = T.lib.load()
    rng = np.random.default_rng(19)
    try:
        L.tenmo_hip_set_tuning(b"gemm_tile", tile)
        for (m, k, n) in [(100, 256, 500), (260, 100, 132), (257, 48, 129), (300, 1000, 68), (1, 64, 4), (4, 4096, 8), (131, 37, 259)]:
            a = rng.standard_normal((m, k), dtype=np.float32)
            b = rng.standard_normal((k, n), dtype=np.float32)
            ref = ref_matmul64(a, b)
            for av in (a, np.ascontiguousarray(a.T).T):
                for bv in (b, np.ascontiguousarray(b.T).T):
                    for sk in (-1, 3):
                        L.tenmo_hip_set_tuning(b"gemm_splitk", sk)
                        got = as_strided_tensor(T, av).matmul(as_strided_tensor(T, bv), track_grad=False).to_numpy()
                        assert rel_fro(got, ref) <= RTOL_FRO, (tile, m, k, n, av.strides, bv.strides, sk)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_tile", -1)
        L.tenmo_hip_set_tuning(b"gemm_splitk", -1)


@pytest.mark.parametrize("smallk", [1, 0])
def test_short_reduction_kernel(T, smallk):
    """C (+)= A . B^T(view) with K a multiple of 16 up to 64 through the kernel-level entry point: the persistent
    short-reduction kernel forced on (and, as the control, off), over whole and ragged tiles, batches, a
    broadcast B, fewer tiles than workgroups and more, with and without accumulation; against fp64."""
    import torch
    L, lib = T.lib.load(), T.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(23)
    cases = [((), 64, 64, 16, 0), ((), 128, 192, 64, 0), ((3,), 100, 130, 32, 0), ((2, 3), 257, 65, 64, 1), ((2,), 333, 777, 48, 1),
             ((), 1000, 1000, 48, 0), ((7,), 1, 1, 16, 0), ((2,), 512, 512, 64, 1), ((9,), 1024, 1024, 64, 0), ((40,), 320, 192, 32, 1),
             ((3, 2), 640, 320, 96, 0)]  # (the last one has K > 64: the ordinary kernel either way)
    try:
        L.tenmo_hip_set_tuning(b"gemm_smallk", smallk)
        for bshape, M, N, K, acc in cases:
            for bcast in (False, True):
                A = torch.randn((*bshape, M, K), generator=gen, device="cuda")
                Bt = torch.randn((*((1,) * len(bshape) if bcast else bshape), N, K), generator=gen, device="cuda")
                Cc = torch.randn((*bshape, M, N), generator=gen, device="cuda")
                ref = A.double() @ Bt.double().transpose(-1, -2) + (Cc.double() if acc else 0)
                ab = [A.stride(i) for i in range(len(bshape))]
                bb = [0 if bcast else Bt.stride(i) for i in range(len(bshape))]
                lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, K, 1, Bt.data_ptr(), 0, 1, K, Cc.data_ptr(), M, N, K, len(bshape),
                                               lib.i64(bshape), lib.i64(ab), lib.i64(bb), acc, 1))
                err = float((Cc.double() - ref).norm() / ref.norm())
                assert err <= RTOL_FRO, (smallk, bshape, M, N, K, acc, bcast, err)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_smallk", -1)


def test_kstream_kernel(T):
    _kstream_cases(T, 1)


def _kstream_cases(T, knob):
    """The persistent K-stream kernel (loading wavefronts of its own, a ring of LDS stages across tiles, stores behind the
    next tile's MFMAs) forced on: every operand layout, whole and ragged tiles, reductions of one step to many, K tails,
    batches with and without a broadcast B, fewer tiles than workgroups and many more, plain and accumulating stores;
    against fp64.  (The same launches are replayed address by address on the CPU in test_kstream_addresses.py.)"""
    import torch
    L, lib = T.lib.load(), T.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31)
    cases = [((), 128, 128, 16, 0), ((), 128, 256, 64, 0), ((3,), 100, 132, 36, 0), ((2, 3), 256, 68, 64, 1), ((5,), 64, 64, 112, 0),
             ((2,), 332, 776, 20, 1), ((), 1000, 1000, 8, 0), ((4,), 72, 52, 84, 1), ((), 256, 50000, 100, 0), ((2,), 512, 512, 52, 1),
             ((9,), 320, 1024, 12, 0), ((), 64, 8192, 104, 0), ((), 132, 72, 4, 0), ((12,), 1024, 1024, 64, 0), ((), 100, 50000, 256, 1),
             ((), 4096, 4096, 512, 0), ((17,), 260, 384, 128, 1)]
    try:
        L.tenmo_hip_set_tuning(b"gemm_panel", knob)
        for bshape, M, N, K, acc in cases:
            for ta in (False, True):
                for tb in (False, True):
                    for bcast in ((False, True) if bshape and M <= 512 else (False,)):
                        A = torch.randn((*bshape, *((K, M) if ta else (M, K))), generator=gen, device="cuda")
                        B = torch.randn((*((1,) * len(bshape) if bcast else bshape), *((N, K) if tb else (K, N))), generator=gen, device="cuda")
                        Cc = torch.randn((*bshape, M, N), generator=gen, device="cuda")
                        a_rs, a_cs = (1, M) if ta else (K, 1)
                        b_rs, b_cs = (1, K) if tb else (N, 1)
                        ref = (A.transpose(-1, -2) if ta else A).double() @ (B.transpose(-1, -2) if tb else B).double() + (Cc.double() if acc else 0)
                        ab = [A.stride(i) for i in range(len(bshape))]
                        bb = [0 if bcast else B.stride(i) for i in range(len(bshape))]
                        lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, Cc.data_ptr(), M, N, K, len(bshape),
                                                       lib.i64(bshape), lib.i64(ab), lib.i64(bb), acc, 1))
                        err = float((Cc.double() - ref).norm() / ref.norm())
                        assert err <= RTOL_FRO, (bshape, M, N, K, acc, ta, tb, bcast, err)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_panel", -1)


def test_raw_abi_arguments(T):
    """Argument checking of the kernel-level entry points (status codes + messages, nothing launched)."""
    L, lib = T.lib.load(), T.lib
    x = T.Tensor.zeros(4, 4)
    p = x.buffer.data_ptr()
    assert L.tenmo_hip_gemm_f32(p, 0, 4, 1, p, 0, 4, 1, p, -1, 4, 4, 0, None, None, None, 0, 0) == -2
    assert b"negative" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_gemm_f32(None, 0, 4, 1, p, 0, 4, 1, p, 4, 4, 4, 0, None, None, None, 0, 0) == -3
    assert L.tenmo_hip_gemm_f32(p, 0, 4, 1, p, 0, 4, 1, p, 4, 4, 4, 7, None, None, None, 0, 0) == -3   # batch rank > 6
    assert L.tenmo_hip_gemm_f32(p, 0, 4, 1, p, 0, 4, 1, p, 4, 4, 4, 1, None, None, None, 0, 0) == -3   # rank 1 without arrays
    assert L.tenmo_hip_set_tuning(b"no_such_knob", 1) == -3
    assert L.tenmo_hip_mv_f32(p, 0, 4, 1, p, 0, 1, p, -2, 4, 0, None, None, None, 0, 0) == -2
    # null pointers are refused before anything is launched
    assert L.tenmo_hip_mv_f32(p, 0, 4, 1, p, 0, 1, None, 4, 4, 0, None, None, None, 0, 0) == -3
    assert L.tenmo_hip_mv_f32(None, 0, 4, 1, p, 0, 1, p, 4, 4, 0, None, None, None, 0, 0) == -3
    assert L.tenmo_hip_vm_f32(p, 0, 1, p, 0, 4, 1, None, 4, 4, 0, None, None, None, 0, 0) == -3
    assert L.tenmo_hip_dot_f32(p, 0, 1, p, 0, 1, 4, None, 0) == -3
    assert L.tenmo_hip_dot_f32(None, 0, 1, p, 0, 1, 4, p, 0) == -3
    assert L.tenmo_hip_gemm_f32(p, 0, 4, 1, p, 0, 4, 1, None, 4, 4, 0, 0, None, None, None, 0, 0) == -3  # K = 0 still writes C
    v = lib.make_view(p, 0, (4, 4), (4, 1))
    nv = lib.make_view(None, 0, (4, 4), (4, 1))
    import ctypes as C
    assert L.tenmo_hip_matmul_nd(C.byref(v), C.byref(v), None, 0) == -3
    assert L.tenmo_hip_matmul_nd(C.byref(nv), C.byref(v), p, 0) == -3
    assert L.tenmo_hip_matrix_vector_nd(C.byref(v), C.byref(lib.make_view(p, 0, (4,), (1,))), None, 0) == -3
    assert L.tenmo_hip_matmul_backward(C.byref(v), C.byref(v), None, p, p, 0) == -3
    # a zero-sized problem is a no-op that succeeds
    assert L.tenmo_hip_gemm_f32(p, 0, 4, 1, p, 0, 4, 1, p, 0, 4, 4, 0, None, None, None, 0, 1) == 0
    # explicit batch arrays: C[b] = A[b] . B (B broadcast with stride 0), accumulate twice doubles
    a = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    b = np.arange(4 * 5, dtype=np.float32).reshape(4, 5)
    A, B, out = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b), T.Tensor.zeros(2, 3, 5)
    for _ in range(2):
        lib.check(L.tenmo_hip_gemm_f32(A.buffer.data_ptr(), 0, 4, 1, B.buffer.data_ptr(), 0, 5, 1, out.buffer.data_ptr(), 3, 5, 4,
                                       1, lib.i64([2]), lib.i64([12]), lib.i64([0]), 1, 1))
    np.testing.assert_array_equal(out.to_numpy(), 2 * np.matmul(a, b))


def test_direct_path_pitch_limits(T):
    """Row pitches the direct global->LDS path cannot address with 32-bit lane offsets (huge, negative)
    fall back to the checked loader and still give the right product; aligned 16-byte rows with a
    large but admissible pitch stay on the direct path."""
    rng = np.random.default_rng(29)
    m, k, n = 6, 64, 40
    b = rng.standard_normal((k, n), dtype=np.float32)
    B = T.Tensor.from_numpy(b)
    for pitch in (3_000_000, 1_000_000):     # above / below the direct path's limit of 2^21 elements
        store = np.zeros(m * pitch, np.float32)
        a = rng.standard_normal((m, k), dtype=np.float32)
        for i in range(m):
            store[i * pitch:i * pitch + k] = a[i]
        dev = T.Tensor.from_numpy(store)
        got = dev.view((m, k), (pitch, 1), 0).matmul(B, track_grad=False).to_numpy()
        assert rel_fro(got, ref_matmul64(a, b)) <= RTOL_FRO, pitch
        # the same rows as the K-major right operand: B2 = a^T through a transposed view
        x = rng.standard_normal((5, m), dtype=np.float32)
        got = T.Tensor.from_numpy(x).matmul(dev.view((m, k), (pitch, 1), 0), track_grad=False).to_numpy()
        assert rel_fro(got, ref_matmul64(x, a)) <= RTOL_FRO, pitch
        del dev
    # rows walked backwards (negative row stride) and columns walked backwards (negative k stride)
    a = rng.standard_normal((70, 64), dtype=np.float32)
    dev = T.Tensor.from_numpy(a.ravel())
    flipped_rows = dev.view((70, 64), (-64, 1), 69 * 64)
    assert rel_fro(flipped_rows.matmul(B, track_grad=False).to_numpy(), ref_matmul64(a[::-1], b)) <= RTOL_FRO
    flipped_cols = dev.view((70, 64), (64, -1), 63)
    assert rel_fro(flipped_cols.matmul(B, track_grad=False).to_numpy(), ref_matmul64(a[:, ::-1], b)) <= RTOL_FRO


@pytest.mark.parametrize("tile", [-1, 0, 2, 3])
def test_fused_epilogue(T, tile):
    """bias + ReLU + ReLU-gradient mask applied in the GEMM store equal the separate steps, on every
    path that can finish a tile: plain store, K slices + reduction, batched, ragged extents."""
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(31)
    try:
        L.tenmo_hip_set_tuning(b"gemm_tile", tile)
        for (bsz, m, k, n, sk) in [(1, 64, 784, 128, -1), (1, 64, 784, 128, 3), (1, 300, 100, 77, -1), (3, 70, 48, 130, -1), (1, 5, 1000, 9, 4)]:
            L.tenmo_hip_set_tuning(b"gemm_splitk", sk)
            a = rng.standard_normal((bsz, m, k), dtype=np.float32)
            b = rng.standard_normal((k, n), dtype=np.float32)
            bias = rng.standard_normal(n).astype(np.float32)
            mask = rng.standard_normal((bsz, m, n)).astype(np.float32)
            A, B, Bi, Mk = (T.Tensor.from_numpy(x) for x in (a, b, bias, mask))
            out = T.Tensor.zeros(bsz, m, n)
            z = ref_matmul64(a, b)
            for relu, use_bias, use_mask in [(0, 1, 0), (1, 1, 0), (1, 0, 0), (0, 0, 1), (1, 1, 1)]:
                lib.check(L.tenmo_hip_gemm_epilogue_f32(
                    A.buffer.data_ptr(), 0, k, 1, B.buffer.data_ptr(), 0, n, 1, out.buffer.data_ptr(), m, n, k,
                    1, lib.i64([bsz]), lib.i64([m * k]), lib.i64([0]),
                    Bi.buffer.data_ptr() if use_bias else None, relu, Mk.buffer.data_ptr() if use_mask else None, 1))
                ref = z + (bias if use_bias else 0.0)
                if relu:
                    ref = np.where(ref > 0, ref, 0.0)
                if use_mask:
                    ref = np.where(mask > 0, ref, 0.0)
                got = out.to_numpy()
                # elements within rounding of the ReLU threshold may legitimately land on either side
                near = np.abs(z + (bias if use_bias else 0.0)) < 1e-4
                assert rel_fro(np.where(near, 0, got), np.where(near, 0, ref)) <= RTOL_FRO, (tile, bsz, m, k, n, sk, relu, use_bias, use_mask)
                if use_mask:
                    assert np.all(got[mask <= 0] == 0)
        # view-level Linear entry against the unfused sequence
        x = rng.standard_normal((4, 33, 50), dtype=np.float32)
        w = rng.standard_normal((50, 20), dtype=np.float32)
        bias = rng.standard_normal(20).astype(np.float32)
        X, W, Bi = T.Tensor.from_numpy(x), T.Tensor.from_numpy(w), T.Tensor.from_numpy(bias)
        got = X.buffer.linear(W.buffer, Bi.buffer, relu=True, sync=True).to_numpy()
        ref = np.maximum(ref_matmul64(x, w) + bias, 0)
        assert got.shape == (4, 33, 20) and rel_fro(got, ref) <= RTOL_FRO
        # accumulate and a fused epilogue exclude each other; K = 0 has no sums to finish
        assert L.tenmo_hip_gemm_epilogue_f32(A.buffer.data_ptr(), 0, 4, 1, B.buffer.data_ptr(), 0, 4, 1, out.buffer.data_ptr(), 2, 2, 0,
                                             0, None, None, None, Bi.buffer.data_ptr(), 0, None, 1) == -2
    finally:
        L.tenmo_hip_set_tuning(b"gemm_tile", -1)
        L.tenmo_hip_set_tuning(b"gemm_splitk", -1)


def test_relu_epilogue_reference_literals(T, golden):
    """The ReLU and ReLU-gradient epilogues on the literals of tests/test_relu.mojo: x.I (+ bias) through the GEMM with the
    ReLU in its store gives the reference's output, ones.I masked by that activation the reference's gradient — exactly
    (products with an identity matrix are exact), in particular 0 at x = 0."""
    L, lib = T.lib.load(), T.lib
    for c in golden["harness"]["relu_literals"]["cases"]:
        x = np.asarray(c["x"], np.float32)[None, :]
        n = x.shape[1]
        bias = np.asarray(c["bias"], np.float32) if "bias" in c else None
        X, I, one = T.Tensor.from_numpy(x), T.Tensor.from_numpy(np.eye(n, dtype=np.float32)), T.Tensor.from_numpy(np.ones((1, n), np.float32))
        Bi = T.Tensor.from_numpy(bias) if bias is not None else None
        h, g = T.Tensor.zeros(1, n), T.Tensor.zeros(1, n)
        lib.check(L.tenmo_hip_gemm_epilogue_f32(X.buffer.data_ptr(), 0, n, 1, I.buffer.data_ptr(), 0, n, 1, h.buffer.data_ptr(), 1, n, n,
                                                0, None, None, None, Bi.buffer.data_ptr() if Bi is not None else None, 1, None, 1))
        want = np.asarray(c["out"], np.float32) if "out" in c else np.maximum(x[0] + (bias if bias is not None else 0), 0)
        np.testing.assert_array_equal(h.to_numpy()[0], want, err_msg=c["source"])
        if "grad" in c:
            lib.check(L.tenmo_hip_gemm_epilogue_f32(one.buffer.data_ptr(), 0, n, 1, I.buffer.data_ptr(), 0, n, 1, g.buffer.data_ptr(), 1, n, n,
                                                    0, None, None, None, None, 0, h.buffer.data_ptr(), 1))
            np.testing.assert_array_equal(g.to_numpy()[0], np.asarray(c["grad"], np.float32), err_msg=c["source"])


def test_column_sum(T):
    """Bias gradient = column sums of the upstream gradient (tenmo/broadcast.mojo:81-87): small, ragged,
    padded rows, accumulate, and a size that takes the K-sliced streaming path."""
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(37)
    for rows, cols, pitch in [(1, 1, 1), (3, 5, 5), (64, 10, 10), (300, 77, 80), (8192, 2304, 2304), (4096, 1000, 1003)]:
        g = rng.standard_normal((rows, pitch), dtype=np.float32)
        G = T.Tensor.from_numpy(g)
        out = T.Tensor.from_numpy(np.ones(cols, np.float32))
        lib.check(L.tenmo_hip_column_sum_f32(G.buffer.data_ptr(), 0, pitch, rows, cols, out.buffer.data_ptr(), 0, 1))
        ref = g[:, :cols].astype(np.float64).sum(axis=0)
        assert rel_fro(out.to_numpy(), ref) <= RTOL_FRO, (rows, cols, pitch)
        lib.check(L.tenmo_hip_column_sum_f32(G.buffer.data_ptr(), 0, pitch, rows, cols, out.buffer.data_ptr(), 1, 1))
        assert rel_fro(out.to_numpy(), 2 * ref) <= RTOL_FRO, (rows, cols, pitch, "accumulate")
    assert L.tenmo_hip_column_sum_f32(None, 0, 4, 4, 4, None, 0, 1) == -3
    assert L.tenmo_hip_column_sum_f32(None, 0, 4, 0, 4, None, 0, 1) == -3     # an empty sum still writes zeros
    out = T.Tensor.from_numpy(np.ones(4, np.float32))
    assert L.tenmo_hip_column_sum_f32(None, 0, 4, 0, 4, out.buffer.data_ptr(), 0, 1) == 0
    assert np.all(out.to_numpy() == 0)


@pytest.mark.parametrize("tile", [0, 1, 2, 3])
def test_stream_k(T, tile):
    """Persistent stream-K launches: tiles shared between workgroups are summed by the fix-up kernel.
    Shapes with fewer tiles than workgroups, with rounds of whole tiles ahead of the shared ones (one
    matrix and batched), with whole rounds only, ragged extents, K tails, transposed views, batches,
    accumulate and the fused epilogue."""
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(53)
    try:
        L.tenmo_hip_set_tuning(b"gemm_tile", tile)
        for wg_per_cu in ((1, 2) if tile <= 1 else (1, 4)):
            L.tenmo_hip_set_tuning(b"gemm_streamk", wg_per_cu)
            for (bsz, m, k, n) in [(1, 768, 2000, 640), (1, 300, 4100, 200), (1, 2048, 512, 1536), (3, 260, 1000, 132), (1, 100, 64, 70), (1, 1500, 8192, 900),
                                      (1, 2304, 400, 2432), (4, 2300, 400, 2432), (1, 2304, 100, 2432), (1, 4096, 48, 4096)]:
                a = rng.standard_normal((bsz, m, k), dtype=np.float32)
                b = rng.standard_normal((k, n), dtype=np.float32)
                ref = ref_matmul64(a, b)
                A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
                got = A.matmul(B, track_grad=False).to_numpy()
                assert rel_fro(got, ref) <= RTOL_FRO, (tile, wg_per_cu, bsz, m, k, n)
                # transposed views of both operands
                At = T.Tensor.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1))).transpose()
                Bt = T.Tensor.from_numpy(np.ascontiguousarray(b.T)).transpose()
                got = At.matmul(Bt, track_grad=False).to_numpy()
                assert rel_fro(got, ref) <= RTOL_FRO, (tile, wg_per_cu, bsz, m, k, n, "views")
            # accumulate twice, then bias + ReLU through the fix-up
            a = rng.standard_normal((700, 3000), dtype=np.float32)
            b = rng.standard_normal((3000, 500), dtype=np.float32)
            bias = rng.standard_normal(500).astype(np.float32)
            A, B, Bi, out = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b), T.Tensor.from_numpy(bias), T.Tensor.zeros(700, 500)
            for _ in range(2):
                lib.check(L.tenmo_hip_gemm_f32(A.buffer.data_ptr(), 0, 3000, 1, B.buffer.data_ptr(), 0, 500, 1, out.buffer.data_ptr(),
                                               700, 500, 3000, 0, None, None, None, 1, 1))
            assert rel_fro(out.to_numpy(), 2 * ref_matmul64(a, b)) <= RTOL_FRO
            lib.check(L.tenmo_hip_gemm_epilogue_f32(A.buffer.data_ptr(), 0, 3000, 1, B.buffer.data_ptr(), 0, 500, 1, out.buffer.data_ptr(),
                                                    700, 500, 3000, 0, None, None, None, Bi.buffer.data_ptr(), 1, None, 1))
            z = ref_matmul64(a, b) + bias
            near = np.abs(z) < 1e-3
            assert rel_fro(np.where(near, 0, out.to_numpy()), np.where(near, 0, np.maximum(z, 0))) <= RTOL_FRO
    finally:
        L.tenmo_hip_set_tuning(b"gemm_tile", -1)
        L.tenmo_hip_set_tuning(b"gemm_streamk", -1)


def test_columns_with_misaligned_row_pitch(T):
    """vm and skinny products against a matrix whose row pitch is not a multiple of 4 floats (rows start
    at every 16-byte phase): the shifted-accumulator kernel, its K slices, its last-row and edge handling,
    batches, and the fall-backs (5..8 left rows, unaligned base)."""
    rng = np.random.default_rng(59)
    for (m, k, n) in [(1, 37, 4099), (1, 1000, 10007), (3, 768, 50257), (4, 129, 2051), (2, 64, 5001), (6, 200, 3001), (4, 5, 7), (1, 4097, 1021)]:
        a = rng.standard_normal((m, k), dtype=np.float32)
        b = rng.standard_normal((k, n), dtype=np.float32)
        ref = ref_matmul64(a, b)
        A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
        if m == 1:
            got = T.Tensor.from_numpy(a[0]).matmul(B, track_grad=False).to_numpy()      # vector x matrix
            assert rel_fro(got, ref[0]) <= RTOL_FRO, ("vm", k, n)
        got = A.matmul(B, track_grad=False).to_numpy()
        assert rel_fro(got, ref) <= RTOL_FRO, (m, k, n)
        # the same matrix one element into its storage: the base is no longer 16-byte aligned
        store = np.zeros(k * n + 1, np.float32)
        store[1:] = b.ravel()
        Bo = T.Tensor.from_numpy(store).view((k, n), (n, 1), 1)
        assert rel_fro(A.matmul(Bo, track_grad=False).to_numpy(), ref) <= RTOL_FRO, (m, k, n, "offset 1")
        # padded rows (pitch n + 2)
        padded = np.zeros((k, n + 2), np.float32)
        padded[:, :n] = b
        Bp = T.Tensor.from_numpy(padded.ravel()).view((k, n), (n + 2, 1), 0)
        assert rel_fro(A.matmul(Bp, track_grad=False).to_numpy(), ref) <= RTOL_FRO, (m, k, n, "padded")
    # batched right operand with an odd pitch and batch stride multiple of 4
    a = rng.standard_normal((2, 768), dtype=np.float32)
    b = rng.standard_normal((4, 768, 2503), dtype=np.float32)
    got = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False).to_numpy()
    assert rel_fro(got, ref_matmul64(a, b)) <= RTOL_FRO


def test_column_kernels_reuse_workspace(T):
    """The column-streaming kernels (vm, skinny) cut K into slices that go through the library's
    workspace.  Same operand storage and workspace reused with new contents call after call, and `+=`."""
    import torch
    from tenmo_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(61)
    for (m, k, n) in [(1, 4096, 4096), (4, 768, 50257), (3, 2000, 3000), (8, 1024, 2048), (1, 16384, 1024)]:
        A = T.Tensor.from_numpy(np.zeros((m, k), np.float32))
        B = T.Tensor.from_numpy(np.zeros((k, n), np.float32))
        for rep in range(3):
            a = rng.standard_normal((m, k), dtype=np.float32)
            b = rng.standard_normal((k, n), dtype=np.float32)
            A.buffer.storage.copy_(torch.from_numpy(a.ravel()))
            B.buffer.storage.copy_(torch.from_numpy(b.ravel()))
            got = A.matmul(B, track_grad=False).to_numpy()
            assert rel_fro(got, ref_matmul64(a, b)) <= RTOL_FRO, (m, k, n, rep)
    a = rng.standard_normal((1, 3000), dtype=np.float32)
    b = rng.standard_normal((3000, 5000), dtype=np.float32)
    c0 = rng.standard_normal((1, 5000), dtype=np.float32)
    out = T.Tensor.from_numpy(c0.copy())
    A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
    _lib.check(L.tenmo_hip_gemm_f32(A.buffer.data_ptr(), 0, 3000, 1, B.buffer.data_ptr(), 0, 5000, 1, out.buffer.data_ptr(),
                                    1, 5000, 3000, 0, None, None, None, 1, 1))
    assert rel_fro(out.to_numpy(), c0.astype(np.float64) + ref_matmul64(a, b)) <= RTOL_FRO


def test_odd_strides_and_overlap(T, oracle):
    """Column stride 2, row stride 0 (broadcast rows), overlapping windows (tests/test_mmnd.mojo:143-175)."""
    rng = np.random.default_rng(23)
    store = rng.standard_normal(4000).astype(np.float32)
    dev = T.Tensor.from_numpy(store)
    cases = [
        ((20, 30), (60, 2), 7, (30, 10), (10, 1), 100),     # A col stride 2
        ((16, 24), (0, 1), 5, (24, 12), (12, 1), 900),      # A rows broadcast
        ((12, 40), (3, 1), 0, (40, 9), (2, 70), 1),         # overlapping A rows, B generic
        ((33, 17), (1, 40), 11, (17, 65), (1, 17), 2000),   # both transposed
    ]
    for ash, ast, aoff, bsh, bst, boff in cases:
        A = dev.view(ash, ast, aoff)
        B = dev.view(bsh, bst, boff)
        an = np.lib.stride_tricks.as_strided(store[aoff:], ash, tuple(4 * s for s in ast))
        bn = np.lib.stride_tricks.as_strided(store[boff:], bsh, tuple(4 * s for s in bst))
        got = A.matmul(B, track_grad=False).to_numpy()
        assert rel_fro(got, ref_matmul64(an, bn)) <= RTOL_FRO
        assert rel_fro(got, oracle.mm2d(oracle.View(store, aoff, ash, ast), oracle.View(store, boff, bsh, bst))) <= 2 * RTOL_FRO
    # inputs are never written
    np.testing.assert_array_equal(dev.to_numpy(), store)


def test_empty_and_degenerate(T):
    z = T.Tensor.zeros(3, 0).matmul(T.Tensor.zeros(0, 4), track_grad=False)  # K = 0 -> zeros (NDBuffer.zeros result)
    assert z.shape() == (3, 4) and np.all(z.to_numpy() == 0)
    e = T.Tensor.zeros(0, 5).matmul(T.Tensor.zeros(5, 4), track_grad=False)
    assert e.shape() == (0, 4)
    one = T.Tensor.d([[2.0]]).matmul(T.Tensor.d([[3.0]]), track_grad=False)
    assert one.to_numpy()[0, 0] == 6.0


def test_shape_errors(T):
    E = T.lib.TenmoHipError
    with pytest.raises(E, match="incompatible shapes"):  # classify_matmul -> invalid -> panic (tenmo/matmul.mojo:226-227)
        T.Tensor.zeros(2, 3).matmul(T.Tensor.zeros(4, 2))
    with pytest.raises(E, match="inner"):  # the NDBuffer-level validator (tenmo/matrixshapevalidator.mojo:58-68)
        T.Tensor.zeros(2, 3).buffer.matmul_2d(T.Tensor.zeros(4, 2).buffer)
    with pytest.raises(E, match="broadcast"):
        T.Tensor.zeros(2, 5, 3).matmul(T.Tensor.zeros(3, 3, 4))
    with pytest.raises(E, match="must match"):
        T.Tensor.zeros(2, 3).matmul(T.Tensor.zeros(4), mode=T.mv)
    with pytest.raises(E, match="must match"):
        T.Tensor.zeros(3).matmul(T.Tensor.zeros(4, 2), mode=T.vm)
    with pytest.raises(E, match="size does not match"):
        T.Tensor.zeros(3).matmul(T.Tensor.zeros(4))


# ---- batched / broadcast ---------------------------------------------------------------------------

def test_batched_broadcast_against_oracle(T, oracle):
    rng = np.random.default_rng(29)
    cases = [((3, 1, 17, 9), (4, 9, 13)), ((2, 5, 70, 33), (2, 5, 33, 41)), ((6, 40, 64), (1, 64, 64)),
             ((1, 2, 4, 8), (3, 2, 8, 4)), ((130, 70), (5, 70, 19)), ((2, 2, 2, 2, 3, 4), (4, 5))]
    for sa, sb in cases:
        a = rng.standard_normal(sa, dtype=np.float32)
        b = rng.standard_normal(sb, dtype=np.float32)
        got = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False).to_numpy()
        assert got.shape == ref_matmul64(a, b).shape
        assert rel_fro(got, ref_matmul64(a, b)) <= RTOL_FRO
        assert rel_fro(got, oracle.matmul(a, b)) <= 2 * RTOL_FRO
    # K^T as a transposed view, attention shape (tests/test_attn_matmul.mojo:106-186)
    q = rng.standard_normal((2, 3, 50, 16), dtype=np.float32)
    k = rng.standard_normal((2, 3, 50, 16), dtype=np.float32)
    s = T.Tensor.from_numpy(q).matmul(T.Tensor.from_numpy(k).transpose(-1, -2), track_grad=False).to_numpy()
    assert rel_fro(s, ref_matmul64(q, np.swapaxes(k, -1, -2))) <= RTOL_FRO
    # a batch-strided view (tests/test_mmnd.mojo:584-593)
    big = rng.standard_normal((4, 6, 5), dtype=np.float32)
    sub = big[::2]
    got = as_strided_tensor(T, sub).matmul(T.Tensor.from_numpy(np.eye(5, dtype=np.float32)), track_grad=False).to_numpy()
    np.testing.assert_array_equal(got, sub)


def test_backward_against_oracle(T, oracle):
    rng = np.random.default_rng(31)
    cases = [((37, 21), (21, 45)), ((3, 18, 9), (3, 9, 14)), ((4, 18, 9), (1, 9, 14)), ((1, 18, 9), (5, 9, 14)),
             ((18, 9), (2, 3, 9, 14)), ((2, 1, 6, 7), (1, 3, 7, 5))]
    for sa, sb in cases:
        a = rng.standard_normal(sa, dtype=np.float32)
        b = rng.standard_normal(sb, dtype=np.float32)
        A, B = T.Tensor.from_numpy(a, True), T.Tensor.from_numpy(b, True)
        out = A.matmul(B)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed), retain_graph=True)
        gA, gB = oracle.matmul_backward(a, b, seed)
        assert A.grad().shape == a.shape and B.grad().shape == b.shape
        assert rel_fro(A.grad(), gA) <= 2 * RTOL_FRO, (sa, sb)
        assert rel_fro(B.grad(), gB) <= 2 * RTOL_FRO, (sa, sb)
        # a second backward accumulates: gradients double (tests/test_mv.mojo:673-692)
        out.backward(T.Tensor.from_numpy(seed))
        assert rel_fro(A.grad(), 2 * gA) <= 2 * RTOL_FRO
        assert rel_fro(B.grad(), 2 * gB) <= 2 * RTOL_FRO
    # only the parent that requires grad receives one (tenmo/matmul.mojo:34,45)
    A, B = T.Tensor.ones(3, 4, requires_grad=False), T.Tensor.ones(4, 2, requires_grad=True)
    out = A.matmul(B)
    out.backward(1.0)
    assert A.grad() is None and np.all(B.grad() == 3.0)


def test_backward_through_transposed_view(T, oracle):
    """x . W^T with W a transposed view (tests/test_tensors.mojo:3443-3466 pattern) on random data."""
    rng = np.random.default_rng(37)
    x = rng.standard_normal((2, 19, 12), dtype=np.float32)
    w = rng.standard_normal((15, 12), dtype=np.float32)
    X = T.Tensor.from_numpy(x, True)
    Wt = T.Tensor.from_numpy(w, True).transpose()
    out = X.matmul(Wt)
    assert rel_fro(out.to_numpy(), ref_matmul64(x, w.T)) <= RTOL_FRO
    seed = rng.standard_normal(out.shape(), dtype=np.float32)
    out.backward(T.Tensor.from_numpy(seed))
    gX, gWt = oracle.matmul_backward(x, w.T, seed)
    assert rel_fro(X.grad(), gX) <= 2 * RTOL_FRO
    assert rel_fro(Wt.grad(), gWt) <= 2 * RTOL_FRO  # gradient at the view's own shape (12, 15)


# ---- mv / vm / dot ---------------------------------------------------------------------------------

def test_mv_vm_forward_all_layouts(T, oracle):
    rng = np.random.default_rng(41)
    M = rng.standard_normal((2, 3, 37, 29), dtype=np.float32)
    v = rng.standard_normal((3, 29), dtype=np.float32)
    u = rng.standard_normal((37,), dtype=np.float32)
    Md = T.Tensor.from_numpy(M)
    got = Md.matmul(T.Tensor.from_numpy(v), mode=T.mv, track_grad=False).to_numpy()
    assert got.shape == (2, 3, 37) and rel_fro(got, oracle.mv_f64(M, v)) <= RTOL_FRO
    assert rel_fro(got, oracle.mv(M, v)) <= 2 * RTOL_FRO
    got = T.Tensor.from_numpy(u).matmul(Md, mode=T.vm, track_grad=False).to_numpy()
    assert got.shape == (2, 3, 29) and rel_fro(got, oracle.vm_f64(u, M)) <= RTOL_FRO
    # transposed matrix view (examples/word2vec_cbow.mojo:531-553), strided vector, padded rows
    got = Md.transpose().matmul(T.Tensor.from_numpy(u), mode=T.mv, track_grad=False).to_numpy()
    assert rel_fro(got, oracle.mv_f64(np.swapaxes(M, -1, -2), u)) <= RTOL_FRO
    got = T.Tensor.from_numpy(v[0]).matmul(Md.transpose(), mode=T.vm, track_grad=False).to_numpy()
    assert rel_fro(got, oracle.vm_f64(v[0], np.swapaxes(M, -1, -2))) <= RTOL_FRO
    w2 = rng.standard_normal((58,), dtype=np.float32)
    got = Md.matmul(as_strided_tensor(T, w2[::2]), mode=T.mv, track_grad=False).to_numpy()
    assert rel_fro(got, oracle.mv_f64(M, w2[::2])) <= RTOL_FRO
    P = rng.standard_normal((45, 64), dtype=np.float32)
    got = as_strided_tensor(T, P[:, 3:60]).matmul(T.Tensor.from_numpy(rng.standard_normal(57, dtype=np.float32) * 0 + 1), mode=T.mv, track_grad=False).to_numpy()
    assert rel_fro(got, P[:, 3:60].astype(np.float64).sum(1)) <= RTOL_FRO
    G = rng.standard_normal((30, 40, 2), dtype=np.float32)[:, :, 0]  # both strides non-unit
    x = rng.standard_normal(40, dtype=np.float32)
    assert rel_fro(as_strided_tensor(T, G).matmul(T.Tensor.from_numpy(x), mode=T.mv, track_grad=False).to_numpy(), oracle.mv_f64(G, x)) <= RTOL_FRO
    y = rng.standard_normal(30, dtype=np.float32)
    assert rel_fro(T.Tensor.from_numpy(y).matmul(as_strided_tensor(T, G), mode=T.vm, track_grad=False).to_numpy(), oracle.vm_f64(y, G)) <= RTOL_FRO
    # sizes that exercise the vector main loops, tails and k splitting
    for m, k in [(1, 1), (5, 3), (300, 1025), (1000, 4100), (7, 9001), (2049, 515)]:
        W = rng.standard_normal((m, k), dtype=np.float32)
        x = rng.standard_normal(k, dtype=np.float32)
        y = rng.standard_normal(m, dtype=np.float32)
        Wd = T.Tensor.from_numpy(W)
        assert rel_fro(Wd.matmul(T.Tensor.from_numpy(x), mode=T.mv, track_grad=False).to_numpy(), oracle.mv_f64(W, x)) <= RTOL_FRO, (m, k)
        assert rel_fro(T.Tensor.from_numpy(y).matmul(Wd, mode=T.vm, track_grad=False).to_numpy(), oracle.vm_f64(y, W)) <= RTOL_FRO, (m, k)


def test_mv_vm_backward_against_oracle(T, oracle):
    rng = np.random.default_rng(43)
    # (a vector shared by every batch of stacked matrices: its gradient is one product with the batch folded into the reduction)
    for ms, vs in [((6, 5), (5,)), ((3, 6, 5), (5,)), ((6, 5), (4, 5)), ((2, 3, 6, 5), (3, 5)), ((1, 6, 5), (4, 5)), ((4, 70, 33), (33,)),
                   ((2, 3, 40, 1030), (1030,))]:
        Mn = rng.standard_normal(ms, dtype=np.float32)
        vn = rng.standard_normal(vs, dtype=np.float32)
        Mt, vt = T.Tensor.from_numpy(Mn, True), T.Tensor.from_numpy(vn, True)
        out = Mt.matmul(vt, mode=T.mv)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed))
        dM, dv = oracle.mv_backward(Mn, vn, seed)
        assert rel_fro(Mt.grad(), dM) <= 2 * RTOL_FRO and rel_fro(vt.grad(), dv) <= 2 * RTOL_FRO, (ms, vs)
    for vs, ms in [((6,), (6, 5)), ((6,), (3, 6, 5)), ((4, 6), (6, 5)), ((3, 6), (2, 3, 6, 5))]:
        Mn = rng.standard_normal(ms, dtype=np.float32)
        vn = rng.standard_normal(vs, dtype=np.float32)
        Mt, vt = T.Tensor.from_numpy(Mn, True), T.Tensor.from_numpy(vn, True)
        out = vt.matmul(Mt, mode=T.vm)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed))
        dv, dM = oracle.vm_backward(vn, Mn, seed)
        assert rel_fro(Mt.grad(), dM) <= 2 * RTOL_FRO and rel_fro(vt.grad(), dv) <= 2 * RTOL_FRO, (vs, ms)


def test_dot(T, oracle):
    rng = np.random.default_rng(47)
    for n in (1, 7, 1000, 300001):
        a = rng.standard_normal(n, dtype=np.float32)
        b = rng.standard_normal(n, dtype=np.float32)
        got = float(T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False).to_numpy())
        ref = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
        assert abs(got - ref) <= 1e-5 * max(1.0, np.linalg.norm(a) * np.linalg.norm(b)), n
    # the streaming form (unit strides, 16-byte loads): every alignment of the two vectors, lengths with a remainder, strides
    import torch
    L = T.lib.load()
    big_a, big_b = rng.standard_normal(2_100_000, dtype=np.float32), rng.standard_normal(2_100_000, dtype=np.float32)
    Ad, Bd, out = torch.from_numpy(big_a).cuda(), torch.from_numpy(big_b).cuda(), torch.zeros(1, device="cuda")
    for (ao, bo, n, sa, sb) in [(0, 0, 2_097_152, 1, 1), (1, 0, 2_000_003, 1, 1), (2, 3, 1_999_998, 1, 1), (3, 1, 4097, 1, 1), (0, 0, 4096, 1, 1),
                                (5, 7, 500_001, 2, 1), (0, 1, 300_000, 3, 2)]:
        T.lib.check(L.tenmo_hip_dot_f32(Ad.data_ptr(), ao, sa, Bd.data_ptr(), bo, sb, n, out.data_ptr(), 1))
        av, bv = big_a[ao:ao + n * sa:sa].astype(np.float64), big_b[bo:bo + n * sb:sb].astype(np.float64)
        assert abs(float(out) - float(av @ bv)) <= 1e-5 * np.linalg.norm(av) * np.linalg.norm(bv), (ao, bo, n, sa, sb)
    a = np.arange(1, 8, dtype=np.float32)
    A, B = T.Tensor.from_numpy(a, True), T.Tensor.from_numpy(2 * a, True)
    out = A.dot(B)
    assert float(out.to_numpy()) == 280.0
    out.backward(3.0)
    np.testing.assert_allclose(A.grad(), 6 * a)
    np.testing.assert_allclose(B.grad(), 3 * a)
    assert float(T.Tensor.d([2.0]).matmul(T.Tensor.from_numpy(a), track_grad=False).to_numpy()) == 56.0


# ---- the reference's CBLAS plugin point ---------------------------------------------------------------

def test_cblas_sgemm(T, golden):
    from tenmo_amd.blashandle import BLASHandle

    h = BLASHandle()
    assert h.is_initialized()
    for c in golden["blas"]:
        if "A_ones" in c:
            A, B = np.ones(c["A_ones"], np.float32), np.ones(c["B_ones"], np.float32)
        else:
            A, B = np.asarray(c["A"], np.float32), np.asarray(c["B"], np.float32)
        tA, tB = c["tA"], c["tB"]
        opA, opB = (A.T if tA else A), (B.T if tB else B)
        out = h.matmul(A, B, tA, tB)
        if "expect" in c:
            np.testing.assert_allclose(out, c["expect"], rtol=1e-5)
        if "expect_00" in c:
            assert abs(out[0, 0] - c["expect_00"]) < 1e-5
        if "expect_value" in c:
            assert out.shape == (opA.shape[0], opB.shape[1]) and np.all(out == c["expect_value"])
        if "grad_A" in c or c.get("equals_native"):
            gA, gB = h.matmul_backward(A, B, np.ones((opA.shape[0], opB.shape[1]), np.float32), tA, tB)
        if "grad_A" in c:
            np.testing.assert_allclose(gA, c["grad_A"])
            np.testing.assert_allclose(gB, c["grad_B"])
        if c.get("equals_native"):  # the reference's BLAS-against-native tests: the plugin entry and the device path on transposed views agree
            At, Bt = T.Tensor.from_numpy(A, True), T.Tensor.from_numpy(B, True)
            Av, Bv = (At.transpose() if tA else At), (Bt.transpose() if tB else Bt)
            nat = Av.matmul(Bv)
            np.testing.assert_array_equal(out, nat.to_numpy())
            nat.backward(1.0)
            np.testing.assert_array_equal(gA, Av.grad().T if tA else Av.grad())   # (the gradient of a transposed view has the view's shape)
            np.testing.assert_array_equal(gB, Bv.grad().T if tB else Bv.grad())
    rs = np.random.default_rng(59)
    for m, k, n in golden["blas_shapes"]["cases"]:
        A, B = rs.standard_normal((m, k), dtype=np.float32), rs.standard_normal((k, n), dtype=np.float32)
        out = h.matmul(A, B)
        nat = T.Tensor.from_numpy(A).matmul(T.Tensor.from_numpy(B), track_grad=False).to_numpy()
        assert rel_fro(out, ref_matmul64(A, B)) <= RTOL_FRO and rel_fro(out, nat) <= RTOL_FRO, (m, k, n)
    assert np.all(h.matmul(np.ones((100, 100), np.float32), np.ones((100, 100), np.float32)) == 100.0)  # tests/test_blas.mojo:216-232
    # four-case backward algebra (tenmo/blashandle.mojo:51-99) against explicit transposes
    rng = np.random.default_rng(53)
    for tA in (False, True):
        for tB in (False, True):
            A = rng.standard_normal((9, 6) if tA else (6, 9), dtype=np.float32)
            B = rng.standard_normal((5, 9) if tB else (9, 5), dtype=np.float32)
            opA, opB = (A.T if tA else A), (B.T if tB else B)
            assert rel_fro(h.matmul(A, B, tA, tB), ref_matmul64(opA, opB)) <= RTOL_FRO
            g = rng.standard_normal((6, 5), dtype=np.float32)
            gA, gB = h.matmul_backward(A, B, g, tA, tB)
            rA, rB = ref_matmul64(g, opB.T), ref_matmul64(opA.T, g)
            assert rel_fro(gA, rA.T if tA else rA) <= RTOL_FRO and rel_fro(gB, rB.T if tB else rB) <= RTOL_FRO
    # raw ABI: column-major, alpha/beta, leading dimensions larger than the extent
    L = T.lib.load()
    A = rng.standard_normal((7, 4), dtype=np.float32)   # column-major 4x7 with lda 4... use explicit ld
    Acm = np.asfortranarray(rng.standard_normal((6, 8), dtype=np.float32))  # M=6, K=8 column-major, lda=6
    Bcm = np.asfortranarray(rng.standard_normal((8, 3), dtype=np.float32))
    Ccm = np.asfortranarray(rng.standard_normal((6, 3), dtype=np.float32))
    want = 0.5 * ref_matmul64(Acm, Bcm) + 2.0 * Ccm
    L.cblas_sgemm(102, 111, 111, 6, 3, 8, 0.5, Acm.ctypes.data, 6, Bcm.ctypes.data, 8, 2.0, Ccm.ctypes.data, 6)
    assert rel_fro(Ccm, want) <= RTOL_FRO
    Ald = np.zeros((6, 11), np.float32)
    Ald[:, :8] = Acm
    out = np.zeros((6, 5), np.float32)
    Brm = np.ascontiguousarray(Bcm)
    L.cblas_sgemm(101, 111, 111, 6, 3, 8, 1.0, Ald.ctypes.data, 11, Brm.ctypes.data, 3, 0.0, out.ctypes.data, 5)
    assert rel_fro(out[:, :3], ref_matmul64(Acm, Bcm)) <= RTOL_FRO and np.all(out[:, 3:] == 0)


# ---- Linear and the MLP training step ---------------------------------------------------------------

def test_linear_layer(T):
    from tenmo_amd.net import Linear

    rng = np.random.default_rng(59)
    lin = Linear(12, 7, rng, init_method="xavier")
    bias = rng.standard_normal(7).astype(np.float32)
    import torch

    lin.bias.buffer.storage.copy_(torch.from_numpy(bias))
    x = rng.standard_normal((5, 12), dtype=np.float32)
    X = T.Tensor.from_numpy(x, True)
    y = lin(X)
    W = lin.weight.to_numpy()
    assert rel_fro(y.to_numpy(), ref_matmul64(x, W) + bias) <= RTOL_FRO
    seed = rng.standard_normal((5, 7), dtype=np.float32)
    y.backward(T.Tensor.from_numpy(seed))
    assert rel_fro(lin.weight.grad(), ref_matmul64(x.T, seed)) <= RTOL_FRO
    assert rel_fro(lin.bias.grad(), seed.astype(np.float64).sum(0)) <= RTOL_FRO
    assert rel_fro(X.grad(), ref_matmul64(seed, W.T)) <= RTOL_FRO
    with pytest.raises(T.lib.TenmoHipError, match="input dim mismatch"):
        lin(T.Tensor.zeros(5, 13))


def test_sgd_vectors(T, golden):
    from tenmo_amd.net import SGD

    for key in ("sgd_single_step", "sgd_three_steps", "sgd_2d"):
        s = golden["harness"][key]
        w = T.Tensor.from_numpy(np.asarray(s["w"], np.float32), True)
        opt = SGD([w], lr=s["lr"])
        for _ in range(s["steps"]):
            w.seed_grad(T.Tensor.from_numpy(np.asarray(s["grad"], np.float32)))
            opt.step()
        np.testing.assert_allclose(w.to_numpy(), s["expect"], rtol=1e-6)


def test_mlp_loss_curve_tracks_cpu(T, oracle):
    """MNIST-shaped MLP 784->128->32->10, batch 64, Xavier, SGD lr=0.01: the per-step loss of the
    GPU run stays within 1e-4 of the CPU restatement for every step."""
    from tenmo_amd import rng as R
    from tenmo_amd.net import MLP

    _mlp_loss_curve(T, oracle, R, MLP)


def _mlp_loss_curve(T, oracle, R, MLP):
    dims, seed, lr = [784, 128, 32, 10], 2024, 0.01
    Ws, bs = R.xavier_mlp(dims, seed)
    gpu, cpu = MLP(dims, Ws, bs, 64), oracle.MLP(dims, Ws, bs, 64)
    worst = 0.0
    for step in range(40):
        x, y = R.mnist_like_batch(64, seed, step)
        lg, lc = gpu.step(x, y, lr), cpu.step(x, y, lr)
        worst = max(worst, abs(lg - lc))
        assert abs(lg - lc) <= 1e-4, (step, lg, lc)
    for l in range(3):
        (Wg, bg), (Wc, bc) = gpu.params(l), cpu.params(l)
        assert rel_fro(Wg, Wc) <= 1e-5 and np.abs(bg - bc).max() <= 1e-5
        (dWg, dbg), (dWc, dbc) = gpu.grads(l), cpu.grads(l)
        assert rel_fro(dWg, dWc) <= 1e-4 and rel_fro(dbg, dbc) <= 1e-4
    x, _ = R.mnist_like_batch(64, seed, 99)
    assert rel_fro(gpu.forward(x), cpu.forward(x)) <= 1e-5
    # a batch larger than one workgroup takes the separate loss-mean / bias-gradient launches
    dims = [40, 24, 5]
    Ws, bs = R.xavier_mlp(dims, seed + 1)
    gpu, cpu = MLP(dims, Ws, bs, 300), oracle.MLP(dims, Ws, bs, 300)
    rs = np.random.default_rng(5)
    for step in range(5):
        x = rs.standard_normal((300, 40)).astype(np.float32)
        y = rs.integers(0, 5, 300).astype(np.int32)
        assert abs(gpu.step(x, y, 0.05) - cpu.step(x, y, 0.05)) <= 1e-4, step
    for l in range(2):
        (dWg, dbg), (dWc, dbc) = gpu.grads(l), cpu.grads(l)
        assert rel_fro(dWg, dWc) <= 1e-4 and rel_fro(dbg, dbc) <= 1e-4
    # batches up to 128 rows: the hidden layers' bias gradients come out of the store of the GEMM that produces their
    # gradient (ragged widths, 65..128 rows take the 128-row tile)
    for batch, dims in ((100, [50, 70, 33, 6]), (128, [20, 200, 64, 130, 4]), (7, [9, 5, 3])):
        Ws, bs = R.xavier_mlp(dims, seed + 2)
        gpu, cpu = MLP(dims, Ws, bs, batch), oracle.MLP(dims, Ws, bs, batch)
        for step in range(4):
            x = rs.standard_normal((batch, dims[0])).astype(np.float32)
            y = rs.integers(0, dims[-1], batch).astype(np.int32)
            assert abs(gpu.step(x, y, 0.05) - cpu.step(x, y, 0.05)) <= 1e-4, (batch, step)
        for l in range(len(dims) - 1):
            (dWg, dbg), (dWc, dbc) = gpu.grads(l), cpu.grads(l)
            assert rel_fro(dWg, dWc) <= 1e-4 and rel_fro(dbg, dbc) <= 1e-4, (batch, l)
    # cross-entropy vector of the reference: uniform logits -> -log(1/3)
    m = MLP([2, 3], [np.zeros((2, 3), np.float32)], [np.ones(3, np.float32)], 2)
    assert abs(m.step(np.ones((2, 2), np.float32), np.asarray([0, 1], np.int32), 0.0) - 1.0986122886681098) < 1e-6


def test_mlp_graph_replay_matches_eager(T, oracle):
    """The captured step replayed many times, with eager library work and synchronisations between
    replays, gives the same losses and parameters as the eager step (and so as the CPU run)."""
    from tenmo_amd import rng as R
    from tenmo_amd.net import MLP

    dims, seed, lr = [784, 128, 32, 10], 77, 0.01
    Ws, bs = R.xavier_mlp(dims, seed)
    eager, graph, cpu = MLP(dims, Ws, bs, 64), MLP(dims, Ws, bs, 64), oracle.MLP(dims, Ws, bs, 64)
    side_a = T.Tensor.from_numpy(np.ones((70, 33), np.float32))
    side_b = T.Tensor.from_numpy(np.ones((33, 20), np.float32))
    for step in range(12):
        x, y = R.mnist_like_batch(64, seed, step)
        le = eager.step(x, y, lr)
        lg = graph.step(x, y, lr, graph=True)
        lc = cpu.step(x, y, lr)
        assert le == lg, (step, le, lg)          # same kernels, same order: bit-identical
        assert abs(lg - lc) <= 1e-4
        # unrelated eager work on the same stream between replays
        assert np.all(side_a.matmul(side_b, track_grad=False).to_numpy() == 33.0)
    for l in range(3):
        (We, be), (Wg, bg) = eager.params(l), graph.params(l)
        np.testing.assert_array_equal(We, Wg)
        np.testing.assert_array_equal(be, bg)
    # a different learning rate re-captures
    x, y = R.mnist_like_batch(64, seed, 99)
    assert eager.step(x, y, 0.05) == graph.step(x, y, 0.05, graph=True)
    np.testing.assert_array_equal(eager.params(0)[0], graph.params(0)[0])


@pytest.mark.gpu
def test_cross_entropy_entries(T, oracle):
    """tenmo_hip_cross_entropy_forward_f32 / _backward_f32 against the CPU restatement: thread-per-row,
    register-resident and streaming (row statistics + flat softmax sweep, wavefront or workgroup per row)
    forward kernels, aligned and unaligned rows, int64 and int32 targets, ignore_index, label smoothing,
    the three reductions, accumulate."""
    import ctypes as C
    import torch

    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(43)
    for M, Cn, ls, is64 in [(2, 3, 0.0, True), (64, 10, 0.0, False), (33, 17, 0.2, True), (5, 1000, 0.05, True),
                            (7, 1001, 0.1, False), (300, 64, 0.0, True), (3, 50257, 0.1, True), (2100, 8009, 0.1, True),
                            (37, 9001, 0.05, False), (130, 40003, 0.0, True), (3, 70001, 0.1, True)]:
        x = (3 * rng.standard_normal((M, Cn))).astype(np.float32)
        t = rng.integers(0, Cn, M)
        t[rng.random(M) < 0.3] = -100
        sm_ref, rows_ref, total_ref, valid_ref = oracle.cross_entropy_forward(x, t, label_smoothing=ls)
        X = torch.from_numpy(x).cuda()
        Tg = torch.from_numpy(t.astype(np.int64 if is64 else np.int32)).cuda()
        sm = torch.empty((M, Cn), dtype=torch.float32, device="cuda")
        rows = torch.empty(M, dtype=torch.float32, device="cuda")
        total = torch.zeros(1, dtype=torch.float32, device="cuda")
        valid = torch.zeros(1, dtype=torch.int32, device="cuda")
        lib.check(L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, M, Cn, -100, ls,
                                                        sm.data_ptr(), rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1))
        case = (M, Cn, ls, is64)
        assert int(valid.item()) == valid_ref, case
        # against fp64 at the stated tolerance; against the CPU restatement a little looser for long
        # rows, whose sum of exponentials the restatement adds serially in fp32 (as the reference does)
        p64, loss64, _ = ce_reference64(x, t, -100, ls)
        assert np.allclose(sm.cpu().numpy(), p64, rtol=1e-5, atol=1e-7), case
        assert np.allclose(rows.cpu().numpy(), loss64, rtol=1e-5, atol=1e-5), case
        assert np.allclose(sm.cpu().numpy(), sm_ref, rtol=2e-4, atol=1e-7), case
        loose = 1e-5 if Cn <= 60000 else 5e-5  # the restatement's serial fp32 sums over 70001 classes are off by 1e-5 themselves
        assert np.allclose(rows.cpu().numpy(), rows_ref, rtol=loose, atol=1e-5), case
        assert abs(float(total.item()) - total_ref) <= loose * max(1.0, abs(total_ref)), case
        assert abs(float(total.item()) - float(np.sum(loss64))) <= 1e-5 * max(1.0, abs(float(np.sum(loss64)))), case
        # a softmax buffer that is not congruent with the logits modulo 16 bytes takes the element-wise path
        sm_odd = torch.empty(M * Cn + 1, dtype=torch.float32, device="cuda")
        lib.check(L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, M, Cn, -100, ls,
                                                        sm_odd.data_ptr() + 4, rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1))
        assert np.allclose(sm_odd[1:].cpu().numpy().reshape(M, Cn), p64, rtol=1e-5, atol=1e-7), case
        g_odd = torch.empty(M * Cn + 1, dtype=torch.float32, device="cuda")
        one = torch.ones(1, dtype=torch.float32, device="cuda")
        lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, one.data_ptr(), M, Cn, -100, ls,
                                                         1, valid_ref, g_odd.data_ptr() + 4, 0, 1))
        ref_odd = oracle.cross_entropy_backward(sm.cpu().numpy(), t, np.ones(1, np.float32), 1, valid_ref, label_smoothing=ls)
        assert np.allclose(g_odd[1:].cpu().numpy().reshape(M, Cn), ref_odd, rtol=1e-5, atol=1e-7), case
        # without a softmax buffer the losses are the same
        rows2 = torch.empty_like(rows)
        lib.check(L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, M, Cn, -100, ls,
                                                        None, rows2.data_ptr(), total.data_ptr(), valid.data_ptr(), 1))
        assert torch.allclose(rows, rows2, rtol=1e-6, atol=1e-6), case
        up = rng.standard_normal(M).astype(np.float32)
        Up = torch.from_numpy(up).cuda()
        grad = torch.empty((M, Cn), dtype=torch.float32, device="cuda")
        for red in (oracle.REDUCTION_NONE, oracle.REDUCTION_SUM, oracle.REDUCTION_MEAN):
            ref = oracle.cross_entropy_backward(sm.cpu().numpy(), t, up if red == 0 else up[:1], red, valid_ref, label_smoothing=ls)
            lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, Up.data_ptr(), M, Cn, -100, ls,
                                                             red, valid_ref, grad.data_ptr(), 0, 1))
            assert np.allclose(grad.cpu().numpy(), ref, rtol=1e-5, atol=1e-7), (case, red)
        lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), Tg.data_ptr(), 1 if is64 else 0, Up.data_ptr(), M, Cn, -100, ls,
                                                         2, valid_ref, grad.data_ptr(), 1, 1))
        assert np.allclose(grad.cpu().numpy(), 2 * ref, rtol=1e-5, atol=1e-7), (case, "accumulate")
    # argument checks
    assert L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1, 3, 0, -100, 0.0, None, rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1) == -2
    assert L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1, 3, 4, -100, 1.5, None, rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1) == -3
    assert b"label_smoothing" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_cross_entropy_forward_f32(None, Tg.data_ptr(), 1, 3, 4, -100, 0.0, None, rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1) == -3
    assert L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), Tg.data_ptr(), 1, Up.data_ptr(), 3, 4, -100, 0.0, 3, 1, grad.data_ptr(), 0, 1) == -3
    # no rows: sum 0, nothing valid
    lib.check(L.tenmo_hip_cross_entropy_forward_f32(None, None, 1, 0, 4, -100, 0.0, None, None, total.data_ptr(), valid.data_ptr(), 1))
    assert float(total.item()) == 0.0 and int(valid.item()) == 0


@pytest.mark.gpu
def test_sgd_entry(T, golden, oracle):
    import torch

    L, lib = T.lib.load(), T.lib
    H = golden["harness"]
    g = H["sgd_momentum_three_steps"]
    w = torch.tensor(g["w"], dtype=torch.float32, device="cuda")
    v = torch.zeros(1, dtype=torch.float32, device="cuda")
    gr = torch.tensor(g["grad"], dtype=torch.float32, device="cuda")
    for want in g["expect_after_each"]:
        lib.check(L.tenmo_hip_sgd_step_f32(w.data_ptr(), gr.data_ptr(), v.data_ptr(), 1, g["lr"], g["momentum"], 0.0, 1))
        assert abs(float(w.item()) - want) < 1e-6
    g = H["sgd_weight_decay"]
    w = torch.tensor(g["w"], dtype=torch.float32, device="cuda")
    gr = torch.tensor(g["grad"], dtype=torch.float32, device="cuda")
    lib.check(L.tenmo_hip_sgd_step_f32(w.data_ptr(), gr.data_ptr(), None, 3, g["lr"], 0.0, g["weight_decay"], 1))
    assert np.allclose(w.cpu().numpy(), g["expect"], rtol=1e-6)
    # a large tensor, both forms, against the CPU restatement
    rng = np.random.default_rng(47)
    n = 1_000_003
    p0, gr0, v0 = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    for vel, mom, wd in [(False, 0.0, 0.0), (False, 0.0, 0.01), (True, 0.9, 0.0), (True, 0.9, 0.01)]:
        p_ref, v_ref = p0.copy(), v0.copy()
        oracle.sgd_step(p_ref, gr0, v_ref if vel else None, 0.05, mom, wd)
        P, G, V = torch.from_numpy(p0.copy()).cuda(), torch.from_numpy(gr0).cuda(), torch.from_numpy(v0.copy()).cuda()
        lib.check(L.tenmo_hip_sgd_step_f32(P.data_ptr(), G.data_ptr(), V.data_ptr() if vel else None, n, 0.05, mom, wd, 1))
        # one rounding of difference per product (fused multiply-add on the GPU): absolute, since sums cancel
        assert np.allclose(P.cpu().numpy(), p_ref, rtol=1e-6, atol=1e-6), (vel, mom, wd)
        if vel:
            assert np.allclose(V.cpu().numpy(), v_ref, rtol=1e-6, atol=1e-6)
    assert L.tenmo_hip_sgd_step_f32(None, G.data_ptr(), None, 4, 0.1, 0.0, 0.0, 1) == -3
    assert L.tenmo_hip_sgd_step_f32(None, None, None, 0, 0.1, 0.0, 0.0, 1) == 0


def test_conv2d_forward(T, golden, oracle):
    """Conv2dFused.forward through tenmo_hip_conv2d_forward_f32 (implicit GEMM): every forward case of
    tests/test_cnn.mojo, then random shapes against the CPU restatement and an fp64 reference at the
    matmul tolerance — channel counts either side of the 64-row tile, K = C_in*KH*KW not a multiple of 4
    or 16, stride / dilation / padding of every kind, and the layer sizes of examples/mnist_conv."""
    import ctypes as C
    import torch
    from helpers import check_conv_case, conv_case_tensors, conv_reference64
    from tenmo_amd.cnn import Conv2dFused

    for case in golden["conv"]["cases"]:
        image, kernel, bias, kw = conv_case_tensors(case)
        out = Conv2dFused.forward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel),
                                  T.Tensor.from_numpy(bias) if bias is not None else None, **kw).to_numpy()
        check_conv_case(case, out)
    rng = np.random.default_rng(73)
    for (n, ci, h, w, co, kh, kww, stride, dil, padding, with_bias) in [
            (2, 3, 9, 11, 4, 3, 3, 1, 1, "valid", True), (1, 2, 8, 8, 3, 3, 2, 2, 1, "same", False),
            (3, 1, 12, 7, 2, 2, 3, 1, 2, 1, True), (2, 4, 10, 10, 5, 3, 3, 2, 2, (2, 1), True),
            (1, 3, 7, 9, 2, 1, 1, 1, 1, "valid", False), (2, 2, 6, 6, 3, 3, 3, 3, 1, [(1, 2), (0, 3)], True),
            (64, 1, 28, 28, 16, 3, 3, 1, 1, "same", True), (16, 16, 14, 14, 32, 3, 3, 1, 1, "same", True),
            (4, 3, 32, 32, 64, 5, 5, 1, 1, 2, True), (2, 64, 16, 16, 130, 3, 3, 2, 1, 1, True),
            (1, 8, 40, 56, 96, 3, 3, 1, 2, "valid", False), (0, 3, 8, 8, 4, 3, 3, 1, 1, "valid", True)]:
        image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
        kernel = rng.standard_normal((co, ci, kh, kww), dtype=np.float32)
        bias = rng.standard_normal(co, dtype=np.float32) if with_bias else None
        case = (n, ci, h, w, co, kh, kww, stride, dil, padding, with_bias)
        got = Conv2dFused.forward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel),
                                  T.Tensor.from_numpy(bias) if bias is not None else None, stride=stride, dilation=dil, padding=padding).to_numpy()
        want = oracle.conv2d_forward(image, kernel, bias, stride=stride, dilation=dil, padding=padding)
        assert got.shape == want.shape, case
        if n == 0:
            continue
        ref = conv_reference64(image, kernel, bias, stride, dil, oracle.conv_padding(h, w, kh, kww, stride, dil, padding))
        assert rel_fro(got, ref) <= RTOL_FRO, case
        assert rel_fro(got, want) <= 2 * RTOL_FRO, case
    # errors: the reference panics with these messages (cnn.mojo:167-176, :237-241, :132-137)
    one = T.Tensor.ones(1, 1, 2, 2)
    with pytest.raises(T.lib.TenmoHipError, match="4D"):
        Conv2dFused.forward(T.Tensor.ones(1, 2, 2), one)
    with pytest.raises(T.lib.TenmoHipError, match="input channels"):
        Conv2dFused.forward(T.Tensor.ones(1, 2, 4, 4), one)
    with pytest.raises(T.lib.TenmoHipError, match="non-positive output"):
        Conv2dFused.forward(one, T.Tensor.ones(1, 1, 3, 3))
    with pytest.raises(T.lib.TenmoHipError, match="bias"):
        Conv2dFused.forward(T.Tensor.ones(1, 1, 4, 4), one, bias=T.Tensor.ones(2))
    L = T.lib.load()
    x = torch.ones(16, device="cuda")
    assert L.tenmo_hip_conv2d_forward_f32(x.data_ptr(), 1, 1, 2, 2, x.data_ptr(), 1, 3, 3, None, 1, 1, x.data_ptr(), 1) == -2
    assert b"Invalid output dimensions" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_conv2d_forward_f32(x.data_ptr(), 1, 1, 4, 4, x.data_ptr(), 1, 2, 2, None, 0, 1, x.data_ptr(), 1) == -3
    assert L.tenmo_hip_conv2d_forward_f32(None, 1, 1, 4, 4, x.data_ptr(), 1, 2, 2, None, 1, 1, x.data_ptr(), 1) == -3


def _random_matrix_view(rng, rows, cols, layout, pad):
    """A rows x cols matrix inside a larger storage: row-major, column-major (a transposed view) or both
    strides > 1, with a padded pitch and a small offset.  Returns (device storage, offset, rs, cs, numpy copy)."""
    import torch
    off = int(rng.integers(0, 5))
    if layout == "row":
        rs, cs = cols + pad, 1
        n = off + rows * rs + 8
    elif layout == "col":
        rs, cs = 1, rows + pad
        n = off + cols * cs + 8
    else:
        cs = int(rng.integers(2, 4))
        rs = cols * cs + pad
        n = off + rows * rs + 8
    st = rng.standard_normal(n).astype(np.float32)
    a = np.lib.stride_tricks.as_strided(st[off:], (rows, cols), (4 * rs, 4 * cs)).copy()
    return torch.from_numpy(st).cuda(), off, rs, cs, a


def test_randomized_gemm_views(T):
    """Seeded sweep of tenmo_hip_gemm_f32: random shapes (ragged against every tile), operand layouts, padded
    pitches, offsets, accumulate, and forced tile / split-K / stream-K choices, against fp64."""
    import torch
    L = T.lib.load()
    rng = np.random.default_rng(101)
    try:
        for case in range(160):
            big = rng.random() < 0.25
            M, N, K = (int(rng.integers(1, 700 if big else 200)), int(rng.integers(1, 700 if big else 200)), int(rng.integers(1, 900 if big else 150)))
            if rng.random() < 0.15:
                K, M, N = int(rng.integers(1000, 5000)), int(rng.integers(1, 130)), int(rng.integers(1, 130))
            la, lb = rng.choice(["row", "col", "gen"], p=[0.45, 0.4, 0.15]), rng.choice(["row", "col", "gen"], p=[0.45, 0.4, 0.15])
            pa, pb = int(rng.choice([0, 0, 1, 3, 4, 8])), int(rng.choice([0, 0, 1, 3, 4, 8]))
            tile, sk, stk = int(rng.choice([-1, -1, 0, 1, 2, 3, 4])), int(rng.choice([-1, -1, -1, 1, 2, 3])), int(rng.choice([-1, -1, -1, 0, 1, 2]))
            acc = int(rng.random() < 0.3)
            A, ao, ars, acs, a = _random_matrix_view(rng, M, K, la, pa)
            B, bo, brs, bcs, b = _random_matrix_view(rng, K, N, lb, pb)
            c0 = rng.standard_normal((M, N)).astype(np.float32)
            Cd = torch.from_numpy(c0.copy()).cuda()
            L.tenmo_hip_set_tuning(b"gemm_tile", tile)
            L.tenmo_hip_set_tuning(b"gemm_splitk", sk)
            L.tenmo_hip_set_tuning(b"gemm_streamk", stk)
            desc = (case, M, N, K, str(la), str(lb), pa, pb, ao, bo, tile, sk, stk, acc)
            T.lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), ao, ars, acs, B.data_ptr(), bo, brs, bcs, Cd.data_ptr(), M, N, K, 0, None, None, None, acc, 1))
            ref = a.astype(np.float64) @ b.astype(np.float64) + (c0 if acc else 0)
            assert rel_fro(Cd.cpu().numpy(), ref) <= RTOL_FRO, desc
    finally:
        for knob in (b"gemm_tile", b"gemm_splitk", b"gemm_streamk"):
            L.tenmo_hip_set_tuning(knob, -1)


def test_randomized_mv_vm_skinny_views(T):
    """Seeded sweep of the view-level mv / vm / skinny / broadcast-batched entries: random sizes, transposed
    storage, padded pitches, offsets and batch shapes, against fp64; the element after the result must stay
    untouched."""
    import ctypes as C
    import torch
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(103)

    def mk(shape, transpose_last=False, pad=0, off=0):
        shape = tuple(shape)
        sshape = shape[:-2] + (shape[-1], shape[-2]) if transpose_last and len(shape) >= 2 else shape
        pshape = sshape[:-1] + (sshape[-1] + pad,)
        st = rng.standard_normal(int(np.prod(pshape)) + off + 4).astype(np.float32)
        strides = [1]
        for d in reversed(pshape[1:]):
            strides.insert(0, strides[0] * d)
        arr = np.lib.stride_tricks.as_strided(st[off:], sshape, tuple(4 * x for x in strides))
        vshape, vstr = list(sshape), list(strides)
        if transpose_last and len(shape) >= 2:
            vstr[-1], vstr[-2] = vstr[-2], vstr[-1]
            vshape[-1], vshape[-2] = vshape[-2], vshape[-1]
            arr = np.swapaxes(arr, -1, -2)
        dev = torch.from_numpy(st).cuda()
        return dev, lib.make_view(dev.data_ptr(), off, vshape, vstr), arr.copy()

    for case in range(40 if os.environ.get("TENMO_TEST_SMALL") == "1" else 120):  # (fewer where the library is the CPU replay)
        kind = str(rng.choice(["mv", "vm", "skinny", "bmm"]))
        pad, off, tr = int(rng.choice([0, 0, 1, 2, 3, 4])), int(rng.choice([0, 0, 1, 2, 4])), bool(rng.random() < 0.4)
        bshape = tuple(int(rng.integers(1, 4)) for _ in range(int(rng.choice([0, 0, 1, 2]))))
        if kind == "mv":
            R, K = int(rng.integers(1, 3000)), int(rng.integers(1, 5000))
            if rng.random() < 0.2:
                R, K = int(rng.integers(1, 40)), int(rng.integers(5000, 70000))
            d1, v1, a = mk(bshape + (R, K), tr, pad, off)
            d2, v2, b = mk((K,), False, 0, int(rng.choice([0, 1])))
            ref, fn = np.einsum("...rk,k->...r", a.astype(np.float64), b.astype(np.float64)), L.tenmo_hip_matrix_vector_nd
        elif kind == "vm":
            K, N = int(rng.integers(1, 3000)), int(rng.integers(1, 6000))
            d1, v1, a = mk((K,), False, 0, int(rng.choice([0, 1])))
            d2, v2, b = mk(bshape + (K, N), tr, pad, off)
            ref, fn = np.einsum("k,...kn->...n", a.astype(np.float64), b.astype(np.float64)), L.tenmo_hip_vector_matmul_nd
        elif kind == "skinny":
            M, K, N = int(rng.integers(1, 9)), int(rng.integers(1, 1500)), int(rng.integers(2048, 9000))
            d1, v1, a = mk((M, K), bool(rng.random() < 0.3), 0, 0)
            d2, v2, b = mk(bshape + (K, N), False, pad, off)
            ref, fn = a.astype(np.float64) @ b.astype(np.float64), L.tenmo_hip_matmul_nd
        else:
            M, K, N = int(rng.integers(1, 150)), int(rng.integers(1, 200)), int(rng.integers(1, 150))
            ba = tuple(1 if rng.random() < 0.3 else x for x in bshape)
            d1, v1, a = mk(ba + (M, K), bool(rng.random() < 0.4), pad, off)
            d2, v2, b = mk(bshape + (K, N), tr, 0, 0)
            ref, fn = a.astype(np.float64) @ b.astype(np.float64), L.tenmo_hip_matmul_nd
        out = torch.full((int(np.prod(ref.shape)) + 1,), 7.0, device="cuda")
        desc = (case, kind, a.shape, b.shape, tr, pad, off)
        lib.check(fn(C.byref(v1), C.byref(v2), out.data_ptr(), 1))
        assert rel_fro(out[:-1].cpu().numpy().reshape(ref.shape), ref) <= RTOL_FRO, desc
        assert float(out[-1]) == 7.0, desc


def test_blocked_tile_order(T):
    """The 256x128 tile's one-workgroup-per-tile launch walks tile grids that divide into 2x32 / 4x16 blocks
    per XCD in block order: every tile must still be computed exactly once (shapes whose grids do and do not
    divide, with K slices and batches on top)."""
    import torch
    L = T.lib.load()
    rng = np.random.default_rng(107)
    try:
        L.tenmo_hip_set_tuning(b"gemm_tile", 0)
        L.tenmo_hip_set_tuning(b"gemm_streamk", 0)
        for (M, N, K, sk, nb) in [(512, 32768, 40, 1, 1), (8192, 6144, 24, 1, 1), (1024, 16384, 130, 2, 1), (512, 8192, 33, 1, 4), (768, 32768, 17, 1, 1), (4096, 4096, 16, 1, 1)]:
            L.tenmo_hip_set_tuning(b"gemm_splitk", sk)
            a = rng.standard_normal((nb, M, K), dtype=np.float32)
            b = rng.standard_normal((K, N), dtype=np.float32)
            A, B = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
            Cd = torch.empty((nb, M, N), dtype=torch.float32, device="cuda")
            T.lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, K, 1, B.data_ptr(), 0, N, 1, Cd.data_ptr(), M, N, K,
                                             1, T.lib.i64([nb]), T.lib.i64([M * K]), T.lib.i64([0]), 0, 1))
            ref = a.astype(np.float64) @ b.astype(np.float64)
            assert rel_fro(Cd.cpu().numpy(), ref) <= RTOL_FRO, (M, N, K, sk, nb)
    finally:
        for knob in (b"gemm_tile", b"gemm_splitk", b"gemm_streamk"):
            L.tenmo_hip_set_tuning(knob, -1)


def test_conv2d_stream_k(T, oracle):
    """The convolution's gathered products through the persistent stream-K launch (rounds of whole tiles, then
    tiles shared between workgroups and summed by the fix-up, which also adds the per-channel bias): forward and
    the three gradients of layers with fewer and more tiles than workgroups, both gather tiles."""
    import torch
    from helpers import conv_backward_reference64
    from tenmo_amd.cnn import Conv2dFused
    L = T.lib.load()
    rng = np.random.default_rng(131)
    try:
        for tile in (2, 3):
            L.tenmo_hip_set_tuning(b"gemm_tile", tile)
            L.tenmo_hip_set_tuning(b"gemm_streamk", 4)
            for (n, ci, h, w, co, k, stride) in [(2, 8, 20, 20, 70, 3, 1), (40, 16, 36, 36, 150, 3, 1), (3, 40, 30, 30, 24, 5, 2)]:
                image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
                kernel = rng.standard_normal((co, ci, k, k), dtype=np.float32)
                bias = rng.standard_normal(co, dtype=np.float32)
                case = (tile, n, ci, h, w, co, k, stride)
                got = Conv2dFused.forward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(bias), stride=stride).to_numpy()
                pads = oracle.conv_padding(h, w, k, k, stride, 1, "valid")
                ref = torch.nn.functional.conv2d(torch.from_numpy(image).double(), torch.from_numpy(kernel).double(),
                                                 torch.from_numpy(bias).double(), stride=stride).numpy()
                assert rel_fro(got, ref) <= RTOL_FRO, case
                up = rng.standard_normal(got.shape, dtype=np.float32)
                gi, gk, gb = Conv2dFused.backward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(up), stride=stride)
                ri, rk, rb = conv_backward_reference64(image, kernel, up, stride, 1, pads)
                assert rel_fro(gi.to_numpy(), ri) <= RTOL_FRO, case + ("image",)
                assert rel_fro(gk.to_numpy(), rk) <= RTOL_FRO, case + ("kernel",)
                assert rel_fro(gb.to_numpy(), rb) <= RTOL_FRO, case + ("bias",)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_tile", -1)
        L.tenmo_hip_set_tuning(b"gemm_streamk", -1)


def test_conv2d_strided_image_gradient_by_phase(T, oracle):
    """The image gradient of a strided convolution computed phase by phase (one small stride-1 convolution per
    residue of the input position modulo the stride) against torch autograd in fp64 and the CPU restatement:
    strides 2-4 with dilations 1-3, kernels smaller than the stride (phases no tap reaches), 1x1 kernels, image
    sizes that leave a remainder, accumulate; the same cases through the single-convolution form must agree."""
    from helpers import conv_backward_reference64
    from tenmo_amd.cnn import Conv2dFused
    L = T.lib.load()
    rng = np.random.default_rng(151)
    cases = [(2, 3, 11, 12, 4, 3, 3, 2, 1), (1, 2, 9, 9, 3, 3, 3, 3, 1), (2, 2, 14, 13, 3, 3, 3, 2, 2), (1, 3, 17, 15, 2, 3, 2, 2, 3),
             (2, 1, 12, 12, 2, 2, 2, 4, 1), (1, 2, 10, 10, 2, 1, 1, 2, 1), (3, 4, 16, 16, 5, 5, 5, 3, 2), (2, 70, 19, 19, 66, 3, 3, 2, 1),
             (1, 2, 13, 11, 2, 4, 3, 4, 3), (2, 2, 8, 8, 2, 3, 3, 6, 1)]
    try:
        for (n, ci, h, w, co, kh, kw, stride, dil) in cases:
            image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
            kernel = rng.standard_normal((co, ci, kh, kw), dtype=np.float32)
            ho, wo = (h - (kh + (kh - 1) * (dil - 1))) // stride + 1, (w - (kw + (kw - 1) * (dil - 1))) // stride + 1
            up = rng.standard_normal((n, co, ho, wo), dtype=np.float32)
            ri, rk, rb = conv_backward_reference64(image, kernel, up, stride, dil, (0, 0, 0, 0))
            want = oracle.conv2d_backward(image, kernel, up, stride=stride, dilation=dil, padding="valid")[0]
            got = {}
            for phases in (1, 0):
                L.tenmo_hip_set_tuning(b"conv_phases", phases)
                gi, gk, gb = Conv2dFused.backward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(up), stride=stride, dilation=dil)
                got[phases] = gi.to_numpy()
                case = (phases, n, ci, h, w, co, kh, kw, stride, dil)
                assert rel_fro(got[phases], ri) <= RTOL_FRO, case
                assert rel_fro(got[phases], want) <= 2 * RTOL_FRO, case
                assert rel_fro(gk.to_numpy(), rk) <= RTOL_FRO, case
            assert rel_fro(got[1], got[0]) <= RTOL_FRO
            # accumulate: gradient added onto what the buffer holds
            L.tenmo_hip_set_tuning(b"conv_phases", 1)
            import torch
            X, K, U = (torch.from_numpy(a).cuda() for a in (image, kernel, up))
            G = torch.ones((n, ci, h, w), dtype=torch.float32, device="cuda")
            T.lib.check(L.tenmo_hip_conv2d_backward_f32(X.data_ptr(), n, ci, h, w, K.data_ptr(), co, kh, kw, stride, dil, U.data_ptr(),
                                                        G.data_ptr(), None, None, 1, 1))
            assert rel_fro(G.cpu().numpy(), ri + 1.0) <= RTOL_FRO, ("accumulate",) + case
    finally:
        L.tenmo_hip_set_tuning(b"conv_phases", -1)


def test_conv2d_backward(T, golden, oracle):
    """FusedCol2ImBackward through tenmo_hip_conv2d_backward_f32: the gradients asserted in tests/test_cnn.mojo,
    then random layers against the CPU restatement and torch autograd in fp64 (stride, dilation, all padding
    forms, one and many images, channel counts around the tile sizes), NULL outputs and accumulate."""
    import torch
    from helpers import check_conv_backward_case, conv_backward_reference64, conv_case_tensors
    from tenmo_amd.cnn import Conv2dFused

    def run(image, kernel, up, **kw):
        gi, gk, gb = Conv2dFused.backward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(up), **kw)
        return gi.to_numpy(), gk.to_numpy(), gb.to_numpy()

    for case in golden["conv"]["backward_cases"]:
        image, kernel, _, kw = conv_case_tensors(case)
        up = conv_case_tensors({"image": case["upstream"], "kernel": case["kernel"]})[0]
        check_conv_backward_case(case, *run(image, kernel, up, **kw))
    rng = np.random.default_rng(83)
    for (n, ci, h, w, co, kh, kww, stride, dil, padding) in [
            (2, 3, 9, 11, 4, 3, 3, 1, 1, "valid"), (1, 2, 8, 8, 3, 3, 2, 2, 1, "same"), (3, 1, 12, 7, 2, 2, 3, 1, 2, 1),
            (2, 4, 10, 10, 5, 3, 3, 2, 2, (2, 1)), (1, 3, 7, 9, 2, 1, 1, 1, 1, "valid"), (2, 2, 6, 6, 3, 3, 3, 3, 1, [(1, 2), (0, 3)]),
            (32, 1, 28, 28, 16, 3, 3, 1, 1, "same"), (8, 16, 14, 14, 32, 3, 3, 1, 1, "same"), (2, 70, 12, 12, 130, 3, 3, 2, 1, 1),
            (1, 8, 20, 36, 96, 5, 5, 1, 1, "valid")]:
        image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
        kernel = rng.standard_normal((co, ci, kh, kww), dtype=np.float32)
        out_shape = oracle.conv2d_forward(image, kernel, None, stride=stride, dilation=dil, padding=padding).shape
        up = rng.standard_normal(out_shape, dtype=np.float32)
        case = (n, ci, h, w, co, kh, kww, stride, dil, padding)
        got = run(image, kernel, up, stride=stride, dilation=dil, padding=padding)
        want = oracle.conv2d_backward(image, kernel, up, stride=stride, dilation=dil, padding=padding)
        ref = conv_backward_reference64(image, kernel, up, stride, dil, oracle.conv_padding(h, w, kh, kww, stride, dil, padding))
        for g, o, r, what in zip(got, want, ref, ("image", "kernel", "bias")):
            assert g.shape == r.shape, (what, case)
            assert rel_fro(g, r) <= RTOL_FRO, (what, case)
            assert rel_fro(g, o) <= 3 * RTOL_FRO, (what, case)
    # NULL outputs are skipped; accumulate adds into what is there
    L = T.lib.load()
    n, ci, h, w, co, k = 3, 4, 9, 9, 6, 3
    image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
    kernel = rng.standard_normal((co, ci, k, k), dtype=np.float32)
    up = rng.standard_normal((n, co, h - k + 1, w - k + 1), dtype=np.float32)
    gi_ref, gk_ref, gb_ref = oracle.conv2d_backward(image, kernel, up)
    X, K, U = torch.from_numpy(image).cuda(), torch.from_numpy(kernel).cuda(), torch.from_numpy(up).cuda()
    gk = torch.ones_like(K)
    gb = torch.full((co,), 2.0, device="cuda")
    gi = torch.full_like(X, 3.0)
    T.lib.check(L.tenmo_hip_conv2d_backward_f32(X.data_ptr(), n, ci, h, w, K.data_ptr(), co, k, k, 1, 1, U.data_ptr(), None, gk.data_ptr(), None, 1, 1))
    assert rel_fro(gk.cpu().numpy(), gk_ref + 1.0) <= RTOL_FRO and float(gb[0]) == 2.0 and float(gi.flatten()[0]) == 3.0
    T.lib.check(L.tenmo_hip_conv2d_backward_f32(None, n, ci, h, w, K.data_ptr(), co, k, k, 1, 1, U.data_ptr(), gi.data_ptr(), None, gb.data_ptr(), 1, 1))
    assert rel_fro(gi.cpu().numpy(), gi_ref + 3.0) <= RTOL_FRO and rel_fro(gb.cpu().numpy(), gb_ref + 2.0) <= RTOL_FRO
    assert L.tenmo_hip_conv2d_backward_f32(None, n, ci, h, w, K.data_ptr(), co, k, k, 1, 1, U.data_ptr(), None, gk.data_ptr(), None, 0, 1) == -3
    assert L.tenmo_hip_conv2d_backward_f32(X.data_ptr(), n, ci, h, w, K.data_ptr(), co, k, k, 1, 1, None, None, gk.data_ptr(), None, 0, 1) == -3


def test_products_with_more_than_2_31_elements(T):
    """Results and operands with more than 2^31 elements: element offsets must be 64-bit everywhere.  The
    inputs are small integers, so every product is exact in fp32 and the check is equality: a GEMM whose
    result has 46400^2 elements, a batched one with 40 x 8192^2, mv and vm over a [65536, 40000] matrix."""
    import torch
    L = T.lib.load()
    gen = torch.Generator(device="cuda").manual_seed(5)
    ints = lambda *shape: torch.randint(-3, 4, shape, generator=gen, device="cuda").float()
    K = 16
    M = N = 46400
    A, B = ints(M, K), ints(K, N)
    Cd = torch.empty((M, N), dtype=torch.float32, device="cuda")
    T.lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, K, 1, B.data_ptr(), 0, N, 1, Cd.data_ptr(), M, N, K, 0, None, None, None, 0, 1))
    for r0 in range(0, M, 5800): # reference in slabs of rows: fp32 sums of small integers are exact in any order
        assert torch.equal(Cd[r0:r0 + 5800], A[r0:r0 + 5800] @ B), ("gemm", r0)
    del Cd
    nb, M, N = 40, 8192, 8192
    A, B = ints(nb, M, K), ints(K, N)
    Cd = torch.empty((nb, M, N), dtype=torch.float32, device="cuda")
    T.lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, K, 1, B.data_ptr(), 0, N, 1, Cd.data_ptr(), M, N, K,
                                     1, T.lib.i64([nb]), T.lib.i64([M * K]), T.lib.i64([0]), 0, 1))
    for b in range(nb):
        assert torch.equal(Cd[b], A[b] @ B), ("batched gemm", b)
    del Cd, A, B
    rows, cols = 65536, 40000
    Mx, x, y = ints(rows, cols), ints(cols), ints(rows)
    out = torch.empty(rows, dtype=torch.float32, device="cuda")
    T.lib.check(L.tenmo_hip_mv_f32(Mx.data_ptr(), 0, cols, 1, x.data_ptr(), 0, 1, out.data_ptr(), rows, cols, 0, None, None, None, 0, 1))
    ref = torch.cat([Mx[r0:r0 + 8192].double() @ x.double() for r0 in range(0, rows, 8192)])
    assert torch.equal(out.double(), ref), "mv"
    out = torch.empty(cols, dtype=torch.float32, device="cuda")
    T.lib.check(L.tenmo_hip_vm_f32(y.data_ptr(), 0, 1, Mx.data_ptr(), 0, cols, 1, out.data_ptr(), rows, cols, 0, None, None, None, 0, 1))
    ref = sum(y[r0:r0 + 8192].double() @ Mx[r0:r0 + 8192].double() for r0 in range(0, rows, 8192))
    assert torch.equal(out.double(), ref), "vm"


def test_more_batches_than_a_grid_dimension(T):
    """mv, vm and a skinny product over more than 65535 batches (a grid's y / z dimension holds 65535): the
    launches are cut into groups of batches; checked against einsum in fp64."""
    import torch
    from tenmo_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(71)
    nb = 70001
    # mv, row kernel: M[nb, 3, 8] . v[nb, 8]
    M = rng.standard_normal((nb, 3, 8), dtype=np.float32)
    v = rng.standard_normal((nb, 8), dtype=np.float32)
    Md, vd = torch.from_numpy(M).cuda(), torch.from_numpy(v).cuda()
    out = torch.empty((nb, 3), device="cuda")
    _lib.check(L.tenmo_hip_mv_f32(Md.data_ptr(), 0, 8, 1, vd.data_ptr(), 0, 1, out.data_ptr(), 3, 8, 1, _lib.i64([nb]), _lib.i64([24]), _lib.i64([8]), 0, 1))
    assert rel_fro(out.cpu().numpy(), np.einsum("bmk,bk->bm", M.astype(np.float64), v.astype(np.float64))) <= RTOL_FRO
    # vm, column kernel: v[nb, 3] . M[nb, 3, 8]
    v3 = rng.standard_normal((nb, 3), dtype=np.float32)
    v3d = torch.from_numpy(v3).cuda()
    out = torch.empty((nb, 8), device="cuda")
    _lib.check(L.tenmo_hip_vm_f32(v3d.data_ptr(), 0, 1, Md.data_ptr(), 0, 8, 1, out.data_ptr(), 3, 8, 1, _lib.i64([nb]), _lib.i64([3]), _lib.i64([24]), 0, 1))
    assert rel_fro(out.cpu().numpy(), np.einsum("bk,bkn->bn", v3.astype(np.float64), M.astype(np.float64))) <= RTOL_FRO
    # generic strides (both non-unit): one thread per output
    out = torch.empty((nb, 2), device="cuda")
    _lib.check(L.tenmo_hip_mv_f32(Md.data_ptr(), 0, 8, 2, vd.data_ptr(), 0, 2, out.data_ptr(), 2, 4, 1, _lib.i64([nb]), _lib.i64([24]), _lib.i64([8]), 0, 1))
    assert rel_fro(out.cpu().numpy(), np.einsum("bmk,bk->bm", M[:, :2, ::2].astype(np.float64), v[:, ::2].astype(np.float64))) <= RTOL_FRO
    # skinny product [2, 4] . [4, 2048] per batch through the view-level entry
    nb2 = 66000
    A = rng.standard_normal((nb2, 2, 4), dtype=np.float32)
    B = rng.standard_normal((4, 2048), dtype=np.float32)
    got = T.Tensor.from_numpy(A).matmul(T.Tensor.from_numpy(B), track_grad=False).to_numpy()
    assert rel_fro(got, ref_matmul64(A, B)) <= RTOL_FRO


def test_kernel_level_entry_routes_skinny_products(T):
    """tenmo_hip_gemm_f32 and tenmo_hip_matmul_nd choose the same kernel for a few rows against a wide
    row-major matrix (the column-streaming one): identical results."""
    import torch
    from tenmo_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(73)
    a = rng.standard_normal((4, 768), dtype=np.float32)
    b = rng.standard_normal((768, 50257), dtype=np.float32)
    via_views = T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False).to_numpy()
    Ad, Bd = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    out = torch.empty((4, 50257), device="cuda")
    _lib.check(L.tenmo_hip_gemm_f32(Ad.data_ptr(), 0, 768, 1, Bd.data_ptr(), 0, 50257, 1, out.data_ptr(), 4, 50257, 768, 0, None, None, None, 0, 1))
    assert np.array_equal(out.cpu().numpy(), via_views)
    assert rel_fro(via_views, ref_matmul64(a, b)) <= RTOL_FRO


def test_clock_probe(T):
    from tenmo_amd import _lib
    L = _lib.load()
    mhz = C.c_float()
    _lib.check(L.tenmo_hip_clock_probe(20000, C.byref(mhz)))
    assert 500.0 < mhz.value < 2600.0, mhz.value   # MI355X: 2400 MHz peak engine clock
    assert L.tenmo_hip_clock_probe(0, C.byref(mhz)) == -3


# ---- written after the last GPU run: checked on the CPU replay only so far (kept late in the file so that a surprise here
# hides as little as possible of the rest under pytest -x) ----

def test_non_finite_values_propagate_as_in_ieee(T):
    """An infinity or a NaN in an operand must come out where, and as what, the reference's plain loops put it: in the
    rows / columns it touches, as +inf, -inf or NaN — never a NaN from a padding lane's 0 x inf.  Poisoned positions are the
    ones tails and clamps handle specially (first and last k, last row, last column) in every product kernel: the GEMM
    tiles with K tails, K slices, stream-K, the short-reduction, K-stream and resident-A kernels, mv / vm / skinny products on
    aligned and odd row pitches."""
    import ctypes as C
    import torch
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(83)

    def classes(x):
        return np.where(np.isnan(x), 2, np.where(np.isposinf(x), 1, np.where(np.isneginf(x), -1, 0)))

    def product(a, b, ta, tb):
        M, K = a.shape
        N = b.shape[1]
        A = torch.from_numpy(np.ascontiguousarray(a.T if ta else a)).cuda()
        B = torch.from_numpy(np.ascontiguousarray(b.T if tb else b)).cuda()
        out = torch.zeros((M, N), device="cuda")
        a_rs, a_cs = (1, M) if ta else (K, 1)
        b_rs, b_cs = (1, K) if tb else (N, 1)
        lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, out.data_ptr(), M, N, K, 0, None, None, None, 0, 1))
        return out.cpu().numpy()

    cases = [(70, 90, 37, (), False, False), (70, 92, 37, (), True, True), (130, 260, 100, (("gemm_panel", 1),), False, False),
             (130, 260, 52, (("gemm_smallk", 1),), False, True), (130, 260, 100, (("gemm_panel", 5),), False, True),
             (256, 3200, 100, (("gemm_resident", 1),), False, False), (100, 3200, 250, (("gemm_resident", 2),), True, False),
             (200, 200, 333, (("gemm_splitk", 3),), False, False), (300, 500, 333, (("gemm_streamk", 1), ("gemm_tile", 1)), False, False),
             (4, 3000, 77, (), False, False), (1, 2049, 515, (), False, False), (3, 2051, 1030, (("cols_join", 1),), False, False),
             (8, 4099, 200, (), False, False), (70, 1, 300, (), False, True), (515, 1, 1030, (), True, False), (33, 1, 6000, (), True, False)]
    for M, N, K, knobs, ta, tb in cases:
        poisons = [("a", (M // 2, K - 1), np.inf), ("a", (0, 0), -np.inf), ("b", (K - 1, N // 2), np.inf), ("b", (0, N - 1), np.nan), ("a", (M - 1, K // 2), np.inf)]
        for which, at, value in poisons:
            a = rng.standard_normal((M, K)).astype(np.float32)
            b = rng.standard_normal((K, N)).astype(np.float32)
            (a if which == "a" else b)[at] = value
            for name, v in knobs:
                L.tenmo_hip_set_tuning(name.encode(), v)
            try:
                got = product(a, b, ta, tb)
            finally:
                for name, _ in knobs:
                    L.tenmo_hip_set_tuning(name.encode(), -1)
            with np.errstate(all="ignore"):
                ref = a.astype(np.float64) @ b.astype(np.float64)
            assert np.array_equal(classes(got), classes(ref)), (M, N, K, knobs, ta, tb, which, at, value)
            finite = np.isfinite(ref)
            assert np.allclose(got[finite], ref[finite], rtol=1e-4, atol=1e-4), (M, N, K, knobs, which, at)


def test_non_finite_values_in_the_gradients(T, oracle):
    """The same for the backward entries (both gradient products, the sum over broadcast batch dimensions inside the product and
    as a separate reduction, the outer-product and transposed-product gradients of mv / vm) and for dot: infinities and NaNs in
    an operand or in the upstream gradient land in the gradients where the reference's loops put them."""
    rng = np.random.default_rng(89)

    def classes(x):
        return np.where(np.isnan(x), 2, np.where(np.isposinf(x), 1, np.where(np.isneginf(x), -1, 0)))

    def same(got, want, what):
        assert got.shape == want.shape, what
        assert np.array_equal(classes(got), classes(want)), what
        finite = np.isfinite(want)
        assert np.allclose(got[finite], want[finite], rtol=1e-4, atol=1e-4), what

    def poisoned(shape, at, value):
        x = rng.standard_normal(shape, dtype=np.float32)
        if at is not None:
            x[at] = value
        return x

    last = lambda shape: tuple(d - 1 for d in shape)
    first = lambda shape: tuple(0 for _ in shape)
    for fold in (1, 0):
        T.lib.load().tenmo_hip_set_tuning(b"fold_reduce", fold)
        try:
            for sa, sb in [((70, 37), (37, 50)), ((3, 40, 24), (24, 36)), ((40, 24), (3, 24, 36)), ((2, 3, 33, 20), (3, 20, 28)), ((2, 1, 64, 64), (1, 4, 64, 128))]:
                sc = tuple(np.broadcast_shapes(sa[:-2], sb[:-2])) + (sa[-2], sb[-1])
                for which, at, value in [("a", last(sa), np.inf), ("a", first(sa), np.nan), ("b", last(sb), -np.inf), ("seed", last(sc), np.inf), ("seed", first(sc), -np.inf)]:
                    a = poisoned(sa, at if which == "a" else None, value)
                    b = poisoned(sb, at if which == "b" else None, value)
                    seed = poisoned(sc, at if which == "seed" else None, value)
                    A, B = T.Tensor.from_numpy(a, True), T.Tensor.from_numpy(b, True)
                    A.matmul(B).backward(T.Tensor.from_numpy(seed))
                    with np.errstate(all="ignore"):
                        gA, gB = oracle.matmul_backward(a, b, seed)
                    same(A.grad(), gA, ("dA", fold, sa, sb, which, at))
                    same(B.grad(), gB, ("dB", fold, sa, sb, which, at))
        finally:
            T.lib.load().tenmo_hip_set_tuning(b"fold_reduce", -1)
    for ms, vs in [((33, 70), (70,)), ((3, 33, 70), (70,)), ((515, 130), (130,)), ((2, 64, 1031), (2, 1031))]:
        so = tuple(np.broadcast_shapes(ms[:-2], vs[:-1])) + (ms[-2],)
        for which, at, value in [("m", last(ms), np.inf), ("v", last(vs), -np.inf), ("v", first(vs), np.nan), ("seed", last(so), np.inf)]:
            Mn = poisoned(ms, at if which == "m" else None, value)
            vn = poisoned(vs, at if which == "v" else None, value)
            seed = poisoned(so, at if which == "seed" else None, value)
            Mt, vt = T.Tensor.from_numpy(Mn, True), T.Tensor.from_numpy(vn, True)
            out = Mt.matmul(vt, mode=T.mv)
            with np.errstate(all="ignore"):
                same(out.to_numpy(), np.einsum("...mk,...k->...m", Mn.astype(np.float64), np.broadcast_to(vn, so[:-1] + (vs[-1],)).astype(np.float64)), ("mv", ms, vs, which, at))
            out.backward(T.Tensor.from_numpy(seed))
            with np.errstate(all="ignore"):
                dM, dv = oracle.mv_backward(Mn, vn, seed)
            same(Mt.grad(), dM, ("mv dM", ms, vs, which, at))
            same(vt.grad(), dv, ("mv dv", ms, vs, which, at))
    for vs, ms in [((70,), (70, 33)), ((70,), (3, 70, 33)), ((1031,), (1031, 515)), ((2, 130), (2, 130, 64))]:
        so = tuple(np.broadcast_shapes(vs[:-1], ms[:-2])) + (ms[-1],)
        for which, at, value in [("m", last(ms), np.inf), ("v", last(vs), -np.inf), ("seed", first(so), np.nan)]:
            Mn = poisoned(ms, at if which == "m" else None, value)
            vn = poisoned(vs, at if which == "v" else None, value)
            seed = poisoned(so, at if which == "seed" else None, value)
            Mt, vt = T.Tensor.from_numpy(Mn, True), T.Tensor.from_numpy(vn, True)
            out = vt.matmul(Mt, mode=T.vm)
            out.backward(T.Tensor.from_numpy(seed))
            with np.errstate(all="ignore"):
                dv, dM = oracle.vm_backward(vn, Mn, seed)
            same(Mt.grad(), dM, ("vm dM", vs, ms, which, at))
            same(vt.grad(), dv, ("vm dv", vs, ms, which, at))
    for n in (7, 1000, 300001):
        a, b = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(n, dtype=np.float32)
        a[n - 1] = np.inf
        got = float(T.Tensor.from_numpy(a).matmul(T.Tensor.from_numpy(b), track_grad=False).to_numpy())
        assert np.isinf(got) and (got > 0) == (b[n - 1] > 0), n


def test_non_finite_logits(T, oracle):
    """Cross-entropy rows that hold an infinity or a NaN: the row's loss and softmax are non-finite exactly where the
    reference's are (a +inf or NaN logit makes its whole row NaN; -inf logits are classes of probability zero), other rows
    are untouched — for every forward kernel (a thread, a wavefront, a workgroup per row; register-resident and streaming;
    with and without the softmax written) and for the gradient computed from that softmax."""
    import torch
    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(97)

    def classes(x):
        return np.where(np.isnan(x), 2, np.where(np.isposinf(x), 1, np.where(np.isneginf(x), -1, 0)))

    for M, Cn in [(9, 10), (70, 64), (33, 1000), (12, 8009), (5, 50257)]:
        x = (3 * rng.standard_normal((M, Cn))).astype(np.float32)
        x[0, Cn - 1] = np.inf
        x[1, 0] = np.nan
        x[2, Cn // 2] = -np.inf
        x[3, :] = -np.inf
        x[3, 1] = 0.5                      # one class carries all the probability
        t = rng.integers(0, Cn, M)
        t[2] = Cn // 2                     # the target is a class of probability zero: the loss is +inf
        with np.errstate(all="ignore"):
            sm_ref, rows_ref, total_ref, valid_ref = oracle.cross_entropy_forward(x, t)
        X, Tg = torch.from_numpy(x).cuda(), torch.from_numpy(t.astype(np.int64)).cuda()
        rows = torch.empty(M, dtype=torch.float32, device="cuda")
        total, valid = torch.zeros(1, dtype=torch.float32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
        for with_softmax in (True, False):
            sm = torch.empty((M, Cn), dtype=torch.float32, device="cuda") if with_softmax else None
            lib.check(L.tenmo_hip_cross_entropy_forward_f32(X.data_ptr(), Tg.data_ptr(), 1, M, Cn, -100, 0.0, sm.data_ptr() if with_softmax else None,
                                                            rows.data_ptr(), total.data_ptr(), valid.data_ptr(), 1))
            got_rows = rows.cpu().numpy()
            assert np.array_equal(classes(got_rows), classes(rows_ref)), (M, Cn, with_softmax, got_rows[:5], rows_ref[:5])
            ok = np.isfinite(rows_ref)
            assert np.allclose(got_rows[ok], rows_ref[ok], rtol=1e-5, atol=1e-5), (M, Cn, with_softmax)
            assert classes(np.float32(total.item())) == classes(np.float32(total_ref)), (M, Cn, with_softmax)
            if with_softmax:
                got = sm.cpu().numpy()
                assert np.array_equal(classes(got), classes(sm_ref)), (M, Cn)
                fin = np.isfinite(sm_ref)
                assert np.allclose(got[fin], sm_ref[fin], rtol=2e-4, atol=1e-7), (M, Cn)
                grad = torch.empty((M, Cn), dtype=torch.float32, device="cuda")
                one = torch.ones(1, dtype=torch.float32, device="cuda")
                lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), Tg.data_ptr(), 1, one.data_ptr(), M, Cn, -100, 0.0, 2, valid_ref, grad.data_ptr(), 0, 1))
                with np.errstate(all="ignore"):
                    g_ref = oracle.cross_entropy_backward(got, t, np.ones(1, np.float32), 2, valid_ref)
                assert np.array_equal(classes(grad.cpu().numpy()), classes(g_ref)), (M, Cn)


def test_non_finite_values_in_a_convolution(T, oracle):
    """The convolution layer forward and backward with an infinity or a NaN in the image, a filter or the upstream gradient:
    non-finite exactly where the reference's loops are (which multiply padded zeros by the filter taps as well)."""
    from tenmo_amd.cnn import Conv2dFused
    rng = np.random.default_rng(101)

    def classes(x):
        return np.where(np.isnan(x), 2, np.where(np.isposinf(x), 1, np.where(np.isneginf(x), -1, 0)))

    for (n, ci, h, w, co, k, stride, padding) in [(2, 3, 9, 11, 4, 3, 1, "valid"), (2, 4, 10, 10, 5, 3, 2, "same"), (3, 16, 12, 12, 32, 3, 1, "same")]:
        for which, value in [("image", np.inf), ("kernel", -np.inf), ("kernel", np.nan), ("up", np.inf)]:
            image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
            kernel = rng.standard_normal((co, ci, k, k), dtype=np.float32)
            bias = rng.standard_normal(co, dtype=np.float32)
            if which == "image":
                image[n - 1, ci - 1, h - 1, w - 1] = value
            if which == "kernel":
                kernel[co - 1, 0, k - 1, 0] = value
            case = (n, ci, h, w, co, k, stride, padding, which, value)
            with np.errstate(all="ignore"):
                want = oracle.conv2d_forward(image, kernel, bias, stride=stride, padding=padding)
            got = Conv2dFused.forward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(bias), stride=stride, padding=padding).to_numpy()
            assert np.array_equal(classes(got), classes(want)), ("forward",) + case
            up = rng.standard_normal(want.shape, dtype=np.float32)
            if which == "up":
                up[0, 0, 0, 0] = value
            with np.errstate(all="ignore"):
                wants = oracle.conv2d_backward(image, kernel, up, stride=stride, padding=padding)
            gi, gk, gb = Conv2dFused.backward(T.Tensor.from_numpy(image), T.Tensor.from_numpy(kernel), T.Tensor.from_numpy(up), stride=stride, padding=padding)
            for g, o, what in zip((gi.to_numpy(), gk.to_numpy(), gb.to_numpy()), wants, ("image", "kernel", "bias")):
                differ = classes(g) != classes(o)
                if what == "image" and which == "kernel":
                    # The one known deviation: the image gradient is computed as a convolution of the zero-padded upstream
                    # gradient with the reversed filter (a gather), the reference scatters; a non-finite filter tap times a
                    # padding zero is NaN here, where the reference never forms that product.  Border positions only.
                    differ &= ~np.isnan(g)
                assert not differ.any(), "%s gradient, case %r" % (what, case)


def test_zz_graph_capture_grows_scratch(T, oracle):
    """A captured training step whose kernel selection wants more library scratch than exists when the capture starts:
    the capture is abandoned, the scratch grown outside it and the step captured again — same losses as the eager step."""
    from tenmo_amd import _lib, rng as R
    from tenmo_amd.net import MLP
    L = _lib.load()
    _lib.check(L.tenmo_hip_shutdown())   # the scratch is grow-only: start from none
    _lib._initialised = False
    _lib.init(0)
    dims, seed, lr, batch = [2048, 1024, 10], 5, 0.01, 1024
    Ws, bs = R.xavier_mlp(dims, seed)
    eager, graph = MLP(dims, Ws, bs, batch), MLP(dims, Ws, bs, batch)
    # stream-K with the 256x128 tile keeps 2 partial tiles per workgroup: 2 * 512 * 256 * 128 * 4 B = 128 MiB of scratch
    _lib.check(L.tenmo_hip_set_tuning(b"gemm_tile", 0))
    _lib.check(L.tenmo_hip_set_tuning(b"gemm_streamk", 2))
    try:
        rng = np.random.default_rng(seed)
        x = rng.random((batch, dims[0]), dtype=np.float32)
        y = rng.integers(0, 10, batch).astype(np.int32)
        lg = graph.step(x, y, lr, graph=True)      # the first library call after the re-initialisation
        le = eager.step(x, y, lr)
        assert lg == le
        assert graph.step(x, y, lr, graph=True) == eager.step(x, y, lr)
    finally:
        _lib.check(L.tenmo_hip_set_tuning(b"gemm_tile", -1))
        _lib.check(L.tenmo_hip_set_tuning(b"gemm_streamk", -1))
    for l in range(2):
        np.testing.assert_array_equal(eager.params(l)[0], graph.params(l)[0])


def test_zz_shutdown_and_reinit(T):
    """tenmo_hip_shutdown releases the library's stream and scratch; after tenmo_hip_init everything works again and
    gives the same results (split-K workspace, column-kernel partial sums and the convolution tables are re-grown)."""
    import torch
    L = T.lib.load()
    rng = np.random.default_rng(109)
    a = rng.standard_normal((96, 4000), dtype=np.float32)
    b = rng.standard_normal((4000, 80), dtype=np.float32)
    img = rng.standard_normal((2, 3, 10, 10), dtype=np.float32)
    ker = rng.standard_normal((5, 3, 3, 3), dtype=np.float32)
    A, B, X, K = (torch.from_numpy(v).cuda() for v in (a, b, img, ker))

    def run():
        out = torch.empty((96, 80), device="cuda")
        L.tenmo_hip_set_tuning(b"gemm_splitk", 4)
        try:
            T.lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, 4000, 1, B.data_ptr(), 0, 80, 1, out.data_ptr(), 96, 80, 4000, 0, None, None, None, 0, 1))
        finally:
            L.tenmo_hip_set_tuning(b"gemm_splitk", -1)
        vm = torch.empty(80, device="cuda")
        T.lib.check(L.tenmo_hip_vm_f32(A.data_ptr(), 0, 1, B.data_ptr(), 0, 80, 1, vm.data_ptr(), 4000, 80, 0, None, None, None, 0, 1))
        conv = torch.empty((2, 5, 8, 8), device="cuda")
        T.lib.check(L.tenmo_hip_conv2d_forward_f32(X.data_ptr(), 2, 3, 10, 10, K.data_ptr(), 5, 3, 3, None, 1, 1, conv.data_ptr(), 1))
        return out.cpu().numpy(), vm.cpu().numpy(), conv.cpu().numpy()

    before = run()
    assert rel_fro(before[0], ref_matmul64(a, b)) <= RTOL_FRO
    assert L.tenmo_hip_shutdown() == 0
    assert L.tenmo_hip_sync() == -1 and b"not initialised" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_shutdown() == 0  # idempotent
    assert L.tenmo_hip_init(0) == 0
    after = run()
    for x, y in zip(before, after):
        assert np.array_equal(x, y)
