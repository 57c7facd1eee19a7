"""GPU parity tests of the kernels and code paths that no GPU has executed yet.

Everything here has passed on the CPU replay of the library (tests/test_replay_parity.py runs this file too) and, where it
matters, on the generated gfx950 code (tests/test_asm_clobbers.py, tests/test_isa_slice_join.py).  The file is collected
after every other GPU test, so that a first GPU run which goes wrong here has already recorded the rest; a test moves
to tests/test_gpu_parity.py once it has passed on a GPU.  In order of collection: the default path first (the batch-
reducing launch behind the gradients of broadcast parents), then the kernels behind knobs that are off by default (K
slices joined inside the column kernels' launch, the fused MLP launches, the K-stream kernel's 64x64 form, the
resident-A kernel), the Linear backward with the bias gradient summed in the weight-gradient launch, last the short-reduction
kernel forced onto reductions that are no multiple of 16 and onto one-step reductions (K <= 16) — the paths that use the masked
direct load (its fault, an undeclared SCC clobber, is fixed; these are the runs that confirm it).
"""
import os

import numpy as np
import pytest

from helpers import RTOL_FRO, ref_matmul64, rel_fro
from test_gpu_parity import T, _kstream_cases, _mlp_loss_curve, as_strided_tensor  # noqa: F401  (T is the module fixture)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fold", [1, 0, -1])
def test_backward_of_broadcast_parents(T, oracle, fold):
    """Gradients of parents that were broadcast over batch dimensions (tenmo/matmul.mojo:115-135: the batched product, then
    sum_over_broadcasted_axes): a shared A, a shared B whose partner's rows do not stack, partially broadcast batches on both
    sides, transposed views, tiles that are whole and ragged.  With the sum folded into the GEMM launch (1), with the
    batched gradient materialised and reduced (0) and with the automatic choice; against the oracle, twice (the second
    backward accumulates)."""
    L = T.lib.load()
    rng = np.random.default_rng(83 + fold)
    cases = [((70, 33), (5, 33, 41), False, False),          # A shared by 5 batches
             ((2, 1, 66, 20), (1, 3, 20, 130), False, False),  # each side broadcast along one batch dim
             ((3, 1, 40, 24), (4, 24, 36), False, False),      # A: one dim kept, one reduced; B: reduced over the leading dim
             ((130, 64), (2, 3, 64, 70), True, False),         # A a transposed view
             ((4, 50, 32), (32, 260), False, True),            # B a transposed view, shared
             ((1, 300, 16), (6, 16, 200), False, False)]
    try:
        L.tenmo_hip_set_tuning(b"fold_reduce", fold)
        for sa, sb, ta, tb in cases:
            a = rng.standard_normal(sa[:-2] + (sa[-1], sa[-2]) if ta else sa, dtype=np.float32)
            b = rng.standard_normal(sb[:-2] + (sb[-1], sb[-2]) if tb else sb, dtype=np.float32)
            A, B = T.Tensor.from_numpy(a, True), T.Tensor.from_numpy(b, True)
            Av, Bv = (A.transpose(-1, -2) if ta else A), (B.transpose(-1, -2) if tb else B)
            al, bl = (np.swapaxes(a, -1, -2) if ta else a), (np.swapaxes(b, -1, -2) if tb else b)
            out = Av.matmul(Bv)
            seed = rng.standard_normal(out.shape(), dtype=np.float32)
            out.backward(T.Tensor.from_numpy(seed), retain_graph=True)
            gA, gB = oracle.matmul_backward(al, bl, seed)
            assert rel_fro(Av.grad(), gA) <= 2 * RTOL_FRO, (fold, sa, sb)
            assert rel_fro(Bv.grad(), gB) <= 2 * RTOL_FRO, (fold, sa, sb)
            out.backward(T.Tensor.from_numpy(seed))
            assert rel_fro(Av.grad(), 2 * gA) <= 2 * RTOL_FRO, (fold, sa, sb)
            assert rel_fro(Bv.grad(), 2 * gB) <= 2 * RTOL_FRO, (fold, sa, sb)
        # a batch-strided A (its matrices do not stack at a constant row pitch) against a shared B: dB through the fold
        big = rng.standard_normal((6, 24, 20), dtype=np.float32)
        w = rng.standard_normal((20, 68), dtype=np.float32)
        sub = big[::2]
        A = as_strided_tensor(T, sub, requires_grad=True)
        W = T.Tensor.from_numpy(w, True)
        out = A.matmul(W)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed))
        gA, gW = oracle.matmul_backward(sub, w, seed)
        assert rel_fro(W.grad(), gW) <= 2 * RTOL_FRO and rel_fro(A.grad(), gA) <= 2 * RTOL_FRO
        # operands without a unit stride (every second row and column of their storage) under a broadcast: the reducing
        # launch takes them through the element-wise loader instead of materialising the batched gradient
        for sa, sb in (((70, 33), (5, 33, 41)), ((3, 1, 40, 24), (4, 24, 36)), ((4, 50, 32), (32, 68))):
            a2 = rng.standard_normal(sa[:-2] + (2 * sa[-2], 2 * sa[-1]), dtype=np.float32)
            b2 = rng.standard_normal(sb[:-2] + (2 * sb[-2], 2 * sb[-1]), dtype=np.float32)
            av, bv = a2[..., ::2, ::2], b2[..., ::2, ::2]
            A, B = as_strided_tensor(T, av, requires_grad=True), as_strided_tensor(T, bv, requires_grad=True)
            out = A.matmul(B)
            seed = rng.standard_normal(out.shape(), dtype=np.float32)
            out.backward(T.Tensor.from_numpy(seed), retain_graph=True)
            out.backward(T.Tensor.from_numpy(seed))
            gA, gB = oracle.matmul_backward(np.ascontiguousarray(av), np.ascontiguousarray(bv), seed)
            assert rel_fro(A.grad(), 2 * gA) <= 2 * RTOL_FRO and rel_fro(B.grad(), 2 * gB) <= 2 * RTOL_FRO, (fold, sa, sb)
        # vector . matrix with the vector shared by the batches (tenmo/vectormatrix.mojo:18-206): its gradient is the sum over
        # the batches of M_b . dy_b; and matrix . vector likewise (tenmo/matrixvector.mojo:19-201)
        for vs, ms in (((48,), (5, 48, 70)), ((1, 33), (3, 2, 33, 20)), ((1030,), (2, 1030, 515))):
            vn = rng.standard_normal(vs, dtype=np.float32)
            mn = rng.standard_normal(ms, dtype=np.float32)
            V, M = T.Tensor.from_numpy(vn, True), T.Tensor.from_numpy(mn, True)
            out = V.matmul(M, mode=T.vm)
            seed = rng.standard_normal(out.shape(), dtype=np.float32)
            out.backward(T.Tensor.from_numpy(seed))
            gv, gm = oracle.vm_backward(vn, mn, seed)
            assert rel_fro(V.grad(), gv) <= 2 * RTOL_FRO and rel_fro(M.grad(), gm) <= 2 * RTOL_FRO, (fold, vs, ms)
            assert rel_fro(V.grad(), np.einsum("...kn,...n->...k", mn.astype(np.float64), seed.astype(np.float64)).reshape(-1, vs[-1]).sum(0).reshape(vs)) <= RTOL_FRO
            mt = np.ascontiguousarray(np.swapaxes(mn, -1, -2))  # [.., n, k] . v[k]
            V, M = T.Tensor.from_numpy(vn, True), T.Tensor.from_numpy(mt, True)
            out = M.matmul(V, mode=T.mv)
            seed = rng.standard_normal(out.shape(), dtype=np.float32)
            out.backward(T.Tensor.from_numpy(seed))
            gm, gv = oracle.mv_backward(mt, vn, seed)
            assert rel_fro(V.grad(), gv) <= 2 * RTOL_FRO and rel_fro(M.grad(), gm) <= 2 * RTOL_FRO, (fold, vs, ms)
    finally:
        L.tenmo_hip_set_tuning(b"fold_reduce", -1)

def test_randomized_backward_of_views_and_broadcast_parents(T, oracle):
    """Seeded sweep of Matmul backward (tenmo/matmul.mojo:24-54, :101-137) at the Tensor level: batch shapes of rank 0 to 3 in which
    each parent keeps, drops or lacks every dimension, operands that are plain, transposed, stepped or offset views of larger
    storage, ragged and whole tiles, the sum over the broadcast dimensions folded into the launch, materialised, or chosen
    automatically; gradients against the oracle on dense copies of the same views, twice (the second backward accumulates)."""
    L = T.lib.load()
    rng = np.random.default_rng(211)

    def operand(rows, cols, own_batch):
        kind = rng.choice(["plain", "transposed", "stepped", "offset"])
        if kind == "plain":
            return rng.standard_normal(tuple(own_batch) + (rows, cols), dtype=np.float32)
        if kind == "transposed":
            return np.swapaxes(rng.standard_normal(tuple(own_batch) + (cols, rows), dtype=np.float32), -1, -2)
        if kind == "stepped":
            return rng.standard_normal(tuple(own_batch) + (2 * rows, 2 * cols), dtype=np.float32)[..., ::2, ::2]
        return rng.standard_normal(tuple(own_batch) + (rows + 3, cols + 4), dtype=np.float32)[..., 2:2 + rows, 4:4 + cols]

    try:
        for case in range(40):
            m, k, n = (int(rng.choice([1, 5, 33, 64, 70, 130, 200])) for _ in range(3))
            batch = [int(rng.integers(2, 5)) for _ in range(int(rng.integers(0, 4)))]

            def own():
                dims = [d if rng.random() < 0.6 else 1 for d in batch]
                return dims[int(rng.integers(0, len(dims) + 1)):]

            a, b = operand(m, k, own()), operand(k, n, own())
            fold = int(rng.choice([-1, 0, 1]))
            L.tenmo_hip_set_tuning(b"fold_reduce", fold)
            A, B = as_strided_tensor(T, a, requires_grad=True), as_strided_tensor(T, b, requires_grad=True)
            out = A.matmul(B)
            desc = (case, a.shape, a.strides, b.shape, b.strides, fold)
            assert rel_fro(out.to_numpy(), ref_matmul64(a, b)) <= RTOL_FRO, desc
            seed = rng.standard_normal(out.shape(), dtype=np.float32)
            out.backward(T.Tensor.from_numpy(seed), retain_graph=True)
            out.backward(T.Tensor.from_numpy(seed))
            gA, gB = oracle.matmul_backward(np.ascontiguousarray(a), np.ascontiguousarray(b), seed)
            assert A.grad().shape == a.shape and B.grad().shape == b.shape, desc
            assert rel_fro(A.grad(), 2 * gA) <= 2 * RTOL_FRO and rel_fro(B.grad(), 2 * gB) <= 2 * RTOL_FRO, desc
    finally:
        L.tenmo_hip_set_tuning(b"fold_reduce", -1)

def test_randomized_mv_vm_backward_of_views(T, oracle):
    """Seeded sweep of the mv / vm gradients (tenmo/matrixvector.mojo:19-201, tenmo/vectormatrix.mojo:18-206) at the Tensor level:
    matrices that are plain, transposed, stepped or offset views, vectors with a step, batch shapes in which matrix and vector each
    keep, drop or lack a dimension (a shared vector's gradient is summed over the batches, a shared matrix's outer products
    likewise); against the oracle on dense copies, twice."""
    rng = np.random.default_rng(223)

    def matrix(rows, cols, own_batch):
        kind = rng.choice(["plain", "transposed", "stepped", "offset"])
        if kind == "plain":
            return rng.standard_normal(tuple(own_batch) + (rows, cols), dtype=np.float32)
        if kind == "transposed":
            return np.swapaxes(rng.standard_normal(tuple(own_batch) + (cols, rows), dtype=np.float32), -1, -2)
        if kind == "stepped":
            return rng.standard_normal(tuple(own_batch) + (2 * rows, 2 * cols), dtype=np.float32)[..., ::2, ::2]
        return rng.standard_normal(tuple(own_batch) + (rows + 3, cols + 4), dtype=np.float32)[..., 2:2 + rows, 4:4 + cols]

    def vector(n, own_batch):
        step = int(rng.choice([1, 1, 2]))
        return rng.standard_normal(tuple(own_batch) + (n * step,), dtype=np.float32)[..., ::step]

    for case in range(40):
        r, c = (int(rng.choice([1, 4, 33, 64, 130, 515, 1030])) for _ in range(2))
        batch = [int(rng.integers(2, 5)) for _ in range(int(rng.integers(0, 3)))]

        def own():
            dims = [d if rng.random() < 0.6 else 1 for d in batch]
            return dims[int(rng.integers(0, len(dims) + 1)):]

        mn = matrix(r, c, own())
        as_mv = rng.random() < 0.5
        vn = vector(c if as_mv else r, own())
        Mt, vt = as_strided_tensor(T, mn, requires_grad=True), as_strided_tensor(T, vn, requires_grad=True)
        out = Mt.matmul(vt, mode=T.mv) if as_mv else vt.matmul(Mt, mode=T.vm)
        desc = (case, "mv" if as_mv else "vm", mn.shape, mn.strides, vn.shape, vn.strides)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed), retain_graph=True)
        out.backward(T.Tensor.from_numpy(seed))
        md, vd = np.ascontiguousarray(mn), np.ascontiguousarray(vn)
        if as_mv:
            dM, dv = oracle.mv_backward(md, vd, seed)
        else:
            dv, dM = oracle.vm_backward(vd, md, seed)
        assert Mt.grad().shape == mn.shape and vt.grad().shape == vn.shape, desc
        assert rel_fro(Mt.grad(), 2 * dM) <= 2 * RTOL_FRO and rel_fro(vt.grad(), 2 * dv) <= 2 * RTOL_FRO, desc


def test_column_kernels_join_slices_in_the_launch(T):
    """vm, mv on a transposed view, skinny and batched skinny products with the K slices added by the last workgroup of
    the streaming launch (cols_join) instead of a second launch: the same bits as the two-launch result — the slices are
    added in the same order — call after call (the arrival counters must be back at zero), with `+=`, and through the
    allocation-free entry."""
    import ctypes as C
    from tenmo_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(67)

    def both(fn):
        apart = fn()
        L.tenmo_hip_set_tuning(b"cols_join", 1)
        try:
            joined, again = fn(), fn()
        finally:
            L.tenmo_hip_set_tuning(b"cols_join", 0)
        assert np.array_equal(apart, joined) and np.array_equal(apart, again)
        return joined

    for (m, k, n) in [(1, 4096, 4096), (4, 768, 50257), (3, 2000, 3001), (8, 1024, 2048), (1, 16384, 1024), (2, 515, 1030), (1, 100, 50000)]:
        a = rng.standard_normal((m, k), dtype=np.float32)
        b = rng.standard_normal((k, n), dtype=np.float32)
        A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
        got = both(lambda: A.matmul(B, track_grad=False).to_numpy())
        assert rel_fro(got, ref_matmul64(a, b)) <= RTOL_FRO, (m, k, n)
        if m == 1:
            v = T.Tensor.from_numpy(a[0])
            got = both(lambda: v.matmul(B, track_grad=False).to_numpy())                      # vector x matrix
            assert rel_fro(got, ref_matmul64(a, b)[0]) <= RTOL_FRO, ("vm", k, n)
            Bt = T.Tensor.from_numpy(b).transpose()                                           # [n, k] view: mv through the column kernel
            got = both(lambda: Bt.matmul(v, track_grad=False).to_numpy())
            assert rel_fro(got, ref_matmul64(a, b)[0]) <= RTOL_FRO, ("mv of a transposed view", k, n)
    # batches of a right operand with an odd pitch
    a = rng.standard_normal((2, 768), dtype=np.float32)
    b = rng.standard_normal((4, 768, 2503), dtype=np.float32)
    A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)
    assert rel_fro(both(lambda: A.matmul(B, track_grad=False).to_numpy()), ref_matmul64(a, b)) <= RTOL_FRO
    # += and the allocation-free entry
    a = rng.standard_normal((1, 3000), dtype=np.float32)
    b = rng.standard_normal((3000, 5000), dtype=np.float32)
    c0 = rng.standard_normal((1, 5000), dtype=np.float32)
    A, B = T.Tensor.from_numpy(a), T.Tensor.from_numpy(b)

    def accumulate(entry):
        out = T.Tensor.from_numpy(c0.copy())
        if entry == "gemm":
            _lib.check(L.tenmo_hip_gemm_f32(A.buffer.data_ptr(), 0, 3000, 1, B.buffer.data_ptr(), 0, 5000, 1, out.buffer.data_ptr(),
                                            1, 5000, 3000, 0, None, None, None, 1, 1))
        else:
            _lib.check(L.tenmo_hip_vm_f32_noalloc(A.buffer.data_ptr(), 0, 1, B.buffer.data_ptr(), 0, 5000, 1, out.buffer.data_ptr(),
                                                  3000, 5000, 0, None, None, None, 1, 1))
        return out.to_numpy()

    for entry in ("gemm", "noalloc"):
        assert rel_fro(both(lambda: accumulate(entry)), c0.astype(np.float64) + ref_matmul64(a, b)) <= RTOL_FRO, entry


def test_mlp_loss_curve_with_the_fused_tail(T, oracle):
    """The same curves with the last two layers, the loss, their backward and their update as one launch (mlp_fused_tail:
    the MNIST shape fits that launch, the other shapes of the curve test fall back to op by op)."""
    from tenmo_amd import rng as R
    from tenmo_amd.net import MLP

    for level in (1, 2, 3):  # 2: the first layer's weight gradient and its update as one launch as well; 3: its forward too
        T.lib.load().tenmo_hip_set_tuning(b"mlp_fused_tail", level)
        try:
            _mlp_loss_curve(T, oracle, R, MLP)
        finally:
            T.lib.load().tenmo_hip_set_tuning(b"mlp_fused_tail", 0)
    # every fused launch on ragged shapes: inputs that end inside an 8-wide k chunk in each way, widths that are no
    # multiples of the 32x32 blocks, batches that do not fill them
    rs = np.random.default_rng(71)
    T.lib.load().tenmo_hip_set_tuning(b"mlp_fused_tail", 3)
    try:
        for batch, dims in ((37, [257, 77, 33, 7]), (64, [1001, 128, 64, 32]), (1, [262, 5, 3, 2]), (100, [518, 130, 40, 9]), (33, [259, 97, 4])):
            Ws, bs = R.xavier_mlp(dims, 11)
            gpu, cpu = MLP(dims, Ws, bs, batch), oracle.MLP(dims, Ws, bs, batch)
            for step in range(3):
                x = rs.standard_normal((batch, dims[0])).astype(np.float32)
                y = rs.integers(0, dims[-1], batch).astype(np.int32)
                assert abs(gpu.step(x, y, 0.05) - cpu.step(x, y, 0.05)) <= 1e-4, (batch, dims, step)
            for l in range(len(dims) - 1):
                (Wg, bg), (Wc, bc) = gpu.params(l), cpu.params(l)
                assert rel_fro(Wg, Wc) <= 1e-5 and np.abs(bg - bc).max() <= 1e-5, (batch, dims, l)
                (dWg, dbg), (dWc, dbc) = gpu.grads(l), cpu.grads(l)
                assert rel_fro(dWg, dWc) <= 1e-4 and rel_fro(dbg, dbc) <= 1e-4, (batch, dims, l)
            assert rel_fro(gpu.forward(x), cpu.forward(x)) <= 1e-5, (batch, dims)
        # the captured step holds the fused launches too, and a change of the knob captures anew
        dims = [784, 128, 32, 10]
        Ws, bs = R.xavier_mlp(dims, 13)
        eager, graph = MLP(dims, Ws, bs, 64), MLP(dims, Ws, bs, 64)
        for step in range(6):
            if step == 3:
                T.lib.load().tenmo_hip_set_tuning(b"mlp_fused_tail", 0)
            x, y = R.mnist_like_batch(64, 13, step)
            assert eager.step(x, y, 0.01) == graph.step(x, y, 0.01, graph=True), step
        np.testing.assert_array_equal(eager.params(0)[0], graph.params(0)[0])
    finally:
        T.lib.load().tenmo_hip_set_tuning(b"mlp_fused_tail", 0)


def test_kstream_kernel_with_64x64_tiles(T):
    """The same cases through the kernel's 64x64-tile variant (a ring of eight stages; two operand fetches behind an MFMA
    where an operand is MN-major)."""
    _kstream_cases(T, 3)


def test_resident_left_operand_kernel(T):
    """The kernel that keeps its tile row of A in LDS for all of K and streams B alone (gemm_resident knob: tiles of 128x64
    and of 64x64), forced on: the CBOW logits and their gradient at full size, K tails, a row-major and a transposed-view A,
    ragged last tile rows and column blocks, several tile rows, a result of fewer tiles than workgroups; and, with the knob
    still on, what the kernel does not take (falls through to the others).  Against fp64; the element behind the result
    stays untouched.  (The same launches run address by address on the CPU in test_replay_addresses.py.)"""
    import torch
    L, lib = T.lib.load(), T.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(37)
    cases = [(256, 50000, 100), (100, 50000, 256), (128, 2052, 32), (64, 4096, 20), (36, 3000, 112), (200, 2500, 132), (1024, 6400, 48),
             (256, 128, 100), (256, 3200, 248), (128, 3200, 272), (128, 3202, 64)]
    try:
        for knob in (1, 2):
            L.tenmo_hip_set_tuning(b"gemm_resident", knob)
            for M, N, K in cases:
                for ta in (False, True):
                    for tb, acc in ((False, 0), (True, 0), (False, 1)) if (M, N, K) == (128, 2052, 32) else ((False, 0),):
                        A = torch.randn(((K, M) if ta else (M, K)), generator=gen, device="cuda")
                        B = torch.randn(((N, K) if tb else (K, N)), generator=gen, device="cuda")
                        out = torch.randn((M * N + 1,), generator=gen, device="cuda")
                        guard = float(out[-1])
                        a_rs, a_cs = (1, M) if ta else (K, 1)
                        b_rs, b_cs = (1, K) if tb else (N, 1)
                        ref = (A.t() if ta else A).double() @ (B.t() if tb else B).double() + (out[:-1].view(M, N).double() if acc else 0)
                        lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, out.data_ptr(), M, N, K, 0,
                                                       None, None, None, acc, 1))
                        err = float((out[:-1].view(M, N).double() - ref).norm() / ref.norm())
                        assert err <= RTOL_FRO, (knob, M, N, K, ta, tb, acc, err)
                        assert float(out[-1]) == guard, (knob, M, N, K, ta, tb, acc)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_resident", 0)


def test_linear_backward_reference_literal(T, golden):
    """The reference's own literal for the gradient of a broadcast bias (tests/test_expand.mojo:229-245): whatever the input and the
    weight, the bias gradient of x.W + b is the upstream gradient summed over its rows — through tenmo_hip_linear_backward (here the
    three rows take the separate pass: in_features <= 8) and through tenmo_hip_column_sum_f32."""
    import ctypes as C

    L, lib = T.lib.load(), T.lib
    case = golden["harness"]["bias_gradient_is_column_sums"]
    up = np.array(case["upstream"], np.float32)
    for k in (2, 20):
        X, W, dY = T.Tensor.from_numpy(np.ones((3, k), np.float32)), T.Tensor.from_numpy(np.ones((k, 4), np.float32)), T.Tensor.from_numpy(up)
        gb = T.Tensor.zeros(4)
        gw = T.Tensor.zeros(k, 4)
        lib.check(L.tenmo_hip_linear_backward(C.byref(X.buffer.c_view()), C.byref(W.buffer.c_view()), dY.buffer.data_ptr(), None, gw.buffer.data_ptr(),
                                              gb.buffer.data_ptr(), 1))
        assert np.array_equal(gb.to_numpy(), np.array(case["expect"], np.float32)), k
        assert np.array_equal(gw.to_numpy(), np.tile(np.array(case["expect"], np.float32), (k, 1))), k  # X = ones: every row of dW is the same sums
    out, upstream = T.Tensor.zeros(4), T.Tensor.from_numpy(up)
    lib.check(L.tenmo_hip_column_sum_f32(upstream.buffer.data_ptr(), 0, 4, 3, 4, out.buffer.data_ptr(), 0, 1))
    assert np.array_equal(out.to_numpy(), np.array(case["expect"], np.float32))


def test_linear_backward_refuses_what_matmul_refuses(T):
    """Same argument errors as the matmul entry points, before anything is launched: an inner-dimension mismatch is the reference's
    panic (tenmo/matmul.mojo:226-227), a gradient asked for without an upstream gradient is an invalid argument; a call that asks for
    no gradient at all is accepted and does nothing."""
    import ctypes as C

    L = T.lib.load()
    X, W, bad = T.Tensor.zeros(5, 7), T.Tensor.zeros(7, 3), T.Tensor.zeros(6, 3)
    g = T.Tensor.from_numpy(np.full(3, 2.0, np.float32))
    assert L.tenmo_hip_linear_backward(C.byref(X.buffer.c_view()), C.byref(bad.buffer.c_view()), X.buffer.data_ptr(), None, None, g.buffer.data_ptr(), 1) < 0
    assert b"incompatible" in L.tenmo_hip_last_error() or b"inner" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_linear_backward(C.byref(X.buffer.c_view()), C.byref(W.buffer.c_view()), None, None, None, g.buffer.data_ptr(), 1) < 0
    assert b"upstream gradient" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_linear_backward(C.byref(X.buffer.c_view()), C.byref(W.buffer.c_view()), None, None, None, None, 1) == 0
    np.testing.assert_array_equal(g.to_numpy(), np.full(3, 2.0, np.float32))


def test_linear_backward_sums_the_bias_gradient_in_the_weight_gradient_launch(T, oracle):
    """tenmo_hip_linear_backward: dX, dW and the bias gradient of x.W + b (tenmo/net.mojo:193-201 = Matmul then Adder; the
    bias gradient is sum_over_broadcasted_axes of the upstream gradient, tenmo/broadcast.mojo:66-88) against the oracle
    and fp64, twice in a row (the second call accumulates), for matrix and batched inputs, whole and ragged tiles — with
    the weight-gradient launch forced through every tile, K slices and stream-K, each of which adds up its dY fragments
    its own way — and for the forms that take the separate pass over dY instead (a transposed-view input, no dW wanted)."""
    import ctypes as C

    L, lib = T.lib.load(), T.lib
    rng = np.random.default_rng(97)
    knobs = [{}, {"gemm_tile": 0}, {"gemm_tile": 1}, {"gemm_tile": 2}, {"gemm_tile": 3}, {"gemm_tile": 4}, {"gemm_tile": 1, "gemm_splitk": 4},
             {"gemm_tile": 0, "gemm_splitk": 3}, {"gemm_tile": 1, "gemm_streamk": 1}, {"gemm_tile": 0, "gemm_streamk": 2}, {"gemm_tile": 3, "gemm_streamk": 2},
             {"gemm_tile": 2, "gemm_streamk": 1}]
    shapes = [((64, 96), 40), ((300, 130), 70), ((3, 50, 64), 36), ((2, 2, 33, 20), 132), ((1000, 260), 200)]
    if not os.environ.get("TENMO_TEST_SMALL"):
        shapes.append(((2048, 768), 1024))

    def run(x, w, dy, xt=None, want=(True, True, True)):
        """One call through the C ABI on fresh zero gradients, then a second one on top; returns the three gradients."""
        X = T.Tensor.from_numpy(x if xt is None else xt)
        Xv = X if xt is None else X.transpose(-1, -2)
        W, dY = T.Tensor.from_numpy(w), T.Tensor.from_numpy(dy)
        outs = [T.Tensor.zeros(*a.shape) if on else None for a, on in zip((x, w, np.zeros(w.shape[-1], np.float32)), want)]
        for _ in range(2):
            lib.check(L.tenmo_hip_linear_backward(C.byref(Xv.buffer.c_view()), C.byref(W.buffer.c_view()), dY.buffer.data_ptr(),
                                                  *[(o.buffer.data_ptr() if o is not None else None) for o in outs], 1))
        return [o.to_numpy() if o is not None else None for o in outs]

    try:
        for xs, n_out in shapes:
            x = rng.standard_normal(xs, dtype=np.float32)
            w = rng.standard_normal((xs[-1], n_out), dtype=np.float32)
            dy = rng.standard_normal(xs[:-1] + (n_out,), dtype=np.float32)
            gx, gw = oracle.matmul_backward(x, w, dy)
            gb = oracle.sum_over_broadcasted_axes(dy, (n_out,))
            gb64 = dy.astype(np.float64).reshape(-1, n_out).sum(0)
            assert rel_fro(gb, gb64) <= RTOL_FRO
            for knob in knobs if len(xs) == 2 or xs == (3, 50, 64) else knobs[:1]:
                for name, value in knob.items():
                    L.tenmo_hip_set_tuning(name.encode(), value)
                try:
                    dx, dw, db = run(x, w, dy)
                finally:
                    for name in knob:
                        L.tenmo_hip_set_tuning(name.encode(), -1)
                assert rel_fro(dx, 2 * gx) <= 2 * RTOL_FRO and rel_fro(dw, 2 * gw) <= 2 * RTOL_FRO, (xs, n_out, knob)
                assert rel_fro(db, 2 * gb64) <= RTOL_FRO and rel_fro(db, 2 * gb.astype(np.float64)) <= 2 * RTOL_FRO, (xs, n_out, knob)
            # what the fused sum does not take: a transposed-view input, and a call that wants no weight gradient
            dx, dw, db = run(x, w, dy, xt=np.ascontiguousarray(np.swapaxes(x, -1, -2)))
            assert rel_fro(dx, 2 * gx) <= 2 * RTOL_FRO and rel_fro(dw, 2 * gw) <= 2 * RTOL_FRO and rel_fro(db, 2 * gb64) <= RTOL_FRO, (xs, n_out)
            dx, dw, db = run(x, w, dy, want=(True, False, True))
            assert dw is None and rel_fro(dx, 2 * gx) <= 2 * RTOL_FRO and rel_fro(db, 2 * gb64) <= RTOL_FRO, (xs, n_out)
            dx, dw, db = run(x, w, dy, want=(False, True, False))
            assert dx is None and db is None and rel_fro(dw, 2 * gw) <= 2 * RTOL_FRO, (xs, n_out)
        # through the layer of the host mirror: Linear forward, backward from a seed, gradients of x, W and b
        from tenmo_amd.net import Linear

        lin = Linear(130, 70, np.random.default_rng(5))
        x = rng.standard_normal((4, 75, 130), dtype=np.float32)
        X = T.Tensor.from_numpy(x, True)
        out = lin(X)
        seed = rng.standard_normal(out.shape(), dtype=np.float32)
        out.backward(T.Tensor.from_numpy(seed))
        w = lin.weight.to_numpy()
        gx, gw = oracle.matmul_backward(x, w, seed)
        assert rel_fro(out.to_numpy(), ref_matmul64(x, w) + lin.bias.to_numpy()) <= RTOL_FRO
        assert rel_fro(X.grad(), gx) <= 2 * RTOL_FRO and rel_fro(lin.weight.grad(), gw) <= 2 * RTOL_FRO
        assert rel_fro(lin.bias.grad(), seed.astype(np.float64).reshape(-1, 70).sum(0)) <= RTOL_FRO
    finally:
        for name in ("gemm_tile", "gemm_splitk", "gemm_streamk"):
            L.tenmo_hip_set_tuning(name.encode(), -1)


@pytest.mark.parametrize("smallk", [0, 1])
def test_short_reduction_kernel_layouts_and_k_tails(T, smallk):
    """The same kernel over every operand layout (row-major and transposed views of A and of B) and reductions that
    are no multiple of 16 (zero-filled K tail; a K-major operand then needs K % 4 == 0, other K fall back to the
    ordinary kernel), whole and ragged tiles, batches, accumulation; against fp64."""
    import torch
    L, lib = T.lib.load(), T.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(29)
    cases = [((), 64, 64, 16, 0), ((), 128, 192, 100, 0), ((3,), 100, 132, 36, 0), ((2, 3), 256, 68, 64, 1), ((5,), 64, 64, 112, 0),
             ((2,), 332, 776, 20, 1), ((), 1000, 1000, 7, 0), ((4,), 72, 52, 84, 0), ((), 256, 5000, 100, 0), ((2,), 512, 512, 50, 1),
             ((9,), 320, 1024, 12, 0), ((), 64, 8192, 104, 0), ((), 130, 70, 33, 0)]
    try:
        L.tenmo_hip_set_tuning(b"gemm_smallk", smallk)
        for bshape, M, N, K, acc in cases:
            for ta in (False, True):
                for tb in (False, True):
                    A = torch.randn((*bshape, *((K, M) if ta else (M, K))), generator=gen, device="cuda")
                    B = torch.randn((*bshape, *((N, K) if tb else (K, N))), generator=gen, device="cuda")
                    Cc = torch.randn((*bshape, M, N), generator=gen, device="cuda")
                    a_rs, a_cs = (1, M) if ta else (K, 1)
                    b_rs, b_cs = (1, K) if tb else (N, 1)
                    ref = (A.transpose(-1, -2) if ta else A).double() @ (B.transpose(-1, -2) if tb else B).double() + (Cc.double() if acc else 0)
                    ab = [A.stride(i) for i in range(len(bshape))]
                    bb = [B.stride(i) for i in range(len(bshape))]
                    lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, Cc.data_ptr(), M, N, K, len(bshape),
                                                   lib.i64(bshape), lib.i64(ab), lib.i64(bb), acc, 1))
                    err = float((Cc.double() - ref).norm() / ref.norm())
                    assert err <= RTOL_FRO, (smallk, bshape, M, N, K, acc, ta, tb, err)
    finally:
        L.tenmo_hip_set_tuning(b"gemm_smallk", -1)


def test_short_reduction_kernel_on_one_step_reductions(T):
    """K <= 16 through the persistent short-reduction kernel (gemm_smallk = 3; the automatic choice keeps such products on the
    ordinary kernel until this has passed on a GPU): several tiles per workgroup, ragged tiles, K tails (the masked direct load
    on every tile), every operand layout, plain and accumulating stores, batches; last the product after which a GPU run
    once ended in a memory fault — [8192,16].[16,8192] with B a transposed view (cause: an undeclared SCC clobber in the masked
    load's asm block, fixed; tests/test_asm_clobbers.py holds the generated code to it).  Against fp64."""
    import torch
    L, lib = T.lib.load(), T.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(41)
    small = bool(os.environ.get("TENMO_TEST_SMALL"))
    cases = [((), 3072, 3072, 16, 0), ((), 3000, 3100, 12, 1), ((3,), 1024, 2052, 8, 0), ((2,), 2048, 2048, 16, 1), ((), 1028, 4100, 4, 0)]
    if small:
        cases = [((), 300, 520, 16, 0), ((), 260, 132, 12, 1), ((3,), 200, 264, 8, 0)]
    try:
        L.tenmo_hip_set_tuning(b"gemm_smallk", 3)
        for bshape, M, N, K, acc in cases:
            for ta in (False, True):
                for tb in (False, True):
                    A = torch.randn((*bshape, *((K, M) if ta else (M, K))), generator=gen, device="cuda")
                    B = torch.randn((*bshape, *((N, K) if tb else (K, N))), generator=gen, device="cuda")
                    Cc = torch.randn((*bshape, M, N), generator=gen, device="cuda")
                    a_rs, a_cs = (1, M) if ta else (K, 1)
                    b_rs, b_cs = (1, K) if tb else (N, 1)
                    ref = (A.transpose(-1, -2) if ta else A).double() @ (B.transpose(-1, -2) if tb else B).double() + (Cc.double() if acc else 0)
                    ab = [A.stride(i) for i in range(len(bshape))]
                    bb = [B.stride(i) for i in range(len(bshape))]
                    lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, Cc.data_ptr(), M, N, K, len(bshape),
                                                   lib.i64(bshape), lib.i64(ab), lib.i64(bb), acc, 1))
                    err = float((Cc.double() - ref).norm() / ref.norm())
                    assert err <= RTOL_FRO, (bshape, M, N, K, acc, ta, tb, err)
        if not small:
            M = N = 8192
            A = torch.randn((M, 16), generator=gen, device="cuda")
            Bt = torch.randn((N, 16), generator=gen, device="cuda")
            Cc = torch.empty((M, N), device="cuda")
            lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, 16, 1, Bt.data_ptr(), 0, 1, 16, Cc.data_ptr(), M, N, 16, 0, None, None, None, 0, 1))
            rows = torch.arange(0, M, 61, device="cuda")
            ref = A[rows].double() @ Bt.double().t()
            assert float((Cc[rows].double() - ref).norm() / ref.norm()) <= RTOL_FRO
    finally:
        L.tenmo_hip_set_tuning(b"gemm_smallk", -1)
