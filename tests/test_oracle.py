"""Pins the CPU oracle (oracle/) before anything trusts it: the reference's own literal test
vectors, fp64 brute force, closed forms and algebraic invariants.  Runs without a GPU."""
import numpy as np
import pytest

from helpers import GOLDEN_GRADIENT_KEYS, ce_reference64, check_golden_extras, exact_product, generated_operand, numpy_view, ref_matmul64, rel_fro, scatter_to_storage, storage_of, strides_of


def _view(O, t):
    return O.View(storage_of(t), t.get("offset", 0), t["shape"], strides_of(t))


def test_golden_forward(golden, oracle):
    O = oracle
    for c in golden["cases"]:
        A, B = _view(O, c["A"]), _view(O, c["B"])
        if c["op"] == "mm":
            got = O.matmul(A, B)
        elif c["op"] == "mv":
            got = O.mv(A, B)
        elif c["op"] == "vm":
            got = O.vm(A, B)
        else:
            got = O.dot(A, B)
        if "expect" in c:
            np.testing.assert_allclose(got, np.asarray(c["expect"], np.float32), rtol=1e-5, atol=1e-8, err_msg=c["name"])
        if "expect_shape" in c:
            assert list(np.shape(got)) == c["expect_shape"], c["name"]
        check_golden_extras(c, got)
    for c in golden["shape_cases"]:  # shapes only (random operands in the reference): the broadcast of the batch dimensions
        assert list(O.result_shape(O.MM, O.View.of(np.zeros(c["A_shape"], np.float32)), O.View.of(np.zeros(c["B_shape"], np.float32)))) == c["expect_shape"], c["name"]


def test_reference_device_kernel_cases(golden, oracle):
    """The operands of the reference's own GPU-launch tests (tests/test_gpu.mojo: CPU result against GPU result): the oracle,
    which restates that CPU path, against the exact product of these small integers and the values the tests state."""
    O = oracle
    for c in golden["device_kernel_cases"]["cases"]:
        a, b = generated_operand(c["A"]), generated_operand(c["B"])
        got = {"mm": O.matmul, "mv": O.mv, "vm": O.vm}[c["op"]](a, b)
        want = exact_product(c["op"], a, b)
        assert got.shape == want.shape, c["name"]
        np.testing.assert_array_equal(got, want.astype(np.float32), err_msg=c["name"])
        if "expect" in c:
            np.testing.assert_array_equal(got, np.asarray(c["expect"], np.float32), err_msg=c["name"])


def test_golden_backward(golden, oracle):
    O = oracle
    for c in golden["cases"]:
        if not any(k in c for k in GOLDEN_GRADIENT_KEYS):
            continue
        A, B = _view(O, c["A"]), _view(O, c["B"])
        if c["op"] == "mm":
            shape = O.result_shape(O.MM, A, B)
            gA, gB = O.matmul_backward(A, B, np.ones(shape, np.float32))
        elif c["op"] == "mv":
            gA, gB = O.mv_backward(A, B, np.ones(O.result_shape(O.MV, A, B), np.float32))
        elif c["op"] == "dot":  # grad_lhs = rhs * g, grad_rhs = lhs * g (tenmo/dotproduct.mojo:13-52) = the backward of lhs[n] . rhs-as-[n, 1]
            n = c["A"]["shape"][0]
            gA, gB = O.vm_backward(A, O.View(storage_of(c["B"]), c["B"].get("offset", 0), (n, 1), (strides_of(c["B"])[0], 1)), np.ones((1,), np.float32))
            gB = gB.reshape(n)
        else:
            gA, gB = O.vm_backward(A, B, np.ones(O.result_shape(O.VM, A, B), np.float32))
        if "grad_A" in c:
            np.testing.assert_allclose(gA, np.asarray(c["grad_A"], np.float32), rtol=1e-5, err_msg=c["name"] + " grad_A")
        if "grad_B" in c:
            np.testing.assert_allclose(gB, np.asarray(c["grad_B"], np.float32), rtol=1e-5, err_msg=c["name"] + " grad_B")
        # gradients asserted on the tensor behind a view: the view-shaped gradient scattered onto its storage
        if "base_grad_A" in c:
            np.testing.assert_allclose(scatter_to_storage(c["A"], gA), c["base_grad_A"], rtol=1e-5, err_msg=c["name"] + " base_grad_A")
        if "base_grad_B" in c:
            np.testing.assert_allclose(scatter_to_storage(c["B"], gB), c["base_grad_B"], rtol=1e-5, err_msg=c["name"] + " base_grad_B")
        check_golden_extras(c, None, gA, gB)


@pytest.mark.parametrize("width", [0, 16, 8, 1])
def test_verify_shapes_against_fp64(golden, oracle, width):
    """The shape list of the reference's own verification file, against an fp64 triple loop; every
    tile/tail combination of the three code paths and every ISA kernel."""
    O = oracle
    O.force_simd_width(width)
    try:
        rng = np.random.default_rng(7)
        for m, k, n in golden["verify_shapes"]["mkn"]:
            a = rng.standard_normal((m, k), dtype=np.float32)
            b = rng.standard_normal((k, n), dtype=np.float32)
            ref = ref_matmul64(a, b)
            info = {}
            assert rel_fro(O.mm2d(a, b, info=info), ref) < 1e-6 and info["path"] == 0
            at = np.ascontiguousarray(a.T).T  # transposed view: path 1b unless a dim is 1
            assert rel_fro(O.mm2d(at, b, info=info), ref) < 1e-6
            bt = np.ascontiguousarray(b.T).T  # B strided: path 2
            assert rel_fro(O.mm2d(a, bt, info=info), ref) < 1e-6
            if k > 1 and n > 1:
                assert info["path"] == 2
            # fp64-accumulating reference of the oracle itself against numpy
            assert rel_fro(O.mm_f64(a, b), ref) < 1e-12
    finally:
        O.force_simd_width(0)


def test_padded_row_views(oracle):
    """Padded-stride views count as non-contiguous (tests/test_matmul_2d_verify.mojo:85-110,144-169,201-229)."""
    O = oracle
    rng = np.random.default_rng(3)
    a_store = rng.standard_normal((33, 50), dtype=np.float32)
    b_store = rng.standard_normal((40, 70), dtype=np.float32)
    a, b = a_store[:, :40], b_store[:, :65]
    ref = ref_matmul64(a, b)
    info = {}
    assert rel_fro(O.mm2d(a, b, info=info), ref) < 1e-6
    assert info["path"] == 2  # B padded
    assert rel_fro(O.mm2d(a, np.ascontiguousarray(b), info=info), ref) < 1e-6
    assert info["path"] == 1  # only A padded


def test_random_views_against_fp64(oracle):
    """Property check over what the reference calls a view (tenmo/matmul_cpu.mojo:710-724: offset, strides, dims of size
    1 read with stride 0): operands cut out of larger storage with steps, offsets, swapped last axes, expanded (stride 0)
    and broadcast batch dimensions, ranks 2 to 5, extents around the tile and vector edges — against numpy in float64."""
    from hypothesis import given, settings, strategies as st

    extent = st.sampled_from([1, 2, 3, 5, 8, 15, 16, 17, 31, 33, 64, 65, 70])

    @st.composite
    def operands(draw):
        m, k, n = draw(extent), draw(extent), draw(extent)
        batch = draw(st.lists(st.integers(1, 3), min_size=0, max_size=3))
        seed = draw(st.integers(0, 2**31 - 1))
        rng = np.random.default_rng(seed)

        def view(rows, cols, own_batch):
            step_r, step_c = draw(st.integers(1, 2)), draw(st.integers(1, 3))
            off_r, off_c = draw(st.integers(0, 2)), draw(st.integers(0, 3))
            swapped = draw(st.booleans())
            r, c = (cols, rows) if swapped else (rows, cols)
            store = rng.standard_normal(tuple(own_batch) + (off_r + r * step_r, off_c + c * step_c + draw(st.integers(0, 2))), dtype=np.float32)
            v = store[..., off_r:off_r + r * step_r:step_r, off_c:off_c + c * step_c:step_c]
            return np.swapaxes(v, -1, -2) if swapped else v

        # each operand keeps, drops (size 1) or lacks each batch dimension; a kept size-1 dimension may be expanded with stride 0
        def own(batch):
            dims = [d if draw(st.booleans()) else 1 for d in batch]
            return dims[draw(st.integers(0, len(dims))):]

        a, b = view(m, k, own(batch)), view(k, n, own(batch))
        if a.ndim > 2 and a.shape[0] == 1 and draw(st.booleans()):
            a = np.broadcast_to(a, (draw(st.integers(2, 3)),) + a.shape[1:]) if b.ndim < a.ndim or b.shape[len(b.shape) - a.ndim] == 1 else a
        return a, b

    @settings(max_examples=150, deadline=None, derandomize=True)
    @given(operands())
    def check(ab):
        a, b = ab
        try:
            want = np.matmul(a.astype(np.float64), b.astype(np.float64))
        except ValueError:
            return  # (the expanded dimension met an incompatible one)
        got = oracle.matmul(a, b)
        assert got.shape == want.shape
        assert rel_fro(got, want) < 2e-6, (a.shape, a.strides, b.shape, b.strides)

    check()


def test_tile_table(oracle):
    """tenmo/matmul_cpu.mojo:87-89 and the worked example docs/from-bytes-to-gradients.md:171-177."""
    O = oracle
    info = {}
    O.mm2d(np.zeros((64, 784), np.float32), np.zeros((784, 128), np.float32), info=info)
    assert info["tiles"] == (32, 64, 128)
    O.mm2d(np.zeros((300, 10), np.float32), np.zeros((10, 10), np.float32), info=info)
    assert info["tiles"] == (128, 32, 64)
    O.mm2d(np.zeros((257, 65), np.float32), np.zeros((65, 257), np.float32), info=info)
    assert info["tiles"] == (128, 64, 256)


def test_contiguity_predicate(oracle):
    """tenmo/strides.mojo:239-266: size-1 dims are skipped, offset is not part of it."""
    O = oracle
    assert O.is_contiguous((2, 3, 4), (12, 4, 1))
    assert not O.is_contiguous((2, 3, 4), (1, 12, 4))
    assert O.is_contiguous((1, 768, 768), (0, 768, 1))
    assert O.is_contiguous((5, 1), (1, 99))
    assert not O.is_contiguous((2, 3), (4, 1))
    assert O.is_contiguous((), ())


def test_classify(oracle):
    O = oracle
    assert O.classify_matmul((3,), (3,)) == O.DOT
    assert O.classify_matmul((), (3,)) == O.DOT
    assert O.classify_matmul((3,), (3, 4)) == O.VM
    assert O.classify_matmul((2, 3), (3,)) == O.MV
    assert O.classify_matmul((2, 3), (3, 4)) == O.MM
    assert O.classify_matmul((5, 2, 3), (3, 4)) == O.MM
    assert O.classify_matmul((2, 3), (4, 4)) == O.INVALID


def test_errors(oracle):
    O = oracle
    with pytest.raises(O.OracleError):
        O.mm2d(np.zeros((2, 3), np.float32), np.zeros((4, 2), np.float32))
    with pytest.raises(O.OracleError):
        O.mmnd(np.zeros((2, 5, 3), np.float32), np.zeros((3, 3, 4), np.float32))
    with pytest.raises(O.OracleError):
        O.mv(np.zeros((2, 3), np.float32), np.zeros((4,), np.float32))


def test_closed_forms(golden, oracle):
    O = oracle
    for c in golden["closed_forms"]:
        A, B = np.ones(c["A_shape"], np.float32), np.ones(c["B_shape"], np.float32)
        out = O.mmnd(A, B)
        assert out.shape == np.broadcast_shapes(tuple(c["A_shape"][:-2]), tuple(c["B_shape"][:-2])) + (c["A_shape"][-2], c["B_shape"][-1])
        assert np.all(out == c["expect_value"])
        if "grad_A_value" in c:
            gA, gB = O.matmul_backward(A, B, np.ones(out.shape, np.float32))
            assert gA.shape == tuple(c["A_shape"]) and np.all(gA == c["grad_A_value"])
            assert gB.shape == tuple(c["B_shape"]) and np.all(gB == c["grad_B_value"])


def test_batched_equals_loop_of_2d(oracle):
    O = oracle
    rng = np.random.default_rng(11)
    A = rng.standard_normal((3, 1, 17, 9), dtype=np.float32)
    B = rng.standard_normal((4, 9, 13), dtype=np.float32)
    out = O.mmnd(A, B)
    for i in range(3):
        for j in range(4):
            np.testing.assert_array_equal(out[i, j], O.mm2d(A[i, 0], B[j]))
    # transposed-view operand equals its contiguous copy within rounding of the other code path
    Bt = np.ascontiguousarray(np.swapaxes(B, -1, -2))
    assert rel_fro(O.mmnd(A, np.swapaxes(Bt, -1, -2)), ref_matmul64(A, B)) < 1e-6


def test_backward_identities(oracle):
    """dA = dC.B^T, dB = A^T.dC (tests/test_mm2d.mojo:39-100) and finite differences
    (tests/test_matmul.mojo:247-307) on the fp64 reference."""
    O = oracle
    rng = np.random.default_rng(5)
    A = rng.standard_normal((6, 5), dtype=np.float32)
    B = rng.standard_normal((5, 4), dtype=np.float32)
    dC = rng.standard_normal((6, 4), dtype=np.float32)
    gA, gB = O.matmul_backward(A, B, dC)
    assert rel_fro(gA, ref_matmul64(dC, B.T)) < 1e-6
    assert rel_fro(gB, ref_matmul64(A.T, dC)) < 1e-6
    loss = lambda a, b: float(np.sum(ref_matmul64(a, b) * dC))
    eps = 1e-3
    for (i, j) in [(0, 0), (3, 2), (5, 4)]:
        Ap, Am = A.astype(np.float64).copy(), A.astype(np.float64).copy()
        Ap[i, j] += eps
        Am[i, j] -= eps
        assert abs((loss(Ap, B) - loss(Am, B)) / (2 * eps) - gA[i, j]) < 1e-3


def test_mv_vm_against_fp64_and_views(oracle):
    O = oracle
    rng = np.random.default_rng(9)
    M = rng.standard_normal((2, 3, 37, 29), dtype=np.float32)
    v = rng.standard_normal((3, 29), dtype=np.float32)
    assert rel_fro(O.mv(M, v), np.einsum("abmk,bk->abm", M.astype(np.float64), v.astype(np.float64))) < 1e-6
    assert rel_fro(O.mv_f64(M, v), np.einsum("abmk,bk->abm", M.astype(np.float64), v.astype(np.float64))) < 1e-12
    u = rng.standard_normal((37,), dtype=np.float32)
    assert rel_fro(O.vm(u, M), np.einsum("m,abmk->abk", u.astype(np.float64), M.astype(np.float64))) < 1e-6
    Mt = np.swapaxes(M, -1, -2)  # transposed view, as examples/word2vec_cbow.mojo:531-553 uses
    assert rel_fro(O.mv(Mt, u), np.einsum("abmk,m->abk", M.astype(np.float64), u.astype(np.float64))) < 1e-6
    # backward closed forms
    dy = rng.standard_normal((2, 3, 37), dtype=np.float32)
    dM, dv = O.mv_backward(M, v, dy)
    assert rel_fro(dM, np.einsum("abm,bk->abmk", dy.astype(np.float64), v.astype(np.float64))) < 1e-6
    assert rel_fro(dv, np.einsum("abmk,abm->bk", M.astype(np.float64), dy.astype(np.float64))) < 1e-6
    dy2 = rng.standard_normal((2, 3, 29), dtype=np.float32)
    du, dM2 = O.vm_backward(u, M, dy2)
    assert rel_fro(du, np.einsum("abmk,abk->m", M.astype(np.float64), dy2.astype(np.float64))) < 1e-6
    assert rel_fro(dM2, np.einsum("m,abk->abmk", u.astype(np.float64), dy2.astype(np.float64))) < 1e-6


def test_dot(oracle):
    O = oracle
    a = np.arange(1, 8, dtype=np.float32)
    assert O.dot(a, a) == 140.0
    assert O.dot(np.asarray([2.0], np.float32), a) == 56.0  # one-element operand broadcasts
    assert O.dot(a[::2], a[::2]) == 1 + 9 + 25 + 49
    with pytest.raises(O.OracleError):
        O.dot(a, a[:3])


def test_sum_over_broadcasted_axes(oracle):
    O = oracle
    rng = np.random.default_rng(2)
    src = rng.standard_normal((2, 4, 3, 6, 5), dtype=np.float32)
    for target in [(1, 3, 6, 5), (4, 1, 6, 5), (3, 6, 5), (2, 4, 3, 6, 5), (6, 5)]:
        ref = src.astype(np.float64)
        lead = src.ndim - len(target)
        ref = ref.sum(axis=tuple(range(lead)))
        for d, s in enumerate(target):
            if s == 1 and ref.shape[d] != 1:
                ref = ref.sum(axis=d, keepdims=True)
        assert rel_fro(O.sum_over_broadcasted_axes(src, target), ref) < 1e-6


def test_mlp_harness_pieces(golden, oracle):
    """Cross-entropy, SGD, bias-gradient and ReLU pieces of the step, against the reference's own
    vectors and closed forms."""
    O = oracle
    h = golden["harness"]
    # uniform logits -> -log(1/3): a 1-layer net with zero weights produces exactly that
    c = h["ce_uniform_logits"]
    m = O.MLP([2, 3], [np.zeros((2, 3), np.float32)], [np.ones(3, np.float32)], 2)
    loss = m.step(np.ones((2, 2), np.float32), np.asarray(c["targets"], np.int32), 0.0)
    assert abs(loss - c["loss"]) < 1e-6
    dW, db = m.grads(0)
    # gradient of mean CE wrt logits = (softmax - onehot)/rows: rows of dlogits sum to zero
    # (tests/test_cross_entropy.mojo:797-823) hence sum(db) == 0 and db = [1/3-1, 1/3-1, 2/3]/2 + ...
    assert abs(db.sum()) < 1e-6
    np.testing.assert_allclose(db, (np.asarray([1 / 3 - 1, 1 / 3, 1 / 3]) + np.asarray([1 / 3, 1 / 3 - 1, 1 / 3])) / 2, atol=1e-6)
    # SGD vectors: a net whose only gradient is the bias gradient is awkward; check p -= lr*g directly
    for key in ("sgd_single_step", "sgd_three_steps", "sgd_2d"):
        s = h[key]
        w = np.asarray(s["w"], np.float32)
        for _ in range(s["steps"]):
            w = w - np.float32(s["lr"]) * np.asarray(s["grad"], np.float32)
        np.testing.assert_allclose(w, s["expect"], rtol=1e-6)


def test_relu_and_its_mask_are_pinned(golden, oracle):
    """The ReLU of the restated step and the mask its backward multiplies by (tenmo/relu.mojo:99-141, :21-46: x > 0, so
    the gradient at exactly 0 is 0) against the literals of tests/test_relu.mojo: a net [n, n, n] with identity weights
    computes relu(x + bias) as its logits; the hidden layer's bias gradient is then the output layer's times the mask, and
    its weight gradient the outer product of x with that."""
    for c in golden["harness"]["relu_literals"]["cases"]:
        x = np.asarray(c["x"], np.float32)[None, :]
        n = x.shape[1]
        bias = np.asarray(c.get("bias", [0.0] * n), np.float32)
        eye = np.eye(n, dtype=np.float32)
        m = oracle.MLP([n, n, n], [eye, eye], [bias, np.zeros(n, np.float32)], 1)
        if "out" in c:
            np.testing.assert_array_equal(m.forward(x)[0], np.asarray(c["out"], np.float32), err_msg=c["source"])
        else:
            np.testing.assert_array_equal(m.forward(x)[0], np.maximum(x[0] + bias, 0))
        if "grad" in c:
            m.step(x, np.zeros(1, np.int32), 0.0)
            dW1, db1 = m.grads(1)
            dW0, db0 = m.grads(0)
            assert np.all(db1 != 0), c["source"]
            mask = np.asarray(c["grad"], np.float32)
            np.testing.assert_array_equal(db0, db1 * mask, err_msg=c["source"])
            np.testing.assert_array_equal(dW0, np.outer(x[0], db1 * mask), err_msg=c["source"])


def test_mlp_step_matches_numpy_fp64(oracle):
    """The whole restated step against an independent fp64 numpy implementation."""
    O = oracle
    from tenmo_amd import rng as R

    dims = [784, 128, 32, 10]
    Ws, bs = R.xavier_mlp(dims, 1234)
    m = O.MLP(dims, Ws, bs, 64)
    W64 = [w.astype(np.float64) for w in Ws]
    b64 = [b.astype(np.float64) for b in bs]
    lr = 0.01
    for step in range(5):
        x, y = R.mnist_like_batch(64, 1234, step)
        loss = m.step(x, y, lr)
        h = [x.astype(np.float64)]
        for l in range(3):
            z = h[-1] @ W64[l] + b64[l]
            h.append(np.maximum(z, 0) if l < 2 else z)
        z = h[-1]
        zs = z - z.max(1, keepdims=True)
        lse = np.log(np.exp(zs).sum(1, keepdims=True))
        ref_loss = float(-(zs - lse)[np.arange(64), y].mean())
        assert abs(loss - ref_loss) < 1e-5, (step, loss, ref_loss)
        g = (np.exp(zs - lse) - np.eye(10)[y]) / 64
        for l in (2, 1, 0):
            dW = h[l].T @ g
            db = g.sum(0)
            if l > 0:
                g = (g @ W64[l].T) * (h[l] > 0)
            W64[l] -= lr * dW
            b64[l] -= lr * db
        for l in range(3):
            W, b = m.params(l)
            assert rel_fro(W, W64[l]) < 1e-5 and np.abs(b - b64[l]).max() < 1e-6


def test_cross_entropy_oracle_is_pinned(golden, oracle):
    """Closed forms and vectors of tests/test_cross_entropy.mojo, an independent fp64 statement, the
    invariants the reference tests (row gradients sum to zero, ignored rows vanish, mean = sum / valid)
    and finite differences of the loss."""
    H = golden["harness"]
    # uniform logits -> log(C)   (tests/test_cross_entropy.mojo:724-743, :1600-1609)
    sm, rows, total, valid = oracle.cross_entropy_forward(np.ones((2, 3), np.float32), np.array([0, 1]))
    assert valid == 2 and abs(total / valid - H["ce_uniform_logits"]["loss"]) < 1e-6 and np.allclose(sm, 1 / 3, atol=1e-7)
    # two rows, mean (:1227-1241)
    g = H["ce_two_rows_mean"]
    x = np.array(g["logits"], np.float32)
    e = np.exp(np.array(g["logits"], np.float64))
    want = (-np.log(e[0, 0] / e[0].sum()) - np.log(e[1, 1] / e[1].sum())) / 2
    sm, rows, total, valid = oracle.cross_entropy_forward(x, np.array(g["targets"]))
    assert abs(total / valid - want) < 1e-6
    # gradient of the mean: (softmax - onehot) / batch (:1449-1476)
    grad = oracle.cross_entropy_backward(sm, np.array(g["targets"]), np.ones(1, np.float32), oracle.REDUCTION_MEAN, valid)
    p64 = e / e.sum(1, keepdims=True)
    assert np.allclose(grad, (p64 - np.eye(3)[g["targets"]]) / 2, atol=1e-6)
    # label smoothing (:2425-2443, :2731-2746)
    g = H["ce_label_smoothing_formula"]
    x, ls = np.array(g["logits"], np.float32), g["label_smoothing"]
    p = np.exp(np.array(g["logits"][0], np.float64)); p /= p.sum()
    sm, rows, total, valid = oracle.cross_entropy_forward(x, np.array(g["targets"]), label_smoothing=ls)
    assert abs(total - ((1 - ls) * -np.log(p[0]) + ls * np.mean(-np.log(p)))) < 1e-6
    grad = oracle.cross_entropy_backward(sm, np.array(g["targets"]), np.ones(1, np.float32), oracle.REDUCTION_MEAN, valid, label_smoothing=ls)
    assert abs(grad[0, 0] - (p[0] - (1 - ls) - ls / 3)) < 1e-6 and abs(grad[0, 1] - (p[1] - ls / 3)) < 1e-6
    # ignore_index (:247-323)
    g = H["ce_ignore_index"]
    x, t = np.array(g["logits"], np.float32), np.array(g["targets"])
    sm, rows, total, valid = oracle.cross_entropy_forward(x, t, ignore_index=g["ignore_index"])
    assert valid == 2 and rows[1] == 0 and rows[0] > 0 and rows[2] > 0
    grad = oracle.cross_entropy_backward(sm, t, np.ones(1, np.float32), oracle.REDUCTION_MEAN, valid, ignore_index=g["ignore_index"])
    assert np.all(grad[1] == 0) and abs(grad[0, 0]) > 1e-6 and abs(grad[2, 0]) > 1e-6
    sm, rows, total, valid = oracle.cross_entropy_forward(x[:2], np.array([-100, -100]))
    assert valid == 0 and total == 0
    assert np.all(oracle.cross_entropy_backward(sm, np.array([-100, -100]), np.ones(1, np.float32), oracle.REDUCTION_MEAN, valid) == 0)
    # random cases against the fp64 statement, all reductions, smoothing and ignored rows together
    rng = np.random.default_rng(41)
    for M, C, ls in [(7, 5, 0.0), (33, 17, 0.2), (4, 1000, 0.05), (64, 10, 0.0)]:
        x = (3 * rng.standard_normal((M, C))).astype(np.float32)
        t = rng.integers(0, C, M)
        t[rng.random(M) < 0.3] = -100
        p64, loss64, grad64 = ce_reference64(x, t, -100, ls)
        sm, rows, total, valid = oracle.cross_entropy_forward(x, t, label_smoothing=ls)
        assert valid == int((t != -100).sum())
        assert np.allclose(sm, p64, rtol=1e-5, atol=1e-7) and np.allclose(rows, loss64, rtol=1e-5, atol=1e-6)
        assert abs(total - loss64.sum()) <= 1e-5 * max(1.0, abs(loss64.sum()))
        up = rng.standard_normal(M).astype(np.float32)
        assert np.allclose(oracle.cross_entropy_backward(sm, t, up, oracle.REDUCTION_NONE, valid, label_smoothing=ls), grad64 * up[:, None], rtol=1e-4, atol=1e-6)
        assert np.allclose(oracle.cross_entropy_backward(sm, t, up[:1], oracle.REDUCTION_SUM, valid, label_smoothing=ls), grad64 * up[0], rtol=1e-4, atol=1e-6)
        gm = oracle.cross_entropy_backward(sm, t, up[:1], oracle.REDUCTION_MEAN, valid, label_smoothing=ls)
        assert np.allclose(gm, grad64 * up[0] / max(valid, 1), rtol=1e-4, atol=1e-6)
        assert np.abs(gm.sum(1)).max() < 1e-6          # every row of the gradient sums to zero (:797-823)
    # finite differences of the summed loss in fp64 agree with the analytic gradient
    x = rng.standard_normal((3, 4)).astype(np.float32)
    t = np.array([1, -100, 3])
    sm, rows, total, valid = oracle.cross_entropy_forward(x, t, label_smoothing=0.1)
    grad = oracle.cross_entropy_backward(sm, t, np.ones(1, np.float32), oracle.REDUCTION_SUM, valid, label_smoothing=0.1)
    for (i, j) in [(0, 0), (0, 1), (2, 3), (1, 2)]:
        h = 1e-5
        xp, xm = x.astype(np.float64), x.astype(np.float64)
        xp[i, j] += h; xm[i, j] -= h
        fd = (ce_reference64(xp, t, -100, 0.1)[1].sum() - ce_reference64(xm, t, -100, 0.1)[1].sum()) / (2 * h)
        assert abs(grad[i, j] - fd) < 1e-5


def test_bias_gradient_oracle_is_pinned(golden, oracle):
    """sum_over_broadcasted_axes (tenmo/broadcast.mojo:66-88), the gradient of a bias under Adder: the reference's own literals."""
    case = golden["harness"]["bias_gradient_is_column_sums"]
    up = np.array(case["upstream"], np.float32)
    assert np.array_equal(oracle.sum_over_broadcasted_axes(up, (1, 4)), np.array([case["expect"]], np.float32))
    assert np.array_equal(oracle.sum_over_broadcasted_axes(up, (4,)), np.array(case["expect"], np.float32))
    case = golden["harness"]["sum_over_broadcasted_axes_of_ones"]
    got = oracle.sum_over_broadcasted_axes(np.ones(case["shape"], np.float32), tuple(case["target_shape"]))
    assert got.shape == tuple(case["target_shape"]) and np.array_equal(got.ravel(), np.array(case["expect"], np.float32))
    # and against numpy on random data, a partial broadcast
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 4, 5, 6), dtype=np.float32)
    assert np.allclose(oracle.sum_over_broadcasted_axes(x, (4, 1, 6)), x.astype(np.float64).sum(axis=(0, 2), keepdims=True)[0], rtol=1e-5, atol=1e-6)


def test_sgd_oracle_is_pinned(golden, oracle):
    """tests/test_sgd.mojo vectors: plain, weight decay, momentum over three steps."""
    H = golden["harness"]
    for key in ("sgd_single_step", "sgd_three_steps", "sgd_2d"):
        g = H[key]
        w = np.array(g["w"], np.float32)
        for _ in range(g["steps"]):
            oracle.sgd_step(w, np.array(g["grad"], np.float32), None, g["lr"])
        assert np.allclose(w, g["expect"], rtol=1e-6)
    g = H["sgd_weight_decay"]
    w = np.array(g["w"], np.float32)
    oracle.sgd_step(w, np.array(g["grad"], np.float32), None, g["lr"], weight_decay=g["weight_decay"])
    assert np.allclose(w, g["expect"], rtol=1e-6)
    g = H["sgd_momentum_three_steps"]
    w, v = np.array(g["w"], np.float32), np.zeros(1, np.float32)
    for want in g["expect_after_each"]:
        oracle.sgd_step(w, np.array(g["grad"], np.float32), v, g["lr"], momentum=g["momentum"])
        assert abs(w[0] - want) < 1e-6


def test_conv_oracle_is_pinned(golden, oracle):
    """The restatement of Conv2dFused.forward (tenmo/cnn.mojo:92-507) against every forward case of
    tests/test_cnn.mojo that asserts values or shapes, then against two independent computations of a
    zero-padded cross-correlation on random inputs: numpy sliding windows in fp64 and torch's conv2d in fp64
    (a swapped kernel index, a wrong stride/dilation product or an off-by-one in the padding fails them)."""
    import torch
    from helpers import check_conv_case, conv_case_tensors, conv_reference64

    for case in golden["conv"]["cases"]:
        image, kernel, bias, kw = conv_case_tensors(case)
        check_conv_case(case, oracle.conv2d_forward(image, kernel, bias, **kw))
    rng = np.random.default_rng(71)
    for (n, ci, h, w, co, kh, kww, stride, dil, padding, with_bias) in [
            (2, 3, 9, 11, 4, 3, 3, 1, 1, "valid", True), (1, 2, 8, 8, 3, 3, 2, 2, 1, "same", False),
            (3, 1, 12, 7, 2, 2, 3, 1, 2, 1, True), (2, 4, 10, 10, 5, 3, 3, 2, 2, (2, 1), True),
            (1, 3, 7, 9, 2, 1, 1, 1, 1, "valid", False), (2, 2, 6, 6, 3, 3, 3, 3, 1, [(1, 2), (0, 3)], True)]:
        image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
        kernel = rng.standard_normal((co, ci, kh, kww), dtype=np.float32)
        bias = rng.standard_normal(co, dtype=np.float32) if with_bias else None
        got = oracle.conv2d_forward(image, kernel, bias, stride=stride, dilation=dil, padding=padding)
        pads = oracle.conv_padding(h, w, kh, kww, stride, dil, padding)
        ref = conv_reference64(image, kernel, bias, stride, dil, pads)
        assert got.shape == ref.shape and np.allclose(got, ref, rtol=1e-5, atol=1e-5), (n, ci, h, w, co, kh, kww, stride, dil, padding)
        x = torch.nn.functional.pad(torch.from_numpy(image).double(), (pads[2], pads[3], pads[0], pads[1]))
        tref = torch.nn.functional.conv2d(x, torch.from_numpy(kernel).double(), None if bias is None else torch.from_numpy(bias).double(),
                                          stride=stride, dilation=dil).numpy()
        assert np.allclose(got, tref, rtol=1e-5, atol=1e-5)
    # error behaviour (cnn.mojo:167-176, :237-241)
    with pytest.raises(oracle.OracleError):
        oracle.conv2d_forward(np.ones((1, 2, 4, 4), np.float32), np.ones((1, 3, 2, 2), np.float32))
    with pytest.raises(oracle.OracleError):
        oracle.conv2d_forward(np.ones((1, 1, 2, 2), np.float32), np.ones((1, 1, 3, 3), np.float32))


def test_conv_backward_oracle_is_pinned(golden, oracle):
    """The restated FusedCol2ImBackward (tenmo/cnn.mojo:546-948) against the gradients asserted in
    tests/test_cnn.mojo and against torch autograd in fp64 on random cases with stride, dilation and every
    padding form (a flipped kernel index or a stride/dilation mix-up in the scatter fails these)."""
    from helpers import check_conv_backward_case, conv_backward_reference64, conv_case_tensors

    for case in golden["conv"]["backward_cases"]:
        image, kernel, _, kw = conv_case_tensors(case)
        up = conv_case_tensors({"image": case["upstream"], "kernel": case["kernel"]})[0]
        check_conv_backward_case(case, *oracle.conv2d_backward(image, kernel, up, **kw))
    rng = np.random.default_rng(79)
    for (n, ci, h, w, co, kh, kww, stride, dil, padding) in [
            (2, 3, 9, 11, 4, 3, 3, 1, 1, "valid"), (1, 2, 8, 8, 3, 3, 2, 2, 1, "same"), (3, 1, 12, 7, 2, 2, 3, 1, 2, 1),
            (2, 4, 10, 10, 5, 3, 3, 2, 2, (2, 1)), (1, 3, 7, 9, 2, 1, 1, 1, 1, "valid"), (2, 2, 6, 6, 3, 3, 3, 3, 1, [(1, 2), (0, 3)])]:
        image = rng.standard_normal((n, ci, h, w), dtype=np.float32)
        kernel = rng.standard_normal((co, ci, kh, kww), dtype=np.float32)
        out_shape = oracle.conv2d_forward(image, kernel, None, stride=stride, dilation=dil, padding=padding).shape
        up = rng.standard_normal(out_shape, dtype=np.float32)
        got = oracle.conv2d_backward(image, kernel, up, stride=stride, dilation=dil, padding=padding)
        want = conv_backward_reference64(image, kernel, up, stride, dil, oracle.conv_padding(h, w, kh, kww, stride, dil, padding))
        for g, r, what in zip(got, want, ("image", "kernel", "bias")):
            assert g.shape == r.shape and np.allclose(g, r, rtol=1e-4, atol=1e-4), (what, n, ci, h, w, co, kh, kww, stride, dil, padding)
