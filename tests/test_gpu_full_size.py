"""The benchmark configurations at their full sizes, checked through properties that do not need
a full CPU recomputation: sampled rows/batches against fp64 dot products, transposed-view ==
contiguous-copy, accumulate twice == 2x, broadcast batch == loop of 2-D products.
Tolerance: relative Frobenius error <= 1e-5 against fp64 on the sampled entries."""
import ctypes as C

import numpy as np
import pytest

from helpers import RTOL_FRO, rel_fro

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    from tenmo_amd import _lib

    _lib.init(0)

    class E:
        L = _lib.load()
        lib = _lib
        t = torch

    return E


def gemm(E, A, a_str, B, b_str, Cc, M, N, K, batch_shape=(), a_b=(), b_b=(), acc=0, a_off=0, b_off=0):
    E.lib.check(E.L.tenmo_hip_gemm_f32(A.data_ptr(), a_off, a_str[0], a_str[1], B.data_ptr(), b_off, b_str[0], b_str[1], Cc.data_ptr(),
                                       M, N, K, len(batch_shape), E.lib.i64(batch_shape), E.lib.i64(a_b), E.lib.i64(b_b), acc, 0))


def randn(E, shape, seed, std=1.0):
    g = E.t.Generator(device="cuda")
    g.manual_seed(seed)
    return E.t.randn(shape, generator=g, device="cuda", dtype=E.t.float32) * std


def sampled_rows_error(E, Cc, A, B, rows, transposed_a=False):
    """fp64 recomputation of a few rows of C = A.B on the host."""
    idx = E.t.tensor(rows, device="cuda")
    a = (A[:, idx].T if transposed_a else A[idx]).double().cpu().numpy()
    ref = a @ B.double().cpu().numpy() if B.shape[0] * B.shape[1] <= 2**27 else None
    if ref is None:  # very wide B: multiply in column chunks to bound host memory
        parts = [a @ B[:, j:j + 8192].double().cpu().numpy() for j in range(0, B.shape[1], 8192)]
        ref = np.concatenate(parts, axis=1)
    return rel_fro(Cc[idx].cpu().numpy(), ref)


@pytest.mark.parametrize("S", [1024, 2048, 4096, 8192])
def test_square_sweep(env, S):
    """config: square GEMM, A row-major and A as a transposed view."""
    E = env
    A, B = randn(E, (S, S), 1), randn(E, (S, S), 2)
    Cc = E.t.empty(S, S, device="cuda")
    rows = [0, 1, S // 3, S // 2 + 5, S - 1]
    gemm(E, A, (S, 1), B, (S, 1), Cc, S, S, S)
    assert sampled_rows_error(E, Cc, A, B, rows) <= RTOL_FRO
    # A given as a transposed view: storage [K, M], strides (1, M)
    Ct = E.t.empty(S, S, device="cuda")
    gemm(E, A, (1, S), B, (S, 1), Ct, S, S, S)
    assert sampled_rows_error(E, Ct, A, B, rows, transposed_a=True) <= RTOL_FRO
    # the view result equals the product of the contiguous copy (same kernel arithmetic, other loader)
    At = A.t().contiguous()
    C2 = E.t.empty(S, S, device="cuda")
    gemm(E, At, (S, 1), B, (S, 1), C2, S, S, S)
    assert rel_fro(Ct.cpu().numpy(), C2.cpu().numpy()) <= 2e-6
    # accumulate: a second pass doubles
    gemm(E, A, (S, 1), B, (S, 1), Cc, S, S, S, acc=1)
    assert sampled_rows_error(E, Cc * 0.5, A, B, rows) <= RTOL_FRO


def test_attention_shapes(env):
    """config: Q[8,12,1024,64] . K^T (transposed view) -> S, P = softmax(S), P . V, and the four backward GEMMs."""
    E = env
    Bn, H, T_, D = 8, 12, 1024, 64
    Q, K, V = randn(E, (Bn, H, T_, D), 3), randn(E, (Bn, H, T_, D), 4), randn(E, (Bn, H, T_, D), 5)
    S_ = E.t.empty(Bn, H, T_, T_, device="cuda")
    bs, st = (Bn, H), (H * T_ * D, T_ * D)
    gemm(E, Q, (D, 1), K, (1, D), S_, T_, T_, D, bs, st, st)
    for (b, h) in [(0, 0), (3, 7), (7, 11)]:
        ref = Q[b, h].double() @ K[b, h].double().T
        assert rel_fro(S_[b, h].cpu().numpy(), ref.cpu().numpy()) <= RTOL_FRO
    P = E.t.softmax(S_ / 8.0, dim=-1)
    O_ = E.t.empty(Bn, H, T_, D, device="cuda")
    pst = (H * T_ * T_, T_ * T_)
    gemm(E, P, (T_, 1), V, (D, 1), O_, T_, D, T_, bs, pst, st)
    for (b, h) in [(0, 0), (5, 2), (7, 11)]:
        ref = P[b, h].double() @ V[b, h].double()
        assert rel_fro(O_[b, h].cpu().numpy(), ref.cpu().numpy()) <= RTOL_FRO
    dO, dS = randn(E, (Bn, H, T_, D), 6), randn(E, (Bn, H, T_, T_), 7)
    dP = E.t.empty(Bn, H, T_, T_, device="cuda")
    gemm(E, dO, (D, 1), V, (1, D), dP, T_, T_, D, bs, st, st)            # dP = dO . V^T
    dV = E.t.empty(Bn, H, T_, D, device="cuda")
    gemm(E, P, (1, T_), dO, (D, 1), dV, T_, D, T_, bs, pst, st)          # dV = P^T . dO
    dQ = E.t.empty(Bn, H, T_, D, device="cuda")
    gemm(E, dS, (T_, 1), K, (D, 1), dQ, T_, D, T_, bs, pst, st)          # dQ = dS . K
    dKt = E.t.empty(Bn, H, D, T_, device="cuda")
    gemm(E, Q, (1, D), dS, (T_, 1), dKt, D, T_, T_, bs, st, pst)         # Q^T . dS
    b, h = 6, 9
    assert rel_fro(dP[b, h].cpu().numpy(), (dO[b, h].double() @ V[b, h].double().T).cpu().numpy()) <= RTOL_FRO
    assert rel_fro(dV[b, h].cpu().numpy(), (P[b, h].double().T @ dO[b, h].double()).cpu().numpy()) <= RTOL_FRO
    assert rel_fro(dQ[b, h].cpu().numpy(), (dS[b, h].double() @ K[b, h].double()).cpu().numpy()) <= RTOL_FRO
    assert rel_fro(dKt[b, h].cpu().numpy(), (Q[b, h].double().T @ dS[b, h].double()).cpu().numpy()) <= RTOL_FRO


def test_readme_broadcast_case(env):
    """config: A[32,512,768] . B[1,768,768] with backward; dB is reduced over the broadcast batch."""
    E = env
    A, B = randn(E, (32, 512, 768), 8), randn(E, (1, 768, 768), 9)
    av = E.lib.make_view(A.data_ptr(), 0, A.shape, A.stride())
    bv = E.lib.make_view(B.data_ptr(), 0, B.shape, B.stride())
    Cc = E.t.empty(32, 512, 768, device="cuda")
    E.lib.check(E.L.tenmo_hip_matmul_nd(C.byref(av), C.byref(bv), Cc.data_ptr(), 0))
    for b in (0, 17, 31):
        assert rel_fro(Cc[b].cpu().numpy(), (A[b].double() @ B[0].double()).cpu().numpy()) <= RTOL_FRO
    dC = randn(E, (32, 512, 768), 10)
    gA, gB = E.t.zeros_like(A), E.t.zeros_like(B)
    E.lib.check(E.L.tenmo_hip_matmul_backward(C.byref(av), C.byref(bv), dC.data_ptr(), gA.data_ptr(), gB.data_ptr(), 0))
    assert rel_fro(gA[5].cpu().numpy(), (dC[5].double() @ B[0].double().T).cpu().numpy()) <= RTOL_FRO
    ref = (A.double().reshape(-1, 768).T @ dC.double().reshape(-1, 768)).cpu().numpy()
    assert gB.shape == (1, 768, 768) and rel_fro(gB[0].cpu().numpy(), ref) <= RTOL_FRO


@pytest.mark.parametrize("name,N", [("qkv", 2304), ("proj", 768), ("up", 3072), ("lm_head", 50257)])
def test_gpt2_linears(env, name, N):
    """config: 8192 tokens, d=768: forward, dX = dY.W^T, dW = X^T.dY."""
    E = env
    Tk, D = 8192, 768
    X, W, dY = randn(E, (Tk, D), 11), randn(E, (D, N), 12, 0.02), randn(E, (Tk, N), 13)
    Y = E.t.empty(Tk, N, device="cuda")
    gemm(E, X, (D, 1), W, (N, 1), Y, Tk, N, D)
    rows = [0, 4095, 8191]
    assert sampled_rows_error(E, Y, X, W, rows) <= RTOL_FRO
    dX = E.t.empty(Tk, D, device="cuda")
    gemm(E, dY, (N, 1), W, (1, N), dX, Tk, D, N)
    idx = E.t.tensor(rows, device="cuda")
    assert rel_fro(dX[idx].cpu().numpy(), (dY[idx].double() @ W.double().T).cpu().numpy()) <= RTOL_FRO
    dW = E.t.empty(D, N, device="cuda")
    gemm(E, X, (1, D), dY, (N, 1), dW, D, N, Tk)
    ridx = E.t.tensor([0, 383, 767], device="cuda")
    ref = X[:, ridx].double().T @ dY.double() if N < 10000 else None
    if ref is None:
        cols = slice(50000, 50257)
        ref = X[:, ridx].double().T @ dY[:, cols].double()
        assert rel_fro(dW[ridx][:, cols].cpu().numpy(), ref.cpu().numpy()) <= RTOL_FRO
    else:
        assert rel_fro(dW[ridx].cpu().numpy(), ref.cpu().numpy()) <= RTOL_FRO


def test_mlp_down_projection(env):
    """config: the MLP down projection [8192,3072].[3072,768], forward and both gradient products
    dX = dY.W^T(view) and dW = X^T(view).dY, through the plain entry and through the backward entry (+=)."""
    E = env
    Tk, D, N = 8192, 3072, 768
    X, W, dY = randn(E, (Tk, D), 14), randn(E, (D, N), 15, 0.02), randn(E, (Tk, N), 23)
    Y = E.t.empty(Tk, N, device="cuda")
    gemm(E, X, (D, 1), W, (N, 1), Y, Tk, N, D)
    rows = [1, 5000, 8190]
    assert sampled_rows_error(E, Y, X, W, rows) <= RTOL_FRO
    idx = E.t.tensor(rows, device="cuda")
    dX = E.t.empty(Tk, D, device="cuda")
    gemm(E, dY, (N, 1), W, (1, N), dX, Tk, D, N)                      # [8192,768] . [768,3072] as a transposed view
    ref_dx = (dY[idx].double() @ W.double().T).cpu().numpy()
    assert rel_fro(dX[idx].cpu().numpy(), ref_dx) <= RTOL_FRO
    dW = E.t.empty(D, N, device="cuda")
    gemm(E, X, (1, D), dY, (N, 1), dW, D, N, Tk)                      # [3072,8192] transposed view . [8192,768]
    ridx = E.t.tensor([0, 1535, 3071], device="cuda")
    ref_dw = (X[:, ridx].double().T @ dY.double()).cpu().numpy()
    assert rel_fro(dW[ridx].cpu().numpy(), ref_dw) <= RTOL_FRO
    # the backward entry accumulates into the gradboxes: called twice it leaves exactly twice the gradient
    xv = E.lib.make_view(X.data_ptr(), 0, X.shape, X.stride())
    wv = E.lib.make_view(W.data_ptr(), 0, W.shape, W.stride())
    gX, gW = E.t.zeros_like(X), E.t.zeros_like(W)
    E.lib.check(E.L.tenmo_hip_matmul_backward(C.byref(xv), C.byref(wv), dY.data_ptr(), gX.data_ptr(), gW.data_ptr(), 0))
    assert rel_fro(gX[idx].cpu().numpy(), ref_dx) <= RTOL_FRO and rel_fro(gW[ridx].cpu().numpy(), ref_dw) <= RTOL_FRO
    E.lib.check(E.L.tenmo_hip_matmul_backward(C.byref(xv), C.byref(wv), dY.data_ptr(), gX.data_ptr(), gW.data_ptr(), 0))
    assert rel_fro(gX[idx].cpu().numpy(), 2 * ref_dx) <= RTOL_FRO and rel_fro(gW[ridx].cpu().numpy(), 2 * ref_dw) <= RTOL_FRO


def test_memory_bound_cases(env):
    """config: mv / vm at 16384^2, skinny [4,768].[768,50257], CBOW [256,100].[100,50000] + A^T.dC."""
    E = env
    n = 16384
    W, x = randn(E, (n, n), 16), randn(E, (n,), 17)
    out = E.t.empty(n, device="cuda")
    E.lib.check(E.L.tenmo_hip_mv_f32(W.data_ptr(), 0, n, 1, x.data_ptr(), 0, 1, out.data_ptr(), n, n, 0, None, None, None, 0, 0))
    assert rel_fro(out.cpu().numpy(), (W.double() @ x.double()).cpu().numpy()) <= RTOL_FRO
    E.lib.check(E.L.tenmo_hip_vm_f32(x.data_ptr(), 0, 1, W.data_ptr(), 0, n, 1, out.data_ptr(), n, n, 0, None, None, None, 0, 0))
    assert rel_fro(out.cpu().numpy(), (x.double() @ W.double()).cpu().numpy()) <= RTOL_FRO
    # mv on the transposed view equals vm on the matrix
    out2 = E.t.empty(n, device="cuda")
    E.lib.check(E.L.tenmo_hip_mv_f32(W.data_ptr(), 0, 1, n, x.data_ptr(), 0, 1, out2.data_ptr(), n, n, 0, None, None, None, 0, 0))
    assert rel_fro(out2.cpu().numpy(), out.cpu().numpy()) <= 1e-6
    del W
    A, B = randn(E, (4, 768), 18), randn(E, (768, 50257), 19)
    av = E.lib.make_view(A.data_ptr(), 0, A.shape, A.stride())
    bv = E.lib.make_view(B.data_ptr(), 0, B.shape, B.stride())
    Cc = E.t.empty(4, 50257, device="cuda")
    E.lib.check(E.L.tenmo_hip_matmul_nd(C.byref(av), C.byref(bv), Cc.data_ptr(), 0))
    assert rel_fro(Cc.cpu().numpy(), (A.double() @ B.double()).cpu().numpy()) <= RTOL_FRO
    A, B, dC = randn(E, (256, 100), 20), randn(E, (100, 50000), 21), randn(E, (256, 50000), 22)
    Cc = E.t.empty(256, 50000, device="cuda")
    gemm(E, A, (100, 1), B, (50000, 1), Cc, 256, 50000, 100)
    assert rel_fro(Cc.cpu().numpy(), (A.double() @ B.double()).cpu().numpy()) <= RTOL_FRO
    dB = E.t.empty(100, 50000, device="cuda")
    gemm(E, A, (1, 100), dC, (50000, 1), dB, 100, 50000, 256)
    assert rel_fro(dB.cpu().numpy(), (A.double().T @ dC.double()).cpu().numpy()) <= RTOL_FRO
