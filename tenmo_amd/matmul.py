"""The matrix-product operators, with the reference's names and dispatch rules:

    classify_matmul, Matmul, Matmul2d, MatmulNd       tenmo/matmul.mojo:58-95, :141-198, :201-272
    Matmul2dBackward, MatmulNdBackward                tenmo/matmul.mojo:22-54, :99-137
    MatrixVectorMulNd (+Backward)                     tenmo/matrixvector.mojo:205-402, :15-201
    VectorMatmulNd (+Backward)                        tenmo/vectormatrix.mojo:210-375, :14-206
    Dot (+Backward)                                   tenmo/dotproduct.mojo:56-123, :13-52

Forward and backward arithmetic is done by ``libtenmo_hip.so``.  A shape the reference panics on
raises ``TenmoHipError`` carrying the library's message.
"""
from __future__ import annotations

import ctypes as C
from typing import List

from . import _lib
from ._lib import TenmoHipError, check
from .ndbuffer import NDBuffer
from .tensor import Tensor, dot, invalid, mm, mv, vm


def classify_matmul(a_shape, b_shape) -> int:
    """tenmo/matmul.mojo:258-272"""
    return _lib.load().tenmo_hip_classify_matmul(len(a_shape), _lib.i64(a_shape), len(b_shape), _lib.i64(b_shape))


def _ptr_or_null(t: Tensor):
    return t.ensure_gradbox().data_ptr() if t.requires_grad else None


def _finish_backward(output: Tensor, retain_graph: bool) -> None:
    if not retain_graph:
        output.zero_grad()  # grad_out.zero_grad(), tenmo/matmul.mojo:53-54


class Matmul2dBackward:
    @staticmethod
    def backward(output: Tensor, retain_graph: bool = False) -> List[Tensor]:
        A, B = output.ancestors[:2]  # a Linear appends its bias as a third parent
        check(_lib.load().tenmo_hip_matmul_backward(C.byref(A.buffer.c_view()), C.byref(B.buffer.c_view()),
                                                    output.gradbox.data_ptr(), _ptr_or_null(A), _ptr_or_null(B), 0))
        _finish_backward(output, retain_graph)
        return [p for p in (A, B) if p.requires_grad]


class MatmulNdBackward(Matmul2dBackward):
    """Same entry point: the library reduces each gradient over the batch axes its parent broadcast
    (sum_over_broadcasted_axes, tenmo/matmul.mojo:121,132) before adding it."""


class Matmul2d:
    @staticmethod
    def forward(A: Tensor, B: Tensor, track_grad: bool = True, sync: bool = True) -> Tensor:
        out = Tensor(A.buffer.matmul_2d(B.buffer, sync=sync), requires_grad=False)
        if track_grad and (A.requires_grad or B.requires_grad):
            out.requires_grad = True
            out.add_ancestry(Matmul2dBackward.backward, A, B)
        return out


class MatmulNd:
    @staticmethod
    def forward(A: Tensor, B: Tensor, track_grad: bool = True, sync: bool = True) -> Tensor:
        if A.rank() == 2 and B.rank() == 2:  # tenmo/matmul.mojo:151-152
            return Matmul2d.forward(A, B, track_grad, sync)
        out = Tensor(A.buffer.matmul_nd(B.buffer, sync=sync), requires_grad=False)
        if track_grad and (A.requires_grad or B.requires_grad):
            out.requires_grad = True
            out.add_ancestry(MatmulNdBackward.backward, A, B)
        return out


class MatrixVectorMulNdBackward:
    @staticmethod
    def backward(output: Tensor, retain_graph: bool = False) -> List[Tensor]:
        M, v = output.ancestors
        check(_lib.load().tenmo_hip_mv_backward(C.byref(M.buffer.c_view()), C.byref(v.buffer.c_view()),
                                                output.gradbox.data_ptr(), _ptr_or_null(M), _ptr_or_null(v), 0))
        _finish_backward(output, retain_graph)
        return [p for p in (M, v) if p.requires_grad]


class MatrixVectorMulNd:
    @staticmethod
    def forward(M: Tensor, v: Tensor, track_grad: bool = True, sync: bool = True) -> Tensor:
        out = Tensor(M.buffer.matrix_vector(v.buffer, sync=sync), requires_grad=False)
        if track_grad and (M.requires_grad or v.requires_grad):
            out.requires_grad = True
            out.add_ancestry(MatrixVectorMulNdBackward.backward, M, v)
        return out


class VectorMatmulNdBackward:
    @staticmethod
    def backward(output: Tensor, retain_graph: bool = False) -> List[Tensor]:
        v, M = output.ancestors
        check(_lib.load().tenmo_hip_vm_backward(C.byref(v.buffer.c_view()), C.byref(M.buffer.c_view()),
                                                output.gradbox.data_ptr(), _ptr_or_null(v), _ptr_or_null(M), 0))
        _finish_backward(output, retain_graph)
        return [p for p in (v, M) if p.requires_grad]


class VectorMatmulNd:
    @staticmethod
    def forward(v: Tensor, M: Tensor, track_grad: bool = True, sync: bool = True) -> Tensor:
        out = Tensor(v.buffer.vector_matrix(M.buffer, sync=sync), requires_grad=False)
        if track_grad and (v.requires_grad or M.requires_grad):
            out.requires_grad = True
            out.add_ancestry(VectorMatmulNdBackward.backward, v, M)
        return out


class DotBackward:
    """grad_lhs += rhs * g, grad_rhs += lhs * g  (tenmo/dotproduct.mojo:13-52): exactly the backward of
    lhs[n] . rhs-as-[n,1], so it runs through the vector x matrix gradient entry."""

    @staticmethod
    def backward(output: Tensor, retain_graph: bool = False) -> List[Tensor]:
        lhs, rhs = output.ancestors
        n = lhs.numels()
        col = NDBuffer(rhs.buffer.storage, (n, 1), (rhs.buffer.strides[0] if rhs.rank() else 0, 1), rhs.buffer.offset)
        check(_lib.load().tenmo_hip_vm_backward(C.byref(lhs.buffer.c_view()), C.byref(col.c_view()),
                                                output.gradbox.data_ptr(), _ptr_or_null(lhs), _ptr_or_null(rhs), 0))
        _finish_backward(output, retain_graph)
        return [p for p in (lhs, rhs) if p.requires_grad]


class Dot:
    @staticmethod
    def forward(lhs: Tensor, rhs: Tensor, track_grad: bool = True, sync: bool = True) -> Tensor:
        if lhs.rank() > 1 or rhs.rank() > 1:
            raise TenmoHipError(-2, "Tensor -> dot: not supported for rank > 1")
        na, nb = lhs.numels(), rhs.numels()
        sa = lhs.buffer.strides[0] if lhs.rank() else 0
        sb = rhs.buffer.strides[0] if rhs.rank() else 0
        broadcast = False
        if na == 1 and nb > 1:      # a one-element operand is broadcast first (tenmo/dotproduct.mojo:67-74)
            na, sa, broadcast = nb, 0, True
        elif nb == 1 and na > 1:
            nb, sb, broadcast = na, 0, True
        if na != nb:
            raise TenmoHipError(-2, f"Tensor -> dot: size does not match {na} vs {nb}")
        out = NDBuffer.empty(())
        check(_lib.load().tenmo_hip_dot_f32(lhs.buffer.data_ptr(), lhs.buffer.offset, sa, rhs.buffer.data_ptr(), rhs.buffer.offset, sb,
                                            na, out.data_ptr(), 1 if sync else 0))
        res = Tensor(out, requires_grad=False)
        if track_grad and (lhs.requires_grad or rhs.requires_grad):
            if broadcast:
                raise TenmoHipError(-5, "gradient through the scalar broadcast of dot belongs to Broadcast, outside the matmul path")
            res.requires_grad = True
            res.add_ancestry(DotBackward.backward, lhs, rhs)
        return res


class Matmul:
    @staticmethod
    def forward(A: Tensor, B: Tensor, track_grad: bool = True, mode: int = mm, sync: bool = True) -> Tensor:
        """tenmo/matmul.mojo:205-241"""
        if mode == mm:
            opcode = classify_matmul(A.shape(), B.shape())
            if opcode == dot:
                return Dot.forward(A, B, track_grad, sync)
            if opcode == vm:
                return VectorMatmulNd.forward(A, B, track_grad, sync)
            if opcode == mv:
                return MatrixVectorMulNd.forward(A, B, track_grad, sync)
            if opcode == mm:
                return MatmulNd.forward(A, B, track_grad, sync)
            raise TenmoHipError(-2, "Matmul: incompatible shapes")
        if mode == dot:
            return Dot.forward(A, B, track_grad, sync)
        if mode == vm:
            return VectorMatmulNd.forward(A, B, track_grad, sync)
        if mode == mv:
            return MatrixVectorMulNd.forward(A, B, track_grad, sync)
        raise TenmoHipError(-2, "Matmul: incompatible shapes")


__all__ = ["classify_matmul", "Matmul", "Matmul2d", "MatmulNd", "Matmul2dBackward", "MatmulNdBackward",
           "MatrixVectorMulNd", "MatrixVectorMulNdBackward", "VectorMatmulNd", "VectorMatmulNdBackward",
           "Dot", "DotBackward", "dot", "vm", "mv", "mm", "invalid"]
