"""BLASHandle: the reference's CBLAS plugin loader pointed at ``libtenmo_hip.so``.

Mirrors tenmo/blashandle.mojo: the library path is a parameter (``BLAS_PATH``, :108-110), the
symbol ``cblas_sgemm`` is looked up by name (:231), operands are HOST arrays passed as raw base
pointers with ``lda = A.shape[1]``, ``ldb = B.shape[1]``, ``ldc = N`` (:353-371), row-major,
alpha = 1, beta = 0, and the four transpose cases of the backward follow :51-99.
A failed load is recorded and reported by ``is_initialized()`` / raised on use (:183-191, :227-228).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import numpy as np

from . import _lib

CblasRowMajor, CblasNoTrans, CblasTrans = 101, 111, 112  # tenmo/blashandle.mojo:130-133


class BLASHandle:
    def __init__(self, path: Optional[str] = None):
        self._path = path or _lib.LIB_PATH
        self._error_msg = ""
        self._handle = None
        try:
            self._handle = C.CDLL(self._path)
        except OSError as e:
            self._error_msg = f"Failed to load BLAS library from {self._path}: {e}"

    def is_initialized(self) -> bool:
        return self._handle is not None

    def error(self) -> str:
        return self._error_msg

    def _sgemm(self):
        if self._handle is None:
            raise RuntimeError("BLASHandle not initialized: " + self._error_msg)
        fn = self._handle.cblas_sgemm  # looked up on every call, as the reference does
        fn.restype = None
        fn.argtypes = [C.c_int] * 6 + [C.c_float, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_int]
        return fn

    def matmul(self, A: np.ndarray, B: np.ndarray, transpose_A: bool = False, transpose_B: bool = False) -> np.ndarray:
        """BLASHandle.matmul (tenmo/blashandle.mojo:295-421): 2-D fp32 dense storage + flags."""
        if A.ndim != 2:
            raise ValueError(f"A must be a 2D tensor, got rank {A.ndim}")
        if B.ndim != 2:
            raise ValueError(f"B must be a 2D tensor, got rank {B.ndim}")
        A = np.ascontiguousarray(A, np.float32)
        B = np.ascontiguousarray(B, np.float32)
        M, K = (A.shape[1], A.shape[0]) if transpose_A else A.shape
        Kb, N = (B.shape[1], B.shape[0]) if transpose_B else B.shape
        if K != Kb:
            raise ValueError(f"Matrix dimensions incompatible for matmul: K mismatch: {K} vs {Kb}")
        Cm = np.zeros((M, N), np.float32)
        self._sgemm()(CblasRowMajor, CblasTrans if transpose_A else CblasNoTrans, CblasTrans if transpose_B else CblasNoTrans,
                      M, N, K, 1.0, A.ctypes.data, A.shape[1], B.ctypes.data, B.shape[1], 0.0, Cm.ctypes.data, N)
        return Cm

    def matmul_backward(self, A: np.ndarray, B: np.ndarray, grad_out: np.ndarray,
                        transpose_A: bool = False, transpose_B: bool = False) -> Tuple[np.ndarray, np.ndarray]:
        """BLASMatmul2dBackward (tenmo/blashandle.mojo:21-105): the four transpose cases."""
        if not transpose_A and not transpose_B:
            gA = self.matmul(grad_out, B, transpose_B=True)
            gB = self.matmul(A, grad_out, transpose_A=True)
        elif transpose_A and not transpose_B:
            gA = self.matmul(B, grad_out, transpose_B=True)
            gB = self.matmul(A, grad_out)
        elif not transpose_A and transpose_B:
            gA = self.matmul(grad_out, B)
            gB = self.matmul(grad_out, A, transpose_A=True)
        else:
            gA = self.matmul(B, grad_out, transpose_A=True, transpose_B=True)
            gB = self.matmul(grad_out, A, transpose_A=True, transpose_B=True)
        return gA, gB
