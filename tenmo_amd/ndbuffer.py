"""NDBuffer: shape / strides / offset over shared device storage.

Host-side mirror of the part of the reference's ``NDBuffer`` (tenmo/ndbuffer.mojo) that the matrix
product path touches: views never copy, ``transpose`` swaps two strides
(tenmo/ndbuffer.mojo:1040-1062), ``is_contiguous`` is the predicate of tenmo/strides.mojo:239-266,
and ``matmul_2d`` / ``matmul_nd`` are the device dispatch points (tenmo/ndbuffer.mojo:2404-2501)
whose GPU branch calls ``libtenmo_hip.so``.

PyTorch is used for one thing only: owning the HIP allocation (a flat fp32 tensor).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from ._lib import OP_MM, OP_MV, OP_VM, TenmoHipError, check


def default_strides(shape: Sequence[int]) -> Tuple[int, ...]:
    """Row-major strides (tenmo/strides.mojo:230-236)."""
    acc, out = 1, []
    for s in reversed(shape):
        out.append(acc)
        acc *= int(s)
    return tuple(reversed(out))


class NDBuffer:
    __slots__ = ("storage", "shape", "strides", "offset")

    def __init__(self, storage: torch.Tensor, shape: Sequence[int], strides: Optional[Sequence[int]] = None, offset: int = 0):
        if storage.dtype != torch.float32 or storage.dim() != 1 or not storage.is_cuda:
            raise TenmoHipError(-3, "NDBuffer storage must be a flat fp32 device tensor")
        self.storage = storage
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in strides) if strides is not None else default_strides(self.shape)
        self.offset = int(offset)
        if len(self.shape) != len(self.strides):
            raise TenmoHipError(-2, "shape and strides differ in rank")

    # ---- construction --------------------------------------------------------------------
    @staticmethod
    def from_numpy(a: np.ndarray) -> "NDBuffer":
        a = np.ascontiguousarray(a, dtype=np.float32)
        _lib.init()
        return NDBuffer(torch.from_numpy(a.reshape(-1).copy()).cuda(), a.shape)

    @staticmethod
    def zeros(shape: Sequence[int]) -> "NDBuffer":
        _lib.init()
        n = int(np.prod(shape)) if len(shape) else 1
        return NDBuffer(torch.zeros(max(n, 1), dtype=torch.float32, device="cuda"), shape)

    @staticmethod
    def empty(shape: Sequence[int]) -> "NDBuffer":
        _lib.init()
        n = int(np.prod(shape)) if len(shape) else 1
        return NDBuffer(torch.empty(max(n, 1), dtype=torch.float32, device="cuda"), shape)

    # ---- metadata --------------------------------------------------------------------------
    def rank(self) -> int:
        return len(self.shape)

    def numels(self) -> int:
        return int(np.prod(self.shape)) if self.shape else 1

    def is_contiguous(self) -> bool:
        expected = 1
        for s, t in zip(reversed(self.shape), reversed(self.strides)):
            if s > 1 and t != expected:
                return False
            expected *= s
        return True

    def view(self, shape: Sequence[int], strides: Sequence[int], offset: int = 0) -> "NDBuffer":
        """A view over the same storage with absolute offset (Tensor.view(shape, strides, offset))."""
        return NDBuffer(self.storage, shape, strides, offset)

    def transpose(self, ax0: int = -1, ax1: int = -2) -> "NDBuffer":
        r = self.rank()
        a, b = ax0 % r, ax1 % r
        sh, st = list(self.shape), list(self.strides)
        sh[a], sh[b] = sh[b], sh[a]
        st[a], st[b] = st[b], st[a]
        return NDBuffer(self.storage, sh, st, self.offset)

    def c_view(self) -> _lib.CView:
        return _lib.make_view(self.storage.data_ptr(), self.offset, self.shape, self.strides)

    def data_ptr(self) -> int:
        return self.storage.data_ptr()

    # ---- host copies (tests) -----------------------------------------------------------------
    def to_numpy(self) -> np.ndarray:
        check(_lib.load().tenmo_hip_sync())
        flat = self.storage.cpu().numpy()
        if not self.shape:
            return flat[self.offset].copy()
        return np.lib.stride_tricks.as_strided(flat[self.offset:], self.shape, tuple(4 * s for s in self.strides)).copy()

    # ---- the device dispatch points ---------------------------------------------------------------
    def _product(self, op: int, other: "NDBuffer", fn_name: str, sync: bool) -> "NDBuffer":
        L = _lib.load()
        _lib.init()
        a, b = self.c_view(), other.c_view()
        oshape = (C.c_int64 * (_lib.MAX_RANK + 2))()
        orank = C.c_int32()
        n = L.tenmo_hip_result_shape(op, C.byref(a), C.byref(b), oshape, C.byref(orank))
        check(n)
        out = NDBuffer.empty(tuple(oshape[i] for i in range(orank.value)))
        check(getattr(L, fn_name)(C.byref(a), C.byref(b), out.data_ptr(), 1 if sync else 0))
        return out

    def matmul_2d(self, other: "NDBuffer", sync: bool = False) -> "NDBuffer":
        """NDBuffer.matmul_2d (tenmo/ndbuffer.mojo:2404-2443): rank-2 x rank-2 only."""
        if self.rank() != 2 or other.rank() != 2:
            raise TenmoHipError(-2, f"validate_matrix_shapes_2d: matmul_2d expects rank == 2. Got A = {self.shape}, B = {other.shape}")
        if self.shape[1] != other.shape[0]:
            raise TenmoHipError(-2, f"validate_matrix_shapes_2d: inner dimensions mismatch in matmul_2d: A(m,{self.shape[1]}) vs B({other.shape[0]},n)")
        return self._product(OP_MM, other, "tenmo_hip_matmul_nd", sync)

    def matmul_nd(self, other: "NDBuffer", sync: bool = False) -> "NDBuffer":
        """NDBuffer.matmul_nd (tenmo/ndbuffer.mojo:2445-2501)."""
        return self._product(OP_MM, other, "tenmo_hip_matmul_nd", sync)

    def linear(self, weight: "NDBuffer", bias: "NDBuffer", relu: bool = False, sync: bool = False) -> "NDBuffer":
        """self . weight + bias (then ReLU) in one launch: Linear.forward, tenmo/net.mojo:193-201."""
        if bias.rank() != 1 or bias.strides[0] != 1 or bias.shape[0] != weight.shape[-1]:
            raise TenmoHipError(-2, f"linear: bias of shape {bias.shape} does not match weight {weight.shape}")
        L = _lib.load()
        a, b = self.c_view(), weight.c_view()
        _lib.init()
        oshape = (C.c_int64 * (_lib.MAX_RANK + 2))()
        orank = C.c_int32()
        check(L.tenmo_hip_result_shape(OP_MM, C.byref(a), C.byref(b), oshape, C.byref(orank)))
        out = NDBuffer.empty(tuple(oshape[i] for i in range(orank.value)))
        check(L.tenmo_hip_linear_nd(C.byref(a), C.byref(b), bias.data_ptr() + 4 * bias.offset, 1 if relu else 0,
                                    out.data_ptr(), 1 if sync else 0))
        return out

    def matrix_vector(self, v: "NDBuffer", sync: bool = False) -> "NDBuffer":
        return self._product(OP_MV, v, "tenmo_hip_matrix_vector_nd", sync)

    def vector_matrix(self, M: "NDBuffer", sync: bool = False) -> "NDBuffer":
        return self._product(OP_VM, M, "tenmo_hip_vector_matmul_nd", sync)
