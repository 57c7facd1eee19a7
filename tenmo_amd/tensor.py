"""Tensor = NDBuffer + requires_grad + gradient box + ancestry: the slice of the reference's
autograd surface that the matrix-product path runs under (tenmo/tensor.mojo:71-75, :1007-1028,
:3154-3247; tenmo/ancestry.mojo:72-105; tenmo/gradbox.mojo:1358-1364).

Only what that path needs is here: leaf construction, views, ``matmul`` in its four modes,
``backward`` (topological walk with fan-in counting) and gradient accumulation.  Every number
is produced by ``libtenmo_hip.so``; this file is bookkeeping.
"""
from __future__ import annotations

from collections import deque
from typing import Callable, List, Optional, Sequence

import numpy as np

from ._lib import TenmoHipError
from .ndbuffer import NDBuffer

# opcodes, tenmo/mnemonics.mojo:26-30
dot, vm, mv, mm, invalid = 0, 1, 2, 3, -1


class Tensor:
    _next_id = 0

    def __init__(self, buffer: NDBuffer, requires_grad: bool = False):
        self.buffer = buffer
        self.requires_grad = requires_grad
        self.gradbox: Optional[NDBuffer] = None  # dense, this tensor's shape, zero offset
        self.ancestors: List["Tensor"] = []
        self.backward_fn: Optional[Callable[["Tensor", bool], List["Tensor"]]] = None
        Tensor._next_id += 1
        self._id = Tensor._next_id

    # ---- construction ----------------------------------------------------------------------
    @staticmethod
    def d(values, requires_grad: bool = False) -> "Tensor":
        """From nested lists / numpy (Tensor.d1 / d2 / d3 ... in the reference's tests)."""
        return Tensor(NDBuffer.from_numpy(np.asarray(values, dtype=np.float32)), requires_grad)

    @staticmethod
    def from_numpy(a: np.ndarray, requires_grad: bool = False) -> "Tensor":
        return Tensor(NDBuffer.from_numpy(a), requires_grad)

    @staticmethod
    def zeros(*shape, requires_grad: bool = False) -> "Tensor":
        return Tensor(NDBuffer.zeros(shape), requires_grad)

    @staticmethod
    def ones(*shape, requires_grad: bool = False) -> "Tensor":
        return Tensor.from_numpy(np.ones(shape, np.float32), requires_grad)

    @staticmethod
    def arange(n: int, requires_grad: bool = False) -> "Tensor":
        return Tensor.from_numpy(np.arange(n, dtype=np.float32), requires_grad)

    # ---- metadata / views ----------------------------------------------------------------------
    def shape(self):
        return self.buffer.shape

    def rank(self) -> int:
        return self.buffer.rank()

    def numels(self) -> int:
        return self.buffer.numels()

    def view(self, shape: Sequence[int], strides: Sequence[int], offset: int = 0, requires_grad: Optional[bool] = None) -> "Tensor":
        """Strided view over the same storage; gradients of a view flow back to positions of the base
        only through an op the path does not own, so views are leaves here (as in the reference's
        matmul tests, which read the view's own gradient)."""
        return Tensor(self.buffer.view(shape, strides, offset), self.requires_grad if requires_grad is None else requires_grad)

    def transpose(self, ax0: int = -1, ax1: int = -2) -> "Tensor":
        return Tensor(self.buffer.transpose(ax0, ax1), self.requires_grad)

    def reshape(self, *shape) -> "Tensor":
        if not self.buffer.is_contiguous():
            raise TenmoHipError(-5, "reshape of a non-contiguous view is outside the matmul path")
        return Tensor(NDBuffer(self.buffer.storage, shape, None, self.buffer.offset), self.requires_grad)

    def to_numpy(self) -> np.ndarray:
        return self.buffer.to_numpy()

    def grad(self) -> Optional[np.ndarray]:
        return None if self.gradbox is None else self.gradbox.to_numpy()

    def zero_grad(self) -> None:
        if self.gradbox is not None:
            self.gradbox.storage.zero_()

    # ---- autograd -------------------------------------------------------------------------------
    def add_ancestry(self, backward_fn, *parents: "Tensor") -> None:
        """tenmo/tensor.mojo:1007-1028"""
        self.backward_fn = backward_fn
        self.ancestors = list(parents)

    def ensure_gradbox(self) -> NDBuffer:
        if self.gradbox is None:
            self.gradbox = NDBuffer.zeros(self.buffer.shape)
        return self.gradbox

    def seed_grad(self, value) -> None:
        g = self.ensure_gradbox()
        if isinstance(value, Tensor):
            src = value.to_numpy()
        else:
            src = np.full(self.buffer.shape, float(value), np.float32)
        import torch

        g.storage.copy_(torch.from_numpy(np.ascontiguousarray(src, np.float32).reshape(-1)))

    def backward(self, start_grad=1.0, retain_graph: bool = False) -> None:
        """Topological sweep with fan-in counting (tenmo/tensor.mojo:3154-3247)."""
        if not self.requires_grad:
            return
        self.seed_grad(start_grad)
        nodes, fanin, stack, seen = {self._id: self}, {}, [self], set()
        while stack:
            n = stack.pop()
            if n._id in seen:
                continue
            seen.add(n._id)
            for p in n.ancestors:
                fanin[p._id] = fanin.get(p._id, 0) + 1
                if p._id not in nodes:
                    nodes[p._id] = p
                    stack.append(p)
        ready = deque([self])
        while ready:
            n = ready.popleft()
            if n.backward_fn is None:
                continue
            for p in n.backward_fn(n, retain_graph):
                fanin[p._id] -= 1
                if fanin[p._id] == 0 and p.backward_fn is not None:
                    ready.append(p)

    # ---- the path -----------------------------------------------------------------------------
    def matmul(self, other: "Tensor", track_grad: bool = True, mode: int = mm, sync: bool = True) -> "Tensor":
        """Tensor.matmul[track_grad, mode] (tenmo/tensor.mojo:4141-4159)."""
        from .matmul import Matmul

        return Matmul.forward(self, other, track_grad=track_grad, mode=mode, sync=sync)

    def dot(self, other: "Tensor", track_grad: bool = True, sync: bool = True) -> "Tensor":
        from .matmul import Dot

        return Dot.forward(self, other, track_grad=track_grad, sync=sync)

    def __matmul__(self, other: "Tensor") -> "Tensor":
        return self.matmul(other)
