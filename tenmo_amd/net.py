"""Callers of the matrix-product path: ``Linear`` and the MNIST-shaped MLP training step.

``Linear``        y = x.W + b with W stored [in, out] (tenmo/net.mojo:49-216, :91-97).  For matrix
                  inputs the bias is added in the GEMM store (one launch); for a vector input it
                  is a rank-1 product on the GEMM entry (ones[rows,1] . b[1,out], accumulated).
                  The backward of a matrix input is one call (tenmo_hip_linear_backward): dX, dW and
                  the bias gradient, the latter summed inside the launch that computes dW; a vector
                  input keeps the separate column sum of dY.  The layer never leaves ``libtenmo_hip.so``.
``MLP``           the whole training step of examples/mnist.mojo:150-162 on the device:
                  Linear -> ReLU -> ... -> Linear -> CrossEntropyLoss(mean) -> backward -> SGD(lr).
``xavier_uniform``  U(+-sqrt(6/(in+out))) weights, zero bias (tenmo/net.mojo:87-114).
"""
from __future__ import annotations

import ctypes as C
import math
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import _lib
from ._lib import TenmoHipError, check
from .matmul import Matmul, Matmul2dBackward, MatmulNdBackward
from .ndbuffer import NDBuffer
from .tensor import Tensor, mm


def xavier_uniform(in_features: int, out_features: int, rng: np.random.Generator) -> np.ndarray:
    limit = math.sqrt(6.0 / float(in_features + out_features))
    return rng.uniform(-limit, limit, size=(in_features, out_features)).astype(np.float32)


class Linear:
    """Fully connected layer (tenmo/net.mojo:49-216)."""

    def __init__(self, in_features: int, out_features: int, rng: Optional[np.random.Generator] = None,
                 init_method: str = "standard", bias: bool = True):
        rng = rng or np.random.default_rng(0)
        if init_method == "xavier":
            w = xavier_uniform(in_features, out_features, rng)
        elif init_method == "he":
            w = (rng.standard_normal((in_features, out_features)) * math.sqrt(2.0 / in_features)).astype(np.float32)
        else:
            w = rng.uniform(-0.1, 0.1, size=(in_features, out_features)).astype(np.float32)
        self.in_features, self.out_features = in_features, out_features
        self.weight = Tensor.from_numpy(w, requires_grad=True)
        self.bias = Tensor.zeros(out_features, requires_grad=True) if bias else None
        self.training = True

    def parameters(self) -> List[Tensor]:
        return [self.weight] + ([self.bias] if self.bias is not None else [])

    def __call__(self, xs: Tensor, sync: bool = True) -> Tensor:
        if xs.shape()[-1] != self.weight.shape()[0]:
            raise TenmoHipError(-2, f"LinearBLAS forward: input dim mismatch: input shape -> {xs.shape()} and weights shape -> {self.weight.shape()}")
        if self.bias is None:
            return Matmul.forward(xs, self.weight, track_grad=self.training, mode=mm, sync=sync)
        L = _lib.load()
        if xs.rank() >= 2:
            # x.W + b in one launch: the bias is added in the GEMM store
            out = Tensor(xs.buffer.linear(self.weight.buffer, self.bias.buffer, relu=False, sync=sync), requires_grad=False)
            if self.training and (xs.requires_grad or self.weight.requires_grad):
                out.requires_grad = True
                out.add_ancestry((Matmul2dBackward if xs.rank() == 2 else MatmulNdBackward).backward, xs, self.weight)
            rows = out.numels() // self.out_features
        else:
            out = Matmul.forward(xs, self.weight, track_grad=self.training, mode=mm, sync=False)
            # out += ones[rows,1] . b[1,out]  — Adder.forward with broadcasting (tenmo/addition.mojo:73-112)
            rows = out.numels() // self.out_features
            ones = torch.ones(rows, dtype=torch.float32, device="cuda")
            check(L.tenmo_hip_gemm_f32(ones.data_ptr(), 0, 1, 1, self.bias.buffer.data_ptr(), self.bias.buffer.offset, self.out_features, 1,
                                       out.buffer.data_ptr(), rows, self.out_features, 1, 0, None, None, None, 1, 1 if sync else 0))
        if self.training and xs.rank() >= 2 and (out.backward_fn is not None or self.bias.requires_grad):
            # Adder backward + Matmul backward in one call of the library: the bias gradient (the upstream gradient summed
            # over its rows, tenmo/broadcast.mojo:81-87) comes out of the launch that computes the weight gradient
            x, w, bias = xs, self.weight, self.bias

            def backward_fused(output: Tensor, retain_graph: bool = False):
                grads = [(p.ensure_gradbox().data_ptr() if p.requires_grad else None) for p in (x, w, bias)]
                check(L.tenmo_hip_linear_backward(C.byref(x.buffer.c_view()), C.byref(w.buffer.c_view()), output.gradbox.data_ptr(), *grads, 0))
                if not retain_graph:
                    output.zero_grad()
                return [p for p in (x, w, bias) if p.requires_grad]

            out.requires_grad = True
            out.backward_fn, out.ancestors = None, []
            out.add_ancestry(backward_fused, x, w, bias)
        elif self.training and (out.backward_fn is not None or self.bias.requires_grad):
            inner, bias, parents = out.backward_fn, self.bias, list(out.ancestors)

            def backward(output: Tensor, retain_graph: bool = False):
                # bias gradient: column sums of the upstream gradient (tenmo/broadcast.mojo:81-87)
                updated = []
                if bias.requires_grad:
                    g = bias.ensure_gradbox()
                    check(L.tenmo_hip_column_sum_f32(output.gradbox.data_ptr(), 0, self.out_features, rows, self.out_features,
                                                     g.data_ptr(), 1, 0))
                    updated.append(bias)
                if inner is not None:
                    updated += inner(output, retain_graph)
                return updated

            out.requires_grad = True
            out.add_ancestry(backward, *parents, bias)
        return out


class SGD:
    """p -= lr * g (tenmo/optim.mojo:93-120), expressed as the rank-1-free GEMM identity
    p += (-lr * I) . g is not worth a launch: parameters here are updated by the MLP harness kernel;
    for stand-alone tensors the update is one accumulate call with a [1,1] scale."""

    def __init__(self, params: Sequence[Tensor], lr: float = 0.01):
        self.params, self.lr = list(params), float(lr)
        self._scale = torch.full((1,), -self.lr, dtype=torch.float32, device="cuda")

    def zero_grad(self) -> None:
        for p in self.params:
            p.zero_grad()

    def step(self) -> None:
        L = _lib.load()
        for p in self.params:
            if p.gradbox is None:
                continue
            n = p.numels()
            # p[n,1] += g[n,1] . scale[1,1]
            check(L.tenmo_hip_gemm_f32(p.gradbox.data_ptr(), 0, 1, 1, self._scale.data_ptr(), 0, 1, 1,
                                       p.buffer.data_ptr() + 4 * p.buffer.offset, n, 1, 1, 0, None, None, None, 1, 0))


class MLP:
    """Device-resident MLP training step through ``tenmo_hip_mlp_*``."""

    def __init__(self, dims: Sequence[int], weights: Sequence[np.ndarray], biases: Sequence[np.ndarray], max_batch: int):
        _lib.init()
        L = _lib.load()
        self.dims = [int(d) for d in dims]
        self.L = len(self.dims) - 1
        self._w = [np.ascontiguousarray(w, np.float32) for w in weights]
        self._b = [np.ascontiguousarray(b, np.float32) for b in biases]
        for l in range(self.L):
            if self._w[l].shape != (self.dims[l], self.dims[l + 1]) or self._b[l].shape != (self.dims[l + 1],):
                raise TenmoHipError(-2, f"layer {l}: weight/bias shapes do not match dims")
        wp = (C.c_void_p * self.L)(*[w.ctypes.data for w in self._w])
        bp = (C.c_void_p * self.L)(*[b.ctypes.data for b in self._b])
        self._h = L.tenmo_hip_mlp_create(self.L, _lib.i64(self.dims), wp, bp, int(max_batch))
        if not self._h:
            raise TenmoHipError(-4, L.tenmo_hip_last_error().decode())
        self.max_batch = int(max_batch)
        self._loss = torch.zeros(1, dtype=torch.float32, device="cuda")

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                _lib.load().tenmo_hip_mlp_destroy(h)
            except Exception:
                pass
            self._h = None

    def step_device(self, x: torch.Tensor, y: torch.Tensor, lr: float, sync: bool = False, graph: bool = False) -> torch.Tensor:
        """x: fp32 [batch, dims[0]] on the device, y: int32 [batch] on the device. Returns the device scalar loss.
        graph=True replays the step from a captured HIP graph (tenmo_hip_mlp_step_graph)."""
        L = _lib.load()
        fn = L.tenmo_hip_mlp_step_graph if graph else L.tenmo_hip_mlp_step
        check(fn(self._h, x.data_ptr(), y.data_ptr(), x.shape[0], float(lr), self._loss.data_ptr(), 1 if sync else 0))
        return self._loss

    def step(self, x: np.ndarray, y: np.ndarray, lr: float, graph: bool = False) -> float:
        xd = torch.from_numpy(np.ascontiguousarray(x, np.float32)).cuda()
        yd = torch.from_numpy(np.ascontiguousarray(y, np.int32)).cuda()
        self.step_device(xd, yd, lr, sync=True, graph=graph)
        return float(self._loss.item())

    def forward(self, x: np.ndarray) -> np.ndarray:
        xd = torch.from_numpy(np.ascontiguousarray(x, np.float32)).cuda()
        out = torch.empty(x.shape[0], self.dims[-1], dtype=torch.float32, device="cuda")
        check(_lib.load().tenmo_hip_mlp_forward(self._h, xd.data_ptr(), x.shape[0], out.data_ptr(), 1))
        return out.cpu().numpy()

    def params(self, layer: int):
        W = np.empty((self.dims[layer], self.dims[layer + 1]), np.float32)
        b = np.empty((self.dims[layer + 1],), np.float32)
        check(_lib.load().tenmo_hip_mlp_get_params(self._h, layer, W.ctypes.data, b.ctypes.data))
        return W, b

    def grads(self, layer: int):
        W = np.empty((self.dims[layer], self.dims[layer + 1]), np.float32)
        b = np.empty((self.dims[layer + 1],), np.float32)
        check(_lib.load().tenmo_hip_mlp_get_grads(self._h, layer, W.ctypes.data, b.ctypes.data))
        return W, b
