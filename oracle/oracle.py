"""ctypes front end of the CPU oracle (``libtenmo_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline.  The product package
never imports it.

A view is ``(storage, offset, shape, strides)`` in elements, the reference's NDBuffer layout
(tenmo/ndbuffer.mojo).  ``View.of(ndarray)`` takes any fp32 numpy view (transposed, sliced,
``as_strided``) and describes it relative to its own first element.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence, Tuple

import numpy as np

MAX_RANK = 8
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtenmo_oracle.so")

DOT, VM, MV, MM, INVALID = 0, 1, 2, 3, -1


class _CView(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("offset", C.c_int64),
        ("rank", C.c_int32),
        ("shape", C.c_int64 * MAX_RANK),
        ("strides", C.c_int64 * MAX_RANK),
    ]


class OracleError(RuntimeError):
    """Raised where the reference panics (shape mismatch, incompatible broadcast ...)."""


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (g++, OpenMP)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-j8"] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp = C.POINTER(_CView)
        i64p, i32p, fp, dp = C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.c_void_p, C.c_void_p
        L.oracle_last_error.restype = C.c_char_p
        L.oracle_simd_width.restype = C.c_int
        L.oracle_force_simd_width.argtypes = [C.c_int]
        L.oracle_num_physical_cores.restype = C.c_int
        L.oracle_is_contiguous.argtypes = [C.c_int32, i64p, i64p]
        L.oracle_classify_matmul.argtypes = [C.c_int32, i64p, C.c_int32, i64p]
        L.oracle_mm2d_f32.argtypes = [vp, vp, fp, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.oracle_mmnd_f32.argtypes = [vp, vp, fp, C.c_int, i64p, i32p, C.c_int64]
        L.oracle_result_shape.argtypes = [C.c_int, vp, vp, i64p, i32p]
        L.oracle_result_shape.restype = C.c_int64
        L.oracle_mv_f32.argtypes = [vp, vp, fp]
        L.oracle_vm_f32.argtypes = [vp, vp, fp]
        L.oracle_mv_backward_f32.argtypes = [vp, vp, fp, fp, fp]
        L.oracle_vm_backward_f32.argtypes = [vp, vp, fp, fp, fp]
        L.oracle_dot_f32.argtypes = [vp, vp, fp]
        L.oracle_sum_over_broadcasted_axes_f32.argtypes = [fp, C.c_int32, i64p, C.c_int32, i64p, fp]
        L.oracle_mmnd_f64acc.argtypes = [vp, vp, dp, C.c_int]
        L.oracle_mv_f64acc.argtypes = [vp, vp, dp]
        L.oracle_vm_f64acc.argtypes = [vp, vp, dp]
        L.oracle_mlp_create.argtypes = [C.c_int, i64p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int64]
        L.oracle_mlp_create.restype = C.c_void_p
        L.oracle_mlp_destroy.argtypes = [C.c_void_p]
        L.oracle_mlp_step.argtypes = [C.c_void_p, fp, C.c_void_p, C.c_int64, C.c_float, C.c_int]
        L.oracle_mlp_step.restype = C.c_float
        L.oracle_mlp_forward.argtypes = [C.c_void_p, fp, C.c_int64, fp, C.c_int]
        L.oracle_mlp_get_params.argtypes = [C.c_void_p, C.c_int, fp, fp]
        L.oracle_mlp_get_grads.argtypes = [C.c_void_p, C.c_int, fp, fp]
        L.oracle_cross_entropy_forward_f32.argtypes = [fp, i64p, C.c_int64, C.c_int64, C.c_int64, C.c_float, fp, fp, fp, i32p]
        L.oracle_cross_entropy_backward_f32.argtypes = [fp, i64p, fp, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_int, C.c_int32, fp]
        L.oracle_sgd_step_f32.argtypes = [fp, fp, fp, C.c_int64, C.c_float, C.c_float, C.c_float]
        L.oracle_conv2d_backward_f32.argtypes = [fp, C.c_int64, C.c_int64, C.c_int64, C.c_int64, fp, C.c_int64, C.c_int64, C.c_int64,
                                                 C.c_int64, C.c_int64, fp, fp, fp, fp]
        L.oracle_conv2d_forward_f32.argtypes = [fp, C.c_int64, C.c_int64, C.c_int64, C.c_int64, fp, C.c_int64, C.c_int64, C.c_int64,
                                                fp, C.c_int64, C.c_int64, fp]
        _lib = L
    return _lib


def _check(rc: int):
    if rc < 0:
        raise OracleError(lib().oracle_last_error().decode())


def _i64(seq: Sequence[int]):
    return (C.c_int64 * max(1, len(seq)))(*[int(x) for x in seq])


class View:
    """(storage, offset, shape, strides) in elements over an fp32 numpy buffer."""

    def __init__(self, storage: np.ndarray, offset: int, shape: Sequence[int], strides: Sequence[int]):
        assert storage.dtype == np.float32 and storage.flags["C_CONTIGUOUS"]
        assert len(shape) == len(strides) <= MAX_RANK
        self.storage = storage
        self.offset = int(offset)
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in strides)

    @staticmethod
    def of(a: np.ndarray) -> "View":
        a = np.asarray(a)
        assert a.dtype == np.float32
        for s in a.strides:
            assert s % 4 == 0
        v = View.__new__(View)
        v.storage = a  # keeps the memory alive; pointer already includes the view's own offset
        v.offset = 0
        v.shape = tuple(a.shape)
        v.strides = tuple(s // 4 for s in a.strides)
        return v

    @property
    def rank(self) -> int:
        return len(self.shape)

    def transpose_last2(self) -> "View":
        """Swap the two trailing dims as a view (NDBuffer.transpose, tenmo/ndbuffer.mojo:1040-1062)."""
        v = View.__new__(View)
        v.storage, v.offset = self.storage, self.offset
        sh, st = list(self.shape), list(self.strides)
        sh[-1], sh[-2] = sh[-2], sh[-1]
        st[-1], st[-2] = st[-2], st[-1]
        v.shape, v.strides = tuple(sh), tuple(st)
        return v

    def c(self) -> _CView:
        cv = _CView()
        cv.data = self.storage.ctypes.data
        cv.offset = self.offset
        cv.rank = self.rank
        for i, (s, t) in enumerate(zip(self.shape, self.strides)):
            cv.shape[i] = s
            cv.strides[i] = t
        return cv

    def numpy(self) -> np.ndarray:
        """Materialise the view (test helper)."""
        base = self.storage.reshape(-1)[self.offset:] if self.offset else self.storage
        return np.lib.stride_tricks.as_strided(base, self.shape, tuple(4 * s for s in self.strides))


def _as_view(x) -> View:
    return x if isinstance(x, View) else View.of(x)


def simd_width() -> int:
    return lib().oracle_simd_width()


def force_simd_width(w: int) -> None:
    lib().oracle_force_simd_width(int(w))


def num_physical_cores() -> int:
    return lib().oracle_num_physical_cores()


def is_contiguous(shape: Sequence[int], strides: Sequence[int]) -> bool:
    return bool(lib().oracle_is_contiguous(len(shape), _i64(shape), _i64(strides)))


def classify_matmul(shape_a: Sequence[int], shape_b: Sequence[int]) -> int:
    return lib().oracle_classify_matmul(len(shape_a), _i64(shape_a), len(shape_b), _i64(shape_b))


def result_shape(mode: int, A, B) -> Tuple[int, ...]:
    A, B = _as_view(A), _as_view(B)
    out = (C.c_int64 * (MAX_RANK + 2))()
    r = C.c_int32()
    _check(lib().oracle_result_shape(mode, C.byref(A.c()), C.byref(B.c()), out, C.byref(r)))
    return tuple(out[i] for i in range(r.value))


def mm2d(A, B, nthreads: int = 0, info: Optional[dict] = None) -> np.ndarray:
    """MmCpu2d.tiled_matmul (tenmo/matmul_cpu.mojo:80-135)."""
    A, B = _as_view(A), _as_view(B)
    if A.rank != 2 or B.rank != 2 or A.shape[1] != B.shape[0]:
        out = np.zeros((1,), np.float32)
    else:
        out = np.empty((A.shape[0], B.shape[1]), np.float32)
    path, tiles = C.c_int(), (C.c_int * 3)()
    _check(lib().oracle_mm2d_f32(C.byref(A.c()), C.byref(B.c()), out.ctypes.data, nthreads, C.byref(path), tiles))
    if info is not None:
        info["path"] = path.value
        info["tiles"] = tuple(tiles)
    return out


def mmnd(A, B, nthreads: int = 0, work_item_limit: int = 0, out: Optional[np.ndarray] = None) -> np.ndarray:
    """MmCpuNd.tiled_matmul (tenmo/matmul_cpu.mojo:568-625)."""
    A, B = _as_view(A), _as_view(B)
    shape = result_shape(MM, A, B)
    if out is None:
        out = np.empty(shape, np.float32)
    _check(lib().oracle_mmnd_f32(C.byref(A.c()), C.byref(B.c()), out.ctypes.data, nthreads, None, None, work_item_limit))
    return out


def matmul(A, B, nthreads: int = 0) -> np.ndarray:
    """NDBuffer-level dispatch of MatmulNd.forward: rank-2 x rank-2 goes to the 2-D kernel
    (tenmo/matmul.mojo:151-152), anything else to the batched one."""
    A, B = _as_view(A), _as_view(B)
    if A.rank == 2 and B.rank == 2:
        return mm2d(A, B, nthreads)
    return mmnd(A, B, nthreads)


def mm_f64(A, B, nthreads: int = 0) -> np.ndarray:
    A, B = _as_view(A), _as_view(B)
    shape = result_shape(MM, A, B)
    out = np.empty(shape, np.float64)
    _check(lib().oracle_mmnd_f64acc(C.byref(A.c()), C.byref(B.c()), out.ctypes.data, nthreads))
    return out


def mv(M, v) -> np.ndarray:
    M, v = _as_view(M), _as_view(v)
    if M.rank < 2 or v.rank < 1:
        _check(lib().oracle_mv_f32(C.byref(M.c()), C.byref(v.c()), None))
    out = np.empty(result_shape(MV, M, v), np.float32)
    _check(lib().oracle_mv_f32(C.byref(M.c()), C.byref(v.c()), out.ctypes.data))
    return out


def vm(v, M) -> np.ndarray:
    v, M = _as_view(v), _as_view(M)
    if M.rank < 2 or v.rank < 1:
        _check(lib().oracle_vm_f32(C.byref(v.c()), C.byref(M.c()), None))
    out = np.empty(result_shape(VM, v, M), np.float32)
    _check(lib().oracle_vm_f32(C.byref(v.c()), C.byref(M.c()), out.ctypes.data))
    return out


def mv_f64(M, v) -> np.ndarray:
    M, v = _as_view(M), _as_view(v)
    out = np.empty(result_shape(MV, M, v), np.float64)
    _check(lib().oracle_mv_f64acc(C.byref(M.c()), C.byref(v.c()), out.ctypes.data))
    return out


def vm_f64(v, M) -> np.ndarray:
    v, M = _as_view(v), _as_view(M)
    out = np.empty(result_shape(VM, v, M), np.float64)
    _check(lib().oracle_vm_f64acc(C.byref(v.c()), C.byref(M.c()), out.ctypes.data))
    return out


def mv_backward(M, v, dy: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """(dM, dv) at the parents' shapes (tenmo/matrixvector.mojo:19-201)."""
    M, v = _as_view(M), _as_view(v)
    dy = np.ascontiguousarray(dy, np.float32)
    dM, dv = np.empty(M.shape, np.float32), np.empty(v.shape, np.float32)
    _check(lib().oracle_mv_backward_f32(C.byref(M.c()), C.byref(v.c()), dy.ctypes.data, dM.ctypes.data, dv.ctypes.data))
    return dM, dv


def vm_backward(v, M, dy: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """(dv, dM) at the parents' shapes (tenmo/vectormatrix.mojo:18-206)."""
    v, M = _as_view(v), _as_view(M)
    dy = np.ascontiguousarray(dy, np.float32)
    dv, dM = np.empty(v.shape, np.float32), np.empty(M.shape, np.float32)
    _check(lib().oracle_vm_backward_f32(C.byref(v.c()), C.byref(M.c()), dy.ctypes.data, dv.ctypes.data, dM.ctypes.data))
    return dv, dM


def dot(a, b) -> np.float32:
    a, b = _as_view(a), _as_view(b)
    out = np.zeros((), np.float32)
    _check(lib().oracle_dot_f32(C.byref(a.c()), C.byref(b.c()), out.ctypes.data))
    return out[()]


def sum_over_broadcasted_axes(src: np.ndarray, target_shape: Sequence[int]) -> np.ndarray:
    src = np.ascontiguousarray(src, np.float32)
    dst = np.empty(tuple(target_shape), np.float32)
    _check(lib().oracle_sum_over_broadcasted_axes_f32(src.ctypes.data, src.ndim, _i64(src.shape),
                                                      len(target_shape), _i64(target_shape), dst.ctypes.data))
    return dst


def matmul_backward(A, B, dC: np.ndarray, nthreads: int = 0) -> Tuple[np.ndarray, np.ndarray]:
    """Matmul2dBackward / MatmulNdBackward (tenmo/matmul.mojo:22-54, :99-137): the two gradient
    GEMMs on transposed views, then the reduction to each parent's shape."""
    A, B = _as_view(A), _as_view(B)
    dCv = View.of(np.ascontiguousarray(dC, np.float32))
    gA = matmul(dCv, B.transpose_last2(), nthreads)
    gB = matmul(A.transpose_last2(), dCv, nthreads)
    if gA.shape != A.shape:
        gA = sum_over_broadcasted_axes(gA, A.shape)
    if gB.shape != B.shape:
        gB = sum_over_broadcasted_axes(gB, B.shape)
    return gA, gB


class MLP:
    """The 4-layer MLP training step of the MNIST example, restated on the oracle's own matmul."""

    def __init__(self, dims: Sequence[int], weights, biases, max_batch: int):
        self.dims = [int(d) for d in dims]
        L = len(dims) - 1
        self._W = [np.ascontiguousarray(w, np.float32) for w in weights]
        self._b = [np.ascontiguousarray(b, np.float32) for b in biases]
        Wp = (C.c_void_p * L)(*[w.ctypes.data for w in self._W])
        bp = (C.c_void_p * L)(*[b.ctypes.data for b in self._b])
        self._h = lib().oracle_mlp_create(L, _i64(self.dims), Wp, bp, max_batch)
        self.L = L

    def __del__(self):
        if getattr(self, "_h", None):
            lib().oracle_mlp_destroy(self._h)
            self._h = None

    def step(self, x: np.ndarray, y: np.ndarray, lr: float, nthreads: int = 0) -> float:
        x = np.ascontiguousarray(x, np.float32)
        y = np.ascontiguousarray(y, np.int32)
        return float(lib().oracle_mlp_step(self._h, x.ctypes.data, y.ctypes.data, x.shape[0], lr, nthreads))

    def forward(self, x: np.ndarray, nthreads: int = 0) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty((x.shape[0], self.dims[-1]), np.float32)
        _check(lib().oracle_mlp_forward(self._h, x.ctypes.data, x.shape[0], out.ctypes.data, nthreads))
        return out

    def params(self, layer: int):
        W = np.empty((self.dims[layer], self.dims[layer + 1]), np.float32)
        b = np.empty((self.dims[layer + 1],), np.float32)
        _check(lib().oracle_mlp_get_params(self._h, layer, W.ctypes.data, b.ctypes.data))
        return W, b

    def grads(self, layer: int):
        W = np.empty((self.dims[layer], self.dims[layer + 1]), np.float32)
        b = np.empty((self.dims[layer + 1],), np.float32)
        _check(lib().oracle_mlp_get_grads(self._h, layer, W.ctypes.data, b.ctypes.data))
        return W, b


REDUCTION_NONE, REDUCTION_SUM, REDUCTION_MEAN = 0, 1, 2


def cross_entropy_forward(logits: np.ndarray, target: np.ndarray, ignore_index: int = -100, label_smoothing: float = 0.0):
    """(softmax [M,C], per-sample loss [M], loss sum, valid count) — tenmo/crossentropy.mojo:285-432."""
    logits = np.ascontiguousarray(logits, np.float32)
    target = np.ascontiguousarray(target, np.int64)
    M, Cn = logits.shape
    sm = np.empty((M, Cn), np.float32)
    rows = np.empty(M, np.float32)
    total = np.zeros(1, np.float32)
    valid = np.zeros(1, np.int32)
    _check(lib().oracle_cross_entropy_forward_f32(logits.ctypes.data_as(C.POINTER(C.c_float)), target.ctypes.data_as(C.POINTER(C.c_int64)),
                                                  M, Cn, ignore_index, label_smoothing,
                                                  sm.ctypes.data_as(C.POINTER(C.c_float)), rows.ctypes.data_as(C.POINTER(C.c_float)),
                                                  total.ctypes.data_as(C.POINTER(C.c_float)), valid.ctypes.data_as(C.POINTER(C.c_int32))))
    return sm, rows, float(total[0]), int(valid[0])


def cross_entropy_backward(softmax: np.ndarray, target: np.ndarray, upstream: np.ndarray, reduction: int, valid_count: int,
                           ignore_index: int = -100, label_smoothing: float = 0.0) -> np.ndarray:
    """Gradient with respect to the logits — tenmo/crossentropy.mojo:744-770, :451-481."""
    softmax = np.ascontiguousarray(softmax, np.float32)
    target = np.ascontiguousarray(target, np.int64)
    upstream = np.ascontiguousarray(np.atleast_1d(upstream), np.float32)
    M, Cn = softmax.shape
    grad = np.empty((M, Cn), np.float32)
    _check(lib().oracle_cross_entropy_backward_f32(softmax.ctypes.data_as(C.POINTER(C.c_float)), target.ctypes.data_as(C.POINTER(C.c_int64)),
                                                   upstream.ctypes.data_as(C.POINTER(C.c_float)), M, Cn, ignore_index, label_smoothing,
                                                   reduction, valid_count, grad.ctypes.data_as(C.POINTER(C.c_float))))
    return grad


def sgd_step(param: np.ndarray, grad: np.ndarray, velocity: Optional[np.ndarray], lr: float, momentum: float = 0.0,
             weight_decay: float = 0.0) -> None:
    """In-place optimiser step on contiguous fp32 arrays — tenmo/optim.mojo:93-160."""
    assert param.dtype == np.float32 and param.flags.c_contiguous and grad.dtype == np.float32
    fpp = C.POINTER(C.c_float)
    _check(lib().oracle_sgd_step_f32(param.ctypes.data_as(fpp), np.ascontiguousarray(grad).ctypes.data_as(fpp),
                                     velocity.ctypes.data_as(fpp) if velocity is not None else None, param.size, lr, momentum, weight_decay))


def conv_padding(h_in: int, w_in: int, kh: int, kw: int, stride: int, dilation: int, padding) -> Tuple[int, int, int, int]:
    """(top, bottom, left, right) zero padding as Conv2dFused.invoke derives it from its `padding` argument
    — tenmo/cnn.mojo:183-222: "valid", "same", an int, a (height, width) pair or [(top, bottom), (left, right)]."""
    dkh, dkw = kh + (kh - 1) * (dilation - 1), kw + (kw - 1) * (dilation - 1)
    if padding == "valid":
        return 0, 0, 0, 0
    if padding == "same":
        h_target, w_target = (h_in + stride - 1) // stride, (w_in + stride - 1) // stride
        ph, pw = (h_target - 1) * stride + dkh - h_in, (w_target - 1) * stride + dkw - w_in
        return ph // 2, ph - ph // 2, pw // 2, pw - pw // 2
    if isinstance(padding, int):
        return padding, padding, padding, padding
    if isinstance(padding, tuple):
        return padding[0], padding[0], padding[1], padding[1]
    if isinstance(padding, list) and len(padding) == 2:
        return padding[0][0], padding[0][1], padding[1][0], padding[1][1]
    raise OracleError("Invalid padding type")


def conv2d_forward(image: np.ndarray, kernel: np.ndarray, bias: Optional[np.ndarray] = None, stride: int = 1, dilation: int = 1,
                   padding="valid") -> np.ndarray:
    """Conv2dFused.forward (tenmo/cnn.mojo:92-273): zero-pad, then the fused im2col convolution (:308-507)."""
    if image.ndim != 4 or kernel.ndim != 4:
        raise OracleError("Image must be 4D: (N, C_in, H_in, W_in); kernel must be 4D: (C_out, C_in, KH, KW)")
    n, c_in, h_in, w_in = image.shape
    c_out, kc, kh, kw = kernel.shape
    if kc != c_in:
        raise OracleError("Kernel input channels must match input channels")
    top, bottom, left, right = conv_padding(h_in, w_in, kh, kw, stride, dilation, padding)
    padded = np.ascontiguousarray(np.pad(image.astype(np.float32), ((0, 0), (0, 0), (top, bottom), (left, right))))
    dkh, dkw = kh + (kh - 1) * (dilation - 1), kw + (kw - 1) * (dilation - 1)
    h_out, w_out = (padded.shape[2] - dkh) // stride + 1, (padded.shape[3] - dkw) // stride + 1
    if h_out <= 0 or w_out <= 0:
        raise OracleError("Invalid convolution parameters lead to non-positive output size")
    out = np.empty((n, c_out, h_out, w_out), np.float32)
    kern = np.ascontiguousarray(kernel, dtype=np.float32)
    fpp = C.POINTER(C.c_float)
    b = np.ascontiguousarray(bias, dtype=np.float32) if bias is not None else None
    if b is not None and b.shape != (c_out,):
        raise OracleError(f"Invalid bias tensor shape: {b.shape}. Should be (C_out,)")
    _check(lib().oracle_conv2d_forward_f32(padded.ctypes.data_as(fpp), n, c_in, padded.shape[2], padded.shape[3], kern.ctypes.data_as(fpp),
                                           c_out, kh, kw, b.ctypes.data_as(fpp) if b is not None else None, stride, dilation,
                                           out.ctypes.data_as(fpp)))
    return out


def conv2d_backward(image: np.ndarray, kernel: np.ndarray, grad_out: np.ndarray, stride: int = 1, dilation: int = 1, padding="valid"):
    """(grad_image, grad_kernel, grad_bias) of Conv2dFused for the upstream gradient `grad_out`: the fused backward
    on the padded image (tenmo/cnn.mojo:546-948), then the border removed as the Pad operator's backward does."""
    n, c_in, h_in, w_in = image.shape
    c_out, _, kh, kw = kernel.shape
    top, bottom, left, right = conv_padding(h_in, w_in, kh, kw, stride, dilation, padding)
    padded = np.ascontiguousarray(np.pad(image.astype(np.float32), ((0, 0), (0, 0), (top, bottom), (left, right))))
    kern = np.ascontiguousarray(kernel, dtype=np.float32)
    go = np.ascontiguousarray(grad_out, dtype=np.float32)
    g_pad, g_k, g_b = np.empty_like(padded), np.empty_like(kern), np.empty(c_out, np.float32)
    fpp = C.POINTER(C.c_float)
    _check(lib().oracle_conv2d_backward_f32(padded.ctypes.data_as(fpp), n, c_in, padded.shape[2], padded.shape[3], kern.ctypes.data_as(fpp),
                                            c_out, kh, kw, stride, dilation, go.ctypes.data_as(fpp),
                                            g_pad.ctypes.data_as(fpp), g_k.ctypes.data_as(fpp), g_b.ctypes.data_as(fpp)))
    return g_pad[:, :, top:top + h_in, left:left + w_in].copy(), g_k, g_b
