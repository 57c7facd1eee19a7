"""ctypes binding of ``libtenmo_hip.so`` — the same symbols a Mojo ``DLHandle`` would bind.

There is no fallback: if the shared library is missing or a symbol is absent the import of any
operator fails loudly.  Nothing here computes; it only marshals pointers and sizes.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Sequence

MAX_RANK = 8
_HERE = os.path.dirname(os.path.abspath(__file__))
# TENMO_HIP_LIBRARY plays the role of the reference's BLAS_PATH define (tenmo/blashandle.mojo:108-110)
LIB_PATH = os.environ.get("TENMO_HIP_LIBRARY") or os.path.join(_HERE, "libtenmo_hip.so")

OP_DOT, OP_VM, OP_MV, OP_MM, OP_INVALID = 0, 1, 2, 3, -1


class TenmoHipError(RuntimeError):
    """An entry point returned a negative status; the text is tenmo_hip_last_error()."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[{status}] {message}")
        self.status = status
        self.message = message


class CView(C.Structure):
    """tenmo_view of include/tenmo_hip.h"""

    _fields_ = [
        ("data", C.c_void_p),
        ("offset", C.c_int64),
        ("rank", C.c_int32),
        ("shape", C.c_int64 * MAX_RANK),
        ("strides", C.c_int64 * MAX_RANK),
    ]


_i64p = C.POINTER(C.c_int64)
_i32p = C.POINTER(C.c_int32)
_vp = C.POINTER(CView)
_ptr = C.c_void_p

# name -> (restype, argtypes); every function include/tenmo_hip.h declares
SIGNATURES = {
    "tenmo_hip_init": (C.c_int, [C.c_int]),
    "tenmo_hip_shutdown": (C.c_int, []),
    "tenmo_hip_sync": (C.c_int, []),
    "tenmo_hip_last_error": (C.c_char_p, []),
    "tenmo_hip_get_stream": (C.c_void_p, []),
    "tenmo_hip_set_stream": (C.c_int, [C.c_void_p]),
    "tenmo_hip_device_info": (C.c_int, [C.POINTER(C.c_int), C.c_char_p, C.c_int]),
    "tenmo_hip_set_tuning": (C.c_int, [C.c_char_p, C.c_int]),
    "tenmo_hip_timer_begin": (C.c_int, []),
    "tenmo_hip_timer_end": (C.c_int, [C.POINTER(C.c_float)]),
    "tenmo_hip_clock_probe": (C.c_int, [C.c_int32, C.POINTER(C.c_float)]),
    "tenmo_hip_gemm_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64,
                                     _ptr, C.c_int64, C.c_int64, C.c_int64, C.c_int32, _i64p, _i64p, _i64p,
                                     C.c_int32, C.c_int32]),
    "tenmo_hip_gemm_epilogue_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64,
                                              _ptr, C.c_int64, C.c_int64, C.c_int64, C.c_int32, _i64p, _i64p, _i64p,
                                              _ptr, C.c_int32, _ptr, C.c_int32]),
    "tenmo_hip_mv_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, _ptr,
                                   C.c_int64, C.c_int64, C.c_int32, _i64p, _i64p, _i64p, C.c_int32, C.c_int32]),
    "tenmo_hip_vm_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64, _ptr,
                                   C.c_int64, C.c_int64, C.c_int32, _i64p, _i64p, _i64p, C.c_int32, C.c_int32]),
    "tenmo_hip_vm_f32_noalloc": (C.c_int, [_ptr, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64, _ptr,
                                           C.c_int64, C.c_int64, C.c_int32, _i64p, _i64p, _i64p, C.c_int32, C.c_int32]),
    "tenmo_hip_column_sum_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int32, C.c_int32]),
    "tenmo_hip_dot_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int32]),
    "tenmo_hip_classify_matmul": (C.c_int, [C.c_int32, _i64p, C.c_int32, _i64p]),
    "tenmo_hip_result_shape": (C.c_int64, [C.c_int32, _vp, _vp, _i64p, _i32p]),
    "tenmo_hip_matmul_nd": (C.c_int, [_vp, _vp, _ptr, C.c_int32]),
    "tenmo_hip_linear_nd": (C.c_int, [_vp, _vp, _ptr, C.c_int32, _ptr, C.c_int32]),
    "tenmo_hip_matrix_vector_nd": (C.c_int, [_vp, _vp, _ptr, C.c_int32]),
    "tenmo_hip_vector_matmul_nd": (C.c_int, [_vp, _vp, _ptr, C.c_int32]),
    "tenmo_hip_matmul_backward": (C.c_int, [_vp, _vp, _ptr, _ptr, _ptr, C.c_int32]),
    "tenmo_hip_linear_backward": (C.c_int, [_vp, _vp, _ptr, _ptr, _ptr, _ptr, C.c_int32]),
    "tenmo_hip_mv_backward": (C.c_int, [_vp, _vp, _ptr, _ptr, _ptr, C.c_int32]),
    "tenmo_hip_vm_backward": (C.c_int, [_vp, _vp, _ptr, _ptr, _ptr, C.c_int32]),
    "tenmo_hip_cross_entropy_forward_f32": (C.c_int, [_ptr, _ptr, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_float,
                                                      _ptr, _ptr, _ptr, _ptr, C.c_int32]),
    "tenmo_hip_cross_entropy_backward_f32": (C.c_int, [_ptr, _ptr, C.c_int32, _ptr, C.c_int64, C.c_int64, C.c_int64, C.c_float,
                                                       C.c_int32, C.c_int32, _ptr, C.c_int32, C.c_int32]),
    "tenmo_hip_conv2d_forward_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64,
                                               _ptr, C.c_int64, C.c_int64, _ptr, C.c_int32]),
    "tenmo_hip_conv2d_backward_f32": (C.c_int, [_ptr, C.c_int64, C.c_int64, C.c_int64, C.c_int64, _ptr, C.c_int64, C.c_int64, C.c_int64,
                                                C.c_int64, C.c_int64, _ptr, _ptr, _ptr, _ptr, C.c_int32, C.c_int32]),
    "tenmo_hip_sgd_step_f32": (C.c_int, [_ptr, _ptr, _ptr, C.c_int64, C.c_float, C.c_float, C.c_float, C.c_int32]),
    "cblas_sgemm": (None, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _ptr, C.c_int,
                           _ptr, C.c_int, C.c_float, _ptr, C.c_int]),
    "tenmo_hip_mlp_create": (C.c_void_p, [C.c_int32, _i64p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int64]),
    "tenmo_hip_mlp_destroy": (None, [C.c_void_p]),
    "tenmo_hip_mlp_step": (C.c_int, [C.c_void_p, _ptr, _ptr, C.c_int64, C.c_float, _ptr, C.c_int32]),
    "tenmo_hip_mlp_step_graph": (C.c_int, [C.c_void_p, _ptr, _ptr, C.c_int64, C.c_float, _ptr, C.c_int32]),
    "tenmo_hip_mlp_forward": (C.c_int, [C.c_void_p, _ptr, C.c_int64, _ptr, C.c_int32]),
    "tenmo_hip_mlp_get_params": (C.c_int, [C.c_void_p, C.c_int32, _ptr, _ptr]),
    "tenmo_hip_mlp_get_grads": (C.c_int, [C.c_void_p, C.c_int32, _ptr, _ptr]),
}

_lib = None


def load() -> C.CDLL:
    """dlopen the library and bind every declared symbol (raises if any is missing)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m tenmo_amd.build` (hipcc, gfx950). "
                "tenmo_amd has no CPU or PyTorch fallback."
            )
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the export is missing
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status: int) -> int:
    if status < 0:
        raise TenmoHipError(int(status), load().tenmo_hip_last_error().decode(errors="replace"))
    return status


def i64(seq: Sequence[int]):
    return (C.c_int64 * max(1, len(seq)))(*[int(x) for x in seq])


_initialised = False


def init(device_id: int = 0) -> None:
    """tenmo_hip_init + route the library onto the caller's current torch stream so that
    allocations and copies made through torch are ordered with the library's kernels."""
    global _initialised
    L = load()
    check(L.tenmo_hip_init(device_id))
    if not _initialised:
        import torch

        check(L.tenmo_hip_set_stream(C.c_void_p(torch.cuda.current_stream(device_id).cuda_stream)))
        _initialised = True


def make_view(data_ptr: int, offset: int, shape: Sequence[int], strides: Sequence[int]) -> CView:
    if len(shape) > MAX_RANK:
        raise TenmoHipError(-2, f"rank {len(shape)} exceeds max_rank {MAX_RANK}")
    v = CView()
    v.data = data_ptr
    v.offset = int(offset)
    v.rank = len(shape)
    for i, (s, t) in enumerate(zip(shape, strides)):
        v.shape[i] = int(s)
        v.strides[i] = int(t)
    return v
