"""tenmo_amd — MI355X (gfx950) implementation of Tenmo's fp32 matrix-product path.

The product is ``libtenmo_hip.so`` (hand-written HIP; C ABI in ``include/tenmo_hip.h``).  The Python
modules mirror the slice of the reference's host API that sits directly above that boundary
(``Tensor.matmul``, ``Matmul*``, ``Linear``, the backward entries, ``BLASHandle``) so that tests read
like the reference's own.  There is no CPU or PyTorch fallback: without the built library, or
without a gfx950 GPU, operators raise.
"""
from ._lib import LIB_PATH, TenmoHipError, init, load  # noqa: F401

__all__ = ["LIB_PATH", "TenmoHipError", "init", "load"]
