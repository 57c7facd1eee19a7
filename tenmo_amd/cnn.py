"""Conv2dFused forward: host-side mirror of tenmo/cnn.mojo:18-273 above ``tenmo_hip_conv2d_forward_f32``.

The reference's layer parses ``padding`` ("valid", "same", int, (h, w) pair, [(top, bottom), (left, right)];
cnn.mojo:183-222), zero-pads the image with its ``Pad`` operator (:229-235) and hands the padded image to
the fused im2col kernel (``FusedIm2Col.forward``, :308-507).  The same split is kept here: the padding is a
device-side copy (plumbing, ``torch.nn.functional.pad``), the convolution itself runs in the library as an
implicit GEMM on the matrix-core kernel.  ``Conv2dFused.backward`` is ``FusedCol2ImBackward`` (cnn.mojo:546-948)
through ``tenmo_hip_conv2d_backward_f32`` followed by the removal of the padding border (the ``Pad`` operator's
backward); it is a plain function here, not wired into the autograd mirror of ``tensor.py``.
"""
from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from . import _lib
from ._lib import TenmoHipError, check
from .ndbuffer import NDBuffer
from .tensor import Tensor

Padding = Union[str, int, Tuple[int, int], List[Tuple[int, int]]]


def parse_padding(h_in: int, w_in: int, kh: int, kw: int, stride: int, dilation: int, padding: Padding) -> Tuple[int, int, int, int]:
    """(top, bottom, left, right) — cnn.mojo:183-222."""
    dkh, dkw = kh + (kh - 1) * (dilation - 1), kw + (kw - 1) * (dilation - 1)
    if isinstance(padding, str):
        if padding == "valid":
            return 0, 0, 0, 0
        if padding == "same":
            h_target, w_target = (h_in + stride - 1) // stride, (w_in + stride - 1) // stride
            ph, pw = (h_target - 1) * stride + dkh - h_in, (w_target - 1) * stride + dkw - w_in
            return ph // 2, ph - ph // 2, pw // 2, pw - pw // 2
        raise TenmoHipError(-3, "Unsupported padding mode: use 'valid' or 'same'")
    if isinstance(padding, int):
        return padding, padding, padding, padding
    if isinstance(padding, tuple):
        return padding[0], padding[0], padding[1], padding[1]
    if isinstance(padding, list):
        if len(padding) != 2:
            raise TenmoHipError(-3, "Padding list must contain exactly 2 tuples")
        return padding[0][0], padding[0][1], padding[1][0], padding[1][1]
    raise TenmoHipError(-3, "Invalid padding type")


class Conv2dFused:
    """``Conv2dFused[dtype].forward(image, kernel, bias, stride, dilation, padding)`` — cnn.mojo:77-100."""

    @staticmethod
    def forward(image: Tensor, kernel: Tensor, bias: Optional[Tensor] = None, stride: int = 1, dilation: int = 1,
                padding: Padding = "valid", sync: bool = False) -> Tensor:
        ish, ksh = image.shape(), kernel.shape()
        if len(ish) != 4:
            raise TenmoHipError(-2, "Image must be 4D: (N, C_in, H_in, W_in)")
        if len(ksh) != 4:
            raise TenmoHipError(-2, "Kernel must be 4D: (C_out, C_in, KH, KW)")
        if ksh[1] != ish[1]:
            raise TenmoHipError(-2, "Kernel input channels must match input channels")
        n, c_in, h_in, w_in = ish
        c_out, _, kh, kw = ksh
        if bias is not None and tuple(bias.shape()) != (c_out,):
            raise TenmoHipError(-2, f"Invalid bias tensor shape: {tuple(bias.shape())}. Should be (C_out,)")
        top, bottom, left, right = parse_padding(h_in, w_in, kh, kw, stride, dilation, padding)
        dkh, dkw = kh + (kh - 1) * (dilation - 1), kw + (kw - 1) * (dilation - 1)
        h_pad, w_pad = h_in + top + bottom, w_in + left + right
        h_out, w_out = (h_pad - dkh) // stride + 1, (w_pad - dkw) // stride + 1
        if h_out <= 0 or w_out <= 0:
            raise TenmoHipError(-2, "Invalid convolution parameters lead to non-positive output size")
        for t, who in ((image, "image"), (kernel, "kernel")) + (((bias, "bias"),) if bias is not None else ()):
            if not t.buffer.is_contiguous():
                raise TenmoHipError(-4, f"Conv2dFused: {who} must be contiguous")
        _lib.init()
        img = image.buffer.storage[image.buffer.offset:image.buffer.offset + n * c_in * h_in * w_in].view(n, c_in, h_in, w_in)
        if top or bottom or left or right:  # the reference's Pad operator (cnn.mojo:229-235): a zero-filled copy
            img = torch.nn.functional.pad(img, (left, right, top, bottom)).contiguous()
        out = NDBuffer.empty((n, c_out, h_out, w_out))
        L = _lib.load()
        check(L.tenmo_hip_conv2d_forward_f32(img.data_ptr(), n, c_in, h_pad, w_pad,
                                             kernel.buffer.data_ptr() + 4 * kernel.buffer.offset, c_out, kh, kw,
                                             (bias.buffer.data_ptr() + 4 * bias.buffer.offset) if bias is not None else None,
                                             stride, dilation, out.data_ptr(), 1 if sync else 0))
        if not sync:
            check(L.tenmo_hip_sync())  # `img` (a temporary when padded) must outlive the launch
        return Tensor(out)

    @staticmethod
    def backward(image: Tensor, kernel: Tensor, grad_out: Tensor, stride: int = 1, dilation: int = 1, padding: Padding = "valid",
                 need_image: bool = True, need_kernel: bool = True, need_bias: bool = True):
        """(grad_image, grad_kernel, grad_bias) for the upstream gradient of ``forward``'s output; entries not needed are None."""
        n, c_in, h_in, w_in = image.shape()
        c_out, _, kh, kw = kernel.shape()
        top, bottom, left, right = parse_padding(h_in, w_in, kh, kw, stride, dilation, padding)
        h_pad, w_pad = h_in + top + bottom, w_in + left + right
        for t, who in ((image, "image"), (kernel, "kernel"), (grad_out, "grad_out")):
            if not t.buffer.is_contiguous():
                raise TenmoHipError(-4, f"Conv2dFused.backward: {who} must be contiguous")
        _lib.init()
        img = image.buffer.storage[image.buffer.offset:image.buffer.offset + n * c_in * h_in * w_in].view(n, c_in, h_in, w_in)
        if top or bottom or left or right:
            img = torch.nn.functional.pad(img, (left, right, top, bottom)).contiguous()
        g_pad = NDBuffer.empty((n, c_in, h_pad, w_pad)) if need_image else None
        g_k = NDBuffer.empty((c_out, c_in, kh, kw)) if need_kernel else None
        g_b = NDBuffer.empty((c_out,)) if need_bias else None
        L = _lib.load()
        check(L.tenmo_hip_conv2d_backward_f32(img.data_ptr(), n, c_in, h_pad, w_pad, kernel.buffer.data_ptr() + 4 * kernel.buffer.offset,
                                              c_out, kh, kw, stride, dilation, grad_out.buffer.data_ptr() + 4 * grad_out.buffer.offset,
                                              g_pad.data_ptr() if g_pad else None, g_k.data_ptr() if g_k else None,
                                              g_b.data_ptr() if g_b else None, 0, 1))
        g_img = None
        if g_pad is not None:  # Pad backward: drop the border
            inner = g_pad.storage[:n * c_in * h_pad * w_pad].view(n, c_in, h_pad, w_pad)[:, :, top:top + h_in, left:left + w_in].contiguous()
            g_img = Tensor(NDBuffer(inner.view(-1), (n, c_in, h_in, w_in)))
        return g_img, Tensor(g_k) if g_k else None, Tensor(g_b) if g_b else None
