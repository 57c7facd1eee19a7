"""Seeded synthetic inputs owned by this build (numpy, host side).

The reference seeds Mojo's stdlib generator (tenmo/tensor.mojo:1320-1332) whose stream cannot be
reproduced without a Mojo runtime, so "same seeded inputs" means: one counter-based generator here
feeds both the CPU restatement and the GPU.  Normal variates are drawn in fp64 and then cast, as the
reference casts fp64 -> fp32 at tenmo/ndbuffer.mojo:228.
"""
from __future__ import annotations

import zlib
from typing import Sequence

import numpy as np


def _generator(seed: int, name: str) -> np.random.Generator:
    # Philox is counter-based: the stream depends only on (seed, name), not on call order
    key = (int(seed) & 0xFFFFFFFF) << 32 | (zlib.crc32(name.encode()) & 0xFFFFFFFF)
    return np.random.Generator(np.random.Philox(key=key))


def randn(shape: Sequence[int], seed: int, name: str, std: float = 1.0) -> np.ndarray:
    g = _generator(seed, name)
    return (g.standard_normal(size=tuple(shape), dtype=np.float64) * std).astype(np.float32)


def uniform(shape: Sequence[int], seed: int, name: str, low: float, high: float) -> np.ndarray:
    g = _generator(seed, name)
    return g.uniform(low, high, size=tuple(shape)).astype(np.float32)


def mnist_like_batch(batch: int, seed: int, step: int):
    """784 uint8 pixels uniform in [0,255] scaled by 1/255, labels uniform in 0..9."""
    g = _generator(seed, f"mnist-batch-{step}")
    x = g.integers(0, 256, size=(batch, 784), dtype=np.uint8).astype(np.float32) * np.float32(1.0 / 255.0)
    y = g.integers(0, 10, size=(batch,), dtype=np.int32)
    return x, y


def xavier_mlp(dims: Sequence[int], seed: int):
    """Xavier-uniform weights [in,out] and zero biases (tenmo/net.mojo:87-114)."""
    Ws, bs = [], []
    for l in range(len(dims) - 1):
        limit = float(np.sqrt(6.0 / float(dims[l] + dims[l + 1])))
        Ws.append(uniform((dims[l], dims[l + 1]), seed, f"xavier-w{l}", -limit, limit))
        bs.append(np.zeros((dims[l + 1],), np.float32))
    return Ws, bs
