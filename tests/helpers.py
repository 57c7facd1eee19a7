"""Shared test helpers: fixture decoding and error measures."""
import numpy as np

RTOL_FRO = 1e-5  # relative Frobenius error against the fp64 reference (the stated tolerance)


def storage_of(t):
    return np.asarray(t["storage"], np.float32)


def strides_of(t):
    if "strides" in t:
        return tuple(t["strides"])
    acc, out = 1, []
    for s in reversed(t["shape"]):
        out.append(acc)
        acc *= s
    return tuple(reversed(out))


def numpy_view(t):
    """Materialise a fixture operand (storage + shape/strides/offset) as a numpy array."""
    st = storage_of(t)
    return np.lib.stride_tricks.as_strided(st[t.get("offset", 0):], tuple(t["shape"]), tuple(4 * s for s in strides_of(t))).copy()


def rel_fro(x, ref):
    x = np.asarray(x, np.float64)
    ref = np.asarray(ref, np.float64)
    d = np.linalg.norm((x - ref).ravel())
    n = np.linalg.norm(ref.ravel())
    return d / n if n > 0 else d


def ref_matmul64(a, b):
    return np.matmul(np.asarray(a, np.float64), np.asarray(b, np.float64))


def ce_reference64(logits, target, ignore_index=-100, ls=0.0):
    """Independent fp64 statement of class-index cross-entropy: per-row loss and d(sum of losses)/d logits."""
    x = np.asarray(logits, np.float64)
    M, C = x.shape
    lse = np.log(np.exp(x - x.max(1, keepdims=True)).sum(1)) + x.max(1)
    logp = x - lse[:, None]
    p = np.exp(logp)
    valid = np.asarray(target) != ignore_index
    t = np.where(valid, target, 0)
    nll = -logp[np.arange(M), t]
    loss = np.where(valid, (1 - ls) * nll + ls * (-logp.mean(1)), 0.0)
    onehot = np.zeros((M, C))
    onehot[np.arange(M), t] = 1.0
    grad = (p - (1 - ls) * onehot - ls / C) * valid[:, None]
    return p, loss, grad
