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


def scatter_to_storage(t, grad):
    """Gradient of a view scattered (added) onto the storage behind it: what the reference's view backward
    leaves in the base tensor's gradbox.  Overlapping strides add up."""
    st = np.zeros(len(t["storage"]), np.float64)
    idx = np.full(tuple(t["shape"]), t.get("offset", 0), np.int64)
    for ax, (n, s) in enumerate(zip(t["shape"], strides_of(t))):
        shape = [1] * len(t["shape"])
        shape[ax] = n
        idx = idx + (np.arange(n, dtype=np.int64) * s).reshape(shape)
    np.add.at(st, idx.ravel(), np.asarray(grad, np.float64).ravel())
    return st


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


def conv_case_tensors(case):
    """image, kernel, bias (or None) and the keyword arguments of one `conv` case of the golden file."""
    def tensor(spec):
        if isinstance(spec, dict):
            return np.full(spec["shape"], spec["fill"], np.float32)
        return np.array(spec, np.float32)
    if "image_per_batch_fill" in case:
        image = np.empty(case["image_shape"], np.float32)
        for b, v in enumerate(case["image_per_batch_fill"]):
            image[b] = v
    elif "image_arange" in case:
        image = np.arange(int(np.prod(case["image_arange"])), dtype=np.float32).reshape(case["image_arange"])
    else:
        image = tensor(case["image"])
    kernel = tensor(case["kernel"])
    bias = np.array(case["bias"], np.float32) if "bias" in case else None
    padding = case.get("padding", "valid")
    if case.get("padding_kind") == "tuple":
        padding = tuple(padding)
    elif case.get("padding_kind") == "list":
        padding = [tuple(p) for p in padding]
    return image, kernel, bias, dict(stride=case.get("stride", 1), dilation=case.get("dilation", 1), padding=padding)


def check_conv_case(case, out):
    """Asserts what the reference's test asserts about the output of one `conv` case."""
    name = case["name"]
    if "expect_shape" in case:
        assert list(out.shape) == case["expect_shape"], name
    if "expect" in case:
        assert np.allclose(out, np.array(case["expect"], np.float32), atol=1e-5), name
    if "expect_all" in case:
        assert np.all(out == case["expect_all"]), name
    if "expect_planes" in case:
        for co, v in enumerate(case["expect_planes"]):
            assert np.all(out[0, co] == v), name
    for n, co, y, x, v in case.get("expect_at", []):
        assert abs(out[n, co, y, x] - v) <= 1e-5, name


def conv_reference64(image, kernel, bias, stride, dilation, pads):
    """Zero-padded cross-correlation in fp64 through numpy's sliding windows — shares nothing with the
    loops of the CPU restatement.  pads = (top, bottom, left, right)."""
    x = np.pad(image.astype(np.float64), ((0, 0), (0, 0), (pads[0], pads[1]), (pads[2], pads[3])))
    kh, kw = kernel.shape[2:]
    dkh, dkw = kh + (kh - 1) * (dilation - 1), kw + (kw - 1) * (dilation - 1)
    win = np.lib.stride_tricks.sliding_window_view(x, (dkh, dkw), axis=(2, 3))       # [N, C, H', W', dkh, dkw]
    win = win[:, :, ::stride, ::stride, ::dilation, ::dilation]                       # [N, C, Ho, Wo, kh, kw]
    out = np.einsum("nchwij,ocij->nohw", win, kernel.astype(np.float64))
    if bias is not None:
        out = out + bias.astype(np.float64)[None, :, None, None]
    return out


def check_conv_backward_case(case, grad_image, grad_kernel, grad_bias):
    """Asserts what the reference's test asserts about the gradients of one `conv.backward_cases` entry."""
    name = case["name"]
    if "grad_image" in case:
        assert np.array_equal(grad_image, np.array(case["grad_image"], np.float32)), name
    if "grad_kernel" in case:
        assert np.array_equal(grad_kernel, np.array(case["grad_kernel"], np.float32)), name
    if "grad_kernel_every_filter_channel" in case:
        want = np.array(case["grad_kernel_every_filter_channel"], np.float32)
        assert all(np.array_equal(grad_kernel[co, ci], want) for co in range(grad_kernel.shape[0]) for ci in range(grad_kernel.shape[1])), name
    if "grad_bias" in case:
        assert np.allclose(grad_bias, np.array(case["grad_bias"], np.float32), atol=1e-5), name
    if "grad_image_shape" in case:
        assert list(grad_image.shape) == case["grad_image_shape"] and list(grad_kernel.shape) == case["grad_kernel_shape"], name


def conv_backward_reference64(image, kernel, grad_out, stride, dilation, pads):
    """Gradients of the zero-padded cross-correlation by torch autograd in fp64 (independent of the restated loops)."""
    import torch
    x = torch.from_numpy(image).double().requires_grad_(True)
    k = torch.from_numpy(kernel).double().requires_grad_(True)
    b = torch.zeros(kernel.shape[0], dtype=torch.float64, requires_grad=True)
    y = torch.nn.functional.conv2d(torch.nn.functional.pad(x, (pads[2], pads[3], pads[0], pads[1])), k, b, stride=stride, dilation=dilation)
    y.backward(torch.from_numpy(grad_out).double())
    return x.grad.numpy(), k.grad.numpy(), b.grad.numpy()


def check_golden_extras(case, out, grad_a=None, grad_b=None):
    """The fixture keys beyond whole-tensor values: a slice of the result or of a gradient at leading indices (the reference asserts
    one batch of it), and shapes of gradients.  `out`, `grad_a`, `grad_b`: numpy arrays (gradients may be None when not computed)."""
    if "expect_slice" in case:
        got = np.asarray(out)[tuple(case["expect_slice"]["index"])]
        np.testing.assert_allclose(got, np.asarray(case["expect_slice"]["expect"], np.float32), rtol=1e-5, atol=1e-8, err_msg=case["name"])
    if "grad_A_slice" in case and grad_a is not None:
        got = np.asarray(grad_a)[tuple(case["grad_A_slice"]["index"])]
        np.testing.assert_allclose(got, np.asarray(case["grad_A_slice"]["expect"], np.float32), rtol=1e-5, err_msg=case["name"] + " grad_A slice")
    if "grad_A_shape" in case and grad_a is not None:
        assert list(np.shape(grad_a)) == case["grad_A_shape"], case["name"]
    if "grad_B_shape" in case and grad_b is not None:
        assert list(np.shape(grad_b)) == case["grad_B_shape"], case["name"]


GOLDEN_GRADIENT_KEYS = ("grad_A", "grad_B", "base_grad_A", "base_grad_B", "grad_A_slice", "grad_A_shape", "grad_B_shape")


def generated_operand(spec):
    """An operand of a `device_kernel_cases` fixture: the reference builds these with ones / zeros / arange / eye / literal values."""
    shape = tuple(spec["shape"])
    kind = spec["gen"]
    if kind == "ones":
        return np.ones(shape, np.float32)
    if kind == "zeros":
        return np.zeros(shape, np.float32)
    if kind == "arange":
        return np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    if kind == "eye":
        return np.eye(shape[0], dtype=np.float32)
    return np.asarray(spec["values"], np.float32).reshape(shape)


def exact_product(op, a, b):
    """The product in float64 (exact for these small integers): mm broadcasts batches; mv / vm broadcast the vector's batch."""
    a, b = a.astype(np.float64), b.astype(np.float64)
    if op == "mm":
        return a @ b
    if op == "mv":
        return (a @ b[..., None])[..., 0]
    return (a[..., None, :] @ b)[..., 0, :]
