"""pytest plugin that lets the GPU parity tests run, unchanged, against the CPU replay of the library.

    TENMO_HIP_LIBRARY=tests/replay/_build/libtenmo_hip_replay.so python -m pytest -p torch_on_host -m gpu tests/test_gpu_parity.py

The replay library's "device memory" is host memory, so a tensor the tests ask for on "cuda" can live on the CPU and its
data_ptr() is what the kernels need.  Loaded with -p (before collection), this module rewrites the few torch calls the
tests and the host mirror make with a cuda device so that they allocate on the CPU instead, and stands in for the
stream and availability queries.  Test infrastructure: it touches nothing unless it is loaded, and tests/test_replay_parity.py
only loads it in a child process of its own.
"""
import torch

_FACTORIES = ["randn", "rand", "zeros", "ones", "empty", "full", "arange", "tensor", "randint", "as_tensor",
              "zeros_like", "ones_like", "empty_like", "full_like", "randn_like", "eye", "linspace"]


def _host(device):
    if device is not None and str(device).startswith("cuda"):
        return "cpu"
    return device


def _wrap_factory(name):
    original = getattr(torch, name)

    def factory(*args, **kwargs):
        if "device" in kwargs:
            kwargs["device"] = _host(kwargs["device"])
        if kwargs.get("generator") is not None and hasattr(kwargs["generator"], "_host_generator"):
            kwargs["generator"] = kwargs["generator"]._host_generator
        return original(*args, **kwargs)

    factory.__name__ = name
    setattr(torch, name, factory)


class _Stream:
    cuda_stream = 0  # the null stream: the replay runs every launch at once


_OriginalGenerator = torch.Generator


class _Generator:
    """torch.Generator(device="cuda") on the host: the same interface, a CPU generator inside."""

    def __init__(self, device=None):
        self._host_generator = _OriginalGenerator(device="cpu")

    def manual_seed(self, seed):
        self._host_generator.manual_seed(seed)
        return self

    def __getattr__(self, name):
        return getattr(self._host_generator, name)


def _install():
    for name in _FACTORIES:
        _wrap_factory(name)
    torch.Generator = _Generator
    # a transfer between host and device is a copy: the two sides must not share memory
    torch.Tensor.cuda = lambda self, *a, **k: self.clone()
    torch.Tensor.cpu = lambda self, *a, **k: self.clone()
    torch.Tensor.is_cuda = property(lambda self: True)
    original_to = torch.Tensor.to

    def to(self, *args, **kwargs):
        args = tuple(_host(a) if isinstance(a, (str, torch.device)) else a for a in args)
        if "device" in kwargs:
            kwargs["device"] = _host(kwargs["device"])
        return original_to(self, *args, **kwargs)

    torch.Tensor.to = to
    torch.cuda.is_available = lambda: True
    torch.cuda.device_count = lambda: 1
    torch.cuda.current_stream = lambda *a, **k: _Stream()
    torch.cuda.synchronize = lambda *a, **k: None
    torch.cuda.empty_cache = lambda *a, **k: None


_install()
