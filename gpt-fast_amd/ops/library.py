"""Loading the compiled HIP libraries and calling their C entry points.

There is no fallback: if a library cannot be built or loaded, or a kernel launch
reports an error, an exception is raised.
"""
import ctypes
from typing import Dict

import torch

from ..csrc import build as _build


class KernelError(RuntimeError):
    pass


_loaded: Dict[str, ctypes.CDLL] = {}


def library(name: str) -> ctypes.CDLL:
    """The shared library of module ``name``, built first if it is not there."""
    lib = _loaded.get(name)
    if lib is None:
        _build.ensure([name])
        path = _build.library_path(name)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the HIP library {path}: {e}") from None
        _loaded[name] = lib
    return lib


def loaded_libraries():
    return {n: _build.library_path(n) for n in _loaded}


def stream_handle() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def check(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what}: HIP error {code}")


def require_device(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("HIP kernels take device tensors only; there is no CPU path")


def require_contiguous(**tensors) -> None:
    for name, t in tensors.items():
        if t is not None and not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous")
