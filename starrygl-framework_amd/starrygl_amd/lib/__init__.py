"""Loader of libsgl_hot.so, the HIP implementation of include/sgl_hot.h.

There is no CPU fallback: if the shared library is missing, `load()` raises.
PyTorch is imported first so that the library binds to the HIP runtime that
PyTorch already mapped (one runtime per process, shared streams and pointers).
"""
import ctypes as C
import os

from . import _abi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libsgl_hot.so")

_lib = None


def load():
    """-> bound entry points of libsgl_hot.so (loaded once per process)."""
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (maps libamdhip64 before our library needs it)
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C starrygl-framework_amd/csrc` "
                "(or __graft_entry__.build()); this package has no CPU fallback")
        _lib = _abi.bind(C.CDLL(LIB_PATH), "sgl_")
    return _lib


_hot = {}


def hot_path(device="cuda:0"):
    """-> HotPath driving libsgl_hot.so on `device` (cached per device)."""
    import torch
    from .driver import HotPath, TorchBackend
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("the sgl hot path runs on a HIP device only (got %s)" % dev)
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    key = str(dev)
    if key not in _hot:
        _hot[key] = HotPath(load(), TorchBackend(dev))
    return _hot[key]
