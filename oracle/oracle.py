"""Loader of the CPU oracle (oracle/libsgl_oracle.so) on numpy arrays.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker / the timed CPU baseline.  The
package under starrygl-framework_amd/ never imports this module.
"""
import ctypes as C
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.join(os.path.dirname(_HERE), "starrygl-framework_amd")
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)

from starrygl_amd.lib import _abi  # noqa: E402
from starrygl_amd.lib.driver import HotPath  # noqa: E402

LIB_PATH = os.path.join(_HERE, "libsgl_oracle.so")


def build(force=False):
    """Compile the oracle when its source is newer than the library (make decides)."""
    have_src = os.path.exists(os.path.join(_HERE, "sgl_oracle.c"))
    if have_src and (force or not os.path.exists(LIB_PATH) or
                     os.path.getmtime(LIB_PATH) < max(os.path.getmtime(os.path.join(_HERE, "sgl_oracle.c")),
                                                      os.path.getmtime(os.path.join(os.path.dirname(_HERE), "include", "sgl_hot.h")))):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []) + ["libsgl_oracle.so"])
    return LIB_PATH


class NumpyBackend:
    _dt = {"i64": np.int64, "i32": np.int32, "f32": np.float32, "u8": np.uint8,
           "bf16": np.uint16, "f16": np.float16}

    def empty(self, shape, dtype="i64"):
        return np.empty(shape, dtype=self._dt[dtype])

    def zeros(self, shape, dtype="i64"):
        return np.zeros(shape, dtype=self._dt[dtype])

    def asarray(self, a, dtype="i64"):
        return np.ascontiguousarray(np.asarray(a, dtype=self._dt[dtype]))

    def ptr(self, a):
        if a is None:
            return None
        assert a.flags["C_CONTIGUOUS"]
        return a.ctypes.data

    def stream(self):
        return None

    def check(self, a, dtype, name):
        if a.dtype != self._dt[dtype]:
            raise TypeError(f"{name} must be {dtype}, got {a.dtype}")
        if not a.flags["C_CONTIGUOUS"]:
            raise ValueError(f"{name} must be contiguous")
        return a

    def tolist(self, a):
        return a.tolist()

    def nbytes(self, a):
        return a.nbytes


_cached = None


def load():
    """-> (HotPath on numpy arrays, raw bound library)."""
    global _cached
    if _cached is None:
        build()
        cdll = C.CDLL(LIB_PATH)
        lib = _abi.bind(cdll, "sglo_")
        cdll.sglo_set_num_threads.argtypes = [C.c_int32]
        cdll.sglo_get_max_threads.restype = C.c_int32
        cdll.sglo_philox4x32_10.argtypes = [C.c_void_p] * 3
        cdll.sglo_draw_bits.restype = C.c_uint64
        cdll.sglo_draw_bits.argtypes = [C.c_uint64, C.c_int32, C.c_int64, C.c_int32]
        cdll.sglo_bounded.restype = C.c_int64
        cdll.sglo_bounded.argtypes = [C.c_uint64, C.c_int64]
        # the indexed CPU sampler (same prototype as sample_khop): the CPU side of an equal-work timing
        cdll.sglo_sample_khop_indexed.restype = lib.sample_khop.restype
        cdll.sglo_sample_khop_indexed.argtypes = lib.sample_khop.argtypes
        _cached = (HotPath(lib, NumpyBackend()), cdll)
    return _cached


def sample_khop_indexed(hp, cdll, g, roots, ts_ptr, root_ts, neg_roots, neg_ts, layers, p):
    """`hp.sample_khop` through sglo_sample_khop_indexed: the oracle's sampler given the next-hop index of
    `g` (g.view.hop_hint) and the root hints of `p`, searching only what those leave open."""
    plain, hp.lib.sample_khop = hp.lib.sample_khop, cdll.sglo_sample_khop_indexed
    try:
        return hp.sample_khop(g, roots, ts_ptr, root_ts, neg_roots, neg_ts, layers, p)
    finally:
        hp.lib.sample_khop = plain
