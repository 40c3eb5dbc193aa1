"""The C-ABI library loads and exports every symbol include/sgl_hot.h declares
(no compute calls: this runs without a GPU)."""
import ctypes as C
import os
import re

from starrygl_amd.lib import LIB_PATH, _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "sgl_hot.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sgl_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 16
    lib = C.CDLL(LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in sgl_hot.h but not exported"
    assert sorted("sgl_" + k for k in _abi.PROTOTYPES) == names


def test_abi_version_and_host_side_errors():
    lib = _abi.bind(C.CDLL(LIB_PATH))
    assert lib.abi_version() == _abi.ABI_VERSION
    # the ctypes mirrors have the layout the library was compiled with
    for which, mirror in enumerate(_abi.STRUCTS):
        assert lib.struct_bytes(which) == C.sizeof(mirror), mirror.__name__
    assert lib.struct_bytes(len(_abi.STRUCTS)) == 0 and lib.struct_bytes(-1) == 0
    # argument validation happens on the host, before any HIP call
    p = _abi.SampleParams(7, 3, -1, 0, 0, 0, 0, 0, None, 0, None, 0, 0)
    g = _abi.TCSR(1, 0, 8, None, None, None, None, None)
    assert lib.sample_hop(C.byref(g), None, None, 0, None, C.byref(p), None, None, 0, None) == _abi.SGL_ENOTSUP
    assert b"undefined sampling strategy" in lib.last_error_string()
    assert lib.sample_hop(None, None, None, 0, None, C.byref(p), None, None, 0, None) == _abi.SGL_EINVAL
    p.type, p.fanout = _abi.SAMPLE_UNIFORM, _abi.UNIFORM_MAX_FANOUT + 1
    assert lib.sample_hop(C.byref(g), None, None, 0, None, C.byref(p), None, None, 0, None) == _abi.SGL_ENOTSUP
    p.type, p.fanout = _abi.SAMPLE_RECENT, _abi.RECENT_MAX_FANOUT + 1     # beyond what a chunk's 32-bit edge offsets hold
    assert lib.sample_hop(C.byref(g), None, None, 0, None, C.byref(p), None, None, 0, None) == _abi.SGL_ENOTSUP
    p.fanout = _abi.RECENT_MAX_FANOUT
    assert lib.sample_hop(C.byref(g), None, None, 0, None, C.byref(p), None, None, 0, None) == _abi.SGL_EINVAL   # (out is NULL)
    c = _abi.Cache(10, 6, -1, None, 0, None, 8, 10, None, None, None)
    assert lib.gather(C.byref(c), 8, 1, None, 8, None, None, None) == _abi.SGL_EINVAL   # row_bytes % 4
    assert lib.time_encode(8, 5, 1, None, 8, 8, 4, 8, None) == _abi.SGL_EINVAL           # bad dtype
    assert lib.remap_init(None, 0, 10, None) == _abi.SGL_EINVAL
    assert lib.remap_state_bytes(64) >= 64 * 8 + 8


def test_oracle_exports_the_same_interface(oracle):
    assert oracle.lib.abi_version() == _abi.ABI_VERSION
