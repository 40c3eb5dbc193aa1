"""ctypes view of include/sgl_hot.h: structs, constants and prototypes.

`bind(cdll, prefix)` attaches argument/return types to every entry point the
header declares.  The product library exports them as ``sgl_*``.
"""
import ctypes as C

ABI_VERSION = 8

SGL_OK, SGL_EINVAL, SGL_ERANGE, SGL_ENOTSUP, SGL_EHIP, SGL_ENOMEM = 0, -1, -2, -3, -4, -5
SAMPLE_RECENT, SAMPLE_UNIFORM = 0, 1
UNIFORM_MAX_FANOUT = 1024
RECENT_MAX_FANOUT = 1 << 21
STATIC_HOP_MAX_SLOTS = 65536
BATCH_MAX = 64
UNIQUE_SORTED, UNIQUE_GROUPED, UNIQUE_PREMARKED, UNIQUE_MULTI_LAUNCH = 0, 1, 0x100, 0x200
SAMPLE_MULTI_LAUNCH = 1
DT_I64, DT_F32 = 0, 1

SAMPLE_TYPES = {"recent": SAMPLE_RECENT, "uniform": SAMPLE_UNIFORM}

i32, i64, u64, vp, sz = C.c_int32, C.c_int64, C.c_uint64, C.c_void_p, C.c_size_t


class TCSR(C.Structure):
    _fields_ = [("n", i64), ("m", i64), ("row_ptr", vp), ("col", vp), ("ts", vp), ("eid", vp), ("hop_hint", vp),
                ("rec", vp)]


class SampleParams(C.Structure):
    _fields_ = [("type", i32), ("fanout", i32), ("allowed_offset", i64),
                ("equal_root_time", i32), ("keep_root_time", i32),
                ("replace", i32), ("hop", i32), ("seed", u64),
                ("mark_state", vp), ("mark_universe", i64), ("root_hint", vp),
                ("flags", i32), ("reserved", i32)]


class HopOut(C.Structure):
    _fields_ = [("capacity_slots", i64), ("capacity_edges", i64),
                ("root_start_ptr", vp), ("root_end_ptr", vp),
                ("neighbors", vp), ("neighbors_ts", vp),
                ("neighbors_eid", vp), ("neighbors_dt", vp), ("counts", vp)]


class Cache(C.Structure):
    _fields_ = [("rows", i64), ("row_bytes", i64), ("id_mask", i64),
                ("g2l", vp), ("g2l_len", i64), ("hot_slot", vp),
                ("hot", vp), ("hot_rows", i64), ("cold", vp),
                ("ts_hot", vp), ("ts_cold", vp), ("cold_stride", i64), ("ts_cold_stride", i64), ("hot_stride", i64)]


class GatherSeg(C.Structure):
    _fields_ = [("cache", C.POINTER(Cache)), ("ids", vp), ("N_max", i64), ("N_dev", vp), ("out", vp), ("out_ts", vp)]


class SeedQuery(C.Structure):
    _fields_ = [("chunk_ptr", vp), ("chunk_nodes", vp), ("num_chunks", i64), ("chunks", vp),
                ("cand_off", vp), ("n_cand", i64), ("t_begin", i64), ("t_end", i64)]


class WindowParams(C.Structure):
    _fields_ = [("lo_offset", i64), ("hi_offset", i64), ("bounded_below", i32), ("keep_slot_time", i32),
                ("first_k", i64), ("edge_tag", vp), ("tag_value", i64)]


# in the order of sgl_struct_bytes(which)
STRUCTS = (TCSR, SampleParams, HopOut, Cache, GatherSeg, SeedQuery, WindowParams)


P = C.POINTER

# name -> (restype, argtypes); the order follows include/sgl_hot.h
PROTOTYPES = {
    "last_error_string": (C.c_char_p, []),
    "abi_version": (i32, []),
    "struct_bytes": (sz, [i32]),
    "set_wait_limit": (i32, [i32]),
    "tcsr_build_workspace_bytes": (sz, [i64, i64]),
    "tcsr_build": (i32, [i64, i64, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]),
    "tcsr_validate": (i32, [P(TCSR), vp, sz, vp]),
    "tcsr_hop_hint_build": (i32, [P(TCSR), vp, vp]),
    "tcsr_records_build": (i32, [P(TCSR), vp, vp]),
    "window_end": (i32, [P(TCSR), vp, vp, i64, vp, vp]),
    "sample_hop_workspace_bytes": (sz, [i64]),
    "sample_hop": (i32, [P(TCSR), vp, vp, i64, vp, P(SampleParams), P(HopOut), vp, sz, vp]),
    "sample_hop_static": (i32, [P(TCSR), vp, vp, i64, vp, P(SampleParams), P(HopOut), vp]),
    "sample_window_workspace_bytes": (sz, [i64]),
    "sample_window": (i32, [P(TCSR), vp, vp, i64, P(WindowParams), P(HopOut), vp, sz, vp]),
    "sample_khop_workspace_bytes": (sz, [i64, i32, i32]),
    "sample_khop": (i32, [P(TCSR), i64, vp, vp, i64, vp, i64, vp, vp, i32,
                          P(SampleParams), vp, vp, P(HopOut), vp, sz, vp]),
    "sample_khop_multi_workspace_bytes": (sz, [i64, i32, i32, i32]),
    "sample_khop_multi": (i32, [P(TCSR), i64, vp, vp, i64, vp, i64, vp, vp, i32, i32,
                                P(SampleParams), vp, vp, P(HopOut), vp, sz, vp]),
    "sample_khop_batched_workspace_bytes": (sz, [i64, i32, i32, i32]),
    "sample_khop_batched": (i32, [P(TCSR), i32, vp, i64, vp, vp, vp, i32, i32, P(SampleParams), P(HopOut), vp, vp, sz, vp]),
    "remap_state_bytes": (sz, [i64]),
    "remap_init": (i32, [vp, sz, i64, vp]),
    "unique_workspace_bytes": (sz, [i64, i32, P(i64)]),
    "unique_compact": (i32, [vp, i64, i32, i32, i32, P(vp), P(i64), P(vp), P(vp),
                             vp, i64, vp, vp, sz, vp]),
    "remap_hashed_state_bytes": (sz, [i64]),
    "remap_hashed_init": (i32, [vp, sz, i64, vp]),
    "unique_hashed_workspace_bytes": (sz, [i64, i32, P(i64)]),
    "unique_compact_hashed": (i32, [vp, i64, i32, i32, i32, P(vp), P(i64), P(vp), P(vp),
                                    vp, i64, vp, vp, sz, vp]),
    "remap_batched_state_bytes": (sz, [i64, i32]),
    "remap_batched_init": (i32, [vp, sz, i64, i32, vp]),
    "unique_batched_workspace_bytes": (sz, [i64, i32]),
    "unique_compact_batched": (i32, [vp, i64, i32, i32, P(vp), P(i64), P(vp), P(vp), vp, i64, vp, vp, sz, vp]),
    "gather": (i32, [P(Cache), vp, i64, vp, vp, vp, vp, vp]),
    "gather_multi": (i32, [i32, P(GatherSeg), vp]),
    "gather_dedup_workspace_bytes": (sz, [i64]),
    "gather_dedup": (i32, [P(Cache), vp, i64, vp, vp, vp, vp, vp, vp, i64, vp, sz, vp]),
    "scatter_update": (i32, [P(Cache), vp, vp, vp, vp, vp, i64, vp, vp, vp]),
    "chunk_index_workspace_bytes": (sz, [i64]),
    "chunk_index_build": (i32, [i64, i64, vp, vp, vp, vp, sz, vp]),
    "seeds_workspace_bytes": (sz, [i64]),
    "seeds_count": (i32, [P(TCSR), P(SeedQuery), vp, vp, sz, vp]),
    "seeds_fill": (i32, [P(TCSR), P(SeedQuery), vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]),
    "unique_pairs_workspace_bytes": (sz, [i64]),
    "unique_pairs": (i32, [vp, vp, i64, vp, vp, vp, vp, vp, vp, sz, vp]),
    "csc_from_pairs_workspace_bytes": (sz, [i64]),
    "csc_from_pairs": (i32, [vp, vp, i64, vp, i64, vp, vp, vp, sz, vp]),
    "slice_workspace_bytes": (sz, [i64, i64]),
    "slice_count": (i32, [P(TCSR), P(SeedQuery), vp, i64, i32, vp, vp, sz, vp]),
    "slice_fill": (i32, [P(TCSR), P(SeedQuery), vp, i64, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]),
    "block_build": (i32, [vp, vp, i64, i64, i64, i64, vp, vp, vp, vp]),
    "segment_max_ts": (i32, [vp, vp, i64, vp, i64, vp, vp, vp, vp]),
    "time_encode": (i32, [vp, i32, i64, vp, vp, vp, i32, vp, vp]),
}


class BoundLib:
    """Entry points of one shared library, addressed without their prefix."""

    def __init__(self, cdll, prefix):
        self._cdll, self._prefix = cdll, prefix
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(cdll, prefix + name)  # AttributeError if a symbol is missing
            fn.restype, fn.argtypes = res, args
            setattr(self, name, fn)

    def error(self):
        msg = self.last_error_string()
        return msg.decode() if msg else ""


def bind(cdll, prefix="sgl_"):
    return BoundLib(cdll, prefix)


class SglError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"sgl status {code}: {msg}")
        self.code = code


_EXC = {SGL_EINVAL: ValueError, SGL_ERANGE: IndexError, SGL_ENOTSUP: RuntimeError,
        SGL_EHIP: RuntimeError, SGL_ENOMEM: MemoryError}


def check(lib, rc):
    """Map a status code to the exception the reference raised for the same
    condition (RuntimeError from C++ exceptions / TORCH_CHECK, export.cu:237-244)."""
    if rc == SGL_OK:
        return
    raise _EXC.get(rc, SglError)(f"sgl status {rc}: {lib.error()}")
