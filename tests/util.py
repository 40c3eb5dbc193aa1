"""Helpers shared by the parity tests: a graph built by the oracle on the host
and mirrored on the GPU, and array comparisons."""
import numpy as np


def to_dev(hot, a, dtype="i64"):
    return hot.be.asarray(a, dtype)


def host_graph(oracle, n, src, dst, ts, eid=None):
    return oracle.tcsr_build(n, *(np.ascontiguousarray(x, dtype=np.int64) for x in (src, dst, ts)),
                             None if eid is None else np.ascontiguousarray(eid, dtype=np.int64))


def mirror_graph(hot, g, validate=True):
    return hot.tcsr_from_sorted(g.n, to_dev(hot, g.row_ptr), to_dev(hot, g.col), to_dev(hot, g.ts),
                                to_dev(hot, g.eid), validate=validate)


def np_of(t):
    return t.cpu().numpy() if hasattr(t, "cpu") else np.asarray(t)


HOP_FIELDS = ("root_start_ptr", "root_end_ptr", "neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt")


def assert_hop_equal(got, want, tag=""):
    assert got.S == want.S, f"{tag} S {got.S} != {want.S}"
    assert got.E == want.E, f"{tag} E {got.E} != {want.E}"
    for f in HOP_FIELDS:
        a, b = np_of(getattr(got, f)), np_of(getattr(want, f))
        assert a.shape == b.shape, f"{tag} {f} shape {a.shape} != {b.shape}"
        if not np.array_equal(a, b):
            bad = np.flatnonzero(a != b)
            raise AssertionError(f"{tag} {f}: {bad.size} mismatches, first at {bad[0]}: {a[bad[0]]} != {b[bad[0]]}")
