"""GPU parity: T-CSR build (stable radix sort by (src, ts, eid)) and validation
through the C ABI vs the CPU oracle / np.lexsort, bit-exact."""
import numpy as np
import pytest

from starrygl_amd.utils import synth
from util import host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


def _check(oracle, hot, n, src, dst, ts, eid=None):
    g = host_graph(oracle, n, src, dst, ts, eid)
    d = hot.tcsr_build(n, to_dev(hot, src), to_dev(hot, dst), to_dev(hot, ts), None if eid is None else to_dev(hot, eid))
    for f in ("row_ptr", "col", "ts", "eid"):
        a, b = np_of(getattr(d, f)), getattr(g, f)
        assert np.array_equal(a, b), f"{f}: first mismatch at {np.flatnonzero(a != b)[:3]}"
    e = np.arange(len(src)) if eid is None else eid
    o = np.lexsort((e, ts, src))
    assert np.array_equal(g.col, np.asarray(dst)[o])
    return d


@pytest.mark.parametrize("n,m", [(1000, 50_000), (1, 300), (100_000, 2_000_000), (7, 0), (300, 1), (5000, 2049)])
def test_build_random_order(oracle, hot, n, m):
    rng = np.random.default_rng(n + m)
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    ts = rng.integers(-10**6, 10**6, m)            # negative timestamps, many ties at small m
    eid = rng.permutation(m).astype(np.int64)      # edge ids in random order
    _check(oracle, hot, n, src, dst, ts, eid)


def test_build_stream_order_skips_sorts(oracle, hot):
    src, dst, ts, eid = synth.graph_stream(10_000, 160_000, 1.2, 2_600_000, 20240)
    _check(oracle, hot, 10_000, src, dst, ts)           # eid = arange, ts ascending: only the src pass runs
    _check(oracle, hot, 10_000, src, dst, ts, eid * 2)  # strictly ascending eids


def test_build_already_sorted_and_heavy_ties(oracle, hot):
    src, dst, ts, eid, row_ptr = synth.graph_by_degree(2000, 100_000, 1.1, 50, 3)   # ts in [0,50): ties everywhere
    d = _check(oracle, hot, 2000, src, dst, ts, eid)
    assert np.array_equal(np_of(d.row_ptr), row_ptr)
    rng = np.random.default_rng(1)
    p = rng.permutation(100_000)
    _check(oracle, hot, 2000, src[p], dst[p], ts[p], eid[p])
    _check(oracle, hot, 2000, src[p], dst[p], ts[p])    # eid = arange over the shuffled order


def test_build_large_keys(oracle, hot):
    rng = np.random.default_rng(2)
    n, m = 50, 10_000
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    ts = rng.integers(-2**62, 2**62, m)
    eid = rng.choice(2**40, m, replace=False).astype(np.int64)
    _check(oracle, hot, n, src, dst, ts, eid)


def test_build_and_validate_errors(oracle, hot):
    n = 10
    ok = np.arange(5, dtype=np.int64)
    with pytest.raises(IndexError):
        hot.tcsr_build(n, to_dev(hot, np.array([0, 10])), to_dev(hot, np.array([1, 1])), to_dev(hot, np.array([0, 1])))
    with pytest.raises(IndexError):
        hot.tcsr_build(n, to_dev(hot, np.array([0, 1])), to_dev(hot, np.array([-1, 1])), to_dev(hot, np.array([0, 1])))
    g = host_graph(oracle, n, ok, ok[::-1].copy(), np.array([5, 4, 3, 2, 1]))
    mirror_graph(hot, g)
    bad = g.ts.copy(); g.row_ptr[1] = 2; bad[0:2] = [9, 1]     # row 0 now holds two edges with descending ts
    with pytest.raises(IndexError):
        hot.tcsr_from_sorted(n, to_dev(hot, g.row_ptr), to_dev(hot, g.col), to_dev(hot, bad), to_dev(hot, g.eid))
    c = g.col.copy(); c[2] = n
    with pytest.raises(IndexError):
        hot.tcsr_from_sorted(n, to_dev(hot, g.row_ptr), to_dev(hot, c), to_dev(hot, g.ts), to_dev(hot, g.eid))
    rp = g.row_ptr.copy(); rp[-1] = 4
    with pytest.raises(IndexError):
        hot.tcsr_from_sorted(n, to_dev(hot, rp), to_dev(hot, g.col), to_dev(hot, g.ts), to_dev(hot, g.eid))
