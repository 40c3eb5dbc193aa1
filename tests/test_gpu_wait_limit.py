"""The error path of the kernels whose blocks wait for each other's totals inside one launch (the
single-launch 2-hop sampler, the numbering pass of the dense unique): with the wait limited to one
poll a block that finds an earlier block's descriptor missing gives up, the call's counts are
poisoned, every kernel still exits, and the host side raises instead of handing out the result."""
import numpy as np
import pytest

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import assert_hop_equal, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu
INT64_MAX = (1 << 63) - 1


def test_sampler_gives_up_cleanly_and_recovers(oracle, hot):
    src, dst, ts, eid = synth.graph_stream(20_000, 600_000, 1.15, 10**9, 41)
    src[:150_000] = 3                                  # one very long row: blocks of very different duration
    g = host_graph(oracle, 20_000, src, dst, ts, eid)
    dg = mirror_graph(hot, g)
    rng = np.random.default_rng(5)
    S0 = 12_000
    roots = rng.integers(0, g.n, S0).astype(np.int64)
    roots[::7] = 3
    root_ts = rng.integers(0, 10**9, S0).astype(np.int64)
    ts_ptr = np.arange(S0 + 1, dtype=np.int64)
    empty = np.zeros(0, dtype=np.int64)
    args = [to_dev(hot, x) for x in (roots, ts_ptr, root_ts, empty, empty)]
    p = hot.params("recent", 10)
    want = oracle.sample_khop(g, roots, ts_ptr, root_ts, empty, empty, 2, oracle.params("recent", 10))
    prev = hot.set_wait_limit(1)
    poisoned = 0
    try:
        assert prev == 1 << 20
        for _ in range(12):
            res = hot.sample_khop(dg, *args, 2, p, finalize=False)
            if int(np_of(res.counts)[2]) == INT64_MAX:
                poisoned += 1
                with pytest.raises(RuntimeError, match="gave up"):
                    res.finalize()
            else:
                # no block gave up (whichever block wrote its count last, a give-up would still show):
                # then the result is the right one
                res.finalize()
                for l in range(2):
                    assert_hop_equal(res.hops[l], want.hops[l], tag=f"hop{l}, wait limit 1, not poisoned")
    finally:
        assert hot.set_wait_limit(0) == 1
    # the limit is back: the same call is right again (nothing of the sampler's is sticky)
    got = hot.sample_khop(dg, *args, 2, p)
    for l in range(2):
        assert_hop_equal(got.hops[l], want.hops[l], tag=f"hop{l} after the limit was restored")
    if not poisoned:
        pytest.skip("no block ever found a descriptor missing: the error path was not reached")


def test_unique_gives_up_cleanly_and_state_stays_poisoned(hot):
    universe = 4_000_000                               # 1954 tiles: the single-launch numbering
    rng = np.random.default_rng(6)
    state = hot.remap_state(universe)
    ids = rng.integers(0, universe, 300_000).astype(np.int64)
    want_u, want_inv = np.unique(ids, return_inverse=True)
    local, uniq, (total, _) = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True)
    assert total == want_u.size and np.array_equal(np_of(local[0]), want_inv)
    hot.set_wait_limit(1)
    poisoned = False
    try:
        for _ in range(20):
            _, _, U = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True, finalize=False)
            if int(np_of(U)[0]) == INT64_MAX:
                poisoned = True
                break
    finally:
        hot.set_wait_limit(0)
    if not poisoned:
        pytest.skip("no tile ever found a descriptor missing: the error path was not reached")
    # sticky: the state reports the failure until it is initialised again
    with pytest.raises(RuntimeError, match="gave up"):
        hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True)
    state = hot.remap_state(universe)
    local, uniq, (total, _) = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True)
    assert total == want_u.size and np.array_equal(np_of(uniq), want_u) and np.array_equal(np_of(local[0]), want_inv)
