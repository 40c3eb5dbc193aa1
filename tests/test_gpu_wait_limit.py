"""The error path of the kernels whose blocks wait for each other's totals inside one launch (the
single-launch 2-hop sampler, the numbering pass of the dense unique): with the wait limited to one
poll (set from the host; every kernel still exits normally) a block that finds an earlier block's
descriptor missing gives up and the call's counts are poisoned.  Through the raw calls the poison is
visible; the host side then re-issues the call through the routes that never wait and hands out the
right result."""
import numpy as np
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import assert_hop_equal, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu
INT64_MAX = (1 << 63) - 1


def _hub_graph(oracle, hot):
    src, dst, ts, eid = synth.graph_stream(20_000, 600_000, 1.15, 10**9, 41)
    src[:150_000] = 3                                  # one very long row: blocks of very different duration
    g = host_graph(oracle, 20_000, src, dst, ts, eid)
    rng = np.random.default_rng(5)
    S0 = 12_000
    roots = rng.integers(0, g.n, S0).astype(np.int64)
    roots[::7] = 3
    root_ts = rng.integers(0, 10**9, S0).astype(np.int64)
    ts_ptr = np.arange(S0 + 1, dtype=np.int64)
    empty = np.zeros(0, dtype=np.int64)
    return (src, dst, ts, eid), g, (roots, ts_ptr, root_ts, empty, empty)


def test_sampler_gives_up_cleanly_and_the_call_is_reissued(oracle, hot):
    _, g, batch = _hub_graph(oracle, hot)
    dg = mirror_graph(hot, g)
    args = [to_dev(hot, x) for x in batch]
    p = hot.params("recent", 10)
    want = oracle.sample_khop(g, *batch, 2, oracle.params("recent", 10))
    prev = hot.set_wait_limit(1)
    poisoned, before = 0, hot.recoveries
    try:
        assert prev == 1 << 20
        for _ in range(12):
            res = hot.sample_khop(dg, *args, 2, p, finalize=False)
            poisoned += int(np_of(res.counts)[2]) == INT64_MAX
            # whether or not a block gave up, reading the result gives the right edges: a poisoned call is
            # re-issued through the launch-per-hop route (the limit of one poll is still in force: that route
            # does not wait)
            res.finalize()
            for l in range(2):
                assert_hop_equal(res.hops[l], want.hops[l], tag=f"hop{l}, wait limit 1")
        assert hot.recoveries - before == poisoned
        # the flag alone keeps a call off the single-launch route: never poisoned
        for _ in range(3):
            res = hot.sample_khop(dg, *args, 2, hot.multi_launch(p), finalize=False)
            assert int(np_of(res.counts)[2]) == 0
    finally:
        assert hot.set_wait_limit(0) == 1
    got = hot.sample_khop(dg, *args, 2, p)
    for l in range(2):
        assert_hop_equal(got.hops[l], want.hops[l], tag=f"hop{l} after the limit was restored")
    if not poisoned:
        pytest.skip("no block ever found a descriptor missing: the error path was not reached")


def test_unique_gives_up_cleanly_and_the_call_is_reissued(hot):
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
        if poisoned:
            # sticky through the raw call: the state reports the failure until it is initialised again
            _, _, U = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True, finalize=False)
            assert int(np_of(U)[0]) == INT64_MAX
            # a call that continues the epoch cannot be re-issued (the epoch's numbering is gone): it raises
            with pytest.raises(RuntimeError, match="void"):
                hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, False)
            # a call that opens an epoch is: state initialised again, numbering in separate launches
            before = hot.recoveries
            local, uniq, (total, _) = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True)
            assert hot.recoveries == before + 1
            assert total == want_u.size and np.array_equal(np_of(uniq), want_u) and np.array_equal(np_of(local[0]), want_inv)
        # with the flag the numbering never waits
        for _ in range(3):
            local, uniq, (total, _) = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED | _abi.UNIQUE_MULTI_LAUNCH, state, True)
            assert total == want_u.size and np.array_equal(np_of(local[0]), want_inv)
    finally:
        hot.set_wait_limit(0)
    local, uniq, (total, _) = hot.unique_compact([to_dev(hot, ids)], _abi.UNIQUE_SORTED, state, True)
    assert total == want_u.size and np.array_equal(np_of(uniq), want_u) and np.array_equal(np_of(local[0]), want_inv)
    if not poisoned:
        pytest.skip("no tile ever found a descriptor missing: the error path was not reached")


def test_pipeline_batch_is_reissued_after_a_give_up(oracle, hot):
    """A MiniBatchPipeline whose captured step (single-launch sampler that records its ids in the remap state,
    single-launch numbering) gives up re-runs the batch through the multi-launch routes when it is read."""
    from starrygl_amd.data import MiniBatchPipeline
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    (src, dst, ts, eid), g, batch = _hub_graph(oracle, hot)
    cg = from_edge_index(g.n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    roots, _, root_ts, _, _ = batch
    pipe = MiniBatchPipeline(cg, roots.shape[0], 0, 2, 10, "recent")
    want = oracle.sample_khop(g, *batch, 2, oracle.params("recent", 10))
    loc, uniq, _ = oracle.unique_compact([want.slot_node0] + [h.neighbors for h in want.hops], _abi.UNIQUE_SORTED, None, True)
    pipe.run(to_dev(hot, roots), to_dev(hot, root_ts)).finalize()            # captures the step's graph
    hot.set_wait_limit(1)     # (the graph was captured with the default limit: capture again under the new one)
    before = hot.recoveries
    try:
        pipe._graph = None
        for _ in range(10):
            mb = pipe.run(to_dev(hot, roots), to_dev(hot, root_ts)).finalize()
            assert mb.E == [h.E for h in want.hops] and np.array_equal(np_of(mb.nid_mapper), uniq)
            for l, h in enumerate(want.hops):
                assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)
                assert np.array_equal(np_of(mb.hops[l]["neighbors_local"]), loc[1 + l])
    finally:
        hot.set_wait_limit(0)
    recovered = hot.recoveries - before
    pipe._graph = None
    mb = pipe.run(to_dev(hot, roots), to_dev(hot, root_ts)).finalize()
    assert np.array_equal(np_of(mb.nid_mapper), uniq)
    if not recovered:
        pytest.skip("no block ever found a descriptor missing: the error path was not reached")


def test_pair_call_gives_up_cleanly_and_the_whole_call_is_reissued(oracle, hot):
    """The most-recent + uniform pair in one launch (sgl_sample_khop_multi) under a wait limit of one poll: whichever
    query was poisoned, finalizing re-issues the whole call with this call's inputs and parameters - also when the
    same buffers served another call before - and re-initialises the remap state the recent query marks ids in."""
    _, g, batch = _hub_graph(oracle, hot)
    dg = mirror_graph(hot, g)
    args = [to_dev(hot, x) for x in batch]
    S0 = batch[0].shape[0]
    state = hot.remap_state(g.n)
    p_rec, p_uni = hot.marking(hot.params("recent", 10), state), hot.params("uniform", 10, seed=4)
    want = {st: oracle.sample_khop(g, *batch, 2, oracle.params(st, 10, seed=4)) for st in ("recent", "uniform")}
    ids = [want["recent"].slot_node0] + [h.neighbors for h in want["recent"].hops]
    want_u, want_inv = np.unique(np.concatenate(ids), return_inverse=True)
    # an earlier, different call on the same buffers leaves its own recovery closure behind
    other = [to_dev(hot, x) for x in (batch[0][::-1].copy(), batch[1], batch[2], batch[3], batch[4])]
    hot.set_wait_limit(1)
    poisoned, before = 0, hot.recoveries
    try:
        for _ in range(10):
            outs = [hot.khop_buffers(S0, 2, 10) for _ in range(2)]
            hot.sample_khop(dg, *other, 2, hot.params("recent", 10), finalize=False, out=outs[0])
            hot.sample_khop_multi(dg, *args, 2, [p_rec, p_uni], outs)
            bad = [int(np_of(o.counts)[2]) == INT64_MAX for o in outs]
            poisoned += any(bad)
            for o, st in zip(outs, ("recent", "uniform")):
                o.finalize()
                for l in range(2):
                    assert_hop_equal(o.hops[l], want[st].hops[l], tag=f"{st} hop{l}, wait limit 1, poisoned {bad}")
            # the marks of the (possibly re-issued) recent query feed the unique stage (whose own numbering pass waits
            # too: it runs under the default limit)
            kr = outs[0]
            hot.set_wait_limit(0)
            local, uniq, (total, _) = hot.unique_compact([kr.slot_node0] + [h.neighbors for h in kr.hops], _abi.UNIQUE_SORTED,
                                                         state, True, premarked=True)
            hot.set_wait_limit(1)
            assert total == want_u.size and np.array_equal(np_of(uniq), want_u)
            assert np.array_equal(np.concatenate([np_of(a) for a in local]), want_inv)
        assert hot.recoveries - before >= (1 if poisoned else 0)
    finally:
        hot.set_wait_limit(0)
    if not poisoned:
        pytest.skip("no block ever found a descriptor missing: the error path was not reached")
