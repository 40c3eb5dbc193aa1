"""GPU: the pre-planned mini-batch unit (sample -> unique -> gathers -> time encoding),
eager and as a replayed HIP graph, against the CPU oracle stage by stage."""
import numpy as np
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import host_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("remap", ["dense", "hashed"])
@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_pipeline_matches_oracle(oracle, hot, use_graph, sample_type, remap):
    from starrygl_amd.data import MiniBatchPipeline
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B = 4000, 80_000, 300
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 500_000, 21)
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    rng = np.random.default_rng(2)
    mem = rng.standard_normal((n, 100)).astype(np.float32)
    mem_ts = rng.integers(0, 10**6, n).astype(np.int64)
    efeat = rng.standard_normal((m, 172)).astype(np.float32)
    hot_ids = rng.permutation(n)[: n // 4]
    slot = np.full(n, -1, np.int32); slot[hot_ids] = np.arange(hot_ids.size, dtype=np.int32)
    c_mem = hot.cache(400, to_dev(hot, mem[hot_ids], "f32"), rows=n, cold=torch.from_numpy(mem).pin_memory(),
                      hot_slot=to_dev(hot, slot, "i32"), ts_hot=to_dev(hot, mem_ts[hot_ids]),
                      ts_cold=torch.from_numpy(mem_ts).pin_memory())
    c_ef = hot.cache(688, to_dev(hot, efeat, "f32"))
    w = (1.0 / 10 ** np.linspace(0, 9, 100, dtype=np.float32)).astype(np.float32)
    b = rng.standard_normal(100).astype(np.float32)
    pipe = MiniBatchPipeline(g, 2 * B, B, 2, 5, sample_type, node_tables={"mem": c_mem}, edge_tables={"f": c_ef},
                             time_encoder=(to_dev(hot, w, "f32"), to_dev(hot, b, "f32")), seed=9, use_graph=use_graph,
                             remap=remap)
    pipe.view("mem", torch.float32).view("f", torch.float32)
    for lo in (20_000, 50_000, 79_000, 30_000):
        roots, ts_ptr, root_ts, neg, neg_ts = synth.link_batch(src, dst, ts, lo, lo + B, n, B, rng)
        mb = pipe.run(to_dev(hot, roots), to_dev(hot, root_ts), to_dev(hot, neg), to_dev(hot, neg_ts)).finalize()
        want = oracle.sample_khop(hg, roots, ts_ptr, root_ts, neg, neg_ts, 2, oracle.params(sample_type, 5, seed=9))
        arrays = [want.slot_node0] + [h.neighbors for h in want.hops]
        loc, uniq, _ = oracle.unique_compact(arrays, _abi.UNIQUE_SORTED, None, True)
        assert mb.E == [h.E for h in want.hops] and mb.num_unique == uniq.shape[0]
        assert np.array_equal(np_of(mb.nid_mapper), uniq) and np.array_equal(np_of(mb.slot_local), loc[0])
        assert np.array_equal(np_of(mb.node_data["mem"]), mem[uniq])
        assert np.array_equal(np_of(mb.node_ts["mem"]), mem_ts[uniq])
        for l, h in enumerate(want.hops):
            assert np.array_equal(np_of(mb.hops[l]["neighbors_local"]), loc[1 + l])
            assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)
            assert np.array_equal(np_of(mb.edge_data[l]["f"]), efeat[h.neighbors_eid])
            y = oracle.time_encode(h.neighbors_dt, w, b)
            assert np.abs(np_of(mb.time_feat[l]) - y).max() <= 1e-6
        blocks = mb.blocks()
        assert [bk.num_edges() for bk in blocks] == mb.E[::-1]
        outer = blocks[0]
        assert outer.num_dst_nodes() == mb.S[0] + mb.E[0] and outer.num_src_nodes() == mb.S[0] + mb.E[0] + mb.E[1]
        assert np.array_equal(uniq[np_of(outer.srcdata["nid"])[-mb.E[1]:]], want.hops[1].neighbors)
    with pytest.raises(ValueError):
        pipe.run(to_dev(hot, roots[:5]), to_dev(hot, root_ts[:5]), to_dev(hot, neg), to_dev(hot, neg_ts))
    if remap == "hashed":     # a hashed state too small for the batch's distinct ids: the result is void, and reading it says so
        small = MiniBatchPipeline(g, 2 * B, B, 2, 5, sample_type, seed=9, use_graph=use_graph, remap="hashed", remap_capacity=50)
        with pytest.raises(RuntimeError, match="capacity"):
            small.run(to_dev(hot, roots), to_dev(hot, root_ts), to_dev(hot, neg), to_dev(hot, neg_ts)).finalize()


def test_pipeline_pool_keeps_batches_in_flight(oracle, hot):
    """Three pipelines on streams of their own: batches are enqueued back to back and only read afterwards;
    each must equal the oracle's result for its own roots (no pipeline sees another one's buffers)."""
    from starrygl_amd.data import MiniBatchPipelinePool
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B = 4000, 80_000, 300
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 500_000, 23)
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    rng = np.random.default_rng(4)
    feat = rng.standard_normal((n, 100)).astype(np.float32)
    c_nf = hot.cache(400, to_dev(hot, feat, "f32"))
    pool = MiniBatchPipelinePool(3, g, 2 * B, B, 2, 5, "recent", node_tables={"x": c_nf})
    for p in pool.pipes:
        p.view("x", torch.float32)
    for rnd in range(3):
        batches = [synth.link_batch(src, dst, ts, lo, lo + B, n, B, rng) for lo in (10_000 + 7_000 * rnd, 40_000, 79_000)]
        inflight = [pool.run(to_dev(hot, b[0]), to_dev(hot, b[2]), to_dev(hot, b[3]), to_dev(hot, b[4])) for b in batches]
        for b, mb in zip(batches, inflight):
            mb.finalize()
            want = oracle.sample_khop(hg, *b, 2, oracle.params("recent", 5))
            arrays = [want.slot_node0] + [h.neighbors for h in want.hops]
            loc, uniq, _ = oracle.unique_compact(arrays, _abi.UNIQUE_SORTED, None, True)
            assert mb.E == [h.E for h in want.hops] and np.array_equal(np_of(mb.nid_mapper), uniq)
            assert np.array_equal(np_of(mb.node_data["x"]), feat[uniq])
            for l, h in enumerate(want.hops):
                assert np.array_equal(np_of(mb.hops[l]["neighbors_local"]), loc[1 + l])
                assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)


def test_pipeline_pool_with_staggered_run_counts(oracle, hot):
    """Rounds of one or two batches on a pool of three: the pipelines' replay counts drift apart (r+1, r, r),
    so that graphs of different pipelines which shared any scratch - the unique stage's epoch stamp, its tile
    sums - would hand each other stale values.  Every batch must still equal the oracle's result."""
    from starrygl_amd.data import MiniBatchPipelinePool
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B = 6000, 120_000, 400
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 500_000, 41)
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    rng = np.random.default_rng(6)
    pool = MiniBatchPipelinePool(3, g, 2 * B, B, 2, 5, "recent")
    assert len({p.uws.data_ptr() for p in pool.pipes}) == 3          # a scratch buffer per pipeline
    lo = 5000
    for rnd, burst in enumerate([1, 2, 2, 1, 1, 2, 1, 2, 2, 1, 1, 1, 2]):
        batches = []
        for _ in range(burst):
            batches.append(synth.link_batch(src, dst, ts, lo, lo + B, n, B, rng))
            lo += 4321
        inflight = [pool.run(to_dev(hot, b[0]), to_dev(hot, b[2]), to_dev(hot, b[3]), to_dev(hot, b[4])) for b in batches]
        for b, mb in zip(batches, inflight):
            mb.finalize()
            want = oracle.sample_khop(hg, *b, 2, oracle.params("recent", 5))
            arrays = [want.slot_node0] + [h.neighbors for h in want.hops]
            loc, uniq, _ = oracle.unique_compact(arrays, _abi.UNIQUE_SORTED, None, True)
            assert np.array_equal(np_of(mb.nid_mapper), uniq), f"round {rnd}"
            assert np.array_equal(np_of(mb.slot_local), loc[0]), f"round {rnd}"
            for l in range(2):
                assert np.array_equal(np_of(mb.hops[l]["neighbors_local"]), loc[1 + l]), f"round {rnd} hop {l}"


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_pipeline_with_root_hints(oracle, hot, sample_type):
    """A pool whose batches carry the window ends of their positive roots (looked up once for the whole
    event stream, as a loader does) gives the oracle's result; a pipeline built for hints refuses a batch
    without them and the other way round."""
    from starrygl_amd.data import MiniBatchPipeline, MiniBatchPipelinePool
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B = 3000, 60_000, 250
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 40_000, 29)          # 40 000 times: ties inside rows
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    # the loader's one-off lookup: (src, ts) and (dst, ts) of every event
    end_src, end_dst = g.window_end(torch.from_numpy(src), torch.from_numpy(ts)), g.window_end(torch.from_numpy(dst), torch.from_numpy(ts))
    rng = np.random.default_rng(6)
    pool = MiniBatchPipelinePool(2, g, 2 * B, B, 2, 6, sample_type, seed=9, root_hints=True)
    for lo in (5_000, 31_000, 59_750):
        b = synth.link_batch(src, dst, ts, lo, lo + B, n, B, rng)           # roots = [src; dst] of events lo..lo+B
        assert np.array_equal(b[0], np.concatenate([src[lo: lo + B], dst[lo: lo + B]]))
        hint = torch.cat([end_src[lo: lo + B], end_dst[lo: lo + B]])
        mb = pool.run(to_dev(hot, b[0]), to_dev(hot, b[2]), to_dev(hot, b[3]), to_dev(hot, b[4]), root_hint=hint).finalize()
        want = oracle.sample_khop(hg, *b, 2, oracle.params(sample_type, 6, seed=9))
        assert mb.E == [h.E for h in want.hops]
        for l, h in enumerate(want.hops):
            assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)
            assert np.array_equal(np_of(mb.hops[l]["neighbors_dt"]), h.neighbors_dt)
    with pytest.raises(ValueError):
        pool.run(to_dev(hot, b[0]), to_dev(hot, b[2]), to_dev(hot, b[3]), to_dev(hot, b[4]))
    plain = MiniBatchPipeline(g, 2 * B, B, 2, 6, sample_type)
    with pytest.raises(ValueError):
        plain.run(to_dev(hot, b[0]), to_dev(hot, b[2]), to_dev(hot, b[3]), to_dev(hot, b[4]), root_hint=hint)


@pytest.mark.parametrize("prefetch", [1, 3, 4])
def test_event_batch_loader(oracle, hot, prefetch):
    """The loader walks the event stream batch by batch with `prefetch` batches in flight and the window ends
    of all event endpoints looked up once; every yielded batch equals the oracle's result for its own events
    and the negatives it drew (read back from the batch), and is still intact while the next ones are in flight."""
    from starrygl_amd.data import EventBatchLoader
    from starrygl_amd.graph.graph import NegSamplingSet
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B, NEG = 2500, 50_000, 200, 150
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 30_000, 31)
    order = np.argsort(ts, kind="stable")
    src, dst, ts, eid = src[order], dst[order], ts[order], eid[order]       # the stream in time order
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    feat = np.random.default_rng(2).standard_normal((n, 100)).astype(np.float32)
    lo_ev = 40_000                                                             # train on the last 10 000 events
    sampler = NegSamplingSet(torch.arange(100, 2000, device="cuda"))
    loader = EventBatchLoader(g, src[lo_ev:], dst[lo_ev:], ts[lo_ev:], B, NEG, 2, 5, "recent",
                              node_tables={"x": hot.cache(400, to_dev(hot, feat, "f32"))}, prefetch=prefetch,
                              negative_sampler=sampler)
    for p in loader.pool.pipes:
        p.view("x", torch.float32)
    assert len(loader) == 10_000 // B
    seen, held = 0, None
    for i, mb in enumerate(loader):
        lo = lo_ev + i * B
        roots = np.concatenate([src[lo: lo + B], dst[lo: lo + B]])
        root_ts = np.concatenate([ts[lo: lo + B], ts[lo: lo + B]])
        neg, neg_ts = np_of(mb.slot_node)[2 * B:], np_of(mb.slot_ts)[2 * B:]
        assert neg.shape[0] == NEG and (neg >= 100).all() and (neg < 2000).all()
        assert np.array_equal(neg_ts, np.resize(ts[lo: lo + B], NEG))
        want = oracle.sample_khop(hg, roots, np.arange(2 * B + 1, dtype=np.int64), root_ts, neg, neg_ts, 2,
                                  oracle.params("recent", 5))
        assert mb.E == [h.E for h in want.hops]
        _, uniq, _ = oracle.unique_compact([want.slot_node0] + [h.neighbors for h in want.hops], _abi.UNIQUE_SORTED, None, True)
        assert np.array_equal(np_of(mb.nid_mapper), uniq) and np.array_equal(np_of(mb.node_data["x"]), feat[uniq])
        for l, h in enumerate(want.hops):
            assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)
        seen += 1
    assert seen == len(loader)


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_group_pipeline_matches_oracle(oracle, hot, use_graph, sample_type):
    """B mini-batches per pass: every batch of a group against the oracle - the batched sampler over the group's
    slots (the uniform strategy is keyed by the slot's place in the call), np.unique per batch, rows, time encoding,
    blocks - for full groups, a short last group and consecutive passes on the same buffers."""
    from starrygl_amd.data import MiniBatchGroupPipeline
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, EV, NEG, B = 4000, 80_000, 120, 70, 5
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 500_000, 21)
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    rng = np.random.default_rng(2)
    mem = rng.standard_normal((n, 100)).astype(np.float32)
    mem_ts = rng.integers(0, 10**6, n).astype(np.int64)
    efeat = rng.standard_normal((m, 172)).astype(np.float32)
    c_mem = hot.cache(400, to_dev(hot, mem, "f32"), ts_hot=to_dev(hot, mem_ts))
    c_ef = hot.cache(688, to_dev(hot, efeat, "f32"))
    w = (1.0 / 10 ** np.linspace(0, 9, 100, dtype=np.float32)).astype(np.float32)
    bias = rng.standard_normal(100).astype(np.float32)
    pipe = MiniBatchGroupPipeline(g, B, 2 * EV, NEG, 2, 5, sample_type, node_tables={"mem": c_mem}, edge_tables={"f": c_ef},
                                  time_encoder=(to_dev(hot, w, "f32"), to_dev(hot, bias, "f32")), seed=9, use_graph=use_graph)
    pipe.view("mem", torch.float32).view("f", torch.float32)
    for live in (B, B, 2, B):
        bts = [synth.link_batch(src, dst, ts, lo, lo + EV, n, NEG, rng) for lo in rng.integers(1000, m - EV, live)]
        stack = lambda i: to_dev(hot, np.stack([b[i] for b in bts]))
        group = pipe.run(stack(0), stack(2), stack(3), stack(4)).finalize()
        assert len(group) == live
        node = np.concatenate([np.concatenate([b[0], b[3]]) for b in bts])
        t = np.concatenate([np.concatenate([b[2], b[4]]) for b in bts])
        ptr = np.arange(live + 1, dtype=np.int64) * (2 * EV + NEG)
        want = oracle.sample_khop_batched(hg, node, t, ptr, 2, [oracle.params(sample_type, 5, seed=9)], finalize=True)
        seg, wq = np.asarray(want.seg_host[0]), want.queries[0]
        for b, mb in enumerate(group):
            assert mb.S[0] == 2 * EV + NEG and mb.E == [int(seg[l + 1][b + 1] - seg[l + 1][b]) for l in range(2)]
            ids = [node[seg[0][b]: seg[0][b + 1]]] + [wq.hops[l].neighbors[seg[l + 1][b]: seg[l + 1][b + 1]] for l in range(2)]
            uniq, inv = np.unique(np.concatenate(ids), return_inverse=True)
            assert np.array_equal(np_of(mb.nid_mapper), uniq) and mb.num_unique == uniq.size, (live, b)
            assert np.array_equal(np_of(mb.slot_local), inv[: ids[0].size])
            assert np.array_equal(np_of(mb.node_data["mem"]), mem[uniq]) and np.array_equal(np_of(mb.node_ts["mem"]), mem_ts[uniq])
            off = ids[0].size
            for l in range(2):
                lo, hi = seg[l + 1][b], seg[l + 1][b + 1]
                h = wq.hops[l]
                assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid[lo:hi])
                assert np.array_equal(np_of(mb.hops[l]["neighbors_local"]), inv[off: off + hi - lo])
                off += hi - lo
                assert np.array_equal(np_of(mb.hops[l]["root_start_ptr"]), h.root_start_ptr[seg[l][b]: seg[l][b + 1] + 1] - lo)
                assert np.array_equal(np_of(mb.edge_data[l]["f"]), efeat[h.neighbors_eid[lo:hi]])
                y = oracle.time_encode(h.neighbors_dt[lo:hi], w, bias)
                assert hi == lo or np.abs(np_of(mb.time_feat[l]) - y).max() <= 1e-6
            blocks = mb.blocks()
            assert [bk.num_edges() for bk in blocks] == mb.E[::-1]
            assert blocks[0].num_dst_nodes() == mb.S[0] + mb.E[0]
    with pytest.raises(ValueError):
        pipe.run(stack(0)[:, :5], stack(2)[:, :5], stack(3), stack(4))


@pytest.mark.parametrize("prefetch,ahead", [(2, 4), (3, 7)])
def test_event_batch_loader_sampling_ahead(oracle, hot, prefetch, ahead):
    """The loader with `sample_ahead` batches per pass: every yielded batch equals the oracle's most-recent sample
    of its own events and negatives (the most-recent strategy does not depend on how batches are grouped)."""
    from starrygl_amd.data import EventBatchLoader
    from starrygl_amd.lib.libstarrygl_comm import from_edge_index
    n, m, B, NEG = 2500, 50_000, 200, 150
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 30_000, 31)
    order = np.argsort(ts, kind="stable")
    src, dst, ts, eid = src[order], dst[order], ts[order], eid[order]
    hg = host_graph(oracle, n, src, dst, ts, eid)
    g = from_edge_index(n, 1, *(torch.from_numpy(x) for x in (src, dst, ts, eid)))
    feat = np.random.default_rng(2).standard_normal((n, 100)).astype(np.float32)
    lo_ev = 44_000                                   # 6000 events = 30 batches: groups of 4 or 7, the last one short
    loader = EventBatchLoader(g, src[lo_ev:], dst[lo_ev:], ts[lo_ev:], B, NEG, 2, 5, "recent",
                              node_tables={"x": hot.cache(400, to_dev(hot, feat, "f32"))}, prefetch=prefetch, sample_ahead=ahead)
    for p in loader.pool.pipes:
        p.view("x", torch.float32)
    seen = 0
    for i, mb in enumerate(loader):
        lo = lo_ev + i * B
        roots = np.concatenate([src[lo: lo + B], dst[lo: lo + B]])
        root_ts = np.concatenate([ts[lo: lo + B], ts[lo: lo + B]])
        assert np.array_equal(np_of(mb.slot_node)[: 2 * B], roots)
        neg, neg_ts = np_of(mb.slot_node)[2 * B:], np_of(mb.slot_ts)[2 * B:]
        assert np.array_equal(neg_ts, np.resize(ts[lo: lo + B], NEG))
        want = oracle.sample_khop(hg, roots, np.arange(2 * B + 1, dtype=np.int64), root_ts, neg, neg_ts, 2, oracle.params("recent", 5))
        assert mb.E == [h.E for h in want.hops]
        _, uniq, _ = oracle.unique_compact([want.slot_node0] + [h.neighbors for h in want.hops], _abi.UNIQUE_SORTED, None, True)
        assert np.array_equal(np_of(mb.nid_mapper), uniq) and np.array_equal(np_of(mb.node_data["x"]), feat[uniq])
        for l, h in enumerate(want.hops):
            assert np.array_equal(np_of(mb.hops[l]["neighbors_eid"]), h.neighbors_eid)
        seen += 1
    assert seen == len(loader) == 30
