"""GPU: the Python façade (pyGraph / AsyncBlock / AsyncGraphBlob / DistNodeState /
TimeEncoder / native-module mirror) against the CPU oracle and plain torch."""
import numpy as np
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import host_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def world(oracle, hot):
    from starrygl_amd.graph.graph import pyGraph
    n, m, C = 3000, 60_000, 8
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 100_000, 11)
    rng = np.random.default_rng(1)
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    # edges arrive shuffled: the façade builds the T-CSR itself
    p = rng.permutation(m)
    g = pyGraph(torch.from_numpy(src[p]), torch.from_numpy(dst[p]), torch.from_numpy(ts[p]), n, C,
                eid=torch.from_numpy(eid[p]), chunk_mapper=torch.from_numpy(chunk_of))
    hg = host_graph(oracle, n, src, dst, ts, eid)
    cp, cn = oracle.chunk_index(n, C, chunk_of)
    return dict(g=g, hg=hg, n=n, C=C, chunk_of=chunk_of, cp=cp, cn=cn, src=src, dst=dst, ts=ts)


def _oracle_query(oracle, w, t0, t1, chunks, neg, neg_ts, policy, state, reset, seed):
    ch = np.asarray(chunks, dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(w["cp"][ch + 1] - w["cp"][ch])]).astype(np.int64)
    roots, ts_ptr, ts, q_ptr, q_eid = oracle.seeds(w["hg"], w["cp"], w["cn"], ch, off, int(off[-1]), t0, t1)
    p = oracle.params(policy["sample_type"], policy["fanout"], policy.get("allowed_offset", -1),
                      policy.get("equal_root_time", False), policy.get("keep_root_time", False), seed=seed)
    res = oracle.sample_khop(w["hg"], roots, ts_ptr, ts, neg, neg_ts, policy["layers"], p)
    arrays = [roots, neg] + [h.neighbors for h in res.hops]
    local, uniq, (tot, before) = oracle.unique_compact(arrays, _abi.UNIQUE_GROUPED, state, reset)
    return dict(roots=roots, ts_ptr=ts_ptr, ts=ts, q_ptr=q_ptr, q_eid=q_eid, res=res, local=local,
                uniq=uniq, tot=tot, before=before)


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_async_sample_matches_oracle_pipeline(oracle, world, sample_type):
    g = world["g"]
    policy = dict(sample_type=sample_type, layers=2, fanout=5, allowed_offset=-1, equal_root_time=False,
                  keep_root_time=False)
    rng = np.random.default_rng(5)
    neg = rng.integers(0, world["n"], 200).astype(np.int64)
    neg_ts = rng.integers(40_000, 60_000, 200).astype(np.int64)
    kw = dict(test_generate_samples=torch.from_numpy(neg), test_generate_samples_ts=torch.from_numpy(neg_ts))
    q0 = g.g._queries
    g.async_sample(50_000, 52_000, torch.tensor([1, 5, 2]), policy, kw, op="r")
    out = g.get_last_sample()
    st = oracle.remap_state(world["n"])
    want = _oracle_query(oracle, world, 50_000, 52_000, [1, 5, 2], neg, neg_ts, policy, st, True, seed=1317 + q0)
    assert out.roots.root_num == want["roots"].shape[0] > 0
    for f in ("ts_ptr", "ts", "q_ptr", "q_eid"):
        assert np.array_equal(np_of(getattr(out.roots, f)), want[f]), f
    assert np.array_equal(np_of(out.roots.roots), want["local"][0])
    assert np.array_equal(np_of(out.neg_roots.roots), want["local"][1])
    assert np.array_equal(np_of(out.nodes_remapper_id), want["uniq"][: want["tot"]])
    assert len(out.neighbors) == 2 and out.neighbors is out.neighbors_list
    for l, layer in enumerate(out.neighbors_list):
        h = want["res"].hops[l]
        assert np.array_equal(np_of(layer.neighbors), want["local"][2 + l])
        for f in ("root_start_ptr", "root_end_ptr", "neighbors_ts", "neighbors_eid", "neighbors_dt"):
            assert np.array_equal(np_of(getattr(layer, f)), getattr(h, f)), (l, f)
        assert layer.neighbor_num == h.E
    # local -> global round trip
    assert np.array_equal(np_of(out.nodes_remapper_id)[np_of(out.neighbors[1].neighbors)], want["res"].hops[1].neighbors)


def test_graph_blob_epochs_and_blocks(oracle, world):
    from starrygl_amd.graph.graph import AsyncBlock, AsyncGraphBlob
    g = world["g"]
    policy = dict(sample_type="recent", layers=2, fanout=4, allowed_offset=-1, equal_root_time=False,
                  keep_root_time=False)
    t0s, t1s = [60_000, 61_000, 62_000], [61_000, 62_000, 63_000]
    chunks = [torch.tensor([0, 1]), torch.tensor([2]), torch.tensor([7, 3])]
    q0 = g.g._queries
    blob = AsyncGraphBlob(g, t0s, t1s, chunks, policy)
    st = oracle.remap_state(world["n"])
    e = np.zeros(0, np.int64)
    mapper_so_far = None
    for i, ab in enumerate(blob.graph):
        out = ab.value()
        want = _oracle_query(oracle, world, t0s[i], t1s[i], chunks[i].tolist(), e, e, policy, st, i == 0, 1317 + q0 + i)
        new = want["uniq"][want["before"]: want["tot"]]
        mapper_so_far = new if i == 0 else np.concatenate([mapper_so_far, new])
        assert np.array_equal(np_of(out.nodes_remapper_id), mapper_so_far)      # one id space across the blob
        assert np.array_equal(np_of(out.roots.roots), want["local"][0])
        root, neg, mfgs, nid = AsyncBlock.to_block(out.roots, out.neg_roots, out.neighbors, out.nodes_remapper_id)
        assert len(mfgs) == 2
        b1, b0 = mfgs            # reversed: outermost hop first
        S0 = out.roots.root_ts_num
        E0, E1 = out.neighbors[0].neighbor_num, out.neighbors[1].neighbor_num
        assert (b0.num_dst_nodes(), b0.num_src_nodes(), b0.num_edges()) == (S0, S0 + E0, E0)
        assert (b1.num_dst_nodes(), b1.num_src_nodes(), b1.num_edges()) == (S0 + E0, S0 + E0 + E1, E1)
        ip0, ip1 = np_of(b0.indptr), np_of(b1.indptr)
        assert np.array_equal(ip0, want["res"].hops[0].root_start_ptr)
        assert np.array_equal(ip1, np.concatenate([np.zeros(S0, np.int64), want["res"].hops[1].root_start_ptr]))
        assert np.array_equal(np_of(b1.indices), S0 + E0 + np.arange(E1))
        # every edge of the outer block joins the sampled neighbour to the slot it was sampled for
        nid1 = np_of(b1.srcdata["nid"])
        dst_of_edge = np.repeat(np.arange(S0 + E0), np.diff(ip1))
        assert np.array_equal(nid1[dst_of_edge], np.repeat(want["local"][2], np.diff(want["res"].hops[1].root_start_ptr)))
        assert np.array_equal(np_of(b1.edata["dt"]), want["res"].hops[1].neighbors_dt)
        assert np.array_equal(np_of(b0.srcdata["ts"])[:S0], want["ts"])


def test_direct_khop_and_errors(oracle, world):
    from starrygl_amd.lib.libstarrygl_comm import TemporalRoot, from_edge_index
    g = world["g"].g
    dev = torch.device("cuda:0")
    roots = torch.tensor([5, 9, 100], device=dev)
    root = TemporalRoot(roots, torch.arange(4, device=dev), torch.tensor([70_000, 80_000, 90_000], device=dev))
    neg = g.get_negative_root(torch.tensor([1, 2]), torch.tensor([50_000, 50_001]))
    res = g.sample_src_in_chunks_khop(root, neg, 3, 1, -1, False, False, "recent")
    want = oracle.sample_khop(world["hg"], np.array([5, 9, 100]), np.arange(4), np.array([70_000, 80_000, 90_000]),
                              np.array([1, 2]), np.array([50_000, 50_001]), 1, oracle.params("recent", 3))
    assert np.array_equal(np_of(res.neighbors_list[0].neighbors), want.hops[0].neighbors)
    with pytest.raises(RuntimeError, match="undefined sampling strategy"):
        g.sample_src_in_chunks_khop(root, neg, 3, 1, -1, False, False, "nearest")
    with pytest.raises(IndexError):
        g.slice_by_chunk_ts(torch.tensor([world["C"]]), 0, 1)
    one = torch.tensor([0, 1])
    with pytest.raises(IndexError):
        from_edge_index(2, 1, one, torch.tensor([1, 2]), one, None)
    with pytest.raises(RuntimeError):
        from_edge_index(2, 1, one.int(), one, one, None)
    with pytest.raises(IndexError):
        from_edge_index(2, 2, one, one, one, None, torch.tensor([0, 2]))
    # a failing query surfaces at get(), later queries still work
    pg = world["g"]
    pol = dict(sample_type="recent", layers=1, fanout=2)
    pg.async_sample(0, 10, torch.tensor([99]), pol, {}, op="r")
    pg.async_sample(0, 100_000, torch.tensor([0]), pol, {}, op="r")
    with pytest.raises(IndexError):
        pg.get_last_sample()
    assert pg.get_last_sample().roots.root_num > 0
    with pytest.raises(ValueError):
        pg.async_sample(0, 1, torch.tensor([0]), dict(sample_type="recent", layers=1), {}, op="r")
    with pytest.raises(TypeError):
        pg.async_sample(0, 1, [0], pol)
    # the wrapper's own call form (graph.py:124-135): chunk list, fanout, hops, window
    res = pg.sample_src_in_chunks_khop(torch.tensor([2, 6]), 4, [4, 4], 50_000, 51_000)
    ch = np.array([2, 6], dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(world["cp"][ch + 1] - world["cp"][ch])]).astype(np.int64)
    r, tp, t, _, _ = oracle.seeds(world["hg"], world["cp"], world["cn"], ch, off, int(off[-1]), 50_000, 51_000)
    e = np.zeros(0, np.int64)
    want = oracle.sample_khop(world["hg"], r, tp, t, e, e, 2, oracle.params("recent", 4))
    assert len(res.neighbors_list) == 2 and res.roots.root_num == r.shape[0] > 0
    for layer, h in zip(res.neighbors_list, want.hops):
        assert np.array_equal(np_of(layer.neighbors), h.neighbors) and np.array_equal(np_of(layer.neighbors_eid), h.neighbors_eid)


@pytest.mark.parametrize("full", [False, True])
def test_slice_by_chunk_ts_matches_oracle(oracle, world, full):
    g = world["g"]
    for chunks, t0, t1 in [([1, 5, 2], 50_000, 50_400), ([0, 1, 2, 3, 4, 5, 6, 7], 10_000, 10_250), ([3], 99_000, 100_000),
                           ([6, 0], 70_000, 70_001), ([], 0, 10), ([4], 500, 500)]:
        ch = np.asarray(chunks, dtype=np.int64)
        off = np.concatenate([[0], np.cumsum(world["cp"][ch + 1] - world["cp"][ch])]).astype(np.int64)
        want = oracle.slice(world["hg"], world["cp"], world["cn"], world["chunk_of"], ch, off, int(off[-1]), t0, t1, full)
        out = g.g.slice_by_chunk_ts(torch.tensor(chunks, dtype=torch.int64), t0, t1, full)
        layer = out.neighbors_list[0]
        got = (out.roots.roots, out.roots.ts_ptr, out.roots.ts, layer.root_start_ptr, layer.neighbors,
               layer.neighbors_ts, layer.neighbors_eid)
        for a, b in zip(got, want):
            assert np.array_equal(np_of(a), b), (chunks, t0, t1)
        assert np.array_equal(np_of(layer.root_end_ptr)[:-1], want[3][1:])
    assert want[0].shape[0] == 0                                      # the empty window
    # seeds with dense timestamps = the slice without a destination filter
    ch = np.array([1, 5, 2], dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(world["cp"][ch + 1] - world["cp"][ch])]).astype(np.int64)
    want = oracle.slice(world["hg"], world["cp"], world["cn"], None, ch, off, int(off[-1]), 50_000, 50_030, True)
    r = g.g.get_seeds_in_chunks(torch.tensor([1, 5, 2]), 50_000, 50_030, True)
    for a, b in zip((r.roots, r.ts_ptr, r.ts, r.q_ptr, r.q_eid), (want[0], want[1], want[2], want[3], want[6])):
        assert np.array_equal(np_of(a), b)
    assert r.root_ts_num == 30 * r.root_num > 0
    # through the query queue: dense timestamps, ids remapped per array (roots, then neighbours)
    g.async_sample(50_000, 50_020, torch.tensor([1, 5, 2]), {"sample_type": "cluster"}, {}, op="r")
    out = g.get_last_sample()
    ch = np.array([1, 5, 2], dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(world["cp"][ch + 1] - world["cp"][ch])]).astype(np.int64)
    want = oracle.slice(world["hg"], world["cp"], world["cn"], world["chunk_of"], ch, off, int(off[-1]), 50_000, 50_020, True)
    assert out.roots.root_ts_num == want[0].shape[0] * 20 > 0
    ids = np_of(out.nodes_remapper_id)
    assert np.array_equal(ids[np_of(out.roots.roots)], want[0])
    assert np.array_equal(ids[np_of(out.neighbors_list[0].neighbors)], want[4])
    assert np.array_equal(np_of(out.neighbors_list[0].root_start_ptr), want[3])


def test_neg_sampling_set():
    from starrygl_amd.graph.graph import NegSamplingSet
    pool = torch.arange(100, 200, device="cuda:0")
    s = NegSamplingSet(pool).sample(50, 3)
    assert s.shape == (50, 3) and int(s.min()) >= 100 and int(s.max()) < 200
    with pytest.raises(TypeError):
        NegSamplingSet([1, 2]).sample(1)


@pytest.mark.parametrize("mode", ["identity", "map", "dist_route_index"])
@pytest.mark.parametrize("tiered", [False, True])
def test_dist_node_state(mode, tiered):
    from starrygl_amd.cache.NodeState import DistNodeState
    from starrygl_amd.utils.partition_book import DistRouteIndex, PartitionState
    rng = np.random.default_rng(3)
    rows, dim, G = 2000, 100, 5000
    loc_ids = torch.from_numpy(rng.permutation(G)[:rows].astype(np.int64)) if mode == "map" else torch.arange(rows)
    st = PartitionState(loc_ids, rows // 2, node_mode=mode, num_nodes=G)
    hot = torch.from_numpy(rng.permutation(rows)[:300].astype(np.int64)) if tiered else None
    ns = DistNodeState(st, dim, hot_ids=hot, ts_dtype=torch.int64 if tiered else torch.float32)
    assert ns.data.is_pinned() and ns.data.shape == (rows, dim) and ns.ts.shape == (rows,)
    ref_data, ref_ts = torch.zeros(rows, dim), torch.zeros(rows, dtype=ns.ts.dtype)
    for it in range(3):
        locs = torch.from_numpy(rng.permutation(rows)[:500].astype(np.int64))
        gids = loc_ids[locs] if mode == "map" else locs
        vals = torch.randn(500, dim)
        t = torch.from_numpy(rng.integers(0, 10**6, 500)).to(ns.ts.dtype)
        key = gids.cuda()
        if mode == "dist_route_index":
            key = DistRouteIndex(gids, torch.from_numpy(rng.integers(0, 8, 500))).dist.cuda()
        ns.update(key, vals.cuda(), t.cuda())
        ref_data[locs], ref_ts[locs] = vals, t
        q_loc = torch.from_numpy(rng.integers(0, rows, 3000).astype(np.int64))
        q = (loc_ids[q_loc] if mode == "map" else q_loc).cuda()
        d, tt = ns[q]
        assert d.is_cuda and torch.equal(d.cpu(), ref_data[q_loc]) and torch.equal(tt.cpu(), ref_ts[q_loc])
        side = torch.cuda.Stream()
        d2, _ = ns.prefetch(q, side)
        side.synchronize()
        assert torch.equal(d2.cpu(), ref_data[q_loc])
    if mode == "map":        # ids that are not stored in this partition read as zero rows and are skipped by update
        absent = torch.tensor(sorted(set(range(G)) - set(loc_ids.tolist()))[:7]).cuda()
        d, tt = ns[absent]
        assert not d.any() and not tt.any()
        ns.update(absent, torch.ones(7, dim).cuda())
    # the tensors of the reference's layout show the rows of the HBM tier after a flush (state_dict flushes)
    sd = ns.state_dict()
    assert torch.equal(sd["data"], ref_data) and torch.equal(sd["ts"], ref_ts)
    with pytest.raises(ValueError, match="repeat"):
        ns.update(q[:1].repeat(2), torch.ones(2, dim).cuda(), check_unique=True)
    ns.to("cuda:0")
    d, tt = ns[q]
    assert torch.equal(d.cpu(), ref_data[q_loc]) and torch.equal(tt.cpu(), ref_ts[q_loc])
    ns.to("cpu")             # back into records of pinned memory (row and time side by side)
    d, tt = ns[q]
    assert ns.data.is_pinned() and torch.equal(d.cpu(), ref_data[q_loc]) and torch.equal(tt.cpu(), ref_ts[q_loc])
    assert torch.equal(ns.data, ref_data) and torch.equal(ns.ts, ref_ts)
    ns.reset()
    assert not ns[q][0].any()


def test_time_encoder_module():
    from starrygl_amd.nn.model.time_encoder import TimeEncoder
    enc = TimeEncoder(100).cuda()
    assert set(enc.state_dict()) == {"w.weight", "w.bias"} and enc.w.weight.shape == (100, 1)
    w_ref = torch.from_numpy((1.0 / 10 ** np.linspace(0, 9, 100, dtype=np.float32)).astype(np.float32))
    assert torch.equal(enc.w.weight.detach().cpu().reshape(-1), w_ref) and not enc.w.bias.any()
    dt = torch.randint(-2_600_000, 0, (4096,), device="cuda")
    y = enc(dt)
    ref = torch.cos(enc.w(dt.float().reshape(-1, 1)))
    assert y.shape == (4096, 100) and (y - ref).abs().max().item() < 5e-4   # Linear may fuse multiply-add
    assert enc(torch.zeros(5, device="cuda")).eq(1).all()
    with torch.no_grad():
        enc.w.bias.normal_()
    y = enc(dt.reshape(64, 64))
    ref = torch.cos(enc.w(dt.float().reshape(-1, 1)))
    g = torch.randn_like(y)
    gw, gb = torch.autograd.grad(y, [enc.w.weight, enc.w.bias], g)
    rw, rb = torch.autograd.grad(ref, [enc.w.weight, enc.w.bias], g)
    assert torch.allclose(gw, rw, rtol=1e-3, atol=1e-2 * rw.abs().max().item())
    assert torch.allclose(gb, rb, rtol=1e-3, atol=1e-2 * rb.abs().max().item())
    frozen = TimeEncoder(16, parameter_requires_grad=False).cuda()
    assert not frozen.w.weight.requires_grad
    want = 1.0 / 4.0 ** np.linspace(0, 4, 16, dtype=np.float32)
    assert np.allclose(frozen.w.weight.detach().cpu().numpy().reshape(-1), want)
    with pytest.raises(RuntimeError):
        TimeEncoder(8)(torch.zeros(1))


def test_segment_max_and_mailbox(oracle, hot):
    rng = np.random.default_rng(6)
    local = rng.integers(-2, 3005, 200_000).astype(np.int64)
    ts = rng.integers(-50, 50, 200_000).astype(np.int64)
    mx, arg = hot.segment_max_ts(to_dev(hot, local), to_dev(hot, ts), 3000)
    omx, oarg = oracle.segment_max_ts(local, ts, 3000)
    assert np.array_equal(np_of(mx), omx) and np.array_equal(np_of(arg), oarg)

    from starrygl_amd.nn.memory.mailbox import mailbox
    n, size, d_out, d_e, B = 500, 2, 8, 4, 300
    mb = mailbox(n, size, d_out, d_e, device="cuda:0")
    assert mb.shape == (n, size, 2 * d_out + d_e)
    ref_box, ref_ts, ref_pos = np.zeros((n, size, 20), np.float32), np.zeros((n, size), np.float32), np.zeros(n, np.int64)
    for it in range(4):
        src, dst = rng.integers(0, n, B), rng.integers(0, n, B)
        t = np.sort(rng.integers(0, 50, B)).astype(np.float32) + it * 50
        ef, ms, md = (rng.standard_normal((B, k)).astype(np.float32) for k in (d_e, d_out, d_out))
        T = lambda a: torch.from_numpy(a).cuda()
        index, mail, mail_ts = mb.get_update_mail(T(src), T(dst), T(t), T(ef), T(ms), T(md))
        # numpy restatement: mails of both endpoints, per node the mail with the largest ts (first on ties)
        idx_all = np.concatenate([src, dst])
        mails = np.concatenate([np.concatenate([ms, md, ef], 1), np.concatenate([md, ms, ef], 1)], 0)
        ts_all = np.concatenate([t, t])
        uniq = np.unique(idx_all)
        pick = np.array([np.flatnonzero(idx_all == u)[np.argmax(ts_all[idx_all == u])] for u in uniq])
        assert np.array_equal(np_of(index), uniq)
        assert np.array_equal(np_of(mail), mails[pick]) and np.array_equal(np_of(mail_ts), ts_all[pick])
        mb.set_mailbox_local(index, mail, mail_ts)
        ref_box[uniq, ref_pos[uniq]] = mails[pick]
        ref_ts[uniq, ref_pos[uniq]] = ts_all[pick]
        ref_pos[uniq] = (ref_pos[uniq] + 1) % size
        assert np.array_equal(np_of(mb.mailbox), ref_box) and np.array_equal(np_of(mb.mailbox_ts), ref_ts)
        assert np.array_equal(np_of(mb.next_mail_pos), ref_pos)
    m, mt = mb.get_message(torch.tensor([3, 4]).cuda())
    assert np.array_equal(np_of(m), ref_box[[3, 4]])
    # 'max' reduction inside set_mailbox_local de-duplicates first
    mb.reset()
    idx = torch.tensor([7, 7, 9]).cuda()
    mb.set_mailbox_local(idx, torch.arange(60, dtype=torch.float32).reshape(3, 20).cuda(), torch.tensor([1.0, 5.0, 2.0]).cuda(), "max")
    assert np_of(mb.mailbox)[7, 0, 0] == 20 and np_of(mb.mailbox_ts)[7, 0] == 5 and np_of(mb.mailbox)[9, 0, 0] == 40


@pytest.mark.parametrize("n,t_max", [(1, 50), (1023, 400), (1025, 400), (5000, 3000)])
def test_seeds_heavy_windows_and_tile_boundaries(oracle, hot, n, t_max):
    """Seed extraction against the oracle where one node holds most of every window (walked by a whole
    wavefront, 64 events per step), timestamps repeat a lot, and the candidate count sits on either side
    of the 1024-candidate tile; windows from empty to the whole history, chunk lists in any order."""
    rng = np.random.default_rng(n)
    m, C = 40_000, 5
    src = rng.integers(0, n, m).astype(np.int64)
    src[rng.random(m) < 0.6] = n // 2                  # the hub
    dst = rng.integers(0, n, m).astype(np.int64)
    ts = np.sort(rng.integers(0, t_max, m)).astype(np.int64)   # m >> t_max: long runs of equal timestamps
    eid = np.arange(m, dtype=np.int64)
    hg = host_graph(oracle, n, src, dst, ts, eid)
    from util import mirror_graph
    dg = mirror_graph(hot, hg)
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    cp, cn = oracle.chunk_index(n, C, chunk_of)
    dcp, dcn = hot.chunk_index(n, C, to_dev(hot, chunk_of))
    assert np.array_equal(np_of(dcp), cp) and np.array_equal(np_of(dcn), cn)
    for chunks in ([0, 1, 2, 3, 4], [3, 0], [int(chunk_of[n // 2])], []):
        ch = np.asarray(chunks, dtype=np.int64)
        off = np.concatenate([[0], np.cumsum(cp[ch + 1] - cp[ch])]).astype(np.int64)
        for t0, t1 in ((0, t_max), (t_max // 3, t_max // 3 + 1), (t_max // 2, t_max // 2 + 7), (5, 5), (t_max, t_max + 9)):
            want = oracle.seeds(hg, cp, cn, ch, off, int(off[-1]), t0, t1, with_window_end=True)
            got = hot.seeds(dg, dcp, dcn, to_dev(hot, ch), to_dev(hot, off), int(off[-1]), t0, t1, with_window_end=True)
            for f, a, b in zip(("roots", "ts_ptr", "ts", "q_ptr", "q_eid", "window_end"), got, want):
                assert np.array_equal(np_of(a), b), (f, chunks, t0, t1)
            # the sixth array is what a window-end lookup of every (root, timestamp) gives
            assert np.array_equal(want[5], oracle.window_end(hg, np.repeat(want[0], np.diff(want[1])), want[2]))


def test_shard_tensor_gathers_rows_of_device_and_host_shards(hot):
    """ShardTensor (feature.cu.hpp:236-422): shards appended in row order, some in HBM, some in pinned host
    memory; st[indices] equals indexing the concatenation."""
    from starrygl_amd.lib.libstarrygl_comm import ShardTensor
    torch.manual_seed(0)
    parts = [torch.randn(700, 25), torch.randn(1200, 25), torch.randn(300, 25), torch.randn(50, 25)]
    full = torch.cat(parts)
    for where in ([0, -1, 0, -1], [0, 0, 0, 0], [-1, -1, -1, -1], [-1, 0, -1, 0]):
        st = ShardTensor(0)
        for p, w in zip(parts, where):
            st.append(p, w)
        assert st.shape() == [2250, 25] and st.size(0) == 2250 and st.numel() == 2250 * 25 and st.stride(0) == 25
        assert st.device() == 0 and st.device_count() == 4
        idx = torch.randint(0, 2250, (5000,))
        got = st[idx.cuda()]
        assert got.is_cuda and torch.equal(got.cpu(), full[idx])
        assert torch.equal(st[idx][:10].cpu(), full[idx][:10])          # host indices are moved over
    st3 = ShardTensor(0)
    st3.append(torch.arange(24, dtype=torch.float32).reshape(4, 2, 3), -1)     # rows of any trailing shape
    assert torch.equal(st3[torch.tensor([3, 0])].cpu(), torch.arange(24, dtype=torch.float32).reshape(4, 2, 3)[[3, 0]])
    with pytest.raises(RuntimeError):
        st3.append(torch.zeros(2, 5), -1)
    with pytest.raises(RuntimeError):
        st3.append(torch.zeros(2, 2, 3), 1)                                    # another GPU
    st3.unregister()
    with pytest.raises(RuntimeError):
        st3[torch.tensor([0])]
