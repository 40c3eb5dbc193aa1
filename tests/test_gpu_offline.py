"""GPU: materialised batches (the reference's offline file layout) built by the HIP path
against a numpy restatement of the reference's builder that samples with the CPU oracle."""
import numpy as np
import pytest
import torch

from starrygl_amd.data import offline
from util import host_graph, np_of, to_dev

pytestmark = pytest.mark.gpu

PAIR = np.dtype([("id", np.int64), ("ts", np.int64)])


def _pairs(ids, ts):
    c = np.empty(len(ids), dtype=PAIR)
    c["id"], c["ts"] = ids, ts
    return c


def _want_layer(oracle, hg, tu, tt, cfg, meta, edge_cluster, cluster_id):
    """One layer as the numba kernel defines it (prepare_sample.py:57-76, 105-170), sampled with the oracle:
    -> (src, edge_ts, eid, dt = t - ts, per-target counts)."""
    st, fanout = cfg["type"], cfg.get("fanout", 10)
    so, eo = meta.get("start_offset", 0), meta.get("end_offset", 0)
    if meta.get("graph_type", "c") == "c":
        if st in ("recent", "uniform"):
            hop = oracle.sample_hop(hg, tu, tt + eo, oracle.params(st, fanout))
        else:
            hop = oracle.sample_window(hg, tu, tt, hi_offset=eo)
    elif st == "cluster":
        hop = oracle.sample_window(hg, tu, tt, lo_offset=so, hi_offset=eo, keep_slot_time=True, edge_tag=edge_cluster,
                                   tag_value=-1 if cluster_id is None else cluster_id)
    else:
        hop = oracle.sample_window(hg, tu, tt, lo_offset=so, hi_offset=eo, keep_slot_time=True,
                                   first_k=fanout if st == "uniform" else -1)
    return hop


def _want_batch(oracle, hg, l0_nodes, l0_ts, layers, meta=None, edge_cluster=None, cluster_id=None):
    """prepare_sample.py:310-371 with numpy: np.unique over (id, ts) records, np.lexsort((ts, dst)).
    layers: fanouts of 'recent' layers, or layer config dicts."""
    meta = meta or {}
    layers = [l if isinstance(l, dict) else {"type": "recent", "fanout": l} for l in layers]
    u, inv = np.unique(_pairs(l0_nodes, l0_ts), return_inverse=True)
    cur_id, cur_ts = u["id"].copy(), u["ts"].copy()
    out = [dict(gids=cur_id, ts=cur_ts, inv_map=inv)]
    last_inv = None
    for cfg in layers:
        tu = cur_id if last_inv is None else cur_id[last_inv]
        tt = cur_ts if last_inv is None else cur_ts[last_inv]
        if tu.size == 0 or not (hg.row_ptr[tu + 1] > hg.row_ptr[tu]).any():
            e = np.zeros(0, np.int64)
            out.append(dict(indptr=np.zeros(1, np.int64), indices=e, eid=e, edge_ts=e, edge_dt=np.zeros(0, np.float32),
                            gids=e, ts=e))
            break
        hop = _want_layer(oracle, hg, tu, tt, cfg, meta, edge_cluster, cluster_id)
        raw_dst = np.repeat(np.arange(tu.size), np.diff(hop.root_start_ptr))
        # t_cut - ts of the edge (prepare_sample.py:130, 145, 157), t_cut the target's own time whatever the offsets
        raw_dt = (tt[raw_dst] - (tt[raw_dst] + hop.neighbors_dt if meta.get("graph_type", "c") != "c" or cfg["type"] in ("full", "cluster")
                                 else hop.neighbors_ts)).astype(np.float32)
        dst_m = raw_dst if last_inv is None else last_inv[raw_dst]
        allp = np.unique(np.concatenate([_pairs(cur_id, cur_ts), _pairs(hop.neighbors, hop.neighbors_ts)]))
        nxt_inv = np.searchsorted(allp, _pairs(hop.neighbors, hop.neighbors_ts))
        perm = np.lexsort((hop.neighbors_ts, dst_m))
        indptr = np.concatenate([[0], np.cumsum(np.bincount(dst_m, minlength=cur_id.size))]).astype(np.int64)
        out.append(dict(indptr=indptr, indices=nxt_inv[perm], eid=hop.neighbors_eid[perm], edge_ts=hop.neighbors_ts[perm],
                        edge_dt=raw_dt[perm], gids=allp["id"].copy(), ts=allp["ts"].copy()))
        cur_id, cur_ts, last_inv = allp["id"].copy(), allp["ts"].copy(), nxt_inv
    return out


def test_pair_unique_and_csc_order(hot):
    rng = np.random.default_rng(2)
    for n in (0, 1, 7, 5000):
        ids, ts = rng.integers(-50, 400, n), rng.integers(-5, 60, n)
        u, inv = np.unique(_pairs(ids, ts), return_inverse=True)
        got = hot.unique_pairs(to_dev(hot, ids), to_dev(hot, ts))
        assert np.array_equal(np_of(got[0]), u["id"]) and np.array_equal(np_of(got[1]), u["ts"])
        assert np.array_equal(np_of(got[2]), inv.reshape(-1))
        d = rng.integers(0, 300, n)
        indptr, perm = hot.csc_from_pairs(to_dev(hot, d), to_dev(hot, ts), 300)
        assert np.array_equal(np_of(perm), np.lexsort((ts, d)))
        assert np.array_equal(np_of(indptr), np.concatenate([[0], np.cumsum(np.bincount(d, minlength=300))]))
    # a live length on the device shorter than the array
    ids, ts = rng.integers(0, 30, 1000), rng.integers(0, 10, 1000)
    n_dev = to_dev(hot, np.array([600]))
    u, inv = np.unique(_pairs(ids[:600], ts[:600]), return_inverse=True)
    got = hot.unique_pairs(to_dev(hot, ids), to_dev(hot, ts), N_dev=n_dev)
    assert np.array_equal(np_of(got[0]), u["id"]) and np.array_equal(np_of(got[2]), inv.reshape(-1))


@pytest.mark.parametrize("layers", [[5], [4, 3]])
def test_link_batch_matches_numpy_builder(oracle, hot, tmp_path, layers):
    rng = np.random.default_rng(8)
    n, m = 400, 9000
    src, dst = rng.integers(0, n, m), rng.integers(0, n - 20, m)     # the last 20 nodes have no in-edges
    ts = np.sort(rng.integers(0, 3000, m))
    eid = rng.permutation(m)
    b = offline.MaterializedMultiLayerBuilder(dict(src=src, dst=dst, ts=ts, eid=eid), n, device=hot.be.device)
    # the oracle's twin of the builder's graph: rows are destinations, ties in arrival order
    hg = host_graph(oracle, n, dst, src, ts, np.arange(m))
    hg.eid[:] = eid[hg.eid]
    lo = 6000
    t_src, t_dst, t_ts = src[lo: lo + 200], dst[lo: lo + 200], ts[lo: lo + 200]
    label, t_eid = np.ones(200, np.int64), eid[lo: lo + 200]
    cfg = {"layer": [{"fanout": f, "type": "recent"} for f in layers], "meta": {"graph_type": "c"}}
    path = tmp_path / "slot_0000.pt"
    task = tuple(torch.from_numpy(np.ascontiguousarray(x)) for x in (t_src, t_dst, t_ts, label, t_eid))
    got = b.build_aligned_batch(("link", task), path, cfg, num_neg=1)
    want = _want_batch(oracle, hg, np.concatenate([t_src, t_dst]), np.concatenate([t_ts, t_ts]), layers)
    assert len(got) == len(want) == len(layers) + 1
    disk = offline.read_batch(path)
    for g, d, w in zip(got, disk, want):
        for k, v in w.items():
            assert np.array_equal(np_of(g[k]), v), k
            assert np.array_equal(np_of(d[k]), v) and d[k].dtype == g[k].dtype, k
    assert got[1]["edge_dt"].dtype == torch.float32 and bool((got[1]["edge_dt"] > 0).all())
    assert disk[0]["num_neg"] == 1 and disk[0]["comm_plan"] == [None] * (len(layers) + 1)
    assert torch.equal(disk[0]["task_src"], task[0]) and torch.equal(disk[0]["task_eid"], task[4])
    # targets come back through inv_map; block view: outermost layer first
    l0 = np.concatenate([t_src, t_dst])
    assert np.array_equal(np_of(got[0]["gids"])[np_of(got[0]["inv_map"])], l0)
    blocks = offline.batch_to_blocks(got)
    assert blocks[-1].num_dst_nodes() == got[0]["gids"].numel() and blocks[0].num_src_nodes() == got[-1]["gids"].numel()


def test_neg_and_node_tasks_and_empty_history(hot, tmp_path):
    rng = np.random.default_rng(3)
    n, m = 100, 2000
    src, dst, ts = rng.integers(0, n, m), rng.integers(0, 50, m), np.sort(rng.integers(0, 500, m))
    b = offline.MaterializedMultiLayerBuilder(dict(src=src, dst=dst, ts=ts), n, device=hot.be.device, seed=5)
    cfg = {"layer": [{"fanout": 3, "type": "uniform"}, {"fanout": 3, "type": "recent"}], "meta": {}}
    pool = np.arange(0, 50)
    t = torch.from_numpy(ts[1000:1050].copy())
    neg = b.build_aligned_batch(("neg", t), tmp_path / "neg.pt", cfg, num_neg=4, global_dst_pool=pool)
    assert neg[0]["task_nodes"].numel() == 200 and neg[0]["task_label"] == "neg_set"
    assert np.array_equal(np_of(neg[0]["ts"])[np_of(neg[0]["inv_map"])], np.repeat(ts[1000:1050], 4))
    lay = neg[1]
    deg = np.diff(np_of(lay["indptr"]))
    assert deg.max() <= 3 and lay["indices"].numel() == deg.sum()
    # every sampled edge is an in-edge of its target strictly before the target's time
    tgt = np.repeat(np.arange(deg.size), deg)
    e_ts, e_dt = np_of(lay["edge_ts"]), np_of(lay["edge_dt"])
    assert (e_ts < np_of(neg[0]["ts"])[tgt]).all() and np.array_equal(e_dt, (np_of(neg[0]["ts"])[tgt] - e_ts).astype(np.float32))
    assert np.array_equal(dst[np_of(lay["eid"])], np_of(neg[0]["gids"])[tgt])
    assert np.array_equal(src[np_of(lay["eid"])], np_of(lay["gids"])[np_of(lay["indices"])])
    assert offline.read_batch(tmp_path / "neg.pt")[0]["task_label"] == "neg_set"
    # targets without any in-edge: one empty layer, then the builder stops (prepare_sample.py:337-347)
    node = b.build_aligned_batch(("node", (torch.tensor([60, 61]), torch.tensor([400, 400]), torch.tensor([0, 1]))),
                                 None, cfg)
    assert len(node) == 2 and node[1]["indptr"].tolist() == [0] and node[1]["gids"].numel() == 0
    with pytest.raises(ValueError):
        b.build_aligned_batch(("graph", None), None, cfg)


@pytest.mark.parametrize("graph_type,types,meta", [
    ("c", ["full", "recent"], {}),
    ("c", ["cluster"], {"end_offset": 40}),
    ("c", ["recent", "full"], {"end_offset": -25}),
    ("d", ["uniform", "full"], {"start_offset": -300, "end_offset": 1}),
    ("d", ["cluster", "uniform"], {"start_offset": -900, "end_offset": 0}),
    ("d", ["recent"], {"start_offset": -120, "end_offset": 5}),
])
def test_every_layer_type_of_both_graph_modes(oracle, hot, graph_type, types, meta):
    """'full' / 'cluster' layers and the discrete-time branch of the offline sampler (prepare_sample.py:57-76,
    105-170) against the numpy restatement of the builder that samples with the oracle."""
    rng = np.random.default_rng(12)
    n, m = 300, 12_000
    src, dst = rng.integers(0, n, m), rng.integers(0, n - 10, m)
    ts = np.sort(rng.integers(0, 2000, m))
    cid = rng.integers(0, 6, m)
    b = offline.MaterializedMultiLayerBuilder(dict(src=src, dst=dst, ts=ts, cid=cid), n, device=hot.be.device)
    hg = host_graph(oracle, n, dst, src, ts, np.arange(m))
    edge_cluster = cid[hg.eid].astype(np.int64)        # the events' clusters in the graph's edge order
    meta = dict(meta, graph_type=graph_type)
    layers = [{"type": t, "fanout": 4} for t in types]
    lo = 9000
    node, t_node = dst[lo: lo + 150], ts[lo: lo + 150]
    task = tuple(torch.from_numpy(np.ascontiguousarray(x)) for x in (node, t_node, np.zeros(150, np.int64)))
    got = b.build_aligned_batch(("node", task), None, {"layer": layers, "meta": meta}, cluster_ids=2)
    want = _want_batch(oracle, hg, node, t_node, layers, meta, edge_cluster, 2)
    assert len(got) == len(want)
    for l, (g, w) in enumerate(zip(got, want)):
        for k, v in w.items():
            assert np.array_equal(np_of(g[k]), v), (l, k)
    assert got[1]["indices"].numel() > 0
    if graph_type == "d":      # a discrete layer reports the target's time as the edge time
        deg = np.diff(np_of(got[1]["indptr"]))
        assert np.array_equal(np_of(got[1]["edge_ts"]), np.repeat(np_of(got[0]["ts"]), deg))
