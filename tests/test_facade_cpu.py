"""Host-side logic of the façade that needs no GPU: id codecs, id mappers, and
the oracle's seed extraction / chunk index / block assembly against brute force."""
import numpy as np
import pytest
import torch

from starrygl_amd.utils.partition_book import DistRouteIndex, IDMapper, PartitionState
from util import host_graph


def test_dist_route_index_codec():
    loc = torch.tensor([0, 5, 2**47 + 3, 2**48 - 1])
    part = torch.tensor([0, 7, 16383, 1])
    d = DistRouteIndex(loc, part)
    assert torch.equal(d.loc, loc) and torch.equal(d.part, part) and not d.is_shared.any()
    d.set_shared(torch.tensor([1, 3]))
    assert d.is_shared.tolist() == [False, True, False, True]
    assert torch.equal(d.loc, loc) and torch.equal(d.part, part)
    assert torch.equal(DistRouteIndex(d.dist).dist, d.dist) and d.shape == loc.shape
    # arithmetic spelled out
    assert int(d.dist[1]) == 5 | (7 << 48) | (1 << 62)


def test_idmapper_modes():
    loc_ids = torch.tensor([10, 3, 7, 25])
    m = IDMapper(loc_ids, num_master=2, mode="map", global_num=30)
    assert m.to_local(torch.tensor([3, 25, 4, 10, 30])).tolist() == [1, 3, -1, 0, -1]
    assert m.loc_nums == 4 and m.num_master == 2 and m.global_nums == 30
    assert m.is_master_by_local(torch.tensor([0, 1, 2, -1])).tolist() == [True, True, False, False]
    assert m.is_remote_ids(torch.tensor([10, 7, 4])).tolist() == [False, True, True]
    assert m.is_store_local(torch.tensor([10, 7, 4])).tolist() == [True, True, False]
    assert m.to_dist(torch.tensor([2, 0])).tolist() == [7, 10]
    assert IDMapper(loc_ids, 4, "identity").to_local(torch.tensor([4, 9])).tolist() == [4, 9]
    assert IDMapper(loc_ids, 4, "offset", offset=100).to_local(torch.tensor([104, 100])).tolist() == [4, 0]
    enc = DistRouteIndex(torch.tensor([4, 9]), torch.tensor([3, 2]))
    assert IDMapper(loc_ids, 4, "dist_route_index").to_local(enc.dist).tolist() == [4, 9]
    assert IDMapper(loc_ids, 4, "identity").to_local(enc).tolist() == [4, 9]
    with pytest.raises(ValueError):
        IDMapper(loc_ids, 4, "hash")
    dm = torch.arange(100, 104)
    assert IDMapper(loc_ids, 4, "identity", dist_mapper=dm).to_dist(torch.tensor([1])).tolist() == [101]


def test_partition_state():
    st = PartitionState(torch.tensor([4, 2, 9]), 2, node_mode="map", num_nodes=10)
    assert st.to_local_nid(torch.tensor([9, 4, 0])).tolist() == [2, 0, -1]
    assert st.is_master_node_by_global(torch.tensor([9, 4])).tolist() == [False, True]
    with pytest.raises(RuntimeError):
        st.to_local_eid(torch.tensor([1]))
    st2 = PartitionState(torch.tensor([4, 2, 9]), 2, loc_eids=torch.tensor([5, 6]), num_master_edges=1)
    assert st2.to_local_eid(torch.tensor([6])).tolist() == [6]
    assert st2.is_master_edge_by_local(torch.tensor([0, 1])).tolist() == [True, False]


def _seed_brute(g, chunk_of, chunks, t0, t1):
    roots, ts_ptr, ts, q_ptr, q_eid = [], [0], [], [0], []
    for c in chunks:
        for v in [v for v in range(g.n) if chunk_of[v] == c]:
            ev = [e for e in range(g.row_ptr[v], g.row_ptr[v + 1]) if t0 <= g.ts[e] < t1]
            if not ev:
                continue
            roots.append(v)
            for t in sorted(set(g.ts[e] for e in ev)):
                ts.append(t)
                q_eid += [g.eid[e] for e in ev if g.ts[e] == t]
                q_ptr.append(len(q_eid))
            ts_ptr.append(len(ts))
    return roots, ts_ptr, ts, q_ptr, q_eid


def test_oracle_seeds_match_brute_force(oracle):
    rng = np.random.default_rng(0)
    n, m, C = 40, 600, 5
    g = host_graph(oracle, n, rng.integers(0, n, m), rng.integers(0, n, m), rng.integers(0, 30, m))
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    chunk_ptr, chunk_nodes = oracle.chunk_index(n, C, chunk_of)
    assert np.array_equal(chunk_ptr, np.concatenate([[0], np.cumsum(np.bincount(chunk_of, minlength=C))]))
    assert np.array_equal(chunk_nodes, np.argsort(chunk_of, kind="stable"))
    for chunks, t0, t1 in [([0, 3], 5, 12), ([4, 4, 1], 0, 30), ([2], 29, 30), ([], 0, 30), ([1], 10, 10)]:
        ch = np.array(chunks, dtype=np.int64)
        sizes = chunk_ptr[ch + 1] - chunk_ptr[ch] if ch.size else np.zeros(0, np.int64)
        off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        got = oracle.seeds(g, chunk_ptr, chunk_nodes, ch, off, int(off[-1]), t0, t1, with_window_end=True)
        want = _seed_brute(g, chunk_of, chunks, t0, t1)
        for a, b in zip(got, want):
            assert a.tolist() == [int(x) for x in b]
        # window end of a (root, timestamp): number of the root's edges before that time, from the row's start
        slot_root = np.repeat(got[0], np.diff(got[1]))
        brute = [int(g.row_ptr[v] + (g.ts[g.row_ptr[v]: g.row_ptr[v + 1]] < t).sum()) for v, t in zip(slot_root, got[2])]
        assert got[5].tolist() == brute
    with pytest.raises(IndexError):
        oracle.chunk_index(3, 2, np.array([0, 2, 1], dtype=np.int64))


def _slice_brute(g, chunk_of, chunks, t0, t1, full):
    sel = set(chunks)
    nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid = [], [0], [], [], [], [], []
    for c in chunks:
        for v in [v for v in range(g.n) if chunk_of[v] == c]:
            ev = [e for e in range(g.row_ptr[v], g.row_ptr[v + 1]) if t0 <= g.ts[e] < t1]
            if not ev:
                continue
            nodes.append(v)
            for t in (range(t0, t1) if full else sorted(set(g.ts[e] for e in ev))):
                ts.append(t)
                edge_ptr.append(len(col))
                for e in ev:
                    if g.ts[e] == t and chunk_of[g.col[e]] in sel:
                        col.append(g.col[e]); col_ts.append(g.ts[e]); col_eid.append(g.eid[e])
            ts_ptr.append(len(ts))
    edge_ptr.append(len(col))
    return nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid


def test_oracle_slice_matches_brute_force(oracle):
    rng = np.random.default_rng(4)
    n, m, C = 40, 900, 5
    g = host_graph(oracle, n, rng.integers(0, n, m), rng.integers(0, n, m), rng.integers(0, 30, m))
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    chunk_ptr, chunk_nodes = oracle.chunk_index(n, C, chunk_of)
    for chunks, t0, t1 in [([0, 3], 5, 12), ([4, 1, 2], 0, 30), ([2], 29, 30), ([], 0, 30), ([1], 10, 10),
                           ([0, 1, 2, 3, 4], 3, 9)]:
        ch = np.array(chunks, dtype=np.int64)
        sizes = chunk_ptr[ch + 1] - chunk_ptr[ch] if ch.size else np.zeros(0, np.int64)
        off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        for full in (False, True):
            got = oracle.slice(g, chunk_ptr, chunk_nodes, chunk_of, ch, off, int(off[-1]), t0, t1, full)
            want = _slice_brute(g, chunk_of, chunks, t0, t1, full)
            for a, b in zip(got, want):
                assert a.tolist() == [int(x) for x in b], (chunks, t0, t1, full)
            # with every chunk selected no edge of the window is dropped
            if len(chunks) == C:
                assert got[4].shape[0] == int(((g.ts >= t0) & (g.ts < t1)).sum())
            # without a destination filter: the seeds of the same query (full: one entry per integer time)
            free = oracle.slice(g, chunk_ptr, chunk_nodes, None, ch, off, int(off[-1]), t0, t1, full)
            roots, ts_ptr, ts_, q_ptr, q_eid = _seed_brute(g, chunk_of, chunks, t0, t1)
            assert free[0].tolist() == [int(x) for x in roots]
            if not full:
                for a, b in zip((free[1], free[2], free[3], free[6]), (ts_ptr, ts_, q_ptr, q_eid)):
                    assert a.tolist() == [int(x) for x in b]
            else:
                assert free[2].tolist() == list(range(t0, t1)) * len(roots) and free[6].tolist() == [int(x) for x in q_eid]
                cnt = np.diff(free[3]).reshape(len(roots), -1) if roots else np.zeros((0, 0))
                for r, v in enumerate(roots):                 # events per (root, integer time)
                    row = g.ts[g.row_ptr[v]: g.row_ptr[v + 1]]
                    assert cnt[r].tolist() == [int((row == t).sum()) for t in range(t0, t1)]


def test_oracle_block_build(oracle):
    rsp = np.array([0, 2, 2, 5], dtype=np.int64)
    counts = np.array([3, 5, 0], dtype=np.int64)
    indptr, indices, edst = oracle.block_build(rsp, counts, 3, 5, 4, 7, with_edge_dst=True)
    assert indptr.tolist() == [0, 0, 0, 0, 0, 2, 2, 5]
    assert indices.tolist() == [7, 8, 9, 10, 11]
    assert edst.tolist() == [4, 4, 6, 6, 6]
    # expanding indptr back gives edge_dst: the CSC and the COO view agree
    assert np.repeat(np.arange(7), np.diff(indptr)).tolist() == edst.tolist()


def test_oracle_segment_max_ts(oracle):
    rng = np.random.default_rng(3)
    local = rng.integers(-1, 12, 500).astype(np.int64)      # -1 and 10, 11 are outside [0, 10)
    ts = rng.integers(0, 20, 500).astype(np.int64)          # many ties
    mx, arg = oracle.segment_max_ts(local, ts, 10)
    for u in range(10):
        pos = np.flatnonzero(local == u)
        assert mx[u] == ts[pos].max() and arg[u] == pos[np.argmax(ts[pos])]     # argmax = first occurrence
    mx, arg = oracle.segment_max_ts(np.array([0, 0], np.int64), np.array([5, 7], np.int64), 3)
    assert arg.tolist() == [1, -1, -1] and mx[0] == 7 and mx[1] == np.iinfo(np.int64).min


def test_oracle_pair_unique_and_csc_order(oracle):
    """np.unique over (id, ts) records and np.lexsort((ts, dst)) are the routines the reference calls
    (prepare_sample.py:205-229); the oracle's restatement must equal them."""
    rng = np.random.default_rng(6)
    dt = np.dtype([("id", np.int64), ("ts", np.int64)])
    for n in (0, 1, 2, 900):
        ids, ts = rng.integers(-9, 40, n).astype(np.int64), rng.integers(-4, 12, n).astype(np.int64)
        c = np.empty(n, dtype=dt)
        c["id"], c["ts"] = ids, ts
        u, inv = np.unique(c, return_inverse=True)
        g_id, g_ts, g_inv = oracle.unique_pairs(ids, ts)
        assert np.array_equal(g_id, u["id"]) and np.array_equal(g_ts, u["ts"]) and np.array_equal(g_inv, inv.reshape(-1))
        d = rng.integers(0, 25, n).astype(np.int64)
        indptr, perm = oracle.csc_from_pairs(d, ts, 25)
        assert np.array_equal(perm, np.lexsort((ts, d)))
        assert np.array_equal(indptr, np.concatenate([[0], np.cumsum(np.bincount(d, minlength=25))]))
    with pytest.raises(IndexError):
        oracle.csc_from_pairs(np.array([3], np.int64), np.array([0], np.int64), 3)


def test_slot_and_batch_files_round_trip(tmp_path):
    from starrygl_amd.data import offline
    src, dst, ts = torch.arange(5), torch.arange(5) + 1, torch.arange(5) * 10
    offline.write_slot(tmp_path / "slot_0001_sub_0000.pt", src, dst, ts, torch.arange(5), torch.tensor([2, 7]), 1, 12)
    d = offline.read_slot(tmp_path / "slot_0001_sub_0000.pt")
    assert sorted(d) == sorted(offline.SLOT_KEYS) and d["slot_id"] == 1 and d["chunk_id"] == 12
    assert torch.equal(d["dst"], dst) and torch.equal(d["cid"], torch.tensor([2, 7]))
    torch.save({"src": src}, tmp_path / "bad.pt")
    with pytest.raises(KeyError):
        offline.read_slot(tmp_path / "bad.pt")
    batch = [{"gids": src, "ts": ts, "inv_map": src, "num_neg": 2, "task_label": "neg_set", "comm_plan": [None, None]},
             {"indptr": torch.tensor([0, 1, 1, 2, 2, 2]), "indices": torch.tensor([0, 3]), "eid": torch.tensor([9, 8]),
              "edge_ts": torch.tensor([1, 2]), "edge_dt": torch.tensor([1.0, 2.0]), "gids": src, "ts": ts}]
    offline.write_batch(tmp_path / "b.pt", batch)
    back = offline.read_batch(tmp_path / "b.pt")
    assert back[0]["task_label"] == "neg_set" and back[0]["comm_plan"] == [None, None]
    assert torch.equal(back[1]["indptr"], batch[1]["indptr"]) and back[1]["edge_dt"].dtype == torch.float32
    blk = offline.batch_to_blocks(back)[0]
    assert blk.num_dst_nodes() == 5 and blk.num_edges() == 2 and torch.equal(blk.edata["eid"], torch.tensor([9, 8]))
