"""GPU parity: two-tier cache gather / scatter-update through the C ABI vs the
CPU oracle and numpy fancy indexing, byte-exact."""
import numpy as np
import pytest
import torch

from util import np_of, to_dev

pytestmark = pytest.mark.gpu


def _tables(rows, dim, dtype, hot_frac, seed):
    rng = np.random.default_rng(seed)
    if dtype == np.uint16:  # bf16 payload: any bit pattern is a valid row
        full = rng.integers(0, 2**16, (rows, dim), dtype=np.uint16)
    else:
        full = rng.standard_normal((rows, dim)).astype(dtype)
    hot_rows = int(rows * hot_frac)
    hot_ids = rng.permutation(rows)[:hot_rows]
    hot_slot = np.full(rows, -1, dtype=np.int32)
    hot_slot[hot_ids] = np.arange(hot_rows, dtype=np.int32)
    hot = full[hot_ids].copy()
    cold = full.copy()
    cold[hot_ids] = 0  # a hot row must never be served from the cold tier
    return full, hot, cold, hot_slot


def _dev_cache(hot_path, full, hot, cold, hot_slot, **kw):
    t_hot = torch.from_numpy(hot).to(hot_path.be.device)
    t_cold = torch.from_numpy(cold).pin_memory()
    t_slot = to_dev(hot_path, hot_slot, "i32")
    rb = full.shape[1] * full.dtype.itemsize
    return hot_path.cache(rb, t_hot, rows=full.shape[0], cold=t_cold, hot_slot=t_slot, **kw), (t_hot, t_cold)


@pytest.mark.parametrize("dim,dtype", [(128, np.uint16), (100, np.float32), (172, np.float32), (1, np.float32),
                                       (3, np.float32), (6, np.float32), (1000, np.float32)])
def test_gather_matches_numpy(oracle, hot, dim, dtype):
    rows, N = 20_000, 50_000
    full, h, c, slot = _tables(rows, dim, dtype, 0.1, dim)
    ids = np.random.default_rng(1).integers(0, rows, N).astype(np.int64)
    cache, keep = _dev_cache(hot, full, h, c, slot)
    out = torch.empty((N, dim), dtype=torch.from_numpy(full[:1]).dtype, device=hot.be.device)
    stats = hot.be.zeros(3)
    hot.gather(cache, to_dev(hot, ids), out, stats=stats)
    assert np.array_equal(np_of(out).view(np.uint8), full[ids].view(np.uint8))
    n_hot = int((slot[ids] >= 0).sum())
    assert np_of(stats).tolist() == [n_hot, N - n_hot, 0]
    # the oracle agrees with numpy on the same tables
    oc = oracle.cache(full.shape[1] * full.dtype.itemsize, h, rows=rows, cold=c, hot_slot=slot)
    o_out = np.empty((N, dim), dtype=full.dtype)
    oracle.gather(oc, ids, o_out)
    assert np.array_equal(o_out.view(np.uint8), full[ids].view(np.uint8))


def test_gather_g2l_mask_ts_and_absent(oracle, hot):
    """global id -> local row through a dense map, DistRouteIndex low-48-bit
    mask, last-update timestamps from both tiers, absent ids -> zero rows."""
    rows, dim, G = 5000, 100, 12_000
    full, h, c, slot = _tables(rows, dim, np.float32, 0.3, 2)
    rng = np.random.default_rng(3)
    loc_ids = rng.permutation(G)[:rows].astype(np.int64)       # global id of each local row
    g2l = np.full(G + 1, -1, dtype=np.int64)
    g2l[loc_ids] = np.arange(rows)
    ts_full = rng.integers(0, 10**9, rows).astype(np.int64)
    hot_rows = h.shape[0]
    ts_hot = np.zeros(hot_rows, dtype=np.int64)
    ts_hot[slot[slot >= 0]] = ts_full[slot >= 0]
    gids = rng.integers(0, G, 30_000).astype(np.int64)
    gids[::97] = -5
    gids[::101] = G + 3
    part = rng.integers(0, 2**14, gids.shape[0]).astype(np.int64)
    enc = np.where(gids >= 0, gids | (part << 48) | (1 << 62), gids)   # DistRouteIndex encoding
    kw = dict(id_mask=0xFFFFFFFFFFFF)
    cache, keep = _dev_cache(hot, full, h, c, slot, g2l=to_dev(hot, g2l), ts_hot=to_dev(hot, ts_hot),
                             ts_cold=torch.from_numpy(ts_full).pin_memory(), **kw)
    out = torch.empty((gids.shape[0], dim), dtype=torch.float32, device=hot.be.device)
    out_ts = hot.be.empty(gids.shape[0])
    stats = hot.be.zeros(3)
    hot.gather(cache, to_dev(hot, enc), out, out_ts=out_ts, stats=stats)
    oc = oracle.cache(dim * 4, h, rows=rows, cold=c, hot_slot=slot, g2l=g2l, ts_hot=ts_hot, ts_cold=ts_full, **kw)
    o_out, o_ts, o_stats = np.empty((gids.shape[0], dim), np.float32), np.empty(gids.shape[0], np.int64), np.zeros(3, np.int64)
    oracle.gather(oc, enc, o_out, out_ts=o_ts, stats=o_stats)
    assert np.array_equal(np_of(out).view(np.uint32), o_out.view(np.uint32))
    assert np.array_equal(np_of(out_ts), o_ts)
    assert np_of(stats).tolist() == o_stats.tolist()
    # numpy closed form
    ok = (gids >= 0) & (gids < G + 1)
    loc = np.where(ok, g2l[np.clip(gids, 0, G)], -1)
    want = np.where((loc >= 0)[:, None], full[np.clip(loc, 0, rows - 1)], 0).astype(np.float32)
    assert np.array_equal(o_out.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(o_ts, np.where(loc >= 0, ts_full[np.clip(loc, 0, rows - 1)], 0))
    assert o_stats[2] == int((loc < 0).sum())


def test_all_hot_table_without_index(hot):
    rows, dim = 3000, 172
    full = np.random.default_rng(0).standard_normal((rows, dim)).astype(np.float32)
    ids = np.random.default_rng(1).integers(0, rows, 10_000).astype(np.int64)
    t = torch.from_numpy(full).to(hot.be.device)
    cache = hot.cache(dim * 4, t)
    out = torch.empty((ids.shape[0], dim), dtype=torch.float32, device=hot.be.device)
    hot.gather(cache, to_dev(hot, ids), out)
    assert np.array_equal(np_of(out), full[ids])
    # a live count on the device shortens the gather
    out.zero_()
    n_dev = to_dev(hot, np.array([123], dtype=np.int64))
    hot.gather(cache, to_dev(hot, ids), out, N_dev=n_dev)
    assert np.array_equal(np_of(out)[:123], full[ids[:123]]) and not np_of(out)[123:].any()


def test_scatter_update_roundtrip(oracle, hot):
    rows, dim = 4000, 100
    full, h, c, slot = _tables(rows, dim, np.float32, 0.25, 7)
    cache, (t_hot, t_cold) = _dev_cache(hot, full, h, c, slot)
    rng = np.random.default_rng(8)
    ids = rng.permutation(rows)[:1500].astype(np.int64)
    ids_bad = ids.copy()
    ids_bad[::50] = -1
    vals = rng.standard_normal((1500, dim)).astype(np.float32)
    ts = rng.integers(0, 10**6, 1500).astype(np.int64)
    ts_hot = hot.be.zeros(h.shape[0])
    ts_cold = torch.zeros(rows, dtype=torch.int64).pin_memory()
    hot.scatter_update(cache, t_hot, t_cold, ts_hot, ts_cold, to_dev(hot, ids_bad), to_dev(hot, vals, "f32"), to_dev(hot, ts))
    torch.cuda.synchronize()
    oh, oc_, oth, otc = h.copy(), c.copy(), np.zeros(h.shape[0], np.int64), np.zeros(rows, np.int64)
    ocache = oracle.cache(dim * 4, oh, rows=rows, cold=oc_, hot_slot=slot)
    oracle.scatter_update(ocache, oh, oc_, oth, otc, ids_bad, vals, ts)
    assert np.array_equal(np_of(t_hot), oh) and np.array_equal(t_cold.numpy(), oc_)
    assert np.array_equal(np_of(ts_hot), oth) and np.array_equal(ts_cold.numpy(), otc)
    # and the gather reads the updated rows back
    out = torch.empty((1500, dim), dtype=torch.float32, device=hot.be.device)
    hot.gather(cache, to_dev(hot, ids), out)
    keep = ids_bad >= 0
    assert np.array_equal(np_of(out)[keep], vals[keep])


@pytest.mark.parametrize("dim", [100, 3, 172])
def test_interleaved_cold_records(oracle, hot, dim):
    """cold tier whose records hold a row and its last-update time side by side (cold_stride / ts_cold_stride of
    sgl_cache): gather with times, scatter_update and a multi-segment gather read and write the records in place;
    byte-exact against numpy on the same values and against the oracle on a numpy copy of the record buffer."""
    rows, N = 6000, 20_000
    full, h, c, slot = _tables(rows, dim, np.float32, 0.2, 40 + dim)
    rng = np.random.default_rng(dim)
    ts_full = rng.integers(1, 10**9, rows).astype(np.int64)
    data, ts, rec = hot.interleaved_cold(rows, dim)
    assert rec.is_pinned() and rec.shape[1] % 128 == 0 and data.shape == (rows, dim) and ts.shape == (rows,)
    data.copy_(torch.from_numpy(c))
    ts.copy_(torch.from_numpy(ts_full))
    hot_ids = np.nonzero(slot >= 0)[0]
    ts_hot_np = np.zeros(h.shape[0], np.int64)
    ts_hot_np[slot[hot_ids]] = ts_full[hot_ids]
    t_hot, t_slot, t_ts_hot = torch.from_numpy(h).to(hot.be.device), to_dev(hot, slot, "i32"), to_dev(hot, ts_hot_np)
    cache = hot.cache(dim * 4, t_hot, rows=rows, cold=data, hot_slot=t_slot, ts_hot=t_ts_hot, ts_cold=ts)
    assert cache.cold_stride == rec.shape[1] and cache.ts_cold_stride == rec.shape[1]
    ids = rng.integers(-2, rows, N).astype(np.int64)
    out = torch.empty((N, dim), dtype=torch.float32, device=hot.be.device)
    out_ts = hot.be.empty(N)
    hot.gather(cache, to_dev(hot, ids), out, out_ts=out_ts)
    ok = ids >= 0
    assert np.array_equal(np_of(out)[ok], full[ids[ok]]) and not np_of(out)[~ok].any()
    assert np.array_equal(np_of(out_ts)[ok], ts_full[ids[ok]]) and not np_of(out_ts)[~ok].any()
    # the oracle on a numpy copy of the same records
    o_rec = rec.numpy().copy()
    o_data = o_rec.view(np.float32)[:, :dim]
    o_ts = o_rec.view(np.int64)[:, (dim * 4 + 7) // 8]
    oh, oth = h.copy(), ts_hot_np.copy()
    oc = oracle.cache(dim * 4, oh, rows=rows, cold=o_data, hot_slot=slot, ts_hot=oth, ts_cold=o_ts)
    o_out, o_out_ts = np.empty((N, dim), np.float32), np.empty(N, np.int64)
    oracle.gather(oc, ids, o_out, out_ts=o_out_ts)
    assert np.array_equal(np_of(out), o_out) and np.array_equal(np_of(out_ts), o_out_ts)
    # rows and times written back in place
    upd = rng.permutation(rows)[:2000].astype(np.int64)
    vals = rng.standard_normal((2000, dim)).astype(np.float32)
    new_ts = rng.integers(10**9, 2 * 10**9, 2000).astype(np.int64)
    hot.scatter_update(cache, t_hot, data, t_ts_hot, ts, to_dev(hot, upd), to_dev(hot, vals, "f32"), to_dev(hot, new_ts))
    torch.cuda.synchronize()
    oracle.scatter_update(oc, oh, o_data, oth, o_ts, upd, vals, new_ts)
    assert np.array_equal(rec.numpy(), o_rec) and np.array_equal(np_of(t_hot), oh) and np.array_equal(np_of(t_ts_hot), oth)
    if dim % 4 == 0:        # a strided segment beside a packed one in one launch
        out2 = torch.empty((N, dim), dtype=torch.float32, device=hot.be.device)
        out_ts2 = hot.be.empty(N)
        other = torch.from_numpy(full).to(hot.be.device)
        out3 = torch.empty((N, dim), dtype=torch.float32, device=hot.be.device)
        ids_d = to_dev(hot, np.where(ids < 0, 0, ids))
        hot.gather_multi(hot.gather_plan([(cache, ids_d, out2, out_ts2, None), (hot.cache(dim * 4, other), ids_d, out3, None, None)]))
        full[upd], ts_full[upd] = vals, new_ts
        idc = np.where(ids < 0, 0, ids)
        assert np.array_equal(np_of(out2), full[idc]) and np.array_equal(np_of(out_ts2), ts_full[idc])


def test_gather_multi_equals_single_gathers(oracle, hot):
    """three segments (tiered 400 B rows with timestamps and a device-side count, all-HBM 688 B
    rows, all-HBM 256 B rows) in one launch == three sgl_gather calls, byte for byte."""
    rng = np.random.default_rng(11)
    rows = 6000
    full, h, c, slot = _tables(rows, 100, np.float32, 0.3, 1)
    ts_full = rng.integers(0, 10**9, rows).astype(np.int64)
    ts_hot = np.zeros(h.shape[0], np.int64); ts_hot[slot[slot >= 0]] = ts_full[slot >= 0]
    c0, keep0 = _dev_cache(hot, full, h, c, slot, ts_hot=to_dev(hot, ts_hot), ts_cold=torch.from_numpy(ts_full).pin_memory())
    t1 = rng.standard_normal((9000, 172)).astype(np.float32)
    t2 = rng.integers(0, 2**16, (3000, 128), dtype=np.uint16)
    d1, d2 = torch.from_numpy(t1).cuda(), torch.from_numpy(t2).cuda()
    c1, c2 = hot.cache(688, d1), hot.cache(256, d2)
    ids = [rng.integers(-1, rows + 1, 20_000).astype(np.int64), rng.integers(0, 9000, 50_000).astype(np.int64),
           rng.integers(0, 3000, 7).astype(np.int64)]
    d_ids = [to_dev(hot, x) for x in ids]
    live0 = to_dev(hot, np.array([12_345], dtype=np.int64))
    outs = [torch.zeros((20_000, 100), device="cuda"), torch.empty((50_000, 172), device="cuda"),
            torch.empty((7, 128), dtype=torch.uint16, device="cuda")]
    out_ts = hot.be.zeros(20_000)
    plan = hot.gather_plan([(c0, d_ids[0], outs[0], out_ts, live0), (c1, d_ids[1], outs[1], None, None),
                            (c2, d_ids[2], outs[2], None, None)])
    hot.gather_multi(plan)
    ref0, ref_ts = torch.zeros((20_000, 100), device="cuda"), hot.be.zeros(20_000)
    hot.gather(c0, d_ids[0], ref0, out_ts=ref_ts, N_dev=live0)
    assert torch.equal(outs[0], ref0) and torch.equal(out_ts, ref_ts) and not np_of(outs[0])[12_345:].any()
    ok = (ids[0][:12_345] >= 0) & (ids[0][:12_345] < rows)
    assert np.array_equal(np_of(outs[0])[:12_345][ok], full[ids[0][:12_345][ok]])
    assert np.array_equal(np_of(out_ts)[:12_345][ok], ts_full[ids[0][:12_345][ok]])
    assert np.array_equal(np_of(outs[1]), t1[ids[1]]) and np.array_equal(np_of(outs[2]), t2[ids[2]])
    # rows that are not a multiple of 16 bytes are refused (the single-gather entry point takes them)
    c3 = hot.cache(12, torch.zeros((10, 3), device="cuda"))
    bad = hot.gather_plan([(c3, d_ids[2], torch.zeros((7, 3), device="cuda"), None, None)])
    with pytest.raises(RuntimeError):
        hot.gather_multi(bad)


def test_gather_multi_large_output(hot):
    """Outputs of 64 MB and more take the multi gather's streaming-store path: same bytes as
    torch.index_select, a device-side count still bounds a segment, and the rows are visible to a
    kernel that reads them right after on the same stream."""
    g = torch.Generator(device="cuda").manual_seed(5)
    t_edge = torch.randn((200_000, 172), device="cuda", generator=g)
    t_node = torch.randn((50_000, 100), device="cuda", generator=g)
    ids_e = torch.randint(0, 200_000, (120_000,), device="cuda", generator=g)      # 120 000 x 688 B = 82.6 MB
    ids_n = torch.randint(0, 50_000, (30_000,), device="cuda", generator=g)
    live_n = torch.tensor([17_003], dtype=torch.int64, device="cuda")
    out_e = torch.empty((120_000, 172), device="cuda")
    out_n = torch.zeros((30_000, 100), device="cuda")
    plan = hot.gather_plan([(hot.cache(400, t_node), ids_n, out_n, None, live_n),
                            (hot.cache(688, t_edge), ids_e, out_e, None, None)])
    for _ in range(2):      # the second launch overwrites rows that the first one streamed out
        hot.gather_multi(plan)
        total = out_e.sum(dtype=torch.float64) + out_n.sum(dtype=torch.float64)       # reads the rows right away
        assert torch.equal(out_e, t_edge.index_select(0, ids_e))
        assert torch.equal(out_n[:17_003], t_node.index_select(0, ids_n[:17_003])) and not out_n[17_003:].any()
        want = t_edge.index_select(0, ids_e).sum(dtype=torch.float64) + t_node.index_select(0, ids_n[:17_003]).sum(dtype=torch.float64)
        assert float(total) == float(want)
        ids_e = ids_e.flip(0).contiguous()
        plan = hot.gather_plan([(hot.cache(400, t_node), ids_n, out_n, None, live_n),
                                (hot.cache(688, t_edge), ids_e, out_e, None, None)])


@pytest.mark.parametrize("dim,dtype,hot_frac,dup", [(128, np.uint16, 0.1, 8), (100, np.float32, 0.3, 3), (172, np.float32, 0.0, 20),
                                                    (128, np.uint16, 1.0, 4), (4, np.float32, 0.5, 2)])
def test_gather_dedup_matches_numpy(oracle, hot, dim, dtype, hot_frac, dup):
    """The gather that fetches every distinct cold row once: same rows, times and (first three) statistics as the
    plain gather, the fourth statistic = np.unique of the cold requests' rows; with a staging buffer that holds all
    distinct cold rows, one that holds a part of them, and none at all; live count on the device; absent ids."""
    rows, N = 30_000, 60_000
    full, h, c, slot = _tables(rows, dim, dtype, hot_frac, dim + dup)
    rng = np.random.default_rng(dup)
    ids = rng.integers(0, rows // dup, N).astype(np.int64) * dup          # every row asked for ~dup times
    ids[::53] = -1
    ids[::59] = rows + 7
    ts_full = rng.integers(0, 10**9, rows).astype(np.int64)
    ts_hot = np.zeros(max(h.shape[0], 1), dtype=np.int64)
    ts_hot[slot[slot >= 0]] = ts_full[slot >= 0]
    cache, keep = _dev_cache(hot, full, h, c, slot, ts_hot=to_dev(hot, ts_hot), ts_cold=torch.from_numpy(ts_full).pin_memory())
    ok = (ids >= 0) & (ids < rows)
    want = np.zeros((N, dim), dtype=full.dtype)
    want[ok] = full[ids[ok]]
    want_ts = np.zeros(N, dtype=np.int64)
    want_ts[ok] = ts_full[ids[ok]]
    cold_req = ok & (slot[np.clip(ids, 0, rows - 1)] < 0)
    distinct = int(np.unique(ids[cold_req]).size)
    tdt = torch.from_numpy(full[:1]).dtype
    for stage_rows, live in ((distinct + 5, N), (max(distinct // 3, 1), N), (0, N), (distinct + 5, N // 2)):
        out = torch.full((N, dim), 7, dtype=tdt, device=hot.be.device)
        out_ts = hot.be.zeros(N)
        stats = hot.be.zeros(4)
        staging = torch.empty((stage_rows, dim), dtype=tdt, device=hot.be.device) if stage_rows else None
        staging_ts = hot.be.empty(stage_rows) if stage_rows else None
        n_dev = to_dev(hot, np.array([live], dtype=np.int64))
        hot.gather_dedup(cache, to_dev(hot, ids), out, staging, out_ts=out_ts, staging_ts=staging_ts, stats=stats, N_dev=n_dev)
        assert np.array_equal(np_of(out)[:live].view(np.uint8), want[:live].view(np.uint8)), (stage_rows, live)
        assert np.array_equal(np_of(out_ts)[:live], want_ts[:live])
        assert (np_of(out)[live:] == 7).all()        # rows beyond the live count stay untouched
        n_hot = int((ok & ~cold_req)[:live].sum())
        assert np_of(stats).tolist() == [n_hot, int(cold_req[:live].sum()), int((~ok)[:live].sum()),
                                         int(np.unique(ids[:live][cold_req[:live]]).size)]
    # the oracle's fourth statistic is pinned by np.unique as well
    oc = oracle.cache(full.shape[1] * full.dtype.itemsize, h, rows=rows, cold=c, hot_slot=slot)
    o_out, o_stats = np.empty((N, dim), dtype=full.dtype), np.zeros(4, dtype=np.int64)
    oracle.gather_dedup(oc, ids, o_out, None, stats=o_stats)
    assert np.array_equal(o_out.view(np.uint8), want.view(np.uint8)) and o_stats[3] == distinct


def test_column_views_of_wider_rows_in_both_tiers(oracle, hot):
    """One record per node in either tier - memory | features (| time, host tier) - gathered whole through one
    cache, and its memory half read and updated through a second cache that is a column view of the same storage
    (row strides travel in sgl_cache: hot_stride, cold_stride, ts_cold_stride).  Against numpy and the oracle."""
    rows, N = 6000, 20_000
    rng = np.random.default_rng(12)
    mem, nf = rng.standard_normal((rows, 100)).astype(np.float32), rng.standard_normal((rows, 100)).astype(np.float32)
    ts_full = rng.integers(0, 10**9, rows).astype(np.int64)
    hot_ids = rng.permutation(rows)[: rows * 7 // 10]
    slot = np.full(rows, -1, np.int32); slot[hot_ids] = np.arange(hot_ids.size, dtype=np.int32)
    dev = hot.be.device
    node_hot = torch.from_numpy(np.concatenate([mem[hot_ids], nf[hot_ids]], axis=1)).to(dev)
    ts_hot = to_dev(hot, ts_full[hot_ids])
    node_cold, ts_cold, rec = hot.interleaved_cold(rows, 200)
    assert rec.shape[1] == 896                              # 800 bytes of rows + 8 of time in seven 128-byte lines
    node_cold.copy_(torch.from_numpy(np.concatenate([mem, nf], axis=1))); ts_cold.copy_(torch.from_numpy(ts_full))
    d_slot = to_dev(hot, slot, "i32")
    c_node = hot.cache(800, node_hot, rows=rows, cold=node_cold, hot_slot=d_slot, ts_hot=ts_hot, ts_cold=ts_cold)
    c_mem = hot.cache(400, node_hot[:, :100], rows=rows, cold=node_cold[:, :100], hot_slot=d_slot, ts_hot=ts_hot, ts_cold=ts_cold)
    c_nf = hot.cache(400, node_hot[:, 100:], rows=rows, cold=node_cold[:, 100:], hot_slot=d_slot)
    assert c_mem.hot_stride == 800 and c_mem.cold_stride == 896 and c_node.hot_stride == 0
    ids = rng.integers(0, rows, N).astype(np.int64)
    d_ids = to_dev(hot, ids)
    out, out_ts = torch.empty((N, 200), device=dev), hot.be.empty(N)
    hot.gather(c_node, d_ids, out, out_ts=out_ts)
    assert np.array_equal(np_of(out), np.concatenate([mem[ids], nf[ids]], axis=1)) and np.array_equal(np_of(out_ts), ts_full[ids])
    o_m, o_f = torch.empty((N, 100), device=dev), torch.empty((N, 100), device=dev)
    hot.gather_multi(hot.gather_plan([(c_mem, d_ids, o_m, out_ts, None), (c_nf, d_ids, o_f, None, None)]))
    assert np.array_equal(np_of(o_m), mem[ids]) and np.array_equal(np_of(o_f), nf[ids]) and np.array_equal(np_of(out_ts), ts_full[ids])
    # memory update through the view: the feature half and the rows of other nodes stay as they are
    upd = np.unique(rng.integers(0, rows, 900)).astype(np.int64)
    vals, new_ts = rng.standard_normal((upd.size, 100)).astype(np.float32), rng.integers(0, 10**9, upd.size).astype(np.int64)
    hot.scatter_update(c_mem, node_hot[:, :100], node_cold[:, :100], ts_hot, ts_cold, to_dev(hot, upd), to_dev(hot, vals, "f32"), to_dev(hot, new_ts))
    mem2, ts2 = mem.copy(), ts_full.copy()
    mem2[upd], ts2[upd] = vals, new_ts
    hot.gather(c_node, d_ids, out, out_ts=out_ts)
    assert np.array_equal(np_of(out), np.concatenate([mem2[ids], nf[ids]], axis=1)) and np.array_equal(np_of(out_ts), ts2[ids])
    # the oracle reads the same views on the host
    oc = oracle.cache(400, np_of(node_hot)[:, :100], rows=rows, cold=node_cold.numpy()[:, :100], hot_slot=slot)
    o_out = np.empty((N, 100), dtype=np.float32)
    oracle.gather(oc, ids, o_out)
    assert np.array_equal(o_out, mem2[ids])
