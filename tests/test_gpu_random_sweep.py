"""GPU: seeded sweeps of random shapes through every stage (T-CSR build, k-hop sampling of both
kinds and both in one call, unique in both modes over the dense table and the hash set, seed extraction,
slicing, pair unique) against the CPU oracle, bit-exact.  The parametrised tests pin chosen edge cases;
this one walks the combinations nobody chose."""
import numpy as np
import pytest

from starrygl_amd.lib import _abi
from util import assert_hop_equal, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


def _one_case(seed, oracle, hot):
    rng = np.random.default_rng(seed)
    n = int(rng.choice([1, 2, 17, 300, 5000, 60000]))
    m = int(rng.choice([0, 1, 50, 4000, 100000, 400000]))
    t_max = int(rng.choice([1, 10, 1000, 10**6, 2**40]))
    if m > 0:
        src = rng.integers(0, n, m)
        dst = rng.integers(0, n, m)
        if rng.random() < 0.5 and n > 2: src[rng.random(m) < 0.4] = n // 2
        ts = rng.integers(0, t_max, m)
        eid = rng.permutation(m)
    else:
        src = dst = ts = eid = np.zeros(0, np.int64)
    src, dst, ts, eid = (np.ascontiguousarray(x, dtype=np.int64) for x in (src, dst, ts, eid))
    g = host_graph(oracle, n, src, dst, ts, eid)
    # build on the device from shuffled input
    dgb = hot.tcsr_build(n, to_dev(hot, src), to_dev(hot, dst), to_dev(hot, ts), to_dev(hot, eid))
    for f in ("row_ptr", "col", "ts", "eid"):
        assert np.array_equal(np_of(getattr(dgb, f)), getattr(g, f)), ("tcsr_build", f)
    dg = mirror_graph(hot, g)
    if seed % 2:        # every other case samples with the graph's next-hop index attached
        hot.build_hop_hint(dg)
        assert np.array_equal(np_of(dg.hop_hint), oracle.build_hop_hint(g).hop_hint), "hop_hint"
    # sampling
    S_pos = int(rng.choice([0, 1, 5, 200, 3000, 20000]))
    N_neg = int(rng.choice([0, 1, 77, 2000]))
    R = S_pos if rng.random() < 0.6 else max(1, S_pos // 3) if S_pos else 0
    if S_pos and R:
        cuts = np.sort(rng.integers(0, S_pos + 1, R - 1)) if R > 1 else np.zeros(0, np.int64)
        ts_ptr = np.concatenate([[0], cuts, [S_pos]]).astype(np.int64)
    else:
        R, S_pos = 0, 0
        ts_ptr = np.zeros(1, np.int64)
    roots = rng.integers(0, n, R).astype(np.int64)
    root_ts = rng.integers(0, t_max + 2, S_pos).astype(np.int64)
    neg = rng.integers(0, n, N_neg).astype(np.int64)
    neg_ts = rng.integers(0, t_max + 2, N_neg).astype(np.int64)
    layers = int(rng.choice([1, 2, 2, 3]))
    fan = int(rng.choice([1, 2, 5, 10, 16, 17, 33]))
    if (S_pos + N_neg) * fan ** layers > 3_000_000: layers = 1
    kw = dict(sample_type=str(rng.choice(["recent", "uniform"])), fanout=fan, seed=int(rng.integers(0, 2**31)),
              allowed_offset=int(rng.choice([-1, 0, 5, t_max // 2 + 1])), equal_root_time=bool(rng.integers(0, 2)),
              keep_root_time=bool(rng.integers(0, 2)), replace=bool(rng.integers(0, 2)))
    host = (roots, ts_ptr, root_ts, neg, neg_ts)
    dev = [to_dev(hot, x) for x in host]
    want = oracle.sample_khop(g, *host, layers, oracle.params(**kw))
    got = hot.sample_khop(dg, *dev, layers, hot.params(**kw))
    for l in range(layers): assert_hop_equal(got.hops[l], want.hops[l], tag=f"khop l{l} {kw}")
    if layers == 2:
        kw2 = dict(kw)
        kw2["sample_type"] = "uniform" if kw["sample_type"] == "recent" else "recent"
        outs = [hot.khop_buffers(S_pos + N_neg, 2, fan) for _ in range(2)]
        hot.sample_khop_multi(dg, *dev, 2, [hot.params(**kw), hot.params(**kw2)], outs)
        want2 = oracle.sample_khop(g, *host, 2, oracle.params(**kw2))
        for res, w in zip(outs, (want, want2)):
            r = res.finalize()
            for l in range(2): assert_hop_equal(r.hops[l], w.hops[l], tag=f"multi l{l}")
    # unique, both modes, dense and hash
    arrays = [want.slot_node0] + [h.neighbors for h in want.hops]
    for mode in (_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED):
        so, sh = oracle.remap_state(n), hot.remap_state(n)
        for reset in (True, False):
            lo, uo, (to_, bo) = oracle.unique_compact(arrays, mode, so, reset)
            lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrays], mode, sh, reset)
            assert (to_, bo) == (th, bh), ("unique counts", mode, reset)
            assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), ("unique list", mode, reset)
            for a, b in zip(lh, lo): assert np.array_equal(np_of(a), b), ("unique local", mode, reset)
            arrays = [a[::-1].copy() for a in arrays]
    lo, uo, _ = oracle.unique_compact(arrays, _abi.UNIQUE_SORTED)
    lh, uh, _ = hot.unique_compact([to_dev(hot, a) for a in arrays], _abi.UNIQUE_SORTED)
    assert np.array_equal(np_of(uh), uo) and all(np.array_equal(np_of(a), b) for a, b in zip(lh, lo)), "hash unique"
    # seeds + slice
    C = int(rng.choice([1, 3, 8]))
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    cp, cn = oracle.chunk_index(n, C, chunk_of)
    dcp, dcn = hot.chunk_index(n, C, to_dev(hot, chunk_of))
    ch = rng.permutation(C)[: int(rng.integers(0, C + 1))].astype(np.int64)
    off = np.concatenate([[0], np.cumsum(cp[ch + 1] - cp[ch])]).astype(np.int64)
    t0 = int(rng.integers(0, t_max + 1))
    t1 = t0 + int(rng.choice([0, 1, 7, t_max]))
    ws = oracle.seeds(g, cp, cn, ch, off, int(off[-1]), t0, t1, with_window_end=True)
    gs = hot.seeds(dg, dcp, dcn, to_dev(hot, ch), to_dev(hot, off), int(off[-1]), t0, t1, with_window_end=True)
    for f, a, b in zip(("roots", "ts_ptr", "ts", "q_ptr", "q_eid", "window_end"), gs, ws): assert np.array_equal(np_of(a), b), ("seeds", f)
    if t1 - t0 <= 1000:
        full = bool(rng.integers(0, 2))
        wsl = oracle.slice(g, cp, cn, chunk_of, ch, off, int(off[-1]), t0, t1, full)
        gsl = hot.slice(dg, dcp, dcn, to_dev(hot, chunk_of), to_dev(hot, ch), to_dev(hot, off), int(off[-1]), t0, t1, full)
        for i, (a, b) in enumerate(zip(gsl, wsl)): assert np.array_equal(np_of(a), b), ("slice", i)
    # pairs
    k = int(rng.choice([0, 1, 100, 30000]))
    ids = rng.integers(-5, max(n, 2), k).astype(np.int64)
    pts = rng.integers(0, min(t_max, 2**40) + 1, k).astype(np.int64)
    wu = oracle.unique_pairs(ids, pts)
    gu = hot.unique_pairs(to_dev(hot, ids), to_dev(hot, pts))
    for a, b in zip(gu, wu): assert np.array_equal(np_of(a), b), "unique_pairs"

@pytest.mark.parametrize("first", [0, 60, 120, 180])
def test_random_shapes_match_the_oracle(oracle, hot, first):
    for seed in range(first, first + 60):
        try:
            _one_case(seed, oracle, hot)
        except AssertionError as exc:
            raise AssertionError(f"seed {seed}: {exc}") from exc


# ---- two-tier gather and multi-segment gather against numpy

def _random_table(rng, hot):
    import torch
    dev = hot.be.device
    rows = int(rng.choice([1, 2, 33, 1000, 20_000]))
    dim = int(rng.choice([1, 2, 3, 4, 6, 16, 100, 172, 64, 500]))
    frac = float(rng.choice([0.0, 0.1, 0.5, 1.0]))
    full = rng.standard_normal((rows, dim)).astype(np.float32)
    ts_full = rng.integers(0, 10**9, rows).astype(np.int64)
    hot_rows = int(rows * frac)
    hot_ids = rng.permutation(rows)[:hot_rows]
    slot = np.full(rows, -1, np.int32)
    slot[hot_ids] = np.arange(hot_rows, dtype=np.int32)
    cold, tsc = full.copy(), ts_full.copy()
    cold[hot_ids] = 0          # a hot row must never be served from the cold tier
    tsc[hot_ids] = 0
    G = rows * 3 + 5
    g2l = None
    if rng.random() < 0.4:     # global id -> local row through a dense map
        g2l = np.full(G + 1, -1, np.int64)
        g2l[rng.permutation(G)[:rows]] = np.arange(rows)
    t_hot = torch.from_numpy(full[hot_ids].copy()).to(dev) if hot_rows else None
    if rng.random() < 0.4:     # row and time side by side in one pinned record
        t_cold, t_tsc, _ = hot.interleaved_cold(rows, dim)
        t_cold.copy_(torch.from_numpy(cold))
        t_tsc.copy_(torch.from_numpy(tsc))
    else:
        t_cold, t_tsc = torch.from_numpy(cold).pin_memory(), torch.from_numpy(tsc).pin_memory()
    kw = {}
    if frac < 1.0 or rng.random() < 0.5:
        kw.update(cold=t_cold, hot_slot=to_dev(hot, slot, "i32"), ts_cold=t_tsc)
        if t_hot is not None:
            kw.update(ts_hot=to_dev(hot, ts_full[hot_ids].copy()))
    else:                      # one HBM table in row order, no index
        t_hot = torch.from_numpy(full).to(dev)
        kw.update(ts_hot=to_dev(hot, ts_full))
    if g2l is not None:
        kw.update(g2l=to_dev(hot, g2l))
    return dict(rows=rows, dim=dim, full=full, ts=ts_full, g2l=g2l, G=G, cache=hot.cache(dim * 4, t_hot, rows=rows, **kw),
                t_hot=t_hot, t_cold=kw.get("cold"), t_ts_hot=kw.get("ts_hot"), t_ts_cold=kw.get("ts_cold"))


def _one_gather_case(seed, hot):
    import torch
    rng = np.random.default_rng(seed)
    dev = hot.be.device
    tabs = [_random_table(rng, hot) for _ in range(int(rng.integers(1, 4)))]
    segs, wants = [], []
    for T in tabs:
        n = int(rng.choice([0, 1, 7, 300, 5000, 40_000]))
        hi = T["G"] + 1 if T["g2l"] is not None else T["rows"]
        ids = rng.integers(0, hi, n).astype(np.int64)
        if n > 3:
            ids[rng.integers(0, n, max(1, n // 50))] = -7
            ids[rng.integers(0, n, max(1, n // 50))] = hi + 11
        ok = (ids >= 0) & (ids < hi)
        loc = np.where(ok, T["g2l"][np.clip(ids, 0, hi - 1)] if T["g2l"] is not None else ids, -1)
        good = loc >= 0
        w_rows = np.where(good[:, None], T["full"][np.clip(loc, 0, T["rows"] - 1)], 0).astype(np.float32)
        w_ts = np.where(good, T["ts"][np.clip(loc, 0, T["rows"] - 1)], 0)
        live = None if rng.random() < 0.5 or n == 0 else int(rng.integers(0, n + 1))
        out = torch.zeros((max(n, 1), T["dim"]), dtype=torch.float32, device=dev)[:n]
        out_ts = hot.be.zeros(max(n, 1))[:n] if rng.random() < 0.5 else None
        n_dev = None if live is None else to_dev(hot, np.array([live], dtype=np.int64))
        segs.append((T["cache"], to_dev(hot, ids), out, out_ts, n_dev))
        wants.append((w_rows, w_ts, n if live is None else live))
    live_segs = [s for s in segs if s[2].shape[0]]
    if rng.random() < 0.5 and live_segs and all(T["dim"] % 4 == 0 for T in tabs):
        hot.gather_multi(hot.gather_plan(live_segs))
    else:
        for c, ids, out, ots, nd in live_segs:
            hot.gather(c, ids, out, out_ts=ots, N_dev=nd)
    for (c, ids, out, ots, nd), (w_rows, w_ts, m) in zip(segs, wants):
        g = np_of(out)
        assert np.array_equal(g[:m].view(np.uint32), w_rows[:m].view(np.uint32)) and not g[m:].any(), f"seed {seed}: rows"
        if ots is not None:
            gt = np_of(ots)
            assert np.array_equal(gt[:m], w_ts[:m]) and not gt[m:].any(), f"seed {seed}: times"


def _one_update_case(seed, hot):
    """scatter_update of distinct rows (some ids absent) into both tiers, read back through the gather"""
    import torch
    rng = np.random.default_rng(seed)
    T = _random_table(rng, hot)
    if T["t_ts_hot"] is None and T["t_hot"] is not None:
        return
    rows, dim = T["rows"], T["dim"]
    hi = T["G"] + 1 if T["g2l"] is not None else rows
    n = int(rng.integers(0, min(rows, 3000) + 1))
    loc = rng.permutation(rows)[:n].astype(np.int64)                   # distinct local rows
    ids = np.nonzero(np.isin(T["g2l"], loc))[0].astype(np.int64) if T["g2l"] is not None else loc.copy()
    if T["g2l"] is not None:
        loc = T["g2l"][ids]
    ids_w = ids.copy()
    if n > 5:
        ids_w[::17] = -3                                               # skipped
    vals = rng.standard_normal((n, dim)).astype(np.float32)
    new_ts = rng.integers(1, 10**9, n).astype(np.int64)
    hot.scatter_update(T["cache"], T["t_hot"], T["t_cold"], T["t_ts_hot"], T["t_ts_cold"], to_dev(hot, ids_w),
                       to_dev(hot, vals, "f32"), to_dev(hot, new_ts))
    want, want_ts = T["full"].copy(), T["ts"].copy()
    keep = ids_w >= 0
    want[loc[keep]] = vals[keep]
    want_ts[loc[keep]] = new_ts[keep]
    probe = rng.integers(0, hi, 4000).astype(np.int64)
    ploc = T["g2l"][probe] if T["g2l"] is not None else probe
    good = ploc >= 0
    out = torch.zeros((4000, dim), dtype=torch.float32, device=hot.be.device)
    out_ts = hot.be.zeros(4000)
    hot.gather(T["cache"], to_dev(hot, probe), out, out_ts=out_ts)
    w_rows = np.where(good[:, None], want[np.clip(ploc, 0, rows - 1)], 0).astype(np.float32)
    assert np.array_equal(np_of(out).view(np.uint32), w_rows.view(np.uint32)), f"seed {seed}: rows after the update"
    assert np.array_equal(np_of(out_ts), np.where(good, want_ts[np.clip(ploc, 0, rows - 1)], 0)), f"seed {seed}: times"


def test_random_updates_read_back(hot):
    for seed in range(120):
        _one_update_case(12000 + seed, hot)


@pytest.mark.parametrize("first", [0, 150])
def test_random_gathers_match_numpy(hot, first):
    """random tables (tiers, index, interleaved cold records, row widths), id lists with absent ids and
    device-side live counts, one launch per table or one for all"""
    for seed in range(first, first + 150):
        _one_gather_case(9000 + seed, hot)


# ---- sequences of calls on a hashed remap state, up to and past its capacity

@pytest.mark.parametrize("first", [0, 200])
def test_random_sequences_on_a_hashed_state(oracle, hot, first):
    """every call of a sequence equals the oracle's; when a sequence outgrows the state, both sides say so"""
    for seq in range(first, first + 200):
        rng = np.random.default_rng(7000 + seq)
        cap = int(rng.choice([1, 7, 300, 5000, 70_000, 400_000]))
        mode = int(rng.choice([_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED]))
        kind = str(rng.choice(["dense", "wide", "encoded", "squares", "neg"]))

        def draw(n):
            if kind == "dense": return rng.integers(0, max(2, cap // 2), n)
            if kind == "wide": return rng.integers(0, 2**62, n)
            if kind == "encoded": return (rng.integers(0, 8, n) << 48) | rng.integers(0, max(2, cap), n)
            if kind == "squares": return rng.integers(0, 50_000, n) ** 2 + (1 << 40)
            x = rng.integers(0, max(2, cap), n)
            x[rng.random(n) < 0.2] = -rng.integers(1, 100)
            return x

        so, sh = oracle.remap_hashed_state(cap), hot.remap_hashed_state(cap)
        for c in range(int(rng.integers(1, 7))):
            G = int(rng.integers(1, 4))
            arrs = [draw(int(rng.choice([0, 1, 5, 300, 4000, 60_000, 9000]))).astype(np.int64) for _ in range(G)]
            reset = bool(rng.random() < 0.4) or c == 0
            try:
                lo, uo, (to_, bo) = oracle.unique_compact([a.copy() for a in arrs], mode, so, reset)
            except RuntimeError:
                lo = None
            try:
                lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, sh, reset)
            except RuntimeError:
                lh = None
            assert (lo is None) == (lh is None), f"sequence {seq} call {c}: only one side reports the outgrown state"
            if lo is None:
                break          # both states are void
            assert (th, bh) == (to_, bo), f"sequence {seq} call {c}"
            assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), f"sequence {seq} call {c}: unique list"
            for g in range(G):
                assert np.array_equal(np_of(lh[g]), lo[g]), f"sequence {seq} call {c} array {g}"


def test_random_sequences_on_a_dense_state(oracle, hot):
    """'r' / 'f' sequences on the dense remap state, ids outside the universe among them"""
    for seq in range(150):
        rng = np.random.default_rng(8000 + seq)
        universe = int(rng.choice([1, 9, 700, 50_000, 3_000_000]))
        mode = int(rng.choice([_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED]))
        so, sh = oracle.remap_state(universe), hot.remap_state(universe)
        for c in range(int(rng.integers(1, 6))):
            G = int(rng.integers(1, 4))
            arrs = []
            for _ in range(G):
                n = int(rng.choice([0, 1, 5, 300, 4000, 60_000]))
                a = rng.integers(0, universe, n).astype(np.int64)
                if n > 4:
                    a[1] = -4
                    a[3] = universe + 2
                arrs.append(a)
            reset = bool(rng.random() < 0.4) or c == 0
            lo, uo, (to_, bo) = oracle.unique_compact([a.copy() for a in arrs], mode, so, reset)
            lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, sh, reset)
            assert (th, bh) == (to_, bo), f"sequence {seq} call {c}"
            assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), f"sequence {seq} call {c}: unique list"
            for g in range(G):
                assert np.array_equal(np_of(lh[g]), lo[g]), f"sequence {seq} call {c} array {g}"


# ---- time encoding over random widths, sizes and live counts

def test_random_time_encodings(oracle, hot):
    for it in range(250):
        rng = np.random.default_rng(5000 + it)
        dim = int(rng.choice([1, 3, 4, 8, 12, 100, 128, 172, 256, 1020, 1024, 1028, int(rng.integers(1, 1100))]))
        N = int(rng.choice([0, 1, 9, 10, 11, 255, 257, 4096, 5121, 40000, int(rng.integers(0, 60000))]))
        N = min(N, 20_000_000 // dim)
        span = int(rng.choice([50, 10**7, 2**40, 2**62]))
        dt = rng.integers(-span, span, N).astype(np.int64)
        w = (1.0 / 10 ** np.linspace(0, 9, dim, dtype=np.float32)).astype(np.float32)
        if rng.random() < 0.3:
            w = rng.standard_normal(dim).astype(np.float32)
        b = rng.standard_normal(dim).astype(np.float32)
        live = None if rng.random() < 0.5 or N == 0 else int(rng.integers(0, N + 1))
        out = hot.be.zeros((max(N, 1), dim), "f32")[:N]
        n_dev = None if live is None else to_dev(hot, np.array([live], dtype=np.int64))
        if rng.random() < 0.3:
            x = dt.astype(np.float32)
            want = oracle.time_encode(x, w, b, dt_dtype=_abi.DT_F32)
            hot.time_encode(to_dev(hot, x, "f32"), to_dev(hot, w, "f32"), to_dev(hot, b, "f32"), dt_dtype=_abi.DT_F32,
                            out=out, N_dev=n_dev)
        else:
            want = oracle.time_encode(dt, w, b)
            hot.time_encode(to_dev(hot, dt), to_dev(hot, w, "f32"), to_dev(hot, b, "f32"), out=out, N_dev=n_dev)
        got = np_of(out)
        n = N if live is None else live
        if n:
            assert np.abs(got[:n].astype(np.float64) - want[:n]).max() <= 1.2e-7, f"case {it}: dim {dim} N {N}"
        assert not got[n:].any(), f"case {it}: rows beyond the live count were written"
