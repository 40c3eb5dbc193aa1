"""GPU parity of the batched calls (B mini-batches per launch sequence) through the C ABI against the CPU oracle,
bit-exact: sgl_sample_khop_batched (both strategies, every output array and the segment table) and
sgl_unique_compact_batched (per-batch local ids, unique lists and their offsets)."""
import numpy as np
import pytest
import torch

from starrygl_amd.utils import synth
from util import assert_hop_equal, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


def concat_slots(batches):
    node = [np.concatenate([b[0], b[3]]) for b in batches]
    t = [np.concatenate([b[2], b[4]]) for b in batches]
    ptr = np.concatenate([[0], np.cumsum([x.size for x in node])]).astype(np.int64)
    return np.concatenate(node).astype(np.int64), np.concatenate(t).astype(np.int64), ptr


def run_both(oracle, hot, g, dg, node, t, ptr, layers, kws, hint=None):
    want = oracle.sample_khop_batched(g, node, t, ptr, layers, [oracle.params(**kw) for kw in kws],
                                      slot_hint=hint, finalize=True)
    got = hot.sample_khop_batched(dg, to_dev(hot, node), to_dev(hot, t), to_dev(hot, ptr), layers,
                                  [hot.params(**kw) for kw in kws],
                                  slot_hint=None if hint is None else to_dev(hot, hint), finalize=True)
    assert np.array_equal(np.asarray(got.seg_host), np.asarray(want.seg_host))
    for q, kw in enumerate(kws):
        for l in range(layers):
            assert_hop_equal(got.queries[q].hops[l], want.queries[q].hops[l], tag=f"query {q} hop {l} {kw}")
    return got, want


@pytest.fixture(scope="module")
def small(oracle, hot):
    n = 4000
    src, dst, ts, eid = synth.graph_stream(n, 120_000, 1.2, 900_000, 21)
    g = host_graph(oracle, n, src, dst, ts, eid)
    dg = mirror_graph(hot, g)
    return (src, dst, ts), g, dg


@pytest.mark.parametrize("with_index", [False, True])
@pytest.mark.parametrize("sizes", [[300, 300, 300, 300], [0, 512, 1, 0, 77, 900], [40], [0, 0], [2000] * 16])
def test_batched_sampler_parity(oracle, hot, small, sizes, with_index):
    (src, dst, ts), g, dg = small
    if with_index:
        dg = mirror_graph(hot, g)
        hot.build_hop_hint(dg)
    rng = np.random.default_rng(len(sizes) * 7 + sum(sizes))
    batches = []
    for sz in sizes:
        lo = int(rng.integers(0, src.size - max(sz, 1)))
        batches.append(synth.link_batch(src, dst, ts, lo, lo + sz, g.n, sz // 2, rng))
    node, t, ptr = concat_slots(batches)
    hint = oracle.window_end(g, node, t)
    hint[rng.random(hint.size) < 0.4] = -1
    kws = [dict(sample_type="recent", fanout=6), dict(sample_type="uniform", fanout=6, seed=5)]
    run_both(oracle, hot, g, dg, node, t, ptr, 2, kws, hint=hint if with_index else None)


@pytest.mark.parametrize("kw", [dict(allowed_offset=5000), dict(equal_root_time=True), dict(keep_root_time=True),
                                dict(replace=True), dict(allowed_offset=0)])
@pytest.mark.parametrize("layers", [1, 3])
def test_batched_sampler_window_flags(oracle, hot, small, kw, layers):
    (src, dst, ts), g, _ = small
    dg = mirror_graph(hot, g)
    hot.build_hop_hint(dg)
    rng = np.random.default_rng(3)
    batches = [synth.link_batch(src, dst, ts, lo, lo + 150, g.n, 60, rng) for lo in (100, 50_000, 119_000)]
    node, t, ptr = concat_slots(batches)
    node[5] = g.n + 3                        # a slot outside [0, n): sampled as empty and counted
    hint = oracle.window_end(g, node, t)
    kws = [dict(sample_type=st, fanout=4, seed=9, **kw) for st in ("uniform", "recent")]
    with pytest.raises(IndexError):
        hot.sample_khop_batched(dg, to_dev(hot, node), to_dev(hot, t), to_dev(hot, ptr), layers,
                                [hot.params(**k_) for k_ in kws], slot_hint=to_dev(hot, hint), finalize=True)
    node[5] = 7
    hint = oracle.window_end(g, node, t)
    run_both(oracle, hot, g, dg, node, t, ptr, layers, kws, hint=hint)


@pytest.mark.parametrize("case", range(6))
def test_batched_pair_side_by_side_sweep(oracle, hot, small, case):
    """Calls of 131072 slots and more take the lane-per-slot kernels, and a most-recent query followed by a uniform
    one with the same fanout runs its kernels of a hop side by side in one launch: random batch sizes (empty ones
    among them), hops, fanouts (16-lane and 32-lane groups), window rules, hints and index on or off."""
    (src, dst, ts), g, _ = small
    rng = np.random.default_rng(900 + case)
    dg = mirror_graph(hot, g)
    with_index = bool(case & 1)
    if with_index:
        hot.build_hop_hint(dg)
    if case & 2:
        hot.build_records(dg)
    B = int(rng.integers(1, 12))
    sizes = rng.multinomial(140_000 + int(rng.integers(0, 20_000)), rng.dirichlet(np.ones(B))).astype(np.int64)
    if B > 2:
        sizes[int(rng.integers(0, B))] = 0
    node = rng.integers(0, g.n, int(sizes.sum())).astype(np.int64)
    t = rng.integers(0, int(ts.max()) + 2, node.size).astype(np.int64)
    ptr = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    hint = oracle.window_end(g, node, t)
    hint[rng.random(hint.size) < 0.5] = -1
    layers = [2, 1, 3, 2, 2, 2][case]
    fan = [5, 10, 3, 20, 7, 16][case]
    extra = [dict(), dict(allowed_offset=40_000), dict(), dict(), dict(keep_root_time=True), dict(replace=True)][case]
    kws = [dict(sample_type="recent", fanout=fan, **{k: v for k, v in extra.items() if k == "allowed_offset"}),
           dict(sample_type="uniform", fanout=fan, seed=11 + case, **extra)]
    if case == 4:           # a pair whose fanouts differ runs its hops one after the other
        kws[0]["fanout"] = 4
    run_both(oracle, hot, g, dg, node, t, ptr, layers, kws, hint=hint if with_index else None)


def test_batched_sampler_refuses_marking_and_bad_sizes(hot, small):
    _, g, dg = small
    node, t = to_dev(hot, np.arange(10)), to_dev(hot, np.arange(10))
    ptr = to_dev(hot, np.array([0, 10]))
    p = hot.marking(hot.params("recent", 3), hot.remap_state(g.n))
    with pytest.raises(ValueError):
        hot.sample_khop_batched(dg, node, t, ptr, 2, [p])
    with pytest.raises(ValueError):
        hot.sample_khop_batched(dg, node, t[:5], ptr, 2, [hot.params("recent", 3)])


@pytest.mark.parametrize("universe,B", [(5000, 6), (16384, 4), (16385, 3), (1_000_000, 16), (3_000_000, 8), (70_000, 64), (9_000_000, 8),
                                        (2000, 1), (50_000, 7), (300, 9), (40_000, 33)])
def test_batched_unique_parity(oracle, hot, universe, B):
    """universes below, at and above one tile of 16384 ids; states of up to 64M ids in all keep a flag byte per id,
    8 x 9M runs on the bitmap; batch counts below, at and above the eight classes of blocks that share the batches out
    (one class per XCD), also ones that do not divide evenly"""
    rng = np.random.default_rng(universe + B)
    hs, ds = oracle.remap_batched_state(universe, B), hot.remap_batched_state(universe, B)
    for trial in range(3):             # consecutive epochs on one state, the last call smaller
        arrays, segs = [], []
        for g in range(3):
            sizes = rng.integers(0, [5000, 3000, 40][trial], B)
            if trial == 1:
                sizes[rng.integers(0, B)] = 0
            seg = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
            a = rng.integers(-2, universe + 3, int(seg[-1]) + 9).astype(np.int64)
            if trial == 0:
                a[: a.size // 2] = rng.zipf(1.3, a.size // 2) % universe           # heavy repeats
            arrays.append(a); segs.append(seg)
        wl, wu, woff = oracle.unique_compact_batched(arrays, segs, hs)
        gl, gu, goff = hot.unique_compact_batched([to_dev(hot, a) for a in arrays], [to_dev(hot, s) for s in segs], ds)
        assert goff == woff, trial
        assert np.array_equal(np_of(gu), wu), trial
        for a, b, s in zip(gl, wl, segs):
            assert np.array_equal(np_of(a)[: s[-1]], b[: s[-1]]), trial


N, M, EV, K = 1_000_000, 20_000_000, 4000, 10


@pytest.fixture(scope="module")
def world(oracle, hot):
    src, dst, ts, eid, row_ptr = synth.graph_by_degree(N, M, 1.1, 1 << 40, 20242)
    hg = oracle.tcsr_from_sorted(N, row_ptr, dst, ts, eid, validate=False)
    dg = hot.tcsr_from_sorted(N, *(to_dev(hot, x) for x in (row_ptr, dst, ts, eid)), validate=True)
    hot.build_hop_hint(dg)
    hot.build_records(dg)
    order = np.argsort(ts, kind="stable")
    yield dict(src=src, dst=dst, ts=ts, hg=hg, dg=dg, order=order)


@pytest.mark.parametrize("B", [4, 16])
def test_configs1_batched_step_parity(oracle, hot, world, B):
    """configs[1] at full size, B batches of 12000 roots per call: both strategies in one library call, the
    segment table, the batched unique over the most-recent query, and the node rows gathered per batch."""
    w, rng = world, np.random.default_rng(B)
    starts = np.sort(rng.integers(M // 2, M - EV, B))
    batches = []
    for s in starts:
        ev = w["order"][s: s + EV]
        batches.append(synth.link_batch(w["src"][ev], w["dst"][ev], w["ts"][ev], 0, EV, N, EV, rng))
    node, t, ptr = concat_slots(batches)
    d_node, d_t, d_ptr = to_dev(hot, node), to_dev(hot, t), to_dev(hot, ptr)
    hint = hot.window_end(w["dg"], d_node, d_t)
    assert np.array_equal(np_of(hint), oracle.window_end(w["hg"], node, t))
    hint_np = np_of(hint).copy()
    for b in range(B):                        # the negatives of a batch carry no hint
        hint_np[ptr[b] + 2 * EV: ptr[b + 1]] = -1
    kws = [dict(sample_type="recent", fanout=K), dict(sample_type="uniform", fanout=K, seed=20242)]
    got, want = run_both(oracle, hot, w["hg"], w["dg"], node, t, ptr, 2, kws, hint=hint_np)
    seg = np.asarray(want.seg_host[0])
    # most recent: every batch's segment is what the oracle samples for that batch alone
    for b in (0, B - 1):
        own = oracle.sample_khop(w["hg"], *batches[b], 2, oracle.params("recent", K))
        for l in range(2):
            lo, hi = seg[l + 1][b], seg[l + 1][b + 1]
            assert np.array_equal(np_of(got.queries[0].hops[l].neighbors_eid)[lo:hi], own.hops[l].neighbors_eid)
    # batched unique over the most-recent query, lengths and offsets read on the device
    kr = got.queries[0]
    arrays = [d_node, kr.hops[0].neighbors, kr.hops[1].neighbors]
    segs = [got.seg[0, 0], got.seg[0, 1], got.seg[0, 2]]
    state = hot.remap_batched_state(N, B)
    local, uniq, off = hot.unique_compact_batched(arrays, [s.contiguous() for s in segs], state)
    wq = want.queries[0]
    ids = [node, wq.hops[0].neighbors, wq.hops[1].neighbors]
    for b in range(B):
        cat = np.concatenate([a[seg[l][b]: seg[l][b + 1]] for l, a in enumerate(ids)])
        u, inv = np.unique(cat, return_inverse=True)
        assert np.array_equal(np_of(uniq[off[b]: off[b + 1]]), u), b
        mine = np.concatenate([np_of(a[seg[l][b]: seg[l][b + 1]]) for l, a in enumerate(local)])
        assert np.array_equal(mine, inv), b
    # node rows of all batches in one gather; a batch's rows are out[off[b]: off[b + 1]]
    g_ = torch.Generator(device="cuda").manual_seed(3)
    feat = torch.randn((N, 100), device="cuda", generator=g_)
    out = torch.empty((off[B], 100), device="cuda")
    hot.gather(hot.cache(400, feat), uniq, out)
    assert torch.equal(out, feat.index_select(0, uniq))
