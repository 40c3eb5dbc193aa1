"""Pins of the oracle's batched entry points (CPU only).

sample_khop_batched is held against (1) the oracle's own single-batch k-hop driver, itself pinned by brute force in
test_oracle.py - for the most-recent strategy a batched call must be the concatenation of the batches' own calls,
for both strategies it must equal one call over the concatenated slots - and (2) a brute-force count of each
batch's edges for the segment table.  unique_compact_batched is held against np.unique per batch."""
import numpy as np
import pytest

from starrygl_amd.utils import synth
from util import host_graph


def _batches(rng, src, dst, ts, n, sizes, n_neg):
    out = []
    for i, sz in enumerate(sizes):
        lo = int(rng.integers(0, src.size - sz)) if sz else 0
        out.append(synth.link_batch(src, dst, ts, lo, lo + sz, n, n_neg if sz else 0, rng))
    return out


def _concat_slots(batches):
    """(slot_node, slot_ts, batch_ptr): per batch its positive root slots, then its negatives"""
    node = [np.concatenate([b[0], b[3]]) for b in batches]      # one timestamp per root in these batches
    t = [np.concatenate([b[2], b[4]]) for b in batches]
    ptr = np.concatenate([[0], np.cumsum([x.size for x in node])]).astype(np.int64)
    return np.concatenate(node).astype(np.int64), np.concatenate(t).astype(np.int64), ptr


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_batched_sampler_is_the_khop_driver_over_all_slots(oracle, sample_type):
    n = 3000
    src, dst, ts, eid = synth.graph_stream(n, 80_000, 1.2, 500_000, 11)
    g = host_graph(oracle, n, src, dst, ts, eid)
    rng = np.random.default_rng(5)
    batches = _batches(rng, src, dst, ts, n, [200, 0, 50, 333, 1], 40)
    node, t, ptr = _concat_slots(batches)
    B, k, L = len(batches), 5, 2
    p = oracle.params(sample_type, k, seed=77)
    res = oracle.sample_khop_batched(g, node, t, ptr, L, [p], finalize=True)
    q = res.queries[0]
    # (1) one call of the pinned driver over the same slots, handed over as negatives
    e = np.zeros(0, np.int64)
    one = oracle.sample_khop(g, e, np.zeros(1, np.int64), e, node, t, L, p)
    for l in range(L):
        for f in ("root_start_ptr", "root_end_ptr", "neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt"):
            assert np.array_equal(getattr(q.hops[l], f), getattr(one.hops[l], f)), (l, f)
    # (2) the segment table by brute force: a batch's edges of hop l are those whose slot belongs to the batch
    seg = np.asarray(res.seg_host[0])
    assert np.array_equal(seg[0], ptr)
    owner = np.repeat(np.arange(B), np.diff(ptr))                # batch of every hop-0 slot
    for l in range(L):
        h = q.hops[l]
        cnt = np.diff(h.root_start_ptr)
        per_batch = np.bincount(owner, weights=cnt, minlength=B).astype(np.int64)
        assert np.array_equal(np.diff(seg[l + 1]), per_batch), l
        assert seg[l + 1][0] == 0 and seg[l + 1][B] == h.E
        owner = np.repeat(owner, cnt)                            # batch of every slot of the next hop
    # (3) most recent: every batch's segment is the batch's own call
    if sample_type == "recent":
        for b, bt in enumerate(batches):
            own = oracle.sample_khop(g, *bt, L, p)
            for l in range(L):
                lo, hi = seg[l + 1][b], seg[l + 1][b + 1]
                for f in ("neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt"):
                    assert np.array_equal(getattr(q.hops[l], f)[lo:hi], getattr(own.hops[l], f)), (b, l, f)


def test_batched_sampler_takes_only_true_window_ends_as_hints(oracle):
    n = 500
    src, dst, ts, eid = synth.graph_stream(n, 9000, 1.1, 50_000, 2)
    g = host_graph(oracle, n, src, dst, ts, eid)
    rng = np.random.default_rng(1)
    node, t, ptr = _concat_slots(_batches(rng, src, dst, ts, n, [60, 70], 10))
    hint = oracle.window_end(g, node, t)
    hint[::3] = -1
    p = oracle.params("recent", 4)
    a = oracle.sample_khop_batched(g, node, t, ptr, 2, [p], slot_hint=hint, finalize=True)
    b = oracle.sample_khop_batched(g, node, t, ptr, 2, [p], finalize=True)
    assert np.array_equal(a.queries[0].hops[1].neighbors_eid, b.queries[0].hops[1].neighbors_eid)
    bad = hint.copy()
    i = int(np.flatnonzero(bad >= 0)[0])
    bad[i] += 1
    if bad[i] != oracle.window_end(g, node[i: i + 1], t[i: i + 1])[0]:
        with pytest.raises(ValueError):
            oracle.sample_khop_batched(g, node, t, ptr, 2, [p], slot_hint=bad)


def test_batched_unique_is_np_unique_per_batch(oracle):
    rng = np.random.default_rng(9)
    universe, B = 5000, 6
    state = oracle.remap_batched_state(universe, B)
    for trial in range(4):
        arrays, segs = [], []
        for g in range(3):
            sizes = rng.integers(0, 400, B)
            if trial == 1:
                sizes[rng.integers(0, B)] = 0
            seg = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
            a = rng.integers(-3, universe + 5, int(seg[-1]) + 17).astype(np.int64)     # a few ids outside the universe, a dead tail
            arrays.append(a); segs.append(seg)
        local, uniq, off = oracle.unique_compact_batched(arrays, segs, state)
        assert off[0] == 0 and len(off) == B + 1
        for b in range(B):
            ids = np.concatenate([a[s[b]: s[b + 1]] for a, s in zip(arrays, segs)])
            ok = (ids >= 0) & (ids < universe)
            u, inv = np.unique(ids[ok], return_inverse=True)
            assert np.array_equal(uniq[off[b]: off[b + 1]], u), (trial, b)
            got = np.concatenate([l[s[b]: s[b + 1]] for l, s in zip(local, segs)])
            assert np.array_equal(got[ok], inv) and np.all(got[~ok] == -1), (trial, b)
