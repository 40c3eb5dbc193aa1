"""GPU parity: temporal sampling through the C ABI vs the CPU oracle, bit-exact
(recent AND uniform: both sides draw from the same counter-based generator)."""
import numpy as np
import pytest

from starrygl_amd.utils import synth
from util import assert_hop_equal, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


def _graph(oracle, hot, n, m, a, t_max, seed, hub=None):
    src, dst, ts, eid = synth.graph_stream(n, m, a, t_max, seed)
    if hub is not None:  # one very long row to exercise the multi-step search
        src[: hub] = 3
    g = host_graph(oracle, n, src, dst, ts, eid)
    return (src, dst, ts, eid), g, mirror_graph(hot, g)


def _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, layers, **kw):
    p = oracle.params(**kw)
    want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, layers, p)
    got = hot.sample_khop(dg, to_dev(hot, roots), to_dev(hot, ts_ptr), to_dev(hot, root_ts),
                          to_dev(hot, neg), to_dev(hot, neg_ts), layers, hot.params(**kw))
    assert np.array_equal(np_of(got.slot_node0), want.slot_node0)
    assert np.array_equal(np_of(got.slot_ts0), want.slot_ts0)
    for l in range(layers):
        assert_hop_equal(got.hops[l], want.hops[l], tag=f"hop{l} {kw}")
    return got, want


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
@pytest.mark.parametrize("layers,fanout", [(1, 10), (2, 10), (2, 5), (1, 20), (1, 1)])
def test_khop_parity_plumbing_graph(oracle, hot, sample_type, layers, fanout):
    """configs[0]: 10k nodes / 160k edges, batches of 600 edges + 600 negatives."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 10_000, 160_000, 1.2, 2_600_000, 20240)
    rng = np.random.default_rng(1)
    for lo in (0, 80_000, 159_400):
        b = synth.link_batch(src, dst, ts, lo, lo + 600, g.n, 600, rng)
        _run_both(oracle, hot, g, dg, *b, layers, sample_type=sample_type, fanout=fanout, seed=7 + lo)


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_window_flags(oracle, hot, sample_type):
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 2_000, 60_000, 1.1, 50_000, 3)
    rng = np.random.default_rng(2)
    b = synth.link_batch(src, dst, ts, 30_000, 30_500, g.n, 300, rng)
    for kw in (dict(allowed_offset=0), dict(allowed_offset=500), dict(allowed_offset=10**9),
               dict(equal_root_time=True), dict(equal_root_time=True, allowed_offset=100),
               dict(keep_root_time=True), dict(replace=True), dict(replace=True, keep_root_time=True)):
        _run_both(oracle, hot, g, dg, *b, 2, sample_type=sample_type, fanout=7, seed=11, **kw)


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
@pytest.mark.parametrize("fanout", [3, 16, 17, 32, 33, 64, 65, 200, 1024])
def test_long_rows_and_wide_fanout(oracle, hot, sample_type, fanout):
    """a 120k-edge row (5 search steps with 16 lanes) and every group width; beyond 64 the uniform
    strategy keeps a slot's picks in LDS."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 500, 150_000, 1.05, 10**12, 5, hub=120_000)
    rng = np.random.default_rng(3)
    roots = np.concatenate([np.full(200, 3), rng.integers(0, g.n, 300)]).astype(np.int64)
    root_ts = rng.integers(0, 10**12, roots.shape[0]).astype(np.int64)
    ts_ptr = np.arange(roots.shape[0] + 1, dtype=np.int64)
    e = np.zeros(0, np.int64)
    _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, e, e, 1, sample_type=sample_type, fanout=fanout, seed=99)


def test_multi_timestamp_roots_and_empty_inputs(oracle, hot):
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 300, 5_000, 1.1, 10_000, 8)
    roots = np.array([5, 7, 7, 250, 0], dtype=np.int64)
    ts_ptr = np.array([0, 3, 3, 4, 9, 10], dtype=np.int64)  # root 1 has no timestamp
    root_ts = np.array([100, 5000, 9999, 7000, 1, 2, 3, 4, 9000, 10_000], dtype=np.int64)
    neg = np.array([299, 0], dtype=np.int64)
    neg_ts = np.array([10_001, 0], dtype=np.int64)
    for st in ("recent", "uniform"):
        _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, 2, sample_type=st, fanout=4, seed=1)
    e = np.zeros(0, np.int64)
    got, _ = _run_both(oracle, hot, g, dg, e, np.zeros(1, np.int64), e, e, e, 2, sample_type="recent", fanout=4)
    assert got.hops[0].E == 0 and got.hops[1].S == 0
    # only negatives
    _run_both(oracle, hot, g, dg, e, np.zeros(1, np.int64), e, neg, neg_ts, 1, sample_type="uniform", fanout=4)


def test_isolated_nodes_and_time_zero(oracle, hot):
    """nodes without edges and roots at t <= every timestamp sample nothing."""
    n = 50
    src = np.array([1, 1, 1, 2], dtype=np.int64)
    dst = np.array([2, 3, 4, 1], dtype=np.int64)
    ts = np.array([10, 10, 20, 5], dtype=np.int64)
    g = host_graph(oracle, n, src, dst, ts)
    dg = mirror_graph(hot, g)
    roots = np.array([0, 1, 1, 1, 2, 49], dtype=np.int64)
    root_ts = np.array([100, 10, 11, 21, 5, 100], dtype=np.int64)
    ts_ptr = np.arange(7, dtype=np.int64)
    e = np.zeros(0, np.int64)
    got, want = _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, e, e, 1, sample_type="recent", fanout=2)
    assert np_of(got.hops[0].root_end_ptr).tolist()[:-1] == [0, 0, 2, 4, 4, 4]
    assert np_of(got.hops[0].neighbors).tolist() == [2, 3, 3, 4]  # ties keep storage (eid) order


def test_out_of_range_root_is_reported(oracle, hot):
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 100, 1_000, 1.1, 1000, 4)
    roots = np.array([5, 100, -1, 7], dtype=np.int64)
    ts_ptr = np.arange(5, dtype=np.int64)
    root_ts = np.full(4, 900, dtype=np.int64)
    e = to_dev(hot, np.zeros(0, np.int64))
    res = hot.sample_khop(dg, to_dev(hot, roots), to_dev(hot, ts_ptr), to_dev(hot, root_ts), e, e, 1,
                          hot.params("recent", 3), finalize=False)
    assert np_of(res.counts).tolist()[2] == 2
    with pytest.raises(IndexError):
        res.finalize()


def test_error_codes(hot):
    with pytest.raises(RuntimeError, match="undefined sampling strategy"):
        hot.params("nearest", 3)
    import ctypes as C
    from starrygl_amd.lib import _abi
    p = hot.params("recent", 3)
    p.type = 9
    assert hot.lib.sample_khop(None, 0, None, None, 0, None, 0, None, None, 1, C.byref(p), None, None, None,
                               None, 0, None) == _abi.SGL_EINVAL


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_large_hops(oracle, hot, sample_type):
    """> 32k slots per hop: the recent strategy switches to 8 lanes per slot, grids
    beyond 1024 blocks use the one-block scan, beyond 8192 blocks every block walks
    several slot groups; a 200k-edge hub row keeps the multi-step search in play."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 2_000, 600_000, 1.05, 10**9, 17, hub=200_000)
    rng = np.random.default_rng(4)
    b = synth.link_batch(src, dst, ts, 500_000, 502_000, g.n, 2000, rng)          # 6k roots -> ~60k -> ~600k slots
    got, want = _run_both(oracle, hot, g, dg, *b, 3, sample_type=sample_type, fanout=10, seed=5)
    assert want.hops[1].S > 32768 and want.hops[2].S > 8192 * 32


@pytest.mark.parametrize("sample_type,fanout,layers", [("recent", 10, 2), ("uniform", 10, 2), ("recent", 20, 1), ("uniform", 33, 1)])
def test_sampler_marks_ids_for_unique(oracle, hot, sample_type, fanout, layers):
    """The sampler records what it emits as pending in a remap state; the unique call that follows
    skips its first pass.  Same local ids and unique list as the oracle's ordinary unique over the
    sampled arrays; the state is clean afterwards (an ordinary call on it still agrees)."""
    from starrygl_amd.lib import _abi
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 10_000, 160_000, 1.2, 2_600_000, 20240)
    rng = np.random.default_rng(5)
    state, ostate = hot.remap_state(g.n), oracle.remap_state(g.n)
    for lo in (80_000, 159_400):
        roots, ts_ptr, root_ts, neg, neg_ts = synth.link_batch(src, dst, ts, lo, lo + 600, g.n, 600, rng)
        roots[:3] = [g.n + 5, -2, 7]                        # out-of-range roots: no neighbours, local id -1
        kw = dict(sample_type=sample_type, fanout=fanout, seed=3 + lo)
        want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, layers, oracle.params(**kw), finalize=False)
        cnt = want.counts
        wa = [want.slot_node0] + [h.neighbors[: int(cnt[3 * l + 1])] for l, h in enumerate(want.hops)]
        wl, wu, (wt, _) = oracle.unique_compact([x.copy() for x in wa], _abi.UNIQUE_SORTED, ostate, True)
        p = hot.marking(hot.params(**kw), state)
        got = hot.sample_khop(dg, to_dev(hot, roots), to_dev(hot, ts_ptr), to_dev(hot, root_ts), to_dev(hot, neg),
                              to_dev(hot, neg_ts), layers, p, finalize=False)
        arrays = [got.slot_node0] + [h.neighbors for h in got.hops]
        lens = [to_dev(hot, np.array([roots.size + neg.size]))] + [h.counts[1:2] for h in got.hops]
        gl, gu, (gt, gb) = hot.unique_compact(arrays, _abi.UNIQUE_SORTED, state, True, lens_dev=lens, premarked=True)
        assert (gt, gb) == (wt, 0) and np.array_equal(np_of(gu), wu[:wt])
        for a, b in zip(gl, wl):
            assert np.array_equal(np_of(a)[: b.size], b)
        assert np_of(gl[0])[:3].tolist()[:2] == [-1, -1]
        # an ordinary call afterwards: nothing left pending from the sampler
        extra = rng.integers(0, g.n, 1000).astype(np.int64)
        l2, u2, (t2, _) = hot.unique_compact([to_dev(hot, extra)], _abi.UNIQUE_SORTED, state, True)
        assert np.array_equal(np_of(u2), np.unique(extra)) and t2 == np.unique(extra).size
    with pytest.raises(ValueError):
        hot.unique_compact([to_dev(hot, extra)], _abi.UNIQUE_GROUPED, state, True, premarked=True)


@pytest.mark.parametrize("fanout", [1, 9, 16, 17])
def test_two_hop_recent_single_launch_boundaries(oracle, hot, fanout):
    """2-hop recent calls of up to 32768 root slots and fanout <= 16 run as one kernel; slot counts
    around the group / block / limit boundaries and fanouts on both sides of the limit must agree
    with the oracle like every other path."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 3_000, 90_000, 1.15, 10**6, 23, hub=20_000)
    rng = np.random.default_rng(9)
    for S0 in (1, 15, 16, 17, 255, 256, 257, 32768, 32769):
        n_neg = S0 // 3
        roots = rng.integers(0, g.n, S0 - n_neg).astype(np.int64)
        root_ts = rng.integers(0, 10**6, S0 - n_neg).astype(np.int64)
        ts_ptr = np.arange(S0 - n_neg + 1, dtype=np.int64)
        neg = rng.integers(0, g.n, n_neg).astype(np.int64)
        neg_ts = rng.integers(0, 10**6, n_neg).astype(np.int64)
        if S0 > 32768 and fanout > 9:
            continue                      # 32769 * 17^2 edges: more than this test needs to allocate
        got, want = _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, 2, sample_type="recent",
                              fanout=fanout, equal_root_time=bool(S0 % 2))
        assert got.hops[1].E == want.hops[1].E


@pytest.mark.parametrize("fanout,layers,S0", [(10, 2, 1), (10, 2, 700), (16, 2, 4099), (17, 2, 300), (10, 1, 500), (5, 3, 200)])
def test_several_policies_in_one_call(oracle, hot, fanout, layers, S0):
    """sgl_sample_khop_multi: every query's result equals the oracle's for that policy.  A recent and a
    uniform 2-hop query of the single-launch size share one kernel; other shapes (fanout 17, one or
    three hops, three queries) run query by query."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 3_000, 90_000, 1.15, 10**6, 29, hub=20_000)
    rng = np.random.default_rng(13)
    n_neg = S0 // 3
    roots = rng.integers(0, g.n, S0 - n_neg).astype(np.int64)
    root_ts = rng.integers(0, 10**6, S0 - n_neg).astype(np.int64)
    ts_ptr = np.arange(S0 - n_neg + 1, dtype=np.int64)
    neg = rng.integers(0, g.n, n_neg).astype(np.int64)
    neg_ts = rng.integers(0, 10**6, n_neg).astype(np.int64)
    dev_args = [to_dev(hot, x) for x in (roots, ts_ptr, root_ts, neg, neg_ts)]
    policies = [dict(sample_type="recent", fanout=fanout, equal_root_time=True),
                dict(sample_type="uniform", fanout=fanout, seed=77, keep_root_time=True),
                dict(sample_type="recent", fanout=max(fanout - 2, 1), allowed_offset=50_000)]
    for sel in ([0, 1], [1, 0], [0, 1, 2], [1]):
        kws = [policies[i] for i in sel]
        outs = [hot.khop_buffers(S0, layers, kw["fanout"]) for kw in kws]
        hot.sample_khop_multi(dg, *dev_args, layers, [hot.params(**kw) for kw in kws], outs)
        for kw, res in zip(kws, outs):
            want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, layers, oracle.params(**kw))
            got = res.finalize()
            assert np.array_equal(np_of(got.slot_node0), want.slot_node0)
            assert np.array_equal(np_of(got.slot_ts0), want.slot_ts0)
            for l in range(layers):
                assert_hop_equal(got.hops[l], want.hops[l], tag=f"hop{l} {kw} of {sel}")


def test_several_policies_with_marks_feed_unique(oracle, hot):
    """The recent query of a shared launch records its ids for the unique stage like a call of its own."""
    from starrygl_amd.lib import _abi
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 5_000, 120_000, 1.1, 10**6, 31)
    rng = np.random.default_rng(17)
    b = synth.link_batch(src, dst, ts, 60_000, 60_400, g.n, 400, rng)
    state = hot.remap_state(g.n)
    p_rec = hot.marking(hot.params("recent", 10), state)
    p_uni = hot.params("uniform", 10, seed=5)
    outs = [hot.khop_buffers(1200, 2, 10), hot.khop_buffers(1200, 2, 10)]
    for _ in range(2):          # twice: the second call starts from the state the first one left
        hot.sample_khop_multi(dg, *[to_dev(hot, x) for x in b], 2, [p_rec, p_uni], outs)
        r = outs[0]
        lens = [r.counts[0:1], r.counts[1:2], r.counts[4:5]]
        arrays = [r.slot_node0, r.hops[0].neighbors, r.hops[1].neighbors]
        local, uniq, U = hot.unique_compact(arrays, _abi.UNIQUE_SORTED, state, True, lens_dev=lens, finalize=False,
                                            premarked=True)
        c = np_of(r.counts)
        ids = np.concatenate([np_of(r.slot_node0), np_of(r.hops[0].neighbors)[: c[1]], np_of(r.hops[1].neighbors)[: c[4]]])
        want_u, want_inv = np.unique(ids, return_inverse=True)
        assert int(np_of(U)[0]) == want_u.size and np.array_equal(np_of(uniq)[: want_u.size], want_u)
        got_inv = np.concatenate([np_of(local[0]), np_of(local[1])[: c[1]], np_of(local[2])[: c[4]]])
        assert np.array_equal(got_inv, want_inv)


@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("layers", [1, 2])
def test_uniform_invariants_and_chi_square_on_the_gpu(hot, replace, layers):
    """The uniform sampler judged on its own output, without the oracle: sampled edges lie strictly
    before the root's time, at most `fanout` per slot and distinct without replacement, (neighbour, ts,
    eid) belong to one edge of the row, and every candidate position is drawn with probability k/cnt
    (chi-square at the 0.999 quantile).  One hop goes through the count/fill kernels, two hops through
    the single-launch kernel (its second hop is tested: a chain 1 -> 0 -> 37 candidates)."""
    import scipy.stats as sps
    cnt, k, trials = 37, 10, 20_000
    # node 0 owns `cnt` edges at times 0..cnt-1 to node 2; node 1 owns one edge to node 0 at time cnt + 1
    src = np.concatenate([np.zeros(cnt, np.int64), [1]])
    dst = np.concatenate([np.full(cnt, 2, np.int64), [0]])
    ts = np.concatenate([np.arange(cnt), [cnt + 1]]).astype(np.int64)
    eid = np.arange(cnt + 1, dtype=np.int64)
    dg = hot.tcsr_build(3, to_dev(hot, src), to_dev(hot, dst), to_dev(hot, ts), to_dev(hot, eid))
    p = hot.params("uniform", k, replace=replace, seed=4242)
    empty = to_dev(hot, np.zeros(0, np.int64))
    if layers == 1:
        roots, t_root = np.zeros(trials, np.int64), np.full(trials, cnt + 5, np.int64)
    else:     # hop 1 of root 1 at time cnt + 3 is its only edge (to node 0, ts cnt + 1); hop 2 samples node 0 before cnt + 1
        roots, t_root = np.ones(trials, np.int64), np.full(trials, cnt + 3, np.int64)
    res = hot.sample_khop(dg, to_dev(hot, roots), to_dev(hot, np.arange(trials + 1)), to_dev(hot, t_root), empty, empty, layers, p)
    h = res.hops[layers - 1]
    assert h.S == trials and h.E == trials * k
    start, end = np_of(h.root_start_ptr), np_of(h.root_end_ptr)
    assert np.array_equal(end[:-1] - start[:-1], np.full(trials, k))
    e, nb, nts, ndt = np_of(h.neighbors_eid), np_of(h.neighbors), np_of(h.neighbors_ts), np_of(h.neighbors_dt)
    t_slot = cnt + 5 if layers == 1 else cnt + 1
    assert (e >= 0).all() and (e < cnt).all() and (nb == 2).all()          # edges of row 0 only: eid <-> dst mapping
    assert np.array_equal(nts, e) and (nts < t_slot).all() and np.array_equal(ndt, nts - t_slot)
    per_slot = e.reshape(trials, k)
    if not replace:
        s = np.sort(per_slot, axis=1)
        assert (s[:, 1:] > s[:, :-1]).all() and np.array_equal(s, per_slot)  # distinct, ascending position
    freq = np.bincount(e, minlength=cnt).astype(np.float64)
    expect = trials * k / cnt
    chi2 = ((freq - expect) ** 2 / expect).sum()
    assert chi2 < sps.chi2.ppf(0.999, cnt - 1), chi2


def test_driver_rejects_arrays_it_cannot_pass_as_pointers(oracle, hot):
    """The ABI takes raw pointers; the array-level driver refuses what would be misread: another
    dtype, a strided view, pageable host memory."""
    import torch
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 500, 5_000, 1.1, 10**5, 43)
    roots = to_dev(hot, np.arange(40))
    tp, t = to_dev(hot, np.arange(41)), to_dev(hot, np.full(40, 9 * 10**4))
    e = to_dev(hot, np.zeros(0, np.int64))
    p = hot.params("recent", 5)
    hot.sample_khop(dg, roots, tp, t, e, e, 1, p)                                   # the well-formed call
    with pytest.raises(TypeError):
        hot.sample_khop(dg, roots.int(), tp, t, e, e, 1, p)
    with pytest.raises(ValueError):
        hot.sample_khop(dg, to_dev(hot, np.arange(80))[::2], tp, t, e, e, 1, p)    # strided view
    with pytest.raises(ValueError):
        hot.sample_khop(dg, torch.arange(40), tp, t, e, e, 1, p)                    # pageable host memory
    with pytest.raises(TypeError):
        hot.unique_compact([roots.float()], 0, hot.remap_state(500), True)
    with pytest.raises(TypeError):
        hot.gather(hot.cache(16, torch.zeros((500, 4), device=roots.device)), roots.int(),
                   torch.empty((40, 4), device=roots.device))


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_next_hop_index_gives_the_same_samples(oracle, hot, sample_type):
    """With sgl_tcsr.hop_hint the slots of hops >= 1 take the end of their window from the index instead
    of searching.  The index itself equals its definition (first position in row col[e] with ts >= ts[e],
    restated by a linear scan); sampling with it equals the oracle in the single-launch kernel, in the
    multi-launch path over two and three hops, and for the parameter sets that must ignore it
    (windows that include the slot's time, uniform slots that keep the root's time)."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 3_000, 90_000, 1.15, 5_000, 47, hub=20_000)   # 5000 times: many ties
    hot.build_hop_hint(dg)
    assert np.array_equal(np_of(dg.hop_hint), oracle.build_hop_hint(g).hop_hint)
    rng = np.random.default_rng(21)
    for S0, layers, fanout in ((700, 2, 10), (40_000, 2, 5), (3_000, 3, 6), (300, 2, 17), (5, 3, 3)):
        n_neg = S0 // 3
        roots = rng.integers(0, g.n, S0 - n_neg).astype(np.int64)
        root_ts = rng.integers(0, 5_000, S0 - n_neg).astype(np.int64)
        ts_ptr = np.arange(S0 - n_neg + 1, dtype=np.int64)
        neg = rng.integers(0, g.n, n_neg).astype(np.int64)
        neg_ts = rng.integers(0, 5_000, n_neg).astype(np.int64)
        for kw in (dict(), dict(allowed_offset=300), dict(equal_root_time=True), dict(keep_root_time=True),
                   dict(replace=True)):
            _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, layers, sample_type=sample_type,
                      fanout=fanout, seed=5, **kw)


@pytest.mark.parametrize("sample_type", ["recent", "uniform"])
def test_root_hints_give_the_same_samples(oracle, hot, sample_type):
    """sgl_window_end equals the oracle's; with its values as sgl_sample_params.root_hint (some entries -1 =
    search, several timestamps per root, negatives behind the positives) the samples equal the oracle's
    un-hinted ones in the single-launch kernel, the multi-launch path, the pair launch, with a lower window
    bound, and when the hints must be ignored (windows that include the root's time)."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 3_000, 90_000, 1.15, 5_000, 53, hub=20_000)   # many ties
    hot.build_hop_hint(dg)
    rng = np.random.default_rng(22)
    for S_pos, n_neg, layers, fanout in ((600, 300, 2, 10), (30_000, 10_000, 2, 5), (2_000, 0, 3, 6), (64, 7, 1, 17)):
        R = max(1, S_pos // 2)
        cuts = np.sort(rng.integers(0, S_pos + 1, R - 1))
        ts_ptr = np.concatenate([[0], cuts, [S_pos]]).astype(np.int64)
        roots = rng.integers(0, g.n, R).astype(np.int64)
        roots[::5] = np.argmax(np.diff(g.row_ptr))                     # the hub: the longest searches
        root_ts = rng.integers(0, 5_001, S_pos).astype(np.int64)
        neg = rng.integers(0, g.n, n_neg).astype(np.int64)
        neg_ts = rng.integers(0, 5_001, n_neg).astype(np.int64)
        slot_node = np.repeat(roots, np.diff(ts_ptr))
        hint = hot.window_end(dg, to_dev(hot, slot_node), to_dev(hot, root_ts))
        assert np.array_equal(np_of(hint), oracle.window_end(g, slot_node, root_ts))
        hint[::4] = -1
        dev = [to_dev(hot, x) for x in (roots, ts_ptr, root_ts, neg, neg_ts)]
        for kw in (dict(), dict(allowed_offset=300), dict(equal_root_time=True), dict(keep_root_time=True)):
            kw = dict(sample_type=sample_type, fanout=fanout, seed=3, **kw)
            want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, layers, oracle.params(**kw))
            got = hot.sample_khop(dg, *dev, layers, hot.with_root_hint(hot.params(**kw), hint))
            for l in range(layers):
                assert_hop_equal(got.hops[l], want.hops[l], tag=f"root hints, hop{l} {kw}")
        if layers == 2 and fanout <= 16:                               # both strategies in one call
            kws = [dict(sample_type=st_, fanout=fanout, seed=3) for st_ in ("recent", "uniform")]
            outs = [hot.khop_buffers(S_pos + n_neg, 2, fanout) for _ in range(2)]
            hot.sample_khop_multi(dg, *dev, 2, [hot.with_root_hint(hot.params(**k_), hint) for k_ in kws], outs)
            for res, k_ in zip(outs, kws):
                want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, 2, oracle.params(**k_))
                res.finalize()
                for l in range(2):
                    assert_hop_equal(res.hops[l], want.hops[l], tag=f"root hints, multi, hop{l} {k_}")
    # hints outside the root's row are clamped to it: the call completes and stays inside its buffers
    wild = to_dev(hot, rng.integers(-5, 2 * g.m, S_pos).astype(np.int64))
    res = hot.sample_khop(dg, *dev, 1, hot.with_root_hint(hot.params(sample_type, 17), wild))
    assert 0 <= res.hops[0].E <= (S_pos + n_neg) * 17
    # ... and the driver's debug check (SGL_CHECK_HINTS=1) refuses them, while it passes hints that are right or -1
    hot.check_hints = True
    try:
        with pytest.raises(ValueError, match="root_hint"):
            hot.sample_khop(dg, *dev, 1, hot.with_root_hint(hot.params(sample_type, 17), wild))
        hot.sample_khop(dg, *dev, 1, hot.with_root_hint(hot.params(sample_type, 17), hint))
    finally:
        hot.check_hints = False


def test_window_end_edge_cases(oracle, hot):
    """No queries, ids that are no node (-1), nodes without edges (their row's start), times before the
    first and after the last edge of a row, and a graph without edges."""
    src = np.array([1, 1, 1, 4], dtype=np.int64)
    dst = np.array([2, 3, 4, 1], dtype=np.int64)
    ts = np.array([10, 10, 20, 5], dtype=np.int64)
    g = host_graph(oracle, 6, src, dst, ts)
    dg = mirror_graph(hot, g)
    node = np.array([-1, 6, 0, 1, 1, 1, 1, 4, 5], dtype=np.int64)
    t = np.array([0, 0, 7, 9, 10, 11, 99, 5, -3], dtype=np.int64)
    want = oracle.window_end(g, node, t)
    assert want.tolist() == [-1, -1, 0, 0, 0, 2, 3, 3, 4]
    assert np.array_equal(np_of(hot.window_end(dg, to_dev(hot, node), to_dev(hot, t))), want)
    e = np.zeros(0, np.int64)
    assert hot.window_end(dg, to_dev(hot, e), to_dev(hot, e)).numel() == 0
    g0 = host_graph(oracle, 3, e, e, e)
    dg0 = mirror_graph(hot, g0)
    assert np_of(hot.window_end(dg0, to_dev(hot, node[:3]), to_dev(hot, t[:3]))).tolist() == [-1, -1, 0]
    with pytest.raises(ValueError):
        hot.window_end(dg, to_dev(hot, node), to_dev(hot, t[:3]))


@pytest.mark.parametrize("index", [False, True])
@pytest.mark.parametrize("layers,fanout,n_roots", [(1, 10, 700), (2, 10, 1800), (3, 4, 900), (2, 20, 40_000), (1, 33, 500)])
def test_interleaved_records_give_the_same_samples(oracle, hot, index, layers, fanout, n_roots):
    """With the graph's interleaved edge records (and, `index`, its next-hop index copied into them) the
    uniform sampler reads its picks from the records: same result as the oracle, through the launch-per-hop
    route, the single-launch 2-hop route and the recent + uniform pair launch; recent is unchanged."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 3_000, 120_000, 1.15, 400_000, 17)
    if index:
        hot.build_hop_hint(dg)
    hot.build_records(dg)
    rec = np_of(dg.rec).reshape(-1, 4)
    assert np.array_equal(rec[:, 0], g.col) and np.array_equal(rec[:, 1], g.ts) and np.array_equal(rec[:, 2], g.eid)
    if index:       # the index entry with the length of the window it ends (+ 1) above bit 40
        hh = np_of(dg.hop_hint)
        assert np.array_equal(rec[:, 3], hh | ((hh - g.row_ptr[g.col] + 1) << 40))
    else:
        assert np.array_equal(rec[:, 3], np.full(g.m, -1))
    rng = np.random.default_rng(5)
    roots = rng.integers(0, g.n, n_roots).astype(np.int64)
    root_ts = rng.integers(0, 400_000, n_roots).astype(np.int64)
    ts_ptr = np.arange(n_roots + 1, dtype=np.int64)
    neg, neg_ts = rng.integers(0, g.n, n_roots // 3).astype(np.int64), rng.integers(0, 400_000, n_roots // 3).astype(np.int64)
    for kw in (dict(), dict(keep_root_time=True), dict(replace=True), dict(allowed_offset=50_000)):
        _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, layers, sample_type="uniform", fanout=fanout, seed=3, **kw)
    _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, neg, neg_ts, layers, sample_type="recent", fanout=fanout)
    if layers == 2 and fanout <= 16:      # both policies in one launch
        S0 = n_roots + n_roots // 3
        outs = [hot.khop_buffers(S0, 2, fanout) for _ in range(2)]
        ps = [hot.params("recent", fanout), hot.params("uniform", fanout, seed=3)]
        hot.sample_khop_multi(dg, *[to_dev(hot, x) for x in (roots, ts_ptr, root_ts, neg, neg_ts)], 2, ps, outs)
        for p, res in zip(ps, outs):
            want = oracle.sample_khop(g, roots, ts_ptr, root_ts, neg, neg_ts, 2, p)
            for l, h in enumerate(res.finalize().hops):
                assert_hop_equal(h, want.hops[l], tag=f"pair hop{l}")


def test_wide_uniform_fanout_over_two_hops_and_flags(oracle, hot):
    """fanout 100 through the k-hop driver (windows shorter and longer than the fanout, with replacement,
    root time kept, lower window bound), from the arrays and from the interleaved records."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 400, 90_000, 1.1, 300_000, 13)
    rng = np.random.default_rng(9)
    roots = rng.integers(0, g.n, 150).astype(np.int64)
    root_ts = rng.integers(0, 300_000, 150).astype(np.int64)
    ts_ptr, e = np.arange(151, dtype=np.int64), np.zeros(0, np.int64)
    for records in (False, True):
        if records:
            hot.build_hop_hint(dg)
            hot.build_records(dg)
        for kw in (dict(), dict(replace=True), dict(keep_root_time=True), dict(allowed_offset=20_000)):
            _run_both(oracle, hot, g, dg, roots, ts_ptr, root_ts, e, e, 2, sample_type="uniform", fanout=100, seed=5, **kw)


def test_sample_window_parity(oracle, hot):
    """Whole-window sampling (the offline sampler's 'full' / 'cluster' layers and its discrete branch) against
    the oracle: hub rows of 100k edges, empty windows, tags, first-k, both time conventions."""
    (src, dst, ts, _), g, dg = _graph(oracle, hot, 800, 200_000, 1.1, 50_000, 19, hub=100_000)
    rng = np.random.default_rng(7)
    tag = rng.integers(0, 5, g.m).astype(np.int64)
    d_tag = to_dev(hot, tag)
    node = np.concatenate([np.full(20, 3), rng.integers(0, g.n, 3000)]).astype(np.int64)
    t = rng.integers(-5, 50_010, node.shape[0]).astype(np.int64)
    for kw in (dict(), dict(first_k=7), dict(lo_offset=-3000), dict(lo_offset=-500, hi_offset=1, first_k=40, keep_slot_time=True),
               dict(tag_value=3, tagged=True), dict(tag_value=0, tagged=True, lo_offset=-8000, first_k=9, keep_slot_time=True)):
        kw = dict(kw)
        tagged = kw.pop("tagged", False)
        want = oracle.sample_window(g, node, t, edge_tag=tag if tagged else None, **kw)
        got = hot.sample_window(dg, to_dev(hot, node), to_dev(hot, t), edge_tag=d_tag if tagged else None, **kw)
        assert_hop_equal(got, want, tag=str(kw))
    bad = hot.sample_window(dg, to_dev(hot, np.array([1, 2])), to_dev(hot, np.array([5, 5])))      # tiny call
    assert bad.S == 2
    with pytest.raises(IndexError):
        hot.sample_window(dg, to_dev(hot, np.array([1, g.n])), to_dev(hot, np.array([5, 5])))
