"""GPU: a seeded sweep of random shapes through every stage (T-CSR build, k-hop sampling of both
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
