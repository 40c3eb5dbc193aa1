"""GPU parity: unique + compaction through the C ABI vs the CPU oracle and vs
np.unique, bit-exact."""
import numpy as np
import pytest

from starrygl_amd.lib import _abi
from starrygl_amd.lib.driver import graph_capture
from util import np_of, to_dev

pytestmark = pytest.mark.gpu


def _both(oracle, hot, arrays, mode, universe, calls=1, resets=None):
    """Run `calls` consecutive unique_compact calls on fresh states on both
    sides; arrays is a list (per call) of lists of id arrays."""
    so, sh = oracle.remap_state(universe), hot.remap_state(universe)
    for c in range(calls):
        reset = True if resets is None else resets[c]
        a = arrays[c]
        lo, uo, (to_, bo) = oracle.unique_compact([x.copy() for x in a], mode, so, reset)
        lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, x) for x in a], mode, sh, reset)
        assert (th, bh) == (to_, bo)
        assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), f"call {c}: unique list differs"
        for g in range(len(a)):
            assert np.array_equal(np_of(lh[g]), lo[g]), f"call {c} array {g}: local ids differ"
        yield a, lo, uo, (to_, bo)


@pytest.mark.parametrize("universe,sizes", [(1000, (50, 500, 5000)), (1_000_000, (12_000, 120_000, 1_200_000)),
                                            (77, (0, 10, 0)), (64, (64,)), (65, (1,)), (5_000_000, (100,)),
                                            # both sides of the flag-byte / flag-bit layout switch (2^24 ids)
                                            (1 << 24, (3000, 70_000)), ((1 << 24) + 1, (3000, 70_000))])
def test_sorted_matches_numpy_unique(oracle, hot, universe, sizes):
    rng = np.random.default_rng(universe)
    arrs = [rng.integers(0, universe, s).astype(np.int64) for s in sizes]
    for a, lo, uo, (tot, _) in _both(oracle, hot, [arrs], _abi.UNIQUE_SORTED, universe):
        cat = np.concatenate(a)
        u, inv = np.unique(cat, return_inverse=True)
        assert np.array_equal(uo[:tot], u)
        assert np.array_equal(np.concatenate(lo), inv)


def test_grouped_matches_setdiff(oracle, hot):
    universe = 50_000
    rng = np.random.default_rng(5)
    arrs = [rng.integers(0, universe, s).astype(np.int64) for s in (1800, 18_000, 180_000)]
    for a, lo, uo, (tot, _) in _both(oracle, hot, [arrs], _abi.UNIQUE_GROUPED, universe):
        seen, want = np.zeros(0, np.int64), []
        for x in a:
            new = np.setdiff1d(np.unique(x), seen)
            want.append(new)
            seen = np.concatenate([seen, new])
        assert np.array_equal(uo[:tot], np.concatenate(want))
        for x, l in zip(a, lo):
            assert np.array_equal(uo[l], x)


@pytest.mark.parametrize("mode", [_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED])
def test_epochs_reset_and_follow(oracle, hot, mode):
    universe = 20_000
    rng = np.random.default_rng(9)
    calls = [[rng.integers(0, universe, s).astype(np.int64) for s in (300, 3000)] for _ in range(5)]
    resets = [True, False, False, True, False]
    seen_u = None
    for c, (a, lo, uo, (tot, before)) in enumerate(_both(oracle, hot, calls, mode, universe, 5, resets)):
        if resets[c]:
            assert before == 0
            seen_u = uo[:tot].copy()
        else:
            assert before == seen_u.shape[0]
            seen_u = np.concatenate([seen_u, uo[before:tot]])
        assert np.unique(seen_u).shape[0] == seen_u.shape[0]
        for x, l in zip(a, lo):
            assert np.array_equal(seen_u[l], x)


def test_invalid_ids_map_to_minus_one(oracle, hot):
    universe = 100
    a = np.array([5, -1, 100, 99, 5, 10**12, 0], dtype=np.int64)
    for _, lo, uo, (tot, _) in _both(oracle, hot, [[a]], _abi.UNIQUE_SORTED, universe):
        assert lo[0].tolist() == [1, -1, -1, 2, 1, -1, 0]
        assert uo[:tot].tolist() == [0, 5, 99]


def test_device_side_lengths(oracle, hot):
    universe = 5000
    rng = np.random.default_rng(4)
    full = [rng.integers(0, universe, 4000).astype(np.int64) for _ in range(2)]
    live = [1234, 0]
    st = hot.remap_state(universe)
    lens = [to_dev(hot, np.array([l], dtype=np.int64)) for l in live]
    lh, uh, (th, _) = hot.unique_compact([to_dev(hot, x) for x in full], _abi.UNIQUE_SORTED, st, True, lens_dev=lens)
    u, inv = np.unique(full[0][:1234], return_inverse=True)
    assert th == u.shape[0] and np.array_equal(np_of(uh), u)
    assert np.array_equal(np_of(lh[0])[:1234], inv)


# ------------------------------------------------------------- hash-set path
@pytest.mark.parametrize("mode", [_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED])
@pytest.mark.parametrize("span,sizes", [(1000, (50, 500, 5000)), (2**40, (12_000, 120_000, 400_000)),
                                        (2**62, (3000, 0, 7)), (3, (4096,)), (10**7, (1_000_000,))])
def test_hash_path_matches_oracle_and_numpy(oracle, hot, mode, span, sizes):
    """no remap state: arbitrary non-negative 63-bit ids, negative ids map to -1."""
    rng = np.random.default_rng(len(sizes) + span % 97)
    pool = rng.integers(0, span, max(sum(sizes) // 3, 1))            # ~3x duplication
    arrs = [pool[rng.integers(0, pool.shape[0], s)].astype(np.int64) for s in sizes]
    if arrs[0].shape[0] > 10:
        arrs[0][::7] = -3
    lo, uo, (to_, _) = oracle.unique_compact([a.copy() for a in arrs], mode, None, True)
    lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, None, True)
    assert (th, bh) == (to_, 0)
    assert np.array_equal(np_of(uh), uo)
    for a, b in zip(lh, lo):
        assert np.array_equal(np_of(a), b)
    if mode == _abi.UNIQUE_SORTED:
        cat = np.concatenate(arrs)
        u = np.unique(cat[cat >= 0])
        assert np.array_equal(uo, u)
    for a, l in zip(arrs, lo):
        assert np.array_equal(uo[l[a >= 0]], a[a >= 0]) and (l[a < 0] == -1).all()


def test_hash_path_rejects_follow(hot):
    a = to_dev(hot, np.arange(10, dtype=np.int64))
    with pytest.raises(RuntimeError):
        hot.unique_compact([a], _abi.UNIQUE_SORTED, None, False)


# ------------------------------------------------- persistent hash-set state
def _encode(rng, n_parts, per_part, count):
    """DistRouteIndex-style ids: partition << 48 | local index (partition_book.py:14-31)."""
    return (rng.integers(0, n_parts, count) << 48) | rng.integers(0, per_part, count)


@pytest.mark.parametrize("mode", [_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED])
@pytest.mark.parametrize("kind", ["encoded", "wide", "dense", "squares"])
def test_hashed_state_epochs_reset_and_follow(oracle, hot, mode, kind):
    """'r' then 'f' calls on a hashed state (Remapper::insert over the queries of a blob) against the oracle,
    call by call; the id distributions include a skewed one whose buckets need the in-place sort."""
    rng = np.random.default_rng(31)
    draw = {"encoded": lambda n: _encode(rng, 8, 300_000, n),
            "wide": lambda n: rng.integers(0, 2**62, n),
            "dense": lambda n: rng.integers(0, 5000, n),
            "squares": lambda n: rng.integers(0, 60_000, n) ** 2 + (1 << 40)}[kind]
    cap = 400_000
    so, sh = oracle.remap_hashed_state(cap), hot.remap_hashed_state(cap)
    resets = [True, False, False, True, False, False]
    sizes = [(500, 5000, 50_000), (3, 0, 2000), (40_000, 40_000, 100_000), (100_000, 7, 7), (1, 1, 1), (0, 90_000, 9)]
    pool = draw(60_000).astype(np.int64)
    for c, (reset, sz) in enumerate(zip(resets, sizes)):
        arrs = [np.where(rng.random(n) < 0.7, pool[rng.integers(0, pool.shape[0], n)], draw(n)).astype(np.int64) for n in sz]
        if arrs[0].shape[0] > 4:
            arrs[0][3] = -9
        lo, uo, (to_, bo) = oracle.unique_compact([a.copy() for a in arrs], mode, so, reset)
        lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, sh, reset)
        assert (th, bh) == (to_, bo), f"call {c}"
        assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), f"call {c}: unique list differs"
        for g in range(len(arrs)):
            assert np.array_equal(np_of(lh[g]), lo[g]), f"call {c} array {g}: local ids differ"


def test_hashed_state_oversized_buckets_are_sorted_in_place(oracle, hot):
    """Ids crowded at the low end of a huge range (one id near 2^62 stretches the key): thousands of ids
    share a bucket and go through the block-wide sort."""
    rng = np.random.default_rng(8)
    a = np.concatenate([rng.integers(0, 3000, 40_000), np.array([2**62 - 5]), rng.integers(2**30, 2**30 + 1500, 9000)]).astype(np.int64)
    rng.shuffle(a)
    sh = hot.remap_hashed_state(60_000)
    lh, uh, (th, _) = hot.unique_compact([to_dev(hot, a)], _abi.UNIQUE_SORTED, sh, True)
    u, inv = np.unique(a, return_inverse=True)
    assert th == u.shape[0] and np.array_equal(np_of(uh), u) and np.array_equal(np_of(lh[0]), inv)


@pytest.mark.parametrize("mode", [_abi.UNIQUE_SORTED, _abi.UNIQUE_GROUPED])
@pytest.mark.parametrize("kind", ["encoded", "wide", "crowded"])
def test_hash_path_of_large_calls_orders_by_radix_passes(oracle, hot, mode, kind):
    """Calls that may add more than 2^20 ids order the new ids with two radix passes on the top bits of the
    squeezed key and rank inside the runs; 'crowded' puts thousands of ids into one run (block-wide sort)."""
    rng = np.random.default_rng(77)
    sizes = (300_000, 900_000, 1_200_000)
    if kind == "encoded":
        pool = _encode(rng, 8, 2_000_000, 900_000)
    elif kind == "wide":
        pool = rng.integers(0, 2**62, 900_000)
    else:
        pool = np.concatenate([rng.integers(0, 40_000, 500_000), rng.integers(0, 2**62, 2000),
                               rng.integers(2**61, 2**61 + 50_000, 400_000)])
    arrs = [pool[rng.integers(0, pool.shape[0], s)].astype(np.int64) for s in sizes]
    arrs[1][::11] = -1
    so, sh = oracle.remap_hashed_state(2_500_000), hot.remap_hashed_state(2_500_000)
    for c, reset in enumerate((True, False)):
        if c == 1:
            arrs = [np.where(rng.random(a.shape[0]) < 0.5, a, a + 1) for a in arrs]
            arrs = [np.where(a == 0, -1, a) for a in arrs]
        lo, uo, (to_, bo) = oracle.unique_compact([a.copy() for a in arrs], mode, so, reset)
        lh, uh, (th, bh) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, sh, reset)
        assert (th, bh) == (to_, bo), f"call {c}"
        assert np.array_equal(np_of(uh)[bh:th], uo[bo:to_]), f"call {c}: unique list differs"
        for g in range(len(arrs)):
            assert np.array_equal(np_of(lh[g]), lo[g]), f"call {c} array {g}: local ids differ"
    # the one-shot call takes the same route
    lh, uh, (th, _) = hot.unique_compact([to_dev(hot, a) for a in arrs], mode, None, True)
    lo, uo, (to_, _) = oracle.unique_compact([a.copy() for a in arrs], mode, None, True)
    assert th == to_ and np.array_equal(np_of(uh), uo) and all(np.array_equal(np_of(a), b) for a, b in zip(lh, lo))


def test_hashed_state_reports_an_outgrown_capacity(hot):
    sh = hot.remap_hashed_state(1000)
    a = to_dev(hot, np.arange(900, dtype=np.int64) * 7)
    hot.unique_compact([a], _abi.UNIQUE_SORTED, sh, True)
    with pytest.raises(RuntimeError, match="void"):
        hot.unique_compact([to_dev(hot, np.arange(200, dtype=np.int64) * 7 + 1)], _abi.UNIQUE_SORTED, sh, False)
    with pytest.raises(RuntimeError, match="void"):
        hot.unique_compact([a], _abi.UNIQUE_SORTED, sh, True)
    with pytest.raises(RuntimeError, match="remap_reinit"):      # the message names the way out
        hot.unique_compact([a], _abi.UNIQUE_SORTED, sh, True)
    # the same state, initialised again in place, works again; so does a fresh one
    lh, uh, (th, _) = hot.unique_compact([a], _abi.UNIQUE_SORTED, hot.remap_reinit(sh), True)
    assert th == 900 and np.array_equal(np_of(lh[0]), np.arange(900))
    lh, uh, (th, _) = hot.unique_compact([a], _abi.UNIQUE_SORTED, hot.remap_hashed_state(1000), True)
    assert th == 900 and np.array_equal(np_of(lh[0]), np.arange(900))
    # remap_reinit picks the initialiser by the kind of state
    d = hot.remap_state(7000)
    hot.unique_compact([a], _abi.UNIQUE_SORTED, d, True)
    lh, uh, (th, _) = hot.unique_compact([a], _abi.UNIQUE_SORTED, hot.remap_reinit(d), False)
    assert th == 900 and np.array_equal(np_of(lh[0]), np.arange(900))


@pytest.mark.parametrize("n_ids,capacity", [(5_000, 50), (30_000, 1_000), (2_000_000, 1_500_000)])
def test_hashed_state_overflow_leaves_scratch_contents_alone(hot, n_ids, capacity):
    """An epoch that outgrows its state (far more distinct ids than the capacity, also more than the table has
    slots; both routes) on a workspace full of 0xFF bytes: whatever the call's scratch held before, nothing of it is
    used as an index - the call completes, reports a void result, and a state of sufficient capacity then numbers
    the same ids correctly with the same workspace."""
    import torch
    ids = to_dev(hot, np.random.default_rng(3).permutation(n_ids).astype(np.int64) * 3)
    lens = (_abi.i64 * 1)(n_ids)
    big = hot.remap_hashed_state(n_ids)
    need = max(int(hot.lib.unique_hashed_workspace_bytes(capacity, 1, lens)), int(hot.lib.unique_hashed_workspace_bytes(n_ids, 1, lens)))
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=ids.device)
    small = hot.remap_hashed_state(capacity)
    out, uniq, U = hot.unique_compact([ids], _abi.UNIQUE_SORTED, small, True, finalize=False, workspace=ws)
    torch.cuda.synchronize()
    assert int(U[0]) == np.iinfo(np.int64).max
    ws.fill_(0xFF)
    lh, uh, (th, _) = hot.unique_compact([ids], _abi.UNIQUE_SORTED, big, True, workspace=ws)
    assert th == n_ids and np.array_equal(np_of(uh), np.arange(n_ids) * 3)
    assert np.array_equal(np_of(uh)[np_of(lh[0])], np_of(ids))


@pytest.mark.parametrize("n", [30_000, 1_300_000])
def test_hash_unique_is_captured_and_replayed_in_a_hip_graph(oracle, hot, n):
    """The hash-set path is a fixed launch sequence without host synchronisation: captured once, replayed
    over new ids of varying live length, with eager work and synchronisations between the replays (the
    larger size takes the radix route)."""
    import torch
    rng = np.random.default_rng(3)
    ids = torch.zeros(n, dtype=torch.int64, device="cuda")
    live = torch.zeros(1, dtype=torch.int64, device="cuda")
    out, uniq, U = torch.empty_like(ids), torch.empty(n, dtype=torch.int64, device="cuda"), torch.zeros(2, dtype=torch.int64, device="cuda")
    state = hot.remap_hashed_state(n)
    lens = (_abi.i64 * 1)(n)
    ws = torch.empty(int(hot.lib.unique_hashed_workspace_bytes(n, 1, lens)), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()

    def call(st):
        hot.unique_compact([ids], _abi.UNIQUE_SORTED, st, True, lens_dev=[live], out_arrays=[out], unique_out=uniq,
                           U_out=U, finalize=False, workspace=ws)

    with torch.cuda.stream(stream):
        call(state)                      # warm-up outside the capture
    stream.synchronize()
    g = torch.cuda.CUDAGraph()
    with graph_capture(g, stream=stream):
        call(state)
    for rep, m in enumerate((n, 17, 12_345, 0, n)):
        a = _encode(rng, 4, n // 3, n).astype(np.int64)
        ids.copy_(torch.from_numpy(a))
        live.fill_(m)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        u, inv = np.unique(a[:m], return_inverse=True)
        tot = int(U[0])
        assert tot == u.shape[0], f"replay {rep}"
        assert np.array_equal(np_of(uniq)[:tot], u) and np.array_equal(np_of(out)[:m], inv), f"replay {rep}"
