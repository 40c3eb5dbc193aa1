"""GPU parity: unique + compaction through the C ABI vs the CPU oracle and vs
np.unique, bit-exact."""
import numpy as np
import pytest

from starrygl_amd.lib import _abi
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
