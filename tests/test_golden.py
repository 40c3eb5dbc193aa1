"""The committed fixture tests/golden/hot_path_v1.npz (written by tests/golden/make_golden.py from the
single-threaded oracle) against today's oracle (CPU) and against the HIP library (GPU), bit-exact
except for the time encoding (1e-6)."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden                                   # noqa: E402
from starrygl_amd.lib import _abi                    # noqa: E402
from util import np_of, to_dev                       # noqa: E402

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hot_path_v1.npz")


@pytest.fixture(scope="module")
def golden():
    return dict(np.load(FIXTURE, allow_pickle=False))


def test_oracle_reproduces_the_fixture(oracle, oracle_cdll, golden):
    got = make_golden.compute(oracle, oracle_cdll, make_golden.case())
    oracle_cdll.sglo_set_num_threads(int(oracle_cdll.sglo_get_max_threads()))
    assert sorted(got) == sorted(golden)
    for k, v in golden.items():
        assert got[k].dtype == v.dtype and np.array_equal(got[k], v), k
    # and the fixture is what the definitions say, on a few direct checks
    c = make_golden.case()
    order = np.lexsort((c["eid"], c["ts"], c["src"]))
    assert np.array_equal(golden["col"], c["dst"][order]) and np.array_equal(golden["ceid"], c["eid"][order])
    u, inv = np.unique(np.concatenate([np.concatenate([c["roots"], c["neg"]]), golden["recent_h0_neighbors"],
                                       golden["recent_h1_neighbors"]]), return_inverse=True)
    assert np.array_equal(golden["unique_sorted"], u) and np.array_equal(golden["local_sorted"], inv)
    assert (golden["recent_h1_neighbors_dt"] < 0).all() and (golden["uniform_h1_neighbors_dt"] < 0).all()
    a = (golden["te_w"].astype(np.float32)[None, :] * golden["recent_h1_neighbors_dt"].astype(np.float32)[:, None])
    a = (a.astype(np.float32) + golden["te_b"][None, :]).astype(np.float32)
    assert np.abs(np.cos(a.astype(np.float64)) - golden["te_out"]).max() <= 1e-6


@pytest.mark.gpu
def test_hip_library_reproduces_the_fixture(hot, golden):
    c = make_golden.case()
    D = lambda a: to_dev(hot, a)
    g = hot.tcsr_build(c["n"], D(c["src"]), D(c["dst"]), D(c["ts"]), D(c["eid"]))
    for f, k in (("row_ptr", "row_ptr"), ("col", "col"), ("ts", "cts"), ("eid", "ceid")):
        assert np.array_equal(np_of(getattr(g, f)), golden[k]), k
    args = [D(c[k]) for k in ("roots", "ts_ptr", "root_ts", "neg", "neg_ts")]
    for name, kw in (("recent", dict(sample_type="recent", fanout=5)),
                     ("uniform", dict(sample_type="uniform", fanout=5, seed=20240)),
                     ("window", dict(sample_type="recent", fanout=3, allowed_offset=400, equal_root_time=True))):
        r = hot.sample_khop(g, *args, 2, hot.params(**kw))
        for l, h in enumerate(r.hops):
            for f in ("root_start_ptr", "neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt"):
                assert np.array_equal(np_of(getattr(h, f)), golden[f"{name}_h{l}_{f}"]), (name, l, f)
        if name == "recent":
            arrays = [r.slot_node0, r.hops[0].neighbors, r.hops[1].neighbors]
            st = hot.remap_state(c["n"])
            for mode, tag in ((_abi.UNIQUE_SORTED, "sorted"), (_abi.UNIQUE_GROUPED, "grouped")):
                local, uniq, (tot, _) = hot.unique_compact(arrays, mode, st, True)
                assert np.array_equal(np_of(uniq), golden[f"unique_{tag}"])
                assert np.array_equal(np.concatenate([np_of(x) for x in local]), golden[f"local_{tag}"])
            local, uniq, _ = hot.unique_compact(arrays, _abi.UNIQUE_SORTED)          # hash-set path
            assert np.array_equal(np_of(uniq), golden["unique_sorted"])
            te = hot.time_encode(r.hops[1].neighbors_dt, to_dev(hot, golden["te_w"], "f32"), to_dev(hot, golden["te_b"], "f32"))
            ref = golden["te_out"]
            assert (np.abs(np_of(te) - ref) <= 1e-6 * np.maximum(1.0, np.abs(ref))).all()
    cp, cn = hot.chunk_index(c["n"], c["C"], D(c["chunk_of"]))
    ch = np.array([2, 0], dtype=np.int64)
    cp_h = np_of(cp)
    off = np.concatenate([[0], np.cumsum(cp_h[ch + 1] - cp_h[ch])]).astype(np.int64)
    for f, a in zip(("roots", "ts_ptr", "ts", "q_ptr", "q_eid"), hot.seeds(g, cp, cn, D(ch), D(off), int(off[-1]), 1000, 1400)):
        assert np.array_equal(np_of(a), golden[f"seeds_{f}"]), f
    for f, a in zip(("nodes", "ts_ptr", "ts", "edge_ptr", "col", "col_ts", "col_eid"),
                    hot.slice(g, cp, cn, D(c["chunk_of"]), D(ch), D(off), int(off[-1]), 1000, 1012, True)):
        assert np.array_equal(np_of(a), golden[f"slice_{f}"]), f
