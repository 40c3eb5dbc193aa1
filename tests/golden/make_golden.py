"""Writes tests/golden/hot_path_v1.npz: inputs and expected outputs of every stage of the hot
path on one small seeded case, computed by the single-threaded CPU oracle (whose functions are
pinned separately against numpy routines, brute force and the published Philox vectors in
tests/test_oracle.py and tests/test_facade_cpu.py).  The reference itself holds no golden
vectors for this path; these fixtures freeze the agreed semantics so that the oracle and the
HIP library cannot drift together unnoticed.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
for p in (ROOT, os.path.join(ROOT, "starrygl-framework_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from oracle import oracle as O                      # noqa: E402
from starrygl_amd.lib import _abi                   # noqa: E402
from starrygl_amd.utils import synth                # noqa: E402


def case():
    """The seeded inputs (also used by the tests to rebuild the graph)."""
    n, m, C = 300, 6000, 4
    src, dst, ts, eid = synth.graph_stream(n, m, 1.15, 5000, 77)
    rng = np.random.default_rng(77)
    eid = rng.permutation(m).astype(np.int64)
    chunk_of = rng.integers(0, C, n).astype(np.int64)
    roots, ts_ptr, root_ts, neg, neg_ts = synth.link_batch(src, dst, ts, 4000, 4040, n, 40, rng)
    return dict(n=n, C=C, src=src, dst=dst, ts=ts, eid=eid, chunk_of=chunk_of, roots=roots, ts_ptr=ts_ptr,
                root_ts=root_ts, neg=neg, neg_ts=neg_ts)


def compute(ora, cdll, c):
    cdll.sglo_set_num_threads(1)
    out = {}
    g = ora.tcsr_build(c["n"], c["src"], c["dst"], c["ts"], c["eid"])
    out.update(row_ptr=g.row_ptr, col=g.col, cts=g.ts, ceid=g.eid)
    for name, kw in (("recent", dict(sample_type="recent", fanout=5)),
                     ("uniform", dict(sample_type="uniform", fanout=5, seed=20240)),
                     ("window", dict(sample_type="recent", fanout=3, allowed_offset=400, equal_root_time=True))):
        r = ora.sample_khop(g, c["roots"], c["ts_ptr"], c["root_ts"], c["neg"], c["neg_ts"], 2, ora.params(**kw))
        for l, h in enumerate(r.hops):
            for f in ("root_start_ptr", "neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt"):
                out[f"{name}_h{l}_{f}"] = getattr(h, f)
        if name == "recent":
            arrays = [r.slot_node0, r.hops[0].neighbors, r.hops[1].neighbors]
            st = ora.remap_state(c["n"])
            for mode, tag in ((_abi.UNIQUE_SORTED, "sorted"), (_abi.UNIQUE_GROUPED, "grouped")):
                local, uniq, (tot, _) = ora.unique_compact([a.copy() for a in arrays], mode, st, True)
                out[f"unique_{tag}"] = uniq[:tot]
                out[f"local_{tag}"] = np.concatenate(local)
            dt = r.hops[1].neighbors_dt
            w = (1.0 / 10 ** np.linspace(0, 9, 12, dtype=np.float32)).astype(np.float32)
            b = np.linspace(-1, 1, 12).astype(np.float32)
            out.update(te_w=w, te_b=b, te_out=ora.time_encode(dt, w, b))
    cp, cn = ora.chunk_index(c["n"], c["C"], c["chunk_of"])
    ch = np.array([2, 0], dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(cp[ch + 1] - cp[ch])]).astype(np.int64)
    for f, a in zip(("roots", "ts_ptr", "ts", "q_ptr", "q_eid"), ora.seeds(g, cp, cn, ch, off, int(off[-1]), 1000, 1400)):
        out[f"seeds_{f}"] = a
    for f, a in zip(("nodes", "ts_ptr", "ts", "edge_ptr", "col", "col_ts", "col_eid"),
                    ora.slice(g, cp, cn, c["chunk_of"], ch, off, int(off[-1]), 1000, 1012, True)):
        out[f"slice_{f}"] = a
    return out


if __name__ == "__main__":
    ora, cdll = O.load()
    c = case()
    res = compute(ora, cdll, c)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_path_v1.npz")
    np.savez_compressed(path, **res)
    print(path, os.path.getsize(path), "bytes,", len(res), "arrays")
