"""GPU parity at the full size of configs[1] (1M nodes / 20M edges, Zipf(1.1) out-degrees, batches of 4000 events +
4000 negatives = 12000 roots, 2-hop 10x10): the step of the benchmark - both samplers in one launch with the
next-hop index and the batch's root hints, unique with the sampler's marks, the three gathers in one launch -
against the CPU oracle and numpy, bit-exact, for batches from the start, the middle and the end of the stream."""
import numpy as np
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import assert_hop_equal, np_of, to_dev

pytestmark = pytest.mark.gpu
N, M, B, K = 1_000_000, 20_000_000, 4000, 10


@pytest.fixture(scope="module")
def world(oracle, hot):
    src, dst, ts, eid, row_ptr = synth.graph_by_degree(N, M, 1.1, 1 << 40, 20242)
    hg = oracle.tcsr_from_sorted(N, row_ptr, dst, ts, eid, validate=False)
    dg = hot.tcsr_from_sorted(N, *(to_dev(hot, x) for x in (row_ptr, dst, ts, eid)), validate=True)
    hot.build_hop_hint(dg)
    order = np.argsort(ts, kind="stable")                     # the event stream: global time order
    yield dict(src=src, dst=dst, ts=ts, hg=hg, dg=dg, order=order)


def test_next_hop_index_on_the_full_graph(oracle, hot, world):
    """every 997th entry against numpy's searchsorted on the destination's row"""
    hg, hint = world["hg"], np_of(world["dg"].hop_hint)
    for e in range(0, M, 997 * 41):
        v, t = hg.col[e], hg.ts[e]
        lo, hi = hg.row_ptr[v], hg.row_ptr[v + 1]
        assert hint[e] == lo + np.searchsorted(hg.ts[lo:hi], t, side="left")


@pytest.mark.parametrize("start", [0, M // 2, M - B])
def test_step_parity(oracle, hot, world, start):
    w, rng = world, np.random.default_rng(start + 1)
    ev = w["order"][start: start + B]
    b = synth.link_batch(w["src"][ev], w["dst"][ev], w["ts"][ev], 0, B, N, B, rng)
    dev = [to_dev(hot, x) for x in b]
    ends = hot.window_end(w["dg"], dev[0], dev[2])
    assert np.array_equal(np_of(ends), oracle.window_end(w["hg"], b[0], b[2]))
    state = hot.remap_state(N)
    p_rec = hot.marking(hot.with_root_hint(hot.params("recent", K), ends), state)
    p_uni = hot.with_root_hint(hot.params("uniform", K, seed=5), ends)
    outs = [hot.khop_buffers(3 * B, 2, K) for _ in range(2)]
    hot.sample_khop_multi(w["dg"], *dev, 2, [p_rec, p_uni], outs)
    kr = outs[0]
    # unique consumes the marks of the recent query (device-side lengths, nothing read back in between)
    arrays = [kr.slot_node0, kr.hops[0].neighbors, kr.hops[1].neighbors]
    lens = [to_dev(hot, np.array([3 * B], dtype=np.int64)), kr.hops[0].counts[1:2], kr.hops[1].counts[1:2]]
    local, uniq, (total, _) = hot.unique_compact(arrays, _abi.UNIQUE_SORTED, state, True, lens_dev=lens, premarked=True)
    want = {st: oracle.sample_khop(w["hg"], *b, 2, oracle.params(st, K, seed=5)) for st in ("recent", "uniform")}
    for res, st in zip(outs, ("recent", "uniform")):
        res.finalize()
        for l in range(2):
            assert_hop_equal(res.hops[l], want[st].hops[l], tag=f"{st} hop{l} start={start}")
    ids = [want["recent"].slot_node0] + [h.neighbors for h in want["recent"].hops]
    u, inv = np.unique(np.concatenate(ids), return_inverse=True)
    assert total == u.size and np.array_equal(np_of(uniq)[:total], u)
    off = 0
    for a, x in zip(local, ids):
        assert np.array_equal(np_of(a)[: x.size], inv[off: off + x.size])
        off += x.size
    # the three gathers of the step in one launch; rows checked through index_select
    g = torch.Generator(device="cuda").manual_seed(3)
    node_feat = torch.randn((N, 100), device="cuda", generator=g)
    edge_feat = torch.randn((2_000_000, 172), device="cuda", generator=g)          # rows of eid mod 2M
    eids = [h.neighbors_eid % 2_000_000 for h in kr.hops]
    out_n = torch.empty((total, 100), device="cuda")
    out_e = [torch.empty((e.numel(), 172), device="cuda") for e in eids]
    plan = hot.gather_plan([(hot.cache(400, node_feat), uniq[:total], out_n, None, None),
                            (hot.cache(688, edge_feat), eids[0], out_e[0], None, None),
                            (hot.cache(688, edge_feat), eids[1], out_e[1], None, None)])
    hot.gather_multi(plan)
    assert torch.equal(out_n, node_feat.index_select(0, uniq[:total]))
    for o, e in zip(out_e, eids):
        assert torch.equal(o, edge_feat.index_select(0, e))
