"""sgl_sample_hop_static, the hop that allocates nothing (its scratch is an array inside the library
image), against sgl_sample_hop with a caller workspace: bit-exact, through the C ABI, on two calls in a
row, the second with a smaller input (the array keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.lib.driver import HopResult
from starrygl_amd.utils import synth
from util import HOP_FIELDS, host_graph, mirror_graph, np_of, to_dev

pytestmark = pytest.mark.gpu


def _hop_pair(hot, dg, node, t, p, S_dev=None):
    S = int(node.shape[0])
    want = hot.sample_hop(dg, node, t, p, S_dev=S_dev, finalize=False)
    got = HopResult(hot.be, S, S * p.fanout)
    # the binding allocates nothing either: the allocator's count of allocations made so far stays put
    # (bytes in use would also move when Python's collector frees another test's tensors during the call)
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    hot.sample_hop_static(dg, node, t, p, got, S_dev=S_dev)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    torch.cuda.synchronize()
    cw, cg = np_of(want.counts), np_of(got.counts)
    assert np.array_equal(cw, cg), (cw, cg)
    S_live, E = int(cw[0]), int(cw[1])
    for f in HOP_FIELDS:
        n = S_live + 1 if "ptr" in f else E
        assert np.array_equal(np_of(getattr(got, f))[:n], np_of(getattr(want, f))[:n]), f
    return S_live, E


@pytest.mark.parametrize("strategy,fanout", [("recent", 10), ("uniform", 10), ("recent", 25), ("uniform", 40)])
def test_static_hop_equals_workspace_hop_twice_in_a_row(hot, oracle, strategy, fanout):
    n, m = 5000, 200_000
    src, dst, ts, eid = synth.graph_stream(n, m, 1.2, 1_000_000, 11)
    dg = mirror_graph(hot, host_graph(oracle, n, src, dst, ts, eid))
    rng = np.random.default_rng(5)
    p = hot.params(strategy, fanout, seed=9)
    # the first call fills a large part of the array (grid beyond 1024 blocks: the scan kernel runs too),
    # the second, smaller one must not see what the first left behind
    for S in (40_000, 700):
        node = to_dev(hot, rng.integers(0, n, S))
        t = to_dev(hot, rng.integers(0, 1_000_000, S))
        S_live, E = _hop_pair(hot, dg, node, t, p)
        assert S_live == S and E > 0
    # a device-side live count below the capacity
    node = to_dev(hot, rng.integers(0, n, 3000))
    t = to_dev(hot, rng.integers(0, 1_000_000, 3000))
    S_live, _ = _hop_pair(hot, dg, node, t, p, S_dev=to_dev(hot, [1234]))
    assert S_live == 1234


def test_static_hop_refuses_more_slots_than_its_array_holds(hot, oracle):
    n = 100
    src, dst, ts, eid = synth.graph_stream(n, 1000, 1.2, 1000, 1)
    dg = mirror_graph(hot, host_graph(oracle, n, src, dst, ts, eid))
    S = _abi.STATIC_HOP_MAX_SLOTS + 1
    node, t = hot.be.zeros(S), hot.be.zeros(S)
    out = HopResult(hot.be, S, S * 2)
    with pytest.raises(MemoryError, match="exceed the limit"):
        hot.sample_hop_static(dg, node, t, hot.params("recent", 2), out)
    # the limit itself is accepted
    node, t = hot.be.zeros(S - 1), hot.be.zeros(S - 1)
    out = HopResult(hot.be, S - 1, (S - 1) * 2)
    hot.sample_hop_static(dg, node, t, hot.params("recent", 2), out)
    torch.cuda.synchronize()
    assert int(np_of(out.counts)[0]) == S - 1
