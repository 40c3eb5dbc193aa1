"""GPU parity at the full size of configs[4]: one GPU's share of a partitioned TGN step - 2.5M local nodes,
60M edges (Zipf(1.1) out-degrees), batches of 2000 events + 2000 negatives; 1-hop most-recent-10 sampling,
unique, gather of TGN memory (+ int64 last-update time), node features and edge features with 30 % of the node
rows served from pinned host memory, cos time encoding to 100 dims - against the CPU oracle and numpy for three
batches, stage by stage (the path of starrygl/graph/graph.py:58-110, starrygl/cache/NodeState.py:36-44 and
starrygl/nn/model/time_encoder.py:29-31)."""
import numpy as np
import psutil
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth
from util import assert_hop_equal, np_of, to_dev

pytestmark = pytest.mark.gpu
N, M, B, K, REMOTE = 2_500_000, 60_000_000, 2000, 10, 0.30


@pytest.fixture(scope="module")
def world(oracle, hot):
    free, _ = torch.cuda.mem_get_info()
    if free < 60 << 30 or psutil.virtual_memory().available < 28 << 30:
        pytest.skip("needs 60 GB of free HBM and 28 GB of host memory")
    dev = hot.be.device
    src, dst, ts, eid, row_ptr = synth.graph_by_degree(N, M, 1.1, 1 << 40, 20245)
    hg = oracle.tcsr_from_sorted(N, row_ptr, dst, ts, eid, validate=False)
    dg = hot.tcsr_from_sorted(N, *(to_dev(hot, x) for x in (row_ptr, dst, ts, eid)), validate=True)
    hot.build_hop_hint(dg)
    rng = np.random.default_rng(9)
    remote = rng.random(N) < REMOTE
    local_ids = np.flatnonzero(~remote)
    slot = np.full(N, -1, dtype=np.int32)
    slot[local_ids] = np.arange(local_ids.size, dtype=np.int32)
    d_slot = to_dev(hot, slot, "i32")
    mem = rng.standard_normal((N, 100), dtype=np.float32)
    mem_ts = rng.integers(0, 1 << 40, N)
    nfeat = rng.standard_normal((N, 100), dtype=np.float32)

    def tiered(full):
        cold = torch.from_numpy(full).pin_memory()
        keep = full.copy()
        hot_t = torch.from_numpy(keep[local_ids]).to(dev)
        return hot_t, cold

    mem_hot, mem_cold = tiered(mem)
    ts_hot, ts_cold = tiered(mem_ts)
    nf_hot, nf_cold = tiered(nfeat)
    c_mem = hot.cache(400, mem_hot, rows=N, cold=mem_cold, hot_slot=d_slot, ts_hot=ts_hot, ts_cold=ts_cold)
    c_nf = hot.cache(400, nf_hot, rows=N, cold=nf_cold, hot_slot=d_slot)
    # the layout of the benchmark's step: one record per node in either tier (memory | features, and the time on the
    # host side: 896 bytes = seven 128-byte lines per remote node instead of 4 + 4 + 1 from three tables)
    node_hot = torch.cat([mem_hot, nf_hot], dim=1).contiguous()
    node_cold, ts_rec, _rec = hot.interleaved_cold(N, 200)
    node_cold[:, :100].copy_(mem_cold); node_cold[:, 100:].copy_(nf_cold); ts_rec.copy_(ts_cold)
    c_node = hot.cache(800, node_hot, rows=N, cold=node_cold, hot_slot=d_slot, ts_hot=ts_hot, ts_cold=ts_rec)
    g = torch.Generator(device=dev).manual_seed(5)
    efeat = torch.empty((M, 172), device=dev)
    for lo in range(0, M, 1 << 22):
        efeat[lo: lo + (1 << 22)].normal_(generator=g)
    c_ef = hot.cache(688, efeat)
    order = np.argsort(ts, kind="stable")
    yield dict(src=src, dst=dst, ts=ts, hg=hg, dg=dg, order=order, mem=mem, mem_ts=mem_ts, nfeat=nfeat, efeat=efeat,
               c_mem=c_mem, c_nf=c_nf, c_ef=c_ef, c_node=c_node, remote=remote)
    torch.cuda.empty_cache()


@pytest.mark.parametrize("start", [M // 2, (3 * M) // 4, M - B])
def test_tgn_step_parity(oracle, hot, world, start):
    w, rng, dev = world, np.random.default_rng(start), hot.be.device
    ev = w["order"][start: start + B]
    b = synth.link_batch(w["src"][ev], w["dst"][ev], w["ts"][ev], 0, B, N, B, rng)
    d = [to_dev(hot, x) for x in b]
    S0 = 3 * B
    # ---- stage 1: 1-hop most-recent-10 with the batch's root hints, ids recorded for unique
    ends = hot.window_end(w["dg"], d[0], d[2])
    state = hot.remap_state(N)
    p = hot.marking(hot.with_root_hint(hot.params("recent", K), ends), state)
    kr = hot.sample_khop(w["dg"], *d, 1, p, finalize=False)
    want = oracle.sample_khop(w["hg"], *b, 1, oracle.params("recent", K))
    # ---- stage 2: unique over roots + neighbours (device-side lengths, the sampler's marks)
    E_dev = kr.hops[0].counts[1:2]
    arrays = [kr.slot_node0, kr.hops[0].neighbors]
    local, uniq, (total, _) = hot.unique_compact(arrays, _abi.UNIQUE_SORTED, state, True,
                                                 lens_dev=[to_dev(hot, np.array([S0])), E_dev], premarked=True)
    kr.finalize()
    assert_hop_equal(kr.hops[0], want.hops[0], tag=f"start={start}")
    E = want.hops[0].E
    u, inv = np.unique(np.concatenate([want.slot_node0, want.hops[0].neighbors]), return_inverse=True)
    assert total == u.size and np.array_equal(np_of(uniq), u)
    assert np.array_equal(np_of(local[0]), inv[:S0]) and np.array_equal(np_of(local[1])[:E], inv[S0:])
    # ---- stage 3: memory (+ last update), node and edge rows in one launch, 30 % of the node rows from the host
    o_mem = torch.empty((total, 100), device=dev)
    o_ts = hot.be.empty(total)
    o_nf = torch.empty((total, 100), device=dev)
    o_ef = torch.empty((E, 172), device=dev)
    stats = hot.be.zeros(3)
    hot.gather_multi(hot.gather_plan([(w["c_mem"], uniq, o_mem, o_ts, None), (w["c_nf"], uniq, o_nf, None, None),
                                      (w["c_ef"], kr.hops[0].neighbors_eid, o_ef, None, None)]))
    hot.gather(w["c_mem"], uniq, torch.empty_like(o_mem), stats=stats)
    assert np.array_equal(np_of(o_mem), w["mem"][u]) and np.array_equal(np_of(o_ts), w["mem_ts"][u])
    assert np.array_equal(np_of(o_nf), w["nfeat"][u])
    assert torch.equal(o_ef, w["efeat"][kr.hops[0].neighbors_eid])
    # the same rows through the one-record-per-node layout: [U, 200] = memory | features, one segment
    o_node, o_ts2 = torch.empty((total, 200), device=dev), hot.be.empty(total)
    hot.gather_multi(hot.gather_plan([(w["c_node"], uniq, o_node, o_ts2, None), (w["c_ef"], kr.hops[0].neighbors_eid, o_ef, None, None)]))
    assert np.array_equal(np_of(o_node[:, :100]), w["mem"][u]) and np.array_equal(np_of(o_node[:, 100:]), w["nfeat"][u])
    assert np.array_equal(np_of(o_ts2), w["mem_ts"][u])
    n_remote = int(w["remote"][u].sum())
    assert np_of(stats).tolist() == [u.size - n_remote, n_remote, 0] and 0.2 < n_remote / u.size < 0.4
    # ---- stage 4: time encoding of the sampled edges' dt
    wv = (1.0 / 10 ** np.linspace(0, 9, 100, dtype=np.float32)).astype(np.float32)
    bias = np.zeros(100, np.float32)
    y = np_of(hot.time_encode(kr.hops[0].neighbors_dt, to_dev(hot, wv, "f32"), to_dev(hot, bias, "f32")))
    y_ref = oracle.time_encode(want.hops[0].neighbors_dt, wv, bias)
    assert np.abs(y - y_ref).max() <= 1e-6        # |y| <= 1: 1e-6 relative of fp32 range
