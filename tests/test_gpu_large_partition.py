"""Full-size run of the 100M-node / 1B-edge single-partition case: 50 000 roots,
2-hop most-recent 20x20, unique/compaction of every sampled id and block
construction, checked through properties that do not need the CPU oracle at
that size:

* the time window of any (node, t) slot is found independently of the CSR by
  one library `searchsorted` over the globally ascending key src << 36 | ts, so
  every output array of both hops is compared bit-exact with index algebra in
  torch;
* unique/compaction: sorted mode (dense-table and hash-set path) equals
  torch.unique(return_inverse); in grouped mode unique[local] gives back every
  input id, there are no duplicates and the groups (roots, hop 1, hop 2) are
  each ascending;
* blocks: expanding indptr gives back edge_dst, indices are consecutive.
"""
import pytest
import torch

from starrygl_amd.lib import _abi
from starrygl_amd.utils import synth

pytestmark = pytest.mark.gpu

N, M, T_BITS, K, R = 100_000_000, 1_000_000_000, 36, 20, 50_000


@pytest.fixture(scope="module")
def big(hot):
    dev = hot.be.device
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 120 << 30:
        pytest.skip("needs 120 GB of free HBM")
    row_ptr, col, ts, eid, key = synth.graph_by_degree_device(torch, dev, N, M, 1.05, 1_000_000, T_BITS, 20243)
    g = hot.tcsr_from_sorted(N, row_ptr, col, ts, eid, validate=True)       # sortedness checked on the device
    gen = torch.Generator(device=dev).manual_seed(1)
    roots = key[torch.randint(0, M, (R,), device=dev, generator=gen)] >> T_BITS
    root_ts = torch.randint(0, 1 << T_BITS, (R,), device=dev, generator=gen)
    yield g, key, roots, root_ts
    del g, key, row_ptr, col, ts, eid
    torch.cuda.empty_cache()


def _expect(g, key, slot_node, slot_ts, k):
    hi = torch.searchsorted(key, (slot_node << T_BITS) | slot_ts)     # first edge of the row at or after t
    lo = torch.maximum(hi - k, g.row_ptr[slot_node])
    cnt = hi - lo
    rsp = torch.zeros(cnt.numel() + 1, dtype=torch.int64, device=cnt.device)
    torch.cumsum(cnt, 0, out=rsp[1:])
    E = int(rsp[-1])
    idx = torch.repeat_interleave(lo - rsp[:-1], cnt, output_size=E) + torch.arange(E, device=cnt.device)
    t_root = torch.repeat_interleave(slot_ts, cnt, output_size=E)
    return rsp, idx, t_root


def test_two_hop_recent_unique_block_at_full_size(hot, big):
    g, key, roots, root_ts = big
    dev = roots.device
    empty = torch.empty(0, dtype=torch.int64, device=dev)
    ts_ptr = torch.arange(R + 1, device=dev)
    kr = hot.sample_khop(g, roots, ts_ptr, root_ts, empty, empty, 2, hot.params("recent", K))
    assert g.m == M and torch.equal(kr.slot_node0, roots)
    slot_node, slot_ts = roots, root_ts
    for l, h in enumerate(kr.hops):
        rsp, idx, t_root = _expect(g, key, slot_node, slot_ts, K)
        assert h.S == slot_node.numel() and h.E == idx.numel(), (l, h.S, h.E, idx.numel())
        assert torch.equal(h.root_start_ptr, rsp)
        assert torch.equal(h.root_end_ptr[:-1], rsp[1:]) and int(h.root_end_ptr[-1]) == h.E
        assert torch.equal(h.neighbors_eid, idx)                 # eid = storage position in this graph
        assert torch.equal(h.neighbors, g.col[idx])
        assert torch.equal(h.neighbors_ts, g.ts[idx])
        assert torch.equal(h.neighbors_dt, g.ts[idx] - t_root)
        assert bool((h.neighbors_dt < 0).all())                  # strictly before the root's time
        slot_node, slot_ts = h.neighbors, h.neighbors_ts
        del rsp, idx, t_root
    assert kr.hops[1].E > 10_000_000                             # the case is the size it claims to be

    arrays = [kr.slot_node0, kr.hops[0].neighbors, kr.hops[1].neighbors]
    state = hot.remap_state(N)
    local, unique, (U, before) = hot.unique_compact(arrays, _abi.UNIQUE_GROUPED, state, True)
    want, inverse = torch.unique(torch.cat(arrays), return_inverse=True)
    assert before == 0 and U == want.numel()
    for a, loc in zip(arrays, local):
        assert torch.equal(unique[loc], a)
    assert torch.unique(unique).numel() == U
    # groups: ids first seen in the roots, then in hop 1, then in hop 2, each ascending
    bounds = [0] + [int(loc.max()) + 1 if loc.numel() else 0 for loc in local]
    bounds = [max(bounds[: i + 1]) for i in range(len(bounds))]
    assert bounds[-1] == U
    for a, b in zip(bounds[:-1], bounds[1:]):
        seg = unique[a:b]
        assert bool((seg[1:] > seg[:-1]).all())

    # the hash-set path (no dense table) in sorted mode is torch.unique(return_inverse) itself,
    # and so is the dense path in sorted mode
    for st in (None, state):
        local_s, unique_s, (U_s, _) = hot.unique_compact(arrays, _abi.UNIQUE_SORTED, st, True)
        assert U_s == U and torch.equal(unique_s, want)
        assert torch.equal(torch.cat(local_s), inverse)

    dst_offset = 0
    for h in kr.hops:
        counts = torch.tensor([h.S, h.E, 0], device=dev)
        indptr, indices, edge_dst = hot.block_build(h.root_start_ptr, counts, h.S, h.E, dst_offset, h.S + dst_offset,
                                                    with_edge_dst=True)
        deg = indptr[1:] - indptr[:-1]
        assert int(indptr[-1]) == h.E and bool((deg[:dst_offset] == 0).all())
        assert torch.equal(torch.repeat_interleave(torch.arange(deg.numel(), device=dev), deg, output_size=h.E), edge_dst)
        assert torch.equal(indices, torch.arange(h.E, device=dev) + h.S + dst_offset)


def test_tcsr_build_at_full_size(hot):
    """T-CSR build from 1B shuffled edges (100M nodes): row_ptr is the cumulated degree sequence, the
    permutation returned as eid maps every output edge to its input edge, rows ascend in (ts, eid)."""
    dev = hot.be.device
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 160 << 30:
        pytest.skip("needs 160 GB of free HBM")
    gen = torch.Generator(device=dev).manual_seed(3)
    src = torch.randint(0, N, (M,), device=dev, generator=gen)
    dst = torch.randint(0, N, (M,), device=dev, generator=gen)
    ts = torch.randint(0, 1 << 20, (M,), device=dev, generator=gen)      # ~1000 edges per timestamp: plenty of ties
    g = hot.tcsr_build(N, src, dst, ts, None)
    deg = torch.bincount(src, minlength=N)
    assert int(g.row_ptr[0]) == 0 and torch.equal(g.row_ptr[1:] - g.row_ptr[:-1], deg)
    assert torch.equal(g.col, dst[g.eid]) and torch.equal(g.ts, ts[g.eid])
    rows = torch.repeat_interleave(torch.arange(N, device=dev), deg, output_size=M)
    assert torch.equal(rows, src[g.eid])
    del deg
    same = rows[1:] == rows[:-1]
    del rows
    assert bool((g.ts[1:][same] >= g.ts[:-1][same]).all())
    tie = same & (g.ts[1:] == g.ts[:-1])
    assert int(tie.sum()) > 0 and bool((g.eid[1:][tie] > g.eid[:-1][tie]).all())
