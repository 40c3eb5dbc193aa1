"""Synthetic power-law temporal graphs and request streams (numpy, seeded).

These generate the workloads the benchmark and the tests run on; every array
is int64 unless stated.  Everything is numpy on the host except
`graph_by_degree_device`, which builds graphs too large for that with torch on
the device it is given.
"""
import numpy as np


def zipf_degrees(n, m, a):
    """Degree sequence deg[r] ~ (r+1)^-a over ranks r, scaled to sum exactly m."""
    w = np.arange(1, n + 1, dtype=np.float64) ** (-a)
    w /= w.sum()
    deg = np.floor(w * m).astype(np.int64)
    rest = int(m - deg.sum())
    if rest > 0:  # hand the remainder to the top ranks, one edge each (wrapping)
        idx = np.arange(rest) % n
        np.add.at(deg, idx, 1)
    return deg


def graph_by_degree(n, m, a, t_max, seed, perm=True):
    """Out-degree follows Zipf(a) by rank; destinations uniform; timestamps
    uniform in [0, t_max), ascending inside every source row; eid = position
    in that (src, ts) order.  Returns (src, dst, ts, eid, row_ptr): the edge
    list is already in T-CSR order."""
    rng = np.random.Generator(np.random.PCG64(seed))
    deg_rank = zipf_degrees(n, m, a)
    ids = rng.permutation(n).astype(np.int64) if perm else np.arange(n, dtype=np.int64)
    deg = np.zeros(n, dtype=np.int64)
    deg[ids] = deg_rank
    row_ptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(deg, out=row_ptr[1:])
    src = np.repeat(np.arange(n, dtype=np.int64), deg)
    dst = rng.integers(0, n, size=m, dtype=np.int64)
    ts = rng.integers(0, t_max, size=m, dtype=np.int64)
    # sort timestamps inside each row: one global sort of (src, ts) keys
    bits = max(int(t_max - 1).bit_length(), 1)
    if bits + max(int(n - 1).bit_length(), 1) <= 62:
        key = (src << bits) | ts
        key.sort()
        ts = key & ((1 << bits) - 1)
    else:
        order = np.lexsort((ts, src))
        ts = ts[order]
    eid = np.arange(m, dtype=np.int64)
    return src, dst, ts, eid, row_ptr


def graph_stream(n, m, a, t_max, seed):
    """Edge stream in arrival order: sources iid Zipf(a) over a fixed rank->id
    permutation, destinations uniform, timestamps ascending uniform draws from
    [0, t_max); eid = arrival index."""
    rng = np.random.Generator(np.random.PCG64(seed))
    w = np.arange(1, n + 1, dtype=np.float64) ** (-a)
    w /= w.sum()
    ids = rng.permutation(n).astype(np.int64)
    src = ids[rng.choice(n, size=m, p=w)]
    dst = rng.integers(0, n, size=m, dtype=np.int64)
    ts = np.sort(rng.integers(0, t_max, size=m, dtype=np.int64))
    eid = np.arange(m, dtype=np.int64)
    return src, dst, ts, eid


def link_batch(src, dst, ts, lo, hi, n, n_neg, rng):
    """Roots of one link-prediction batch over events [lo, hi): sources, then
    destinations (positives), plus n_neg uniform negative destinations that
    reuse the event timestamps.  Every positive root has one timestamp."""
    roots = np.concatenate([src[lo:hi], dst[lo:hi]])
    root_ts = np.concatenate([ts[lo:hi], ts[lo:hi]])
    ts_ptr = np.arange(roots.shape[0] + 1, dtype=np.int64)
    neg = rng.integers(0, n, size=n_neg, dtype=np.int64)
    neg_ts = np.resize(ts[lo:hi], n_neg).astype(np.int64) if n_neg else np.zeros(0, np.int64)
    return roots, ts_ptr, root_ts, neg, neg_ts


def zipf_requests(rows, count, a, seed):
    """`count` row ids drawn Zipf(a) by access rank; rank r maps to row id r, so
    the hottest rows are the lowest ids (callers permute if they need to)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    # inverse-CDF sampling on the continuous approximation of the rank law,
    # then clipped: exact enough for a request stream and O(count) in memory
    u = rng.random(count)
    if abs(a - 1.0) < 1e-9:
        r = np.exp(u * np.log(rows + 1.0))
    else:
        b = 1.0 - a
        r = (1.0 + u * ((rows + 1.0) ** b - 1.0)) ** (1.0 / b)
    return np.clip(np.floor(r).astype(np.int64) - 1, 0, rows - 1)


def graph_by_degree_device(torch, device, n, m, a, max_deg, t_bits, seed, dst_by_degree=True):
    """A T-CSR of n nodes and m edges generated on `device` with torch: out-degree
    Zipf(a) by rank, capped at max_deg and scaled to sum m, node ids a random
    permutation of the ranks; timestamps uniform in [0, 2^t_bits), ascending
    inside every row; destinations drawn in proportion to out-degree (or
    uniformly); eid = storage position.  Needs bit_length(n - 1) + t_bits <= 63.
    Returns (row_ptr, col, ts, eid, key) with key[e] = src[e] << t_bits | ts[e],
    ascending over the whole edge list: a searchsorted over it finds any row's
    time window without walking the CSR."""
    assert max(int(n - 1).bit_length(), 1) + t_bits <= 63
    gen = torch.Generator(device=device).manual_seed(seed)
    w = torch.arange(1, n + 1, device=device, dtype=torch.float64).pow_(-a)

    def degrees(c):
        return torch.clamp((w * c).floor_(), max=float(max_deg)).to(torch.int64)

    lo, hi = 0.0, max_deg / float(w[-1])
    for _ in range(60):           # largest scale whose floor-and-cap degrees stay within m
        mid = 0.5 * (lo + hi)
        if int(degrees(mid).sum()) <= m:
            lo = mid
        else:
            hi = mid
    deg_rank = degrees(lo)
    rest = m - int(deg_rank.sum())
    deg_rank += rest // n
    if rest % n:
        deg_rank[n - rest % n:] += 1          # the remainder goes to the tail ranks, one edge each
    del w
    ids = torch.randperm(n, device=device, generator=gen)
    deg = torch.empty_like(deg_rank)
    deg[ids] = deg_rank
    del ids, deg_rank
    row_ptr = torch.zeros(n + 1, dtype=torch.int64, device=device)
    torch.cumsum(deg, 0, out=row_ptr[1:])
    key = torch.repeat_interleave(torch.arange(n, device=device), deg, output_size=m)
    del deg
    key.mul_(1 << t_bits)
    key.add_(torch.randint(0, 1 << t_bits, (m,), device=device, generator=gen))
    key = torch.sort(key).values
    ts = key & ((1 << t_bits) - 1)
    if dst_by_degree:
        col = key[torch.randint(0, m, (m,), device=device, generator=gen)]
        col >>= t_bits
    else:
        col = torch.randint(0, n, (m,), device=device, generator=gen)
    eid = torch.arange(m, device=device)
    return row_ptr, col, ts, eid, key


def zipf_exponent_for_duplicates(rows, count, target_dup, seed, tol=0.01):
    """The exponent a for which `count` requests drawn Zipf(a) over `rows` ranks (zipf_requests) repeat an
    earlier request with probability ~ target_dup (found by bisection on the measured duplicate fraction;
    Zipf(1.1) itself gives about 0.8 at 2M requests over 50M rows)."""
    lo, hi = 0.0, 2.0
    a = 1.0
    for _ in range(24):
        a = 0.5 * (lo + hi)
        dup = 1.0 - np.unique(zipf_requests(rows, count, a, seed)).size / count
        if abs(dup - target_dup) <= tol:
            break
        if dup < target_dup:
            lo = a
        else:
            hi = a
    return a


def row_content(torch, ids, dim):
    """int16 payload (any bit pattern is a valid bf16 row) of the rows `ids` of a synthetic table: a function of
    the row id alone, so that a gathered row can be checked without keeping a second copy of the table."""
    base = (ids * 2654435761 % 65521).to(torch.int32).unsqueeze(1)
    return ((base + torch.arange(dim, device=ids.device, dtype=torch.int32)) & 0x7FFF).to(torch.int16)


def two_tier_table(torch, device, rows, dim, hot_frac, seed):
    """A rows x dim int16 table whose hottest hot_frac of rows by access rank live on `device` and all rows
    in pinned host memory; rank r maps to row rank_to_id[r] (a random permutation), content = row_content.
    Returns (rank_to_id, hot_slot[int32], hot_table, cold_table)."""
    g = torch.Generator(device=device).manual_seed(seed)
    hot_rows = int(rows * hot_frac)
    rank_to_id = torch.randperm(rows, device=device, generator=g)
    hot_slot = torch.full((rows,), -1, dtype=torch.int32, device=device)
    hot_slot[rank_to_id[:hot_rows]] = torch.arange(hot_rows, dtype=torch.int32, device=device)
    hot_tab = torch.empty((hot_rows, dim), dtype=torch.int16, device=device)
    for lo in range(0, hot_rows, 1 << 20):
        hot_tab[lo: lo + (1 << 20)] = row_content(torch, rank_to_id[lo: min(lo + (1 << 20), hot_rows)], dim)
    cold = torch.empty((rows, dim), dtype=torch.int16, pin_memory=True)
    for lo in range(0, rows, 1 << 22):
        hi = min(lo + (1 << 22), rows)
        cold[lo:hi].copy_(row_content(torch, torch.arange(lo, hi, device=device), dim))
    torch.cuda.synchronize(device)
    return rank_to_id, hot_slot, hot_tab, cold
