#!/usr/bin/env python3
"""Benchmark of the temporal mini-batch hot path on one MI355X.

A step is one pass of the hot path over one batch of the 1M-node / 20M-edge
synthetic power-law graph: 2-hop most-recent 10x10 sampling, unique/compaction
of the sampled node ids, node + edge feature gather, and 2-hop uniform 10x10
sampling.  All inputs (graph, features, batches) are resident in HBM before the
timed region starts; nothing inside the region synchronises with the host.

Prints ONE JSON line: whole-step sampled edges/s as `value`, per-stage figures
under `stages`, the HBM roofline of the dominant kernel (the hop-2 edge-feature
gather) under `roofline`, and the CPU oracle sampler timed on the host cores
under `cpu_baseline`.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "starrygl-framework_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--nodes", type=int, default=1_000_000)
    ap.add_argument("--edges", type=int, default=20_000_000)
    ap.add_argument("--batch-edges", type=int, default=4000)
    ap.add_argument("--fanout", type=int, default=10)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--no-edge-feat", action="store_true", help="skip the 13.8 GB edge feature table (debug)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one 1 GiB device-to-device copy (known traffic) so that rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings can be scaled")
    ap.add_argument("--serial", action="store_true", help="capture the step as one serial chain of kernels")
    ap.add_argument("--eager", action="store_true", help="launch every kernel from the host instead of replaying a HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs the hot path of ONE GPU's partition; --gpus must be 1 "
            "(multi-GPU sharding is by graph partition and is not part of this build)")
        sys.exit(2)

    import numpy as np
    import torch
    from starrygl_amd.lib import _abi, hot_path
    from starrygl_amd.utils import synth

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(2)
    dev = torch.device("cuda:0")
    hot = hot_path(dev)
    n, m, B, k = args.nodes, args.edges, args.batch_edges, args.fanout
    t0 = time.time()
    src, dst, ts, eid, row_ptr = synth.graph_by_degree(n, m, 1.1, 1 << 40, 20242)
    log(f"[setup] graph n={n} m={m} generated in {time.time() - t0:.1f}s, max degree {int(np.diff(row_ptr).max())}")
    D = lambda a, dt="i64": hot.be.asarray(a, dt)
    dg = hot.tcsr_from_sorted(n, D(row_ptr), D(dst), D(ts), D(eid), validate=True)
    gen = torch.Generator(device=dev).manual_seed(20242)
    node_feat = torch.randn((n, 100), device=dev, generator=gen)
    edge_feat = None
    if not args.no_edge_feat:
        edge_feat = torch.empty((m, 172), device=dev)
        for lo in range(0, m, 1 << 22):
            edge_feat[lo: lo + (1 << 22)].normal_(generator=gen)
    node_cache = hot.cache(400, node_feat)
    edge_cache = hot.cache(688, edge_feat) if edge_feat is not None else None

    # batches: B consecutive events of the global time order, from the later half
    order = np.argsort(ts, kind="stable")
    NB = min(args.steps + args.warmup, 64)
    rng = np.random.default_rng(7)
    starts = np.sort(rng.integers(m // 2, m - B, NB))
    bt = [synth.link_batch(src[order[s: s + B]], dst[order[s: s + B]], ts[order[s: s + B]], 0, B, n, B, rng)
          for s in starts]
    roots = D(np.stack([b[0] for b in bt]))
    root_ts = D(np.stack([b[2] for b in bt]))
    neg = D(np.stack([b[3] for b in bt]))
    neg_ts = D(np.stack([b[4] for b in bt]))
    ts_ptr = D(bt[0][1])
    S0 = 3 * B
    log(f"[setup] {NB} batches of {B} events + {B} negatives = {S0} roots; setup {time.time() - t0:.1f}s")

    p_rec = hot.params("recent", k)
    p_uni = hot.params("uniform", k, seed=20242)
    kr, ku = hot.khop_buffers(S0, 2, k), hot.khop_buffers(S0, 2, k)
    state = hot.remap_state(n)
    total_ids = S0 + S0 * k + S0 * k * k
    local = [hot.be.empty(S0), hot.be.empty(S0 * k), hot.be.empty(S0 * k * k)]
    ubuf, U = hot.be.empty(min(total_ids, n)), hot.be.zeros(2)
    S0_dev = D(np.array([S0], dtype=np.int64))
    node_out = torch.empty((min(total_ids, n), 100), device=dev)
    e_out = [torch.empty((S0 * k, 172), device=dev), torch.empty((S0 * k * k, 172), device=dev)] if edge_cache else None
    # pre-size the shared workspace so no step allocates
    hot._workspace(max(hot.lib.sample_khop_workspace_bytes(S0, 2, k),
                       hot.lib.unique_workspace_bytes(n, 3, (_abi.i64 * 3)(S0, S0 * k, S0 * k * k))))

    # static input buffers: a step copies its batch here (4 small D2D copies), the stages read them
    s_roots, s_root_ts, s_neg, s_neg_ts = (torch.empty_like(roots[0]), torch.empty_like(root_ts[0]),
                                           torch.empty_like(neg[0]), torch.empty_like(neg_ts[0]))
    acc = torch.zeros(5, dtype=torch.int64, device=dev)   # running sums of E0, E1 (recent), E0, E1 (uniform), U

    def stage_inputs(b):
        s_roots.copy_(roots[b]); s_root_ts.copy_(root_ts[b]); s_neg.copy_(neg[b]); s_neg_ts.copy_(neg_ts[b])

    def st_recent():
        hot.sample_khop(dg, s_roots, ts_ptr, s_root_ts, s_neg, s_neg_ts, 2, p_rec, finalize=False, out=kr)

    def st_unique():
        hot.unique_compact([kr.slot_node0, kr.hops[0].neighbors, kr.hops[1].neighbors], _abi.UNIQUE_SORTED, state,
                           True, lens_dev=[S0_dev, kr.hops[0].counts[1:2], kr.hops[1].counts[1:2]],
                           out_arrays=local, finalize=False, unique_out=ubuf, U_out=U)

    def st_node():
        hot.gather(node_cache, ubuf, node_out, N_dev=U[0:1])

    def st_edge0():
        if edge_cache is not None:
            hot.gather(edge_cache, kr.hops[0].neighbors_eid, e_out[0], N_dev=kr.hops[0].counts[1:2])

    def st_edge1():
        if edge_cache is not None:
            hot.gather(edge_cache, kr.hops[1].neighbors_eid, e_out[1], N_dev=kr.hops[1].counts[1:2])

    def st_uniform():
        hot.sample_khop(dg, s_roots, ts_ptr, s_root_ts, s_neg, s_neg_ts, 2, p_uni, finalize=False, out=ku)

    def st_account():
        acc[0:2].add_(kr.counts[1::3]); acc[2:4].add_(ku.counts[1::3]); acc[4:5].add_(U[0:1])

    stages_fn = [st_recent, st_unique, st_node, st_edge0, st_edge1, st_uniform]

    def body():
        for f in stages_fn:
            f()
        st_account()

    K, W = args.steps, args.warmup
    stage_inputs(0)
    body()
    torch.cuda.synchronize()
    if args.pmc_calibration:
        cal_src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        cal_dst = torch.empty_like(cal_src)
        cal_dst.copy_(cal_src)          # 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del cal_src, cal_dst
    mode = "eager"
    graphs = None
    if not args.eager:
        # one HIP graph for the whole step (timed region) + one per stage (per-stage GPU time)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g_step = torch.cuda.CUDAGraph()
        if args.serial:
            with torch.cuda.graph(g_step):
                body()
        else:
            # independent stages become parallel branches of the graph: the uniform sampler
            # runs beside the recent one, the edge gathers beside unique + node gather
            br = [torch.cuda.Stream() for _ in range(3)]
            with torch.cuda.graph(g_step):
                cur = torch.cuda.current_stream()
                br[0].wait_stream(cur)
                with torch.cuda.stream(br[0]):
                    st_uniform()
                st_recent()
                br[1].wait_stream(cur)
                br[2].wait_stream(cur)
                with torch.cuda.stream(br[1]):
                    st_edge0()
                with torch.cuda.stream(br[2]):
                    st_edge1()
                st_unique()
                st_node()
                for b_ in br:
                    cur.wait_stream(b_)
                st_account()
        graphs = []
        for f in stages_fn:
            gs = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gs):
                f()
            graphs.append(gs)
        mode = "hipgraph" if args.serial else "hipgraph, independent stages on parallel branches"
        run_step = g_step.replay
    else:
        run_step = body
    for i in range(W):
        stage_inputs(i % NB)
        run_step()
    torch.cuda.synchronize()
    acc.zero_()
    torch.cuda.synchronize()
    # ---- timed region: exactly K steps, wall clock, no host synchronisation inside
    t_start = time.perf_counter()
    for i in range(K):
        stage_inputs((W + i) % NB)
        run_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_start
    tot = acc.cpu().numpy().astype(np.float64)
    # ---- per-stage GPU time: the same K steps, HIP events between the stages
    NEV = len(stages_fn) + 1
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(NEV)] for _ in range(K)]
    cl = np.zeros((K, 5))
    cnt_log = torch.zeros((K, 5), dtype=torch.int64, device=dev)
    for i in range(K):
        stage_inputs((W + i) % NB)
        evs[i][0].record()
        for j in range(len(stages_fn)):
            graphs[j].replay() if graphs is not None else stages_fn[j]()
            evs[i][j + 1].record()
        cnt_log[i, 0:2].copy_(kr.counts[1::3]); cnt_log[i, 2:4].copy_(ku.counts[1::3]); cnt_log[i, 4:5].copy_(U[0:1])
    torch.cuda.synchronize()
    cl = cnt_log.cpu().numpy()
    assert np.array_equal(cl.sum(axis=0).astype(np.float64), tot), "the two passes over the batches disagree"
    st = np.array([[evs[i][j].elapsed_time(evs[i][j + 1]) for j in range(NEV - 1)] for i in range(K)])  # ms
    med = np.median(st, axis=0)
    e_rec, e_uni = cl[:, 0] + cl[:, 1], cl[:, 2] + cl[:, 3]
    edges_total = int(e_rec.sum() + e_uni.sum())
    ms_per_step = wall / K * 1e3
    value = edges_total / wall

    def gbps(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0

    E0, E1, Um = float(np.median(cl[:, 0])), float(np.median(cl[:, 1])), float(np.median(cl[:, 4]))
    # algorithmic bytes: id 8 + row read + row write (all rows are HBM resident, no index entry)
    b_node, b_e0, b_e1 = Um * (8 + 800), E0 * (8 + 1376), E1 * (8 + 1376)
    # sampling: per slot 16 (node, t) + 16 row_ptr + 16 start/end ptr, per edge 24 read + 32 written
    samp_bytes = lambda S, E: S * 48 + E * 56
    b_rec = samp_bytes(S0, E0) + samp_bytes(E0, E1)
    ids_in = S0 + E0 + E1
    stages = {
        "sample_recent_2hop": {"ms": med[0], "edges_per_s": (E0 + E1) / (med[0] * 1e-3), "GBps": gbps(b_rec, med[0])},
        "unique_compact": {"ms": med[1], "ids_per_s": ids_in / (med[1] * 1e-3), "GBps": gbps(16 * ids_in + 8 * Um, med[1])},
        "gather_node_feat": {"ms": med[2], "rows": Um, "GBps": gbps(b_node, med[2])},
        "gather_edge_feat_hop1": {"ms": med[3], "rows": E0, "GBps": gbps(b_e0, med[3])},
        "gather_edge_feat_hop2": {"ms": med[4], "rows": E1, "GBps": gbps(b_e1, med[4])},
        "sample_uniform_2hop": {"ms": med[5], "edges_per_s": float(np.median(e_uni)) / (med[5] * 1e-3)},
    }
    for v in stages.values():
        for kk in v:
            v[kk] = float(round(v[kk], 4))
    dom = "gather_edge_feat_hop2" if edge_cache is not None else "gather_node_feat"
    ach = stages[dom]["GBps"]
    roofline = {"kernel": "gather_kernel<u32x4> (" + dom + ")", "bound": "hbm", "achieved": ach,
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": None,
                "avg_launch_ms": stages[dom]["ms"],
                "algorithmic_bytes_per_launch": int(b_e1 if edge_cache is not None else b_node)}

    # ---- CPU baseline: the oracle's 2-hop recent sampler on the host cores, same batches
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import oracle as O
        ora, cdll = O.load()
        threads = min(int(cdll.sglo_get_max_threads()), os.cpu_count() or 1)
        cdll.sglo_set_num_threads(threads)
        hg = ora.tcsr_from_sorted(n, row_ptr, dst, ts, eid, validate=False)
        po = ora.params("recent", k)
        # parity of batch 0 against the GPU result (the oracle as the checker)
        want = ora.sample_khop(hg, *bt[W % NB], 2, po)
        stage_inputs(W % NB)
        st_recent()
        c = kr.counts.cpu().numpy()
        assert int(c[1]) == want.hops[0].E and int(c[4]) == want.hops[1].E, "GPU and oracle disagree on edge counts"
        assert np.array_equal(kr.hops[1].neighbors_eid[: int(c[4])].cpu().numpy(), want.hops[1].neighbors_eid)
        t_cpu, edges_cpu, nb_cpu = 0.0, 0, 0
        while t_cpu < args.cpu_seconds:
            b = bt[nb_cpu % NB]
            t1 = time.perf_counter()
            r = ora.sample_khop(hg, *b, 2, po)
            t_cpu += time.perf_counter() - t1
            edges_cpu += r.hops[0].E + r.hops[1].E
            nb_cpu += 1
        cpu = {"value": round(edges_cpu / t_cpu, 1), "unit": "sampled edges/s (2-hop recent 10x10)", "cores": threads,
               "kind": "port", "sample": f"{nb_cpu} batches of {S0} roots, {edges_cpu} edges in {t_cpu:.2f}s",
               "gpu_over_cpu_sampler": round(stages["sample_recent_2hop"]["edges_per_s"] / (edges_cpu / t_cpu), 1)}

    out = {
        "metric": "sampled edges/sec (2-hop recent & uniform) + feature-gather GB/s vs HBM peak",
        "value": round(value, 1), "unit": "sampled edges/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int64", "data": "synthetic", "launch_mode": mode,
        "config": {"workload": "configs[1]: 1M nodes / 20M edges Zipf(1.1) out-degree, batches of 4000 events + 4000 "
                               "negatives (12000 roots): 2-hop recent 10x10 + unique + node/edge gather + 2-hop uniform 10x10",
                   "nodes": n, "edges": m, "roots_per_batch": S0, "fanout": [k, k],
                   "node_feat": "100xfp32", "edge_feat": "172xfp32" if edge_cache is not None else None},
        "edges_per_step": {"recent": float(np.mean(e_rec)), "uniform": float(np.mean(e_uni))},
        "stages": stages, "roofline": roofline, "cpu_baseline": cpu,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
