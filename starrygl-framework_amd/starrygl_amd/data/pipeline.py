"""One mini-batch of the temporal hot path as a single pre-planned unit.

The reference assembles a training batch in its (unpublished) `starrygl.data`
package: `AsyncPipelineLoader` asks the graph engine for samples and a
`GraphCollator` turns them into blocks plus feature / memory futures
(call sites: test/test.py:201-221, test/test_dataloader.py:119-149; consumers
starrygl/nn/model/tgn.py:119-196).  `MiniBatchPipeline` is that unit for one GPU:

    roots (+ negatives) -> k-hop sampling -> unique / local ids -> node, memory
    and edge row gathers -> cos time encoding of every hop's dt

All buffers are allocated once for the worst case, no stage synchronises with
the host, live sizes stay on the device; with `use_graph=True` the whole chain
is captured into one HIP graph on the first batch and replayed afterwards (a
batch then costs a few small copies plus one graph launch).
"""
import torch

from ..graph.graph import Block
from ..lib import _abi, hot_path
from ..lib.driver import POISON, check_sample_bad, check_unique_total, graph_capture


class MiniBatch:
    """Result of one pipeline run.  Device tensors are worst-case sized until
    `finalize()` reads the live counts once and narrows them."""

    def __init__(self, pipe):
        self._p = pipe
        self.final = False

    def finalize(self):
        if self.final:
            return self
        p = self._p
        if p._done is not None:      # the batch ran on the pipeline's own stream
            p._done.synchronize()
        c = p.live.tolist()
        u_total = int(c[3 * p.layers])
        if u_total == POISON or max(c[3 * l + 2] for l in range(p.layers)) >= POISON:
            # a block of a single-launch kernel gave up its bounded wait: the batch (still in the pipeline's input
            # buffers) is re-issued through the launch-per-stage routes, which have no such wait
            p._recover()
            c = p.live.tolist()
            u_total = int(c[3 * p.layers])
        check_unique_total(u_total)
        check_sample_bad(max(c[3 * l + 2] for l in range(p.layers)))
        check_sample_bad(sum(c[3 * l + 2] for l in range(p.layers)))
        self.S = [c[3 * l] for l in range(p.layers)]
        self.E = [c[3 * l + 1] for l in range(p.layers)]
        self.num_unique = u_total
        self.slot_node, self.slot_ts = p.kr.slot_node0[: self.S[0]], p.kr.slot_ts0[: self.S[0]]
        self.slot_local = p.local[0][: self.S[0]]
        self.nid_mapper = p.ubuf[:u_total]
        self.hops = []
        for l, h in enumerate(p.kr.hops):
            S, E = self.S[l], self.E[l]
            self.hops.append(dict(root_start_ptr=h.root_start_ptr[: S + 1], root_end_ptr=h.root_end_ptr[: S + 1],
                                  neighbors=h.neighbors[:E], neighbors_local=p.local[1 + l][:E],
                                  neighbors_ts=h.neighbors_ts[:E], neighbors_eid=h.neighbors_eid[:E],
                                  neighbors_dt=h.neighbors_dt[:E]))
        self.node_data = {k: v[:u_total] for k, v in p.node_out.items()}
        self.node_ts = {k: v[:u_total] for k, v in p.node_ts_out.items()}
        self.edge_data = [{k: v[l][: self.E[l]] for k, v in p.edge_out.items()} for l in range(p.layers)]
        self.time_feat = [t[: self.E[l]] for l, t in enumerate(p.te_out)] if p.te_out else None
        self.final = True
        return self

    def blocks(self, self_loop=True):
        """Message-flow blocks, outermost hop first (AsyncBlock.to_block order);
        node ids inside the blocks are LOCAL ids (rows of node_data)."""
        self.finalize()
        hp = self._p.hp
        last_nodes, last_ts = self.slot_local, self.slot_ts
        out = []
        for l, h in enumerate(self.hops):
            S, E, n_prev = self.S[l], self.E[l], int(last_nodes.numel())
            dst_off = n_prev - S if self_loop else 0
            num_dst = n_prev if self_loop else S
            src_off = num_dst if self_loop else 0
            counts = self._p.kr.hops[l].counts
            indptr, indices, _ = hp.block_build(h["root_start_ptr"], counts, S, E, dst_off, src_off)
            b = Block(indptr, indices, src_off + E, num_dst)
            if self_loop:
                b.srcdata["nid"] = torch.cat([last_nodes, h["neighbors_local"]])
                b.srcdata["ts"] = torch.cat([last_ts, h["neighbors_ts"]])
            else:
                b.srcdata["nid"], b.srcdata["ts"] = h["neighbors_local"], h["neighbors_ts"]
            b.edata["eid"], b.edata["dt"] = h["neighbors_eid"], h["neighbors_dt"]
            for k, v in self.edge_data[l].items():
                b.edata[k] = v
            if self.time_feat is not None:
                b.edata["time_feat"] = self.time_feat[l]
            last_nodes, last_ts = b.srcdata["nid"], b.srcdata["ts"]
            out.append(b)
        out.reverse()
        return out


class MiniBatchPipeline:
    def __init__(self, graph, num_pos_slots, num_neg, layers, fanout, sample_type="recent", node_tables=None,
                 edge_tables=None, time_encoder=None, allowed_offset=-1, equal_root_time=False,
                 keep_root_time=False, seed=0, use_graph=True, stream=None, root_hints=False, remap="dense",
                 remap_capacity=None):
        """graph: the native graph object (`pyGraph.g`, i.e. `CUDAGraph`).
        num_pos_slots / num_neg: positive root timestamps and negatives per batch
        (fixed, they size every buffer).  node_tables / edge_tables: name ->
        `sgl_cache` (from `HotPath.cache`) gathered for the unique nodes / the
        sampled edge ids; a node table with timestamps also yields node_ts[name].
        time_encoder: (w, b) fp32 device tensors, or a TimeEncoder module.
        root_hints: every run() also takes `root_hint`, the window ends of the positive slots
        (`graph.window_end(roots, root_ts)`, which a loader looks up once for all the events it will
        train on; -1 = search): those roots are then sampled without a search.
        remap: "dense" numbers the batch's ids through a table over the graph's n nodes (the sampler marks the ids
        it emits there, unique skips its first pass); "hashed" through the LDS-staged hash set, whose state is sized
        by `remap_capacity` distinct ids per batch (default: the batch's worst case) and not by n - for graphs whose
        id space has no room for a table per pipeline.  Same local ids either way.
        stream: run every batch on this stream instead of the caller's current one (see
        MiniBatchPipelinePool); inputs handed to run() must then be complete on the host side
        or long-lived, and results are read through MiniBatch.finalize(), which waits for it."""
        self.g = graph
        self.hp = hp = graph._hp
        self.dev = hp.be.device
        self.layers, self.fanout = int(layers), int(fanout)
        self.S_pos, self.N_neg = int(num_pos_slots), int(num_neg)
        self.S0 = self.S_pos + self.N_neg
        self.p = hp.params(sample_type, fanout, allowed_offset, equal_root_time, keep_root_time, seed=seed)
        self.node_tables, self.edge_tables = dict(node_tables or {}), dict(edge_tables or {})
        if time_encoder is not None and not isinstance(time_encoder, tuple):
            time_encoder = (time_encoder.w.weight.detach().reshape(-1).contiguous(),
                            time_encoder.w.bias.detach().contiguous())
        self.te = time_encoder
        be = hp.be
        # static inputs
        self.in_roots, self.in_ts = be.empty(self.S_pos), be.empty(self.S_pos)
        self.in_neg, self.in_neg_ts = be.empty(self.N_neg), be.empty(self.N_neg)
        self.ts_ptr = torch.arange(self.S_pos + 1, dtype=torch.int64, device=self.dev)
        self.in_hint = be.empty(self.S_pos) if root_hints else None
        if root_hints:
            self.p = hp.with_root_hint(self.p, self.in_hint)
        # outputs
        # every device-side count of a batch in one array: finalize() reads them with one copy
        self.live = be.zeros(3 * self.layers + 2)
        self.kr = hp.khop_buffers(self.S0, self.layers, self.fanout, counts=self.live[: 3 * self.layers])
        caps = [self.S0] + [self.S0 * self.fanout ** (l + 1) for l in range(self.layers)]
        self.local = [be.empty(c) for c in caps]
        self.ucap = min(sum(caps), graph._n)
        self.ubuf, self.U = be.empty(max(self.ucap, 1)), self.live[3 * self.layers:]
        if remap not in ("dense", "hashed"):
            raise ValueError("remap must be 'dense' or 'hashed'")
        self.hashed = remap == "hashed"
        if self.hashed:
            self.state = hp.remap_hashed_state(int(remap_capacity) if remap_capacity else max(self.ucap, 1))
        else:
            self.state = hp.remap_state(graph._n)
            # the sampler records the ids it emits as pending in the remap state: unique skips its first pass
            self.p = hp.marking(self.p, self.state)
        self.S0_dev = torch.tensor([self.S0], dtype=torch.int64, device=self.dev)
        f32 = torch.float32
        self.node_out, self.node_ts_out, self.edge_out = {}, {}, {}
        for name, c in self.node_tables.items():
            self.node_out[name] = torch.empty((self.ucap, c.row_bytes), dtype=torch.uint8, device=self.dev)
            if c.ts_hot or c.ts_cold:
                self.node_ts_out[name] = be.empty(self.ucap)
        for name, c in self.edge_tables.items():
            self.edge_out[name] = [torch.empty((caps[l + 1], c.row_bytes), dtype=torch.uint8, device=self.dev)
                                   for l in range(self.layers)]
        self.te_out = None
        if self.te is not None:
            dim = int(self.te[0].numel())
            self.te_out = [torch.empty((caps[l + 1], dim), dtype=f32, device=self.dev) for l in range(self.layers)]
        self._views = {}
        # the unique stage's scratch belongs to this pipeline: its pointer is baked into the pipeline's HIP
        # graph, and graphs of different pipelines replay side by side on different streams
        lens_c = (_abi.i64 * (1 + self.layers))(*caps)
        need = (hp.lib.unique_hashed_workspace_bytes(self.state.universe, 1 + self.layers, lens_c) if self.hashed
                else hp.lib.unique_workspace_bytes(graph._n, 1 + self.layers, lens_c))
        self.uws = be.empty(max(int(need), 256), "u8")
        self.use_graph, self._graph = use_graph, None
        self._plans, self._slow = None, []
        self.stream = stream
        self._done = torch.cuda.Event() if stream is not None else None

    def view(self, name, dtype):
        """Reinterpret the byte output buffers of table `name` as rows of `dtype`."""
        key = (name, dtype)
        if key not in self._views:
            if name in self.node_out:
                self.node_out[name] = self.node_out[name].view(dtype)
            if name in self.edge_out:
                self.edge_out[name] = [t.view(dtype) for t in self.edge_out[name]]
            self._views[key] = True
        return self

    def _recover(self):
        """Run the batch in the input buffers again, eagerly, with every kernel that exchanges totals inside one
        launch replaced by its multi-launch route, after initialising the remap state again."""
        hp = self.hp
        cur = torch.cuda.current_stream(self.dev)
        with torch.cuda.stream(self.stream if self.stream is not None else cur):
            hp._reinit_marked(self.p)
            if self.hashed:          # a hashed state whose capacity an epoch outgrew stays void until it is initialised again
                be = hp.be
                hp._ck(hp.lib.remap_hashed_init(be.ptr(self.state.buf), be.nbytes(self.state.buf), self.state.universe, be.stream()))
            self._chain(multi_launch=True)
            torch.cuda.current_stream(self.dev).synchronize()
        hp.recoveries += 1

    def _chain(self, multi_launch=False):
        hp, kr = self.hp, self.kr
        hp.sample_khop(self.g._g, self.in_roots, self.ts_ptr, self.in_ts, self.in_neg, self.in_neg_ts, self.layers,
                       hp.multi_launch(self.p) if multi_launch else self.p, finalize=False, out=kr)
        arrays = [kr.slot_node0] + [h.neighbors for h in kr.hops]
        lens = [self.S0_dev] + [h.counts[1:2] for h in kr.hops]
        hp.unique_compact(arrays, _abi.UNIQUE_SORTED | (_abi.UNIQUE_MULTI_LAUNCH if multi_launch and not self.hashed else 0), self.state, True,
                          lens_dev=lens, out_arrays=self.local, finalize=False, unique_out=self.ubuf, U_out=self.U,
                          premarked=not self.hashed, workspace=self.uws)
        if self._plans is None:      # every gather of the batch in as few launches as possible
            segs = [(c, self.ubuf, self.node_out[name], self.node_ts_out.get(name), self.U[0:1])
                    for name, c in self.node_tables.items()]
            segs += [(c, h.neighbors_eid, self.edge_out[name][l], None, h.counts[1:2])
                     for l, h in enumerate(kr.hops) for name, c in self.edge_tables.items()]
            fast = [s for s in segs if s[0].row_bytes % 16 == 0]
            self._slow = [s for s in segs if s[0].row_bytes % 16 != 0]
            self._plans = [hp.gather_plan(fast[i: i + 8]) for i in range(0, len(fast), 8)]
        for plan in self._plans:
            hp.gather_multi(plan)
        for c, ids, out, out_ts, n_dev in self._slow:
            hp.gather(c, ids, out, out_ts=out_ts, N_dev=n_dev)
        for l, h in enumerate(kr.hops):
            if self.te is not None:
                hp.time_encode(h.neighbors_dt, self.te[0], self.te[1], out=self.te_out[l], N_dev=h.counts[1:2])

    def run(self, roots, root_ts, neg_roots=None, neg_ts=None, root_hint=None):
        """Enqueue one batch (asynchronous).  `roots`/`root_ts`: S_pos ids and
        timestamps (one timestamp per root); `neg_roots`/`neg_ts`: N_neg each; `root_hint`: S_pos
        window ends, for a pipeline built with root_hints=True."""
        if roots.numel() != self.S_pos or root_ts.numel() != self.S_pos:
            raise ValueError(f"this pipeline was planned for {self.S_pos} positive slots")
        if (self.in_hint is None) != (root_hint is None) or (root_hint is not None and root_hint.numel() != self.S_pos):
            raise ValueError("root_hint goes with a pipeline built with root_hints=True, one entry per positive slot")
        if self.N_neg and (neg_roots is None or neg_roots.numel() != self.N_neg or neg_ts.numel() != self.N_neg):
            raise ValueError(f"this pipeline was planned for {self.N_neg} negatives")
        if self.stream is not None:
            with torch.cuda.stream(self.stream):
                out = self._run(roots, root_ts, neg_roots, neg_ts, root_hint)
                self._done.record(self.stream)
            return out
        return self._run(roots, root_ts, neg_roots, neg_ts, root_hint)

    def _run(self, roots, root_ts, neg_roots, neg_ts, root_hint):
        dsts, srcs = [self.in_roots, self.in_ts], [roots, root_ts]
        if root_hint is not None:
            dsts.append(self.in_hint); srcs.append(root_hint)
        if self.N_neg:
            dsts += [self.in_neg, self.in_neg_ts]; srcs += [neg_roots, neg_ts]
        if all(t.is_cuda and t.dtype == torch.int64 and t.is_contiguous() for t in srcs):
            torch._foreach_copy_(dsts, [t.reshape(-1) for t in srcs], non_blocking=True)   # one launch for all inputs
        else:
            for d, t in zip(dsts, srcs):
                d.copy_(t.reshape(-1), non_blocking=True)
        if not self.use_graph:
            self._chain()
        elif self._graph is None:
            self._chain()                      # warm-up outside capture (also the result of this call)
            torch.cuda.current_stream(self.dev).synchronize()
            side = torch.cuda.Stream(self.dev)
            side.wait_stream(torch.cuda.current_stream(self.dev))
            with torch.cuda.stream(side):
                self._chain()
            torch.cuda.current_stream(self.dev).wait_stream(side)
            torch.cuda.current_stream(self.dev).synchronize()
            g = torch.cuda.CUDAGraph()
            with graph_capture(g):
                self._chain()
            self._graph = g
            g.replay()
        else:
            self._graph.replay()
        return MiniBatch(self)


def bound_streams(n, device):
    """n streams, each used once: a HIP stream gets its hardware queue at first use, and streams that
    share a queue take turns instead of overlapping.  Call this before other streams are created."""
    streams = [torch.cuda.Stream(device) for _ in range(n)]
    for st in streams:
        with torch.cuda.stream(st):
            torch.zeros(1, device=device).add_(1)
    torch.cuda.synchronize(device)
    return streams


class MiniBatchPipelinePool:
    """`n` MiniBatchPipeline objects on streams of their own; run() hands the batches to them in
    turn, so that up to `n` batches are in flight: the latency-bound sampling of one batch overlaps
    the bandwidth-bound gathers of another (12 000 roots, 2-hop recent 10x10, node and edge rows
    of a 1M-node / 20M-edge graph: 0.071 ms per batch with three in flight against 0.094 ms one at a time).  A MiniBatch stays valid until the `n`-th
    following run().  Create the pool before any other stream of the process."""

    def __init__(self, n, graph, *args, **kwargs):
        if n < 1:
            raise ValueError("a pool needs at least one pipeline")
        dev = graph._hp.be.device
        self.pipes = [MiniBatchPipeline(graph, *args, stream=st, **kwargs) for st in bound_streams(n, dev)]
        self._next = 0

    def run(self, roots, root_ts, neg_roots=None, neg_ts=None, root_hint=None):
        p = self.pipes[self._next]
        self._next = (self._next + 1) % len(self.pipes)
        return p.run(roots, root_ts, neg_roots, neg_ts, root_hint)


class GroupedMiniBatch:
    """One mini-batch of a `MiniBatchGroupPipeline` pass: views of the group's buffers (same attributes as a
    finalized MiniBatch).  `root_start_ptr` / `root_end_ptr` of a hop count from the batch's first edge."""

    final = True

    def __init__(self, pipe, b, seg, uoff):
        p, self._p, self.index = pipe, pipe, b
        L = p.layers
        self.S = [seg[l][b + 1] - seg[l][b] for l in range(L)]
        self.E = [seg[l + 1][b + 1] - seg[l + 1][b] for l in range(L)]
        self.num_unique = uoff[b + 1] - uoff[b]
        s0, s1 = seg[0][b], seg[0][b + 1]
        self.slot_node, self.slot_ts, self.slot_local = p.in_node[s0:s1], p.in_ts[s0:s1], p.local[0][s0:s1]
        self.nid_mapper = p.ubuf[uoff[b]: uoff[b + 1]]
        self.hops = []
        kr = p.kb.queries[0]
        for l, h in enumerate(kr.hops):
            a0, a1, e0, e1 = seg[l][b], seg[l][b + 1], seg[l + 1][b], seg[l + 1][b + 1]
            self.hops.append(dict(root_start_ptr=h.root_start_ptr[a0: a1 + 1] - e0, root_end_ptr=h.root_end_ptr[a0: a1] - e0,
                                  neighbors=h.neighbors[e0:e1], neighbors_local=p.local[1 + l][e0:e1],
                                  neighbors_ts=h.neighbors_ts[e0:e1], neighbors_eid=h.neighbors_eid[e0:e1],
                                  neighbors_dt=h.neighbors_dt[e0:e1]))
        self.node_data = {k: v[uoff[b]: uoff[b + 1]] for k, v in p.node_out.items()}
        self.node_ts = {k: v[uoff[b]: uoff[b + 1]] for k, v in p.node_ts_out.items()}
        self.edge_data = [{k: v[l][seg[l + 1][b]: seg[l + 1][b + 1]] for k, v in p.edge_out.items()} for l in range(L)]
        self.time_feat = ([t[seg[l + 1][b]: seg[l + 1][b + 1]] for l, t in enumerate(p.te_out)] if p.te_out else None)

    def finalize(self):
        return self

    def blocks(self, self_loop=True):
        """Message-flow blocks, outermost hop first, local node ids (as MiniBatch.blocks)."""
        hp = self._p.hp
        last_nodes, last_ts = self.slot_local, self.slot_ts
        out = []
        for l, h in enumerate(self.hops):
            S, E, n_prev = self.S[l], self.E[l], int(last_nodes.numel())
            dst_off = n_prev - S if self_loop else 0
            num_dst = n_prev if self_loop else S
            src_off = num_dst if self_loop else 0
            counts = torch.tensor([S, E, 0], dtype=torch.int64, device=last_nodes.device)
            indptr, indices, _ = hp.block_build(h["root_start_ptr"].contiguous(), counts, S, E, dst_off, src_off)
            b = Block(indptr, indices, src_off + E, num_dst)
            if self_loop:
                b.srcdata["nid"] = torch.cat([last_nodes, h["neighbors_local"]])
                b.srcdata["ts"] = torch.cat([last_ts, h["neighbors_ts"]])
            else:
                b.srcdata["nid"], b.srcdata["ts"] = h["neighbors_local"], h["neighbors_ts"]
            b.edata["eid"], b.edata["dt"] = h["neighbors_eid"], h["neighbors_dt"]
            for k, v in self.edge_data[l].items():
                b.edata[k] = v
            if self.time_feat is not None:
                b.edata["time_feat"] = self.time_feat[l]
            last_nodes, last_ts = b.srcdata["nid"], b.srcdata["ts"]
            out.append(b)
        out.reverse()
        return out


class MiniBatchGroup:
    """Result of one `MiniBatchGroupPipeline.run`: `finalize()` reads the segment table, the unique offsets and
    the counts once (one synchronisation for the whole group) and returns the per-batch views in order."""

    def __init__(self, pipe, live):
        self._p, self.live, self.batches = pipe, live, None

    def finalize(self):
        if self.batches is None:
            p = self._p
            if p._done is not None:
                p._done.synchronize()
            # (the k-hop buffers are reused by the next pass: read the tables, leave the buffers at full size)
            counts = p.kb.counts.tolist()
            for l in range(p.layers):
                check_sample_bad(counts[3 * l + 2])
            seg, uoff = p.kb.seg[0].tolist(), p.uoff.tolist()
            self.batches = [GroupedMiniBatch(p, b, seg, uoff) for b in range(self.live)]
        return self.batches


class MiniBatchGroupPipeline:
    """B mini-batches per pass of the library calls: `sgl_sample_khop_batched` over the concatenated root slots,
    `sgl_unique_compact_batched` (a local-id space per batch), one gather launch per 8 row lists over all batches'
    rows, one time-encoding launch per hop.  What a loader that samples B batches ahead runs instead of B
    MiniBatchPipeline passes: the reference keeps several windows queued (AsyncGraphBlob, graph.py:274-293;
    prefetch_factor, test/test.py:212-221) but samples them one by one.  A 12 000-root batch alone is bound by
    launch floors and chains of dependent loads; 16 of them per pass are bound by throughput (the most-recent
    2-hop sampler: 6 us per batch instead of 25).  Same constructor arguments as MiniBatchPipeline after
    `batches`; the remap is always the dense one."""

    def __init__(self, graph, batches, num_pos_slots, num_neg, layers, fanout, sample_type="recent", node_tables=None,
                 edge_tables=None, time_encoder=None, allowed_offset=-1, equal_root_time=False, keep_root_time=False,
                 seed=0, use_graph=True, stream=None, root_hints=False):
        self.g = graph
        self.hp = hp = graph._hp
        self.dev = hp.be.device
        self.B, self.layers, self.fanout = int(batches), int(layers), int(fanout)
        self.S_pos, self.N_neg = int(num_pos_slots), int(num_neg)
        self.S0 = self.S_pos + self.N_neg
        B, S0 = self.B, self.S0
        self.p = hp.params(sample_type, fanout, allowed_offset, equal_root_time, keep_root_time, seed=seed)
        self.node_tables, self.edge_tables = dict(node_tables or {}), dict(edge_tables or {})
        if time_encoder is not None and not isinstance(time_encoder, tuple):
            time_encoder = (time_encoder.w.weight.detach().reshape(-1).contiguous(),
                            time_encoder.w.bias.detach().contiguous())
        self.te = time_encoder
        be = hp.be
        self.in_node, self.in_ts = be.empty(B * S0), be.empty(B * S0)
        self.in_hint = torch.full((B * S0,), -1, dtype=torch.int64, device=self.dev) if root_hints else None
        self.ptr_host = [b * S0 for b in range(B + 1)]
        self.ptr = torch.tensor(self.ptr_host, dtype=torch.int64, device=self.dev)
        self._ptr_by_live = {B: self.ptr.clone()}
        self.kb = hp.khop_batched_buffers(B * S0, B, self.layers, self.fanout, 1)
        caps = [B * S0] + [B * S0 * self.fanout ** (l + 1) for l in range(self.layers)]
        self.local = [be.empty(c) for c in caps]
        self.ucap = min(sum(caps), B * graph._n)
        self.ubuf, self.uoff = be.empty(max(self.ucap, 1)), be.zeros(B + 1)
        self.state = hp.remap_batched_state(graph._n, B)
        self.uws = be.empty(max(int(hp.lib.unique_batched_workspace_bytes(graph._n, B)), 256), "u8")
        self.node_out, self.node_ts_out, self.edge_out = {}, {}, {}
        for name, c in self.node_tables.items():
            self.node_out[name] = torch.empty((self.ucap, c.row_bytes), dtype=torch.uint8, device=self.dev)
            if c.ts_hot or c.ts_cold:
                self.node_ts_out[name] = be.empty(self.ucap)
        for name, c in self.edge_tables.items():
            self.edge_out[name] = [torch.empty((caps[l + 1], c.row_bytes), dtype=torch.uint8, device=self.dev)
                                   for l in range(self.layers)]
        self.te_out = None
        if self.te is not None:
            dim = int(self.te[0].numel())
            self.te_out = [torch.empty((caps[l + 1], dim), dtype=torch.float32, device=self.dev) for l in range(self.layers)]
        self._views = {}
        self.use_graph, self._graph = use_graph, None
        self._plans, self._slow = None, []
        self.stream = stream
        self._done = torch.cuda.Event() if stream is not None else None

    view = MiniBatchPipeline.view

    def _chain(self):
        hp, kr = self.hp, self.kb.queries[0]
        hp.sample_khop_batched(self.g._g, self.in_node, self.in_ts, self.ptr, self.layers, [self.p], out=self.kb,
                               slot_hint=self.in_hint)
        arrays = [self.in_node] + [h.neighbors for h in kr.hops]
        hp.unique_compact_batched(arrays, [self.kb.seg[0, l] for l in range(self.layers + 1)], self.state,
                                  out_arrays=self.local, unique_out=self.ubuf, U_off=self.uoff, workspace=self.uws,
                                  finalize=False)
        if self._plans is None:
            n_u = self.uoff[self.B: self.B + 1]
            segs = [(c, self.ubuf, self.node_out[name], self.node_ts_out.get(name), n_u)
                    for name, c in self.node_tables.items()]
            segs += [(c, h.neighbors_eid, self.edge_out[name][l], None, h.counts[1:2])
                     for l, h in enumerate(kr.hops) for name, c in self.edge_tables.items()]
            fast = [s for s in segs if s[0].row_bytes % 16 == 0]
            self._slow = [s for s in segs if s[0].row_bytes % 16 != 0]
            self._plans = [hp.gather_plan(fast[i: i + 8]) for i in range(0, len(fast), 8)]
        for plan in self._plans:
            hp.gather_multi(plan)
        for c, ids, out, out_ts, n_dev in self._slow:
            hp.gather(c, ids, out, out_ts=out_ts, N_dev=n_dev)
        if self.te is not None:
            for l, h in enumerate(kr.hops):
                hp.time_encode(h.neighbors_dt, self.te[0], self.te[1], out=self.te_out[l], N_dev=h.counts[1:2])

    def run(self, roots, root_ts, neg_roots=None, neg_ts=None, root_hint=None):
        """Enqueue one group (asynchronous).  roots / root_ts: [live, S_pos]; neg_roots / neg_ts: [live, N_neg];
        root_hint: [live, S_pos] window ends for a pipeline built with root_hints=True.  live <= B batches (a
        stream's last group may be short: the remaining batches of the pass are empty)."""
        live = int(roots.shape[0]) if roots.dim() == 2 else -1
        if live < 1 or live > self.B or tuple(roots.shape) != (live, self.S_pos) or tuple(root_ts.shape) != (live, self.S_pos):
            raise ValueError(f"this pipeline was planned for up to {self.B} batches of {self.S_pos} positive slots")
        if (self.in_hint is None) != (root_hint is None) or (root_hint is not None and tuple(root_hint.shape) != (live, self.S_pos)):
            raise ValueError("root_hint goes with a pipeline built with root_hints=True, one entry per positive slot")
        if self.N_neg and (neg_roots is None or tuple(neg_roots.shape) != (live, self.N_neg) or tuple(neg_ts.shape) != (live, self.N_neg)):
            raise ValueError(f"this pipeline was planned for {self.N_neg} negatives per batch")
        if self.stream is not None:
            with torch.cuda.stream(self.stream):
                out = self._run(live, roots, root_ts, neg_roots, neg_ts, root_hint)
                self._done.record(self.stream)
            return out
        return self._run(live, roots, root_ts, neg_roots, neg_ts, root_hint)

    def _run(self, live, roots, root_ts, neg_roots, neg_ts, root_hint):
        B, S0, Sp = self.B, self.S0, self.S_pos
        rows = lambda t: t.view(B, S0)[:live]
        dsts, srcs = [rows(self.in_node)[:, :Sp], rows(self.in_ts)[:, :Sp]], [roots, root_ts]
        if root_hint is not None:
            dsts.append(rows(self.in_hint)[:, :Sp]); srcs.append(root_hint)
        if self.N_neg:
            dsts += [rows(self.in_node)[:, Sp:], rows(self.in_ts)[:, Sp:]]; srcs += [neg_roots, neg_ts]
        for d, t in zip(dsts, srcs):
            d.copy_(t, non_blocking=True)
        if live not in self._ptr_by_live:
            self._ptr_by_live[live] = torch.tensor([min(b, live) * S0 for b in range(B + 1)], dtype=torch.int64, device=self.dev)
        self.ptr.copy_(self._ptr_by_live[live], non_blocking=True)
        if not self.use_graph:
            self._chain()
        elif self._graph is None:
            self._chain()
            torch.cuda.current_stream(self.dev).synchronize()
            g = torch.cuda.CUDAGraph()
            with graph_capture(g):
                self._chain()
            self._graph = g
            g.replay()
        else:
            self._graph.replay()
        return MiniBatchGroup(self, live)


class MiniBatchGroupPool:
    """`n` MiniBatchGroupPipeline objects on streams of their own, taking the groups in turn (as MiniBatchPipelinePool)."""

    def __init__(self, n, graph, *args, **kwargs):
        if n < 1:
            raise ValueError("a pool needs at least one pipeline")
        dev = graph._hp.be.device
        self.pipes = [MiniBatchGroupPipeline(graph, *args, stream=st, **kwargs) for st in bound_streams(n, dev)]
        self._next = 0

    def run(self, *args, **kwargs):
        p = self.pipes[self._next]
        self._next = (self._next + 1) % len(self.pipes)
        return p.run(*args, **kwargs)
