"""Sampler façade with the class names, signatures and attribute names of the
reference's starrygl/graph/graph.py, running on libsgl_hot.so (MI355X).

    NegSamplingSet   graph.py:15-26
    pyGraph          graph.py:30-136
    AsyncBlock       graph.py:139-271
    AsyncGraphBlob   graph.py:274-293

`to_block` returns `Block` objects (CSC indptr/indices + srcdata/edata dicts);
`Block.to_dgl()` converts to a DGL block when dgl is importable.
"""
from typing import List, Optional

import torch

from ..lib import hot_path
from ..lib import libstarrygl_comm as starrygl_ops
from ..utils.context import DistributedContext


class NegSamplingSet:
    def __init__(self, node_set):
        self.node_set = node_set

    def sample(self, num_samples: int, num_groups: int = 1) -> torch.Tensor:
        """`num_samples x num_groups` negatives drawn uniformly (with repetition)
        from the node set."""
        if not isinstance(self.node_set, torch.Tensor):
            raise TypeError("node_set must be a torch.Tensor")
        pick = torch.randint(0, len(self.node_set), (num_samples, num_groups), device=self.node_set.device)
        return self.node_set[pick]


class pyGraph:
    def __init__(self, src, dst, ts, node_num: int, chunk_size: int, eid=None,
                 chunk_mapper: Optional[torch.Tensor] = None, weights: Optional[torch.Tensor] = None,
                 add_inverse_edge: bool = False, stream: Optional[torch.cuda.Stream] = None):
        ctx = DistributedContext.get_default_context()
        if eid is None:
            eid = torch.arange(src.size(0), dtype=torch.long, device=ctx.device)
        self.add_inverse_edge = add_inverse_edge
        # construction errors propagate (the reference prints them and leaves the
        # object without a graph, graph.py:49-55)
        self.g = starrygl_ops.from_edge_index(node_num, chunk_size, src.to(ctx.device), dst.to(ctx.device),
                                              ts.to(ctx.device), eid.to(ctx.device), chunk_mapper,
                                              stream if stream is not None else 0, ctx.local_rank)

    def async_sample(self, time_start: int, time_end: int, chunk_list: torch.Tensor, policy: dict = {},
                     test_generate_kwargs: dict = {}, op: Optional[str] = None):
        """Queue one sampling query; results come back in order from
        get_last_sample()."""
        if not isinstance(chunk_list, torch.Tensor):
            raise TypeError("chunk_list must be a torch.Tensor")
        if not isinstance(policy, dict):
            raise TypeError("policy must be a dict")
        if not isinstance(test_generate_kwargs, dict):
            raise TypeError("test_generate_kwargs must be a dict")
        if op is not None and not isinstance(op, str):
            raise TypeError("op must be a str")
        dev = DistributedContext.get_default_context().device
        empty = torch.empty(0, dtype=torch.long, device=dev)
        neg = test_generate_kwargs.get("test_generate_samples", empty).to(dev)
        neg_ts = test_generate_kwargs.get("test_generate_samples_ts", empty).to(dev)
        if policy["sample_type"] == "cluster":
            return self.g.submit_query(time_start, time_end, chunk_list, neg, neg_ts, "cluster",
                                       1, 0, 0, 0, 0, op)
        for key in ("fanout", "layers"):
            if key not in policy:
                raise ValueError(f"policy must contain '{key}' for non-c sampling")
        return self.g.submit_query(time_start, time_end, chunk_list, neg, neg_ts, policy["sample_type"],
                                   policy["layers"], policy["fanout"], policy.get("allowed_offset", -1),
                                   policy.get("equal_root_time", False), policy.get("keep_root_time", False), op)

    def get_last_sample(self):
        return self.g.get()

    def slice_by_chunk_ts(self, chunk_list: torch.Tensor, time_begin: float, time_end: float):
        return self.g.slice_by_chunk_ts(chunk_list, time_begin, time_end)

    def sample_src_in_chunks_khop(self, postive_root, negative_root, k=None, layers=None, allowed_offset=-1,
                                  equal_root_time=False, keep_root_time=False, sample_type="recent"):
        """Bound signature of the native method (export.cu:194-201).  The reference's wrapper of the same
        name passes (chunk_list, k, layers, time_begin, time_end) to it (graph.py:124-135), which the
        native method does not accept; that form is served here as what it spells: the seeds of the
        chunks in [time_begin, time_end), then k most recent neighbours per hop (`layers`: a hop count
        or one entry per hop), no negatives."""
        if isinstance(postive_root, torch.Tensor):
            chunk_list, fanout, hops, time_begin, time_end = postive_root, negative_root, k, layers, allowed_offset
            hops = len(hops) if isinstance(hops, (list, tuple)) else int(hops)
            roots = self.g.get_seeds_in_chunks(chunk_list, int(time_begin), int(time_end))
            return self.g.sample_src_in_chunks_khop(roots, None, int(fanout), hops, -1, False, False, "recent")
        return self.g.sample_src_in_chunks_khop(postive_root, negative_root, k, layers, allowed_offset,
                                                equal_root_time, keep_root_time, sample_type)


class Block:
    """One message-flow block in CSC form: dst node d has in-edges
    indptr[d]..indptr[d+1]; edge e comes from src node indices[e].  The first
    num_dst src nodes are the dst nodes themselves when self_loop is on."""

    def __init__(self, indptr, indices, num_src, num_dst):
        self.indptr, self.indices = indptr, indices
        self._num_src, self._num_dst = int(num_src), int(num_dst)
        self.srcdata, self.edata, self.dstdata = {}, {}, {}

    def num_src_nodes(self):
        return self._num_src

    def num_dst_nodes(self):
        return self._num_dst

    def num_edges(self):
        return int(self.indices.numel())

    def to_dgl(self):
        import dgl
        b = dgl.create_block(("csc", (self.indptr, self.indices, self.indices.new_empty(0))),
                             num_src_nodes=self._num_src, num_dst_nodes=self._num_dst)
        for k, v in self.srcdata.items():
            b.srcdata[k] = v
        for k, v in self.edata.items():
            b.edata[k] = v
        return b

    def __repr__(self):
        return f"<Block src={self._num_src} dst={self._num_dst} edges={self.num_edges()}>"


class AsyncBlock:
    def __init__(self, graph: pyGraph, index: int):
        self.graph = graph
        self.index = index

    def value(self):
        return self.graph.get_last_sample()

    @staticmethod
    def to_block(root, neg_roots, neighbors, nid_mapper, self_loop=True, add_inverse_edge=False):
        """Layer i's destinations are the previous layer's source set (layer 0:
        the hop-0 slots = root timestamps then negatives); its sources are
        [destinations (self-loop prefix, if self_loop)] ++ the sampled edges.
        srcdata['nid'|'ts'], edata['eid' (// 2 if add_inverse_edge) | 'dt'].
        Returns (root, neg_roots, blocks in reversed order, nid_mapper)."""
        dev = root.roots.device
        hp = hot_path(dev)
        # hop-0 slots: every (root, timestamp) pair, then the negatives
        reps = root.ts_ptr[1:] - root.ts_ptr[:-1]
        last_nodes = torch.cat([torch.repeat_interleave(root.roots, reps, output_size=int(root.ts.numel())),
                                neg_roots.roots])
        last_ts = torch.cat([root.ts, neg_roots.ts])
        mfgs = []
        for layer in neighbors:
            S, E = int(layer.root_start_ptr.numel()) - 1, int(layer.neighbors.numel())
            n_prev = int(last_nodes.numel())
            # the layer's slots are the newest S entries of the previous source set
            dst_offset = n_prev - S if self_loop else 0
            num_dst = n_prev if self_loop else S
            src_offset = num_dst if self_loop else 0
            counts = torch.tensor([S, E], dtype=torch.int64, device=dev)
            indptr, indices, _ = hp.block_build(layer.root_start_ptr, counts, S, E, dst_offset, src_offset)
            b = Block(indptr, indices, src_offset + E, num_dst)
            if self_loop:
                b.srcdata["ts"] = torch.cat([last_ts, layer.neighbors_ts])
                b.srcdata["nid"] = torch.cat([last_nodes, layer.neighbors])
            else:
                b.srcdata["ts"], b.srcdata["nid"] = layer.neighbors_ts, layer.neighbors
            b.edata["eid"] = layer.neighbors_eid // 2 if add_inverse_edge else layer.neighbors_eid
            b.edata["dt"] = layer.neighbors_dt
            last_nodes, last_ts = b.srcdata["nid"], b.srcdata["ts"]
            mfgs.append(b)
        mfgs.reverse()
        return root, neg_roots, mfgs, nid_mapper


class AsyncGraphBlob:
    def __init__(self, graph: pyGraph, time_start: List[int], time_end: List[int],
                 chunk_list: List[torch.Tensor], policy: dict = {}, test_generate_kwargs: dict = {}):
        """Submits one query per time window; the first starts a new local-id
        epoch ('r'), the following ones continue it ('f')."""
        self.graph = []
        for i in range(len(time_start)):
            graph.async_sample(time_start[i], time_end[i], chunk_list[i], policy=policy,
                               test_generate_kwargs=test_generate_kwargs, op=("f" if i > 0 else "r"))
            self.graph.append(AsyncBlock(graph, i))
