"""Materialised mini-batches in the reference's on-disk layout, built on the GPU.

`MaterializedMultiLayerBuilder` mirrors the class of the same name in the
reference's offline sampler (prepare_sample.py:178-406): same constructor
arguments, same `build_aligned_batch(task_param, save_path, layer_configs, ...)`
call, same file content - a list whose entry 0 describes the task and the
unique (node, time) targets and whose entries 1.. are the sampled layers as CSC
blocks:

    [0]  gids, ts, inv_map, num_neg, task_* ..., comm_plan
    [l]  indptr, indices, eid, edge_ts, edge_dt (fp32), gids, ts

The sampling (most recent / uniform before t over the in-edges of each target),
the (id, ts) pair unique and the (destination, time) edge order run in
libsgl_hot.so; only concatenations and permutation indexing are torch glue.

Layer types (prepare_sample.py:57-76, 105-170), with the window of a target
(v, t) = its in-edges with ts < t + meta['end_offset'] (continuous graphs:
from the first edge; discrete graphs, meta graph_type != 'c': from
t + meta['start_offset']):
  continuous  'recent'  the last `fanout` window edges     'uniform' `fanout` of them at random
              'full', 'cluster'  every window edge
  discrete    'uniform' the first `fanout` window edges    'full' every window edge
              'cluster' the window edges whose event cluster ('cid' of the partition data) is `cluster_ids`
              'recent'  as 'full' (the reference counts the whole window for it and then writes nothing,
                        prepare_sample.py:75, 147-170: its output arrays stay uninitialised)
              every edge of a discrete layer reports the target's time as its own (edge_ts = t).

Differences from the reference
  * `comm_plan` entries are None: routing plans between partitions belong to
    the multi-GPU exchange, which this library does not build;
  * uniform draws come from the library's counter-based generator (the
    reference draws from numpy's unseeded global generator).

`write_slot` / `read_slot` cover the event-slot files the partitioner writes
(prepare_nparts_louvain.py:442-451).
"""
import torch

from ..graph.graph import Block
from ..lib import hot_path
from ..lib.driver import TCSRArrays

SLOT_KEYS = ("src", "dst", "ts", "eid", "cid", "slot_id", "chunk_id")


def _dev_i64(x, device):
    t = torch.as_tensor(x)
    return t.to(device=device, dtype=torch.int64).contiguous()


class MaterializedMultiLayerBuilder:
    def __init__(self, partition_data, num_nodes, node_parts=None, rep_table=None, pid=0, num_parts=1,
                 device=None, seed=0):
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        self.hp = hp = hot_path(self.device)
        dev = self.device
        src, dst, ts = (_dev_i64(partition_data[k], dev) for k in ("src", "dst", "ts"))
        m = src.numel()
        eid = _dev_i64(partition_data["eid"], dev) if "eid" in partition_data else torch.arange(m, device=dev)
        self.num_nodes, self.pid, self.num_parts = int(num_nodes), pid, num_parts
        self.node_parts, self.rep_table = node_parts, rep_table
        self.seed, self._calls = int(seed), 0
        # in-edges of every node in (time, arrival) order - np.lexsort((ts, dst)) of the
        # reference (prepare_sample.py:193-198): rows are destinations, columns sources
        with torch.cuda.device(dev):
            g = hp.tcsr_build(self.num_nodes, dst, src, ts, torch.arange(m, device=dev))
            self.g = TCSRArrays(hp.be, self.num_nodes, g.row_ptr, g.col, g.ts, eid[g.eid])
            # the events' cluster ids in the same order (sorted_cluster, prepare_sample.py:183, 198)
            cid = _dev_i64(partition_data["cid"], dev) if "cid" in partition_data else torch.zeros(m, dtype=torch.int64, device=dev)
            self.edge_cluster = cid[g.eid].contiguous()

    # ---- one layer -----------------------------------------------------------
    def _sample_layer(self, target_nodes, target_ts, fanout, sample_type, seed, meta=None, cluster_id=None):
        """-> (raw_src, raw_dst, raw_ts, raw_dt, raw_eid) or None when no target has an in-edge at all
        (prepare_sample.py:248-265; the kernel's branches :57-76, :105-170)."""
        hp, g = self.hp, self.g
        meta = meta or {}
        if sample_type not in ("recent", "uniform", "cluster", "full"):
            sample_type = "recent"                  # the reference's .get(sample_type, 0)
        if target_nodes.numel() == 0 or not bool((g.row_ptr[target_nodes + 1] > g.row_ptr[target_nodes]).any()):
            return None
        start_off, end_off = int(meta.get("start_offset", 0)), int(meta.get("end_offset", 0))
        discrete = meta.get("graph_type", "c") != "c"
        if not discrete and sample_type in ("recent", "uniform"):
            # the k-hop sampler's windows end strictly before the slot time: shift it by end_offset
            p = hp.params(sample_type, int(fanout), seed=seed)
            hop = hp.sample_hop(g, target_nodes, target_ts + end_off if end_off else target_ts, p)
        elif not discrete:                           # 'cluster' and 'full': every edge before the cut
            hop = hp.sample_window(g, target_nodes, target_ts, hi_offset=end_off)
        elif sample_type == "cluster":
            hop = hp.sample_window(g, target_nodes, target_ts, lo_offset=start_off, hi_offset=end_off, keep_slot_time=True,
                                   edge_tag=self.edge_cluster, tag_value=-1 if cluster_id is None else int(cluster_id))
        else:                                        # discrete 'uniform': the first `fanout`; 'full' / 'recent': all
            hop = hp.sample_window(g, target_nodes, target_ts, lo_offset=start_off, hi_offset=end_off, keep_slot_time=True,
                                   first_k=int(fanout) if sample_type == "uniform" else -1)
        counts = torch.tensor([hop.S, hop.E, 0], device=self.device)
        raw_dst = hp.block_build(hop.root_start_ptr, counts, hop.S, hop.E, 0, 0, with_edge_dst=True)[2]
        if not discrete and sample_type in ("recent", "uniform") and end_off:
            raw_dt = (target_ts[raw_dst[: hop.E]] - hop.neighbors_ts).to(torch.float32)
        else:
            raw_dt = (-hop.neighbors_dt).to(torch.float32)      # t_cut - ts, prepare_sample.py:130, 145
        return hop.neighbors, raw_dst[: hop.E], hop.neighbors_ts, raw_dt, hop.neighbors_eid

    def build_aligned_batch(self, task_param, save_path, layer_configs, num_neg=1, global_dst_pool=None,
                            cluster_ids=None):
        hp, dev = self.hp, self.device
        task_type, task_nodes = task_param
        meta = layer_configs.get("meta", {})
        extra = {}
        if task_type == "link":
            task_src, task_dst, task_ts, task_label, task_eid = task_nodes
            l0_nodes = torch.cat([_dev_i64(task_src, dev), _dev_i64(task_dst, dev)])
            l0_ts = torch.cat([_dev_i64(task_ts, dev)] * 2)
            extra = {"task_ts": task_ts, "task_src": task_src, "task_dst": task_dst, "task_label": task_label,
                     "task_eid": task_eid}
        elif task_type == "node":
            task_node, task_ts, task_label = task_nodes
            l0_nodes, l0_ts = _dev_i64(task_node, dev), _dev_i64(task_ts, dev)
            extra = {"task_node": task_node, "task_ts": task_ts, "task_label": task_label}
        elif task_type == "neg":
            if num_neg <= 0 or global_dst_pool is None:
                raise ValueError("a 'neg' task needs num_neg > 0 and a destination pool")
            task_ts = _dev_i64(task_nodes, dev)
            pool = _dev_i64(global_dst_pool, dev)
            gen = torch.Generator(device=dev).manual_seed(self.seed + 7919 * self._calls)
            pick = torch.randint(0, pool.numel(), (task_ts.numel() * num_neg,), device=dev, generator=gen)
            l0_nodes = pool[pick]
            l0_ts = torch.repeat_interleave(task_ts, num_neg)
            extra = {"task_nodes": l0_nodes, "task_ts": task_ts, "task_label": "neg_set"}
        else:
            raise ValueError(f"Unsupported task type: {task_type}")
        self._calls += 1

        with torch.cuda.device(dev):
            curr_uid, curr_uts, l0_inv = hp.unique_pairs(l0_nodes, l0_ts)
            batch = [{"gids": curr_uid, "ts": curr_uts, "inv_map": l0_inv, "num_neg": num_neg}]
            routes = [None]
            last_inv = None
            for l, cfg in enumerate(layer_configs["layer"]):
                target_u = curr_uid if last_inv is None else curr_uid[last_inv]
                target_t = curr_uts if last_inv is None else curr_uts[last_inv]
                raw = self._sample_layer(target_u, target_t, cfg.get("fanout", 10), cfg["type"],
                                         seed=self.seed + 104729 * self._calls + l, meta=meta, cluster_id=cluster_ids)
                if raw is None:
                    e = curr_uid.new_empty(0)
                    batch.append({"indptr": curr_uid.new_zeros(1), "indices": e, "eid": e, "edge_ts": e,
                                  "edge_dt": torch.empty(0, dtype=torch.float32, device=dev), "gids": e, "ts": e})
                    routes.append(None)
                    break
                raw_src, raw_dst, raw_ts, raw_dt, raw_eid = raw
                dst_mapped = raw_dst if last_inv is None else last_inv[raw_dst]
                n_curr = curr_uid.numel()
                next_uid, next_uts, inv_all = hp.unique_pairs(torch.cat([curr_uid, raw_src]),
                                                              torch.cat([curr_uts, raw_ts]))
                next_inv = inv_all[n_curr:]
                indptr, perm = hp.csc_from_pairs(dst_mapped, raw_ts, n_curr)
                batch.append({"indptr": indptr, "indices": next_inv[perm], "eid": raw_eid[perm], "edge_ts": raw_ts[perm],
                              "edge_dt": raw_dt[perm], "gids": next_uid, "ts": next_uts})
                routes.append(None)
                curr_uid, curr_uts, last_inv = next_uid, next_uts, next_inv
        batch[0].update(extra)
        batch[0]["comm_plan"] = routes
        if save_path is not None:
            write_batch(save_path, batch)
        return batch


def _to_cpu(v):
    return v.detach().cpu() if isinstance(v, torch.Tensor) else (torch.as_tensor(v) if hasattr(v, "dtype") else v)


def write_batch(path, batch):
    """One batch file: the list of dicts, tensors on the host (prepare_sample.py:383-406)."""
    torch.save([{k: _to_cpu(v) for k, v in d.items()} for d in batch], path)


def read_batch(path, device=None):
    """Load a batch file without executing anything from it (tensors, numbers, strings, None only)."""
    batch = torch.load(path, map_location="cpu", weights_only=True)
    if device is not None:
        batch = [{k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in d.items()} for d in batch]
    return batch


def batch_to_blocks(batch):
    """Layer l of a batch as a Block: destinations are the previous entry's (gid, ts) targets,
    sources this entry's; returned outermost layer first, the order a model consumes them in."""
    blocks = []
    for prev, cur in zip(batch[:-1], batch[1:]):
        b = Block(cur["indptr"], cur["indices"], cur["gids"].numel(), cur["indptr"].numel() - 1)
        b.srcdata["nid"], b.srcdata["ts"] = cur["gids"], cur["ts"]
        b.dstdata["nid"], b.dstdata["ts"] = prev["gids"], prev["ts"]
        b.edata["eid"], b.edata["ts"], b.edata["dt"] = cur["eid"], cur["edge_ts"], cur["edge_dt"]
        blocks.append(b)
    return blocks[::-1]


def write_slot(path, src, dst, ts, eid, cid, slot_id, chunk_id, route=None):
    """One event-slot file of the partitioner (prepare_nparts_louvain.py:442-451)."""
    d = dict(zip(SLOT_KEYS, (src, dst, ts, eid, cid, slot_id, chunk_id)))
    if route is not None:
        d["route"] = route
    torch.save({k: _to_cpu(v) for k, v in d.items()}, path)


def read_slot(path, device=None):
    d = torch.load(path, map_location="cpu", weights_only=True)
    missing = [k for k in SLOT_KEYS[:4] if k not in d]
    if missing:
        raise KeyError(f"slot file lacks {missing}")
    if device is not None:
        d = {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in d.items()}
    return d
