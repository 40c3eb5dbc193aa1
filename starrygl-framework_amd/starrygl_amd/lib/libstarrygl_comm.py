"""Drop-in for the reference's pybind module `starrygl.lib.libstarrygl_comm`
(csrc/srcs/starrygl/export.cu:20-253), sampler part: the same functions,
classes, attribute names and argument order, running on libsgl_hot.so.

Differences a caller can observe
  * result attributes are views of the result's own tensors, not fresh copies
    (export.cu:29-162 copies device-to-device on every attribute read);
  * `root_start_ptr` / `root_end_ptr` both have S+1 entries: `root_start_ptr` is
    the exclusive prefix (a CSC indptr), `root_end_ptr[s] = root_start_ptr[s+1]`
    with a repeated last entry, so `ptr[:-1]` (graph.py:166-168) is per slot;
  * `op='r'` starts a new local-id epoch and `op='f'` continues it, as
    `AsyncGraphBlob` (graph.py:291) and the comment at sample.cu.hpp:1874 say;
  * time windows of `get_seeds_in_chunks` and `slice_by_chunk_ts` are half open,
    [time_begin, time_end).
"""
import ctypes as C
import queue
import threading

import torch

from . import _abi, hot_path
from .driver import POISON, check_unique_total


class TemporalRoot:
    """export.cu:28-79 / sample.cu.hpp:849-871."""

    def __init__(self, roots, ts_ptr, ts, q_ptr=None, q_eid=None, window_end=None):
        e = roots.new_empty(0)
        self.roots, self.ts_ptr, self.ts = roots, ts_ptr, ts
        self.q_ptr = e if q_ptr is None else q_ptr
        self.q_eid = e if q_eid is None else q_eid
        # not in the reference: per (root, timestamp) where the window strictly before it ends; roots
        # that come out of get_seeds_in_chunks carry it, and sampling them then needs no search
        self.window_end = window_end

    @property
    def root_num(self):
        return int(self.roots.numel())

    @property
    def root_ts_num(self):
        return int(self.ts.numel())

    def __repr__(self):
        return f"<TemporalRoot with {self.root_num} roots>"


class NegativeRoot:
    """export.cu:82-106 / sample.cu.hpp:872-881."""

    def __init__(self, roots, ts):
        self.roots, self.ts = roots, ts

    @property
    def root_num(self):
        return int(self.roots.numel())

    def __repr__(self):
        return f"<NegativeRoot with {self.root_num} roots>"


class TemporalNeighbor:
    """export.cu:109-167 / sample.cu.hpp:882-915."""

    def __init__(self, hop):
        self.root_start_ptr, self.root_end_ptr = hop.root_start_ptr, hop.root_end_ptr
        self.neighbors, self.neighbors_ts = hop.neighbors, hop.neighbors_ts
        self.neighbors_eid, self.neighbors_dt = hop.neighbors_eid, hop.neighbors_dt

    @classmethod
    def from_arrays(cls, root_start_ptr, root_end_ptr, neighbors, neighbors_ts, neighbors_eid, neighbors_dt):
        self = cls.__new__(cls)
        self.root_start_ptr, self.root_end_ptr = root_start_ptr, root_end_ptr
        self.neighbors, self.neighbors_ts = neighbors, neighbors_ts
        self.neighbors_eid, self.neighbors_dt = neighbors_eid, neighbors_dt
        return self

    @property
    def neighbor_num(self):
        return int(self.neighbors.numel())

    def __repr__(self):
        return f"<TemporalNeighbor with {self.neighbor_num} neighbors>"


class TemporalResult:
    """export.cu:170-184 / sample.cu.hpp:916-934."""

    def __init__(self, roots, neg_roots, neighbors_list, nodes_remapper_id=None):
        self.roots, self.neg_roots, self.neighbors_list = roots, neg_roots, neighbors_list
        self.nodes_remapper_id = roots.roots.new_empty(0) if nodes_remapper_id is None else nodes_remapper_id

    @property
    def neighbors(self):
        return self.neighbors_list

    def __repr__(self):
        return f"<TemporalResult with {len(self.neighbors_list)} neighbor layers>"


def _i64(t, device, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != torch.int64:
        raise RuntimeError(f"{name} must be int64")          # sample.cu.hpp:1001-1013
    return t.to(device).contiguous()


class CUDAGraph:
    """The sampler object of export.cu:186-227 on one HIP device."""

    def __init__(self, hp, tcsr, chunk_size, mapper, stream=None, seed=1317):
        self._hp, self._g = hp, tcsr
        self._n, self._chunks = tcsr.n, int(chunk_size)
        self._stream = stream
        self._seed, self._queries = int(seed), 0
        self._state = None
        self._mapper = mapper
        self._chunk_index = None
        self._tasks, self._results = queue.Queue(), queue.Queue()
        self._worker = None

    # ---- direct (synchronous) entry points ---------------------------------
    def get_negative_root(self, negative_root, negative_time):
        dev = self._hp.be.device
        return NegativeRoot(_i64(negative_root, dev, "negative_root"), _i64(negative_time, dev, "negative_time"))

    def sample_src_in_chunks_khop(self, postive_root, negative_root, k, layers, allowed_offset, equal_root_time,
                                  keep_root_time, sample_type, seed=None, _defer=None):
        """k-hop sampling from explicit roots (sample.cu.hpp:1532-1716).  Ids in
        the result are global; `submit_query` adds the remap.  (`_defer`: the query
        worker passes a device array for the counts and reads them later, together with
        the unique count, in one copy.)"""
        hp = self._hp
        p = hp.params(sample_type, k, allowed_offset, equal_root_time, keep_root_time,
                      seed=self._seed if seed is None else seed)
        w_end = getattr(postive_root, "window_end", None)
        if w_end is not None and w_end.numel() == postive_root.ts.numel():
            p = hp.with_root_hint(p, w_end)
        neg = negative_root if negative_root is not None else self._empty_neg()
        if _defer is None:
            res = hp.sample_khop(self._g, postive_root.roots, postive_root.ts_ptr, postive_root.ts, neg.roots, neg.ts,
                                 int(layers), p)
            return TemporalResult(postive_root, neg, [TemporalNeighbor(h) for h in res.hops])
        S0 = int(postive_root.ts.numel() + neg.roots.numel())
        out = hp.khop_buffers(S0, int(layers), int(k), counts=_defer)
        return hp.sample_khop(self._g, postive_root.roots, postive_root.ts_ptr, postive_root.ts, neg.roots, neg.ts,
                              int(layers), p, finalize=False, out=out)

    def window_end(self, node, t):
        """Where the strictly-before window of every slot (node[i], t[i]) ends (not in the reference;
        sgl_window_end): a loader looks this up once for the events it trains on and hands a batch's
        values to MiniBatchPipeline.run(root_hint=...)."""
        dev = self._hp.be.device
        return self._hp.window_end(self._g, _i64(node, dev, "node"), _i64(t, dev, "t"))

    def get_seeds_in_chunks(self, chunks, time_begin, time_end, using_full_timestamp=False):
        from .seeds import seeds_in_chunks
        return seeds_in_chunks(self, chunks, int(time_begin), int(time_end), bool(using_full_timestamp))

    def slice_by_chunk_ts(self, chunks, time_begin, time_end, using_full_timestamp=False, stream=0):
        from .seeds import slice_in_chunks
        return slice_in_chunks(self, chunks, int(time_begin), int(time_end), bool(using_full_timestamp))

    # ---- asynchronous FIFO pipeline (sample.cu.hpp:1856-2031) ---------------
    def submit_query(self, time_start, time_end, chunk_list, test_generate_samples, test_generate_samples_ts,
                     sample_type, layers, fanout, allowed_offset, equal_root_time, keep_root_time, op):
        if sample_type != "cluster" and sample_type not in _abi.SAMPLE_TYPES:
            raise RuntimeError("undefined sampling strategy")
        if self._worker is None:
            self._worker = threading.Thread(target=self._run, name="sgl-sampler", daemon=True)
            self._worker.start()
        fut = _Future()
        self._results.put(fut)
        self._tasks.put((fut, int(time_start), int(time_end), chunk_list, test_generate_samples,
                         test_generate_samples_ts, sample_type, int(layers), int(fanout), int(allowed_offset),
                         bool(equal_root_time), bool(keep_root_time), op, self._queries))
        self._queries += 1

    def get(self):
        """Oldest unfinished query's result (blocks); a failed query re-raises here."""
        return self._results.get().result()

    def close(self):
        if self._worker is not None:
            self._tasks.put(None)
            self._worker.join()
            self._worker = None

    def _run(self):
        dev = self._hp.be.device
        torch.cuda.set_device(dev)
        stream = self._stream if isinstance(self._stream, torch.cuda.Stream) else torch.cuda.Stream(dev)
        while True:
            task = self._tasks.get()
            if task is None:
                return
            fut = task[0]
            try:
                with torch.cuda.stream(stream):
                    fut.set_result(self._execute(*task[1:]))
            except BaseException as exc:  # forwarded to get(), like promise.set_exception
                fut.set_exception(exc)

    def _execute(self, t0, t1, chunk_list, neg_nodes, neg_ts, sample_type, layers, fanout, allowed_offset,
                 equal_root_time, keep_root_time, op, query_index):
        if sample_type == "cluster":     # sample.cu.hpp:1953-1961: dense timestamps, no negatives
            return self.remap(self.slice_by_chunk_ts(chunk_list, t0, t1, True), reset=(op != "f"))
        roots = self.get_seeds_in_chunks(chunk_list, t0, t1)
        neg = self.get_negative_root(neg_nodes, neg_ts)
        if layers < 1:
            raise ValueError("layers must be at least 1")
        # sampling and unique are chained on the device; their counts come back in one copy
        hp = self._hp
        live = hp.be.zeros(3 * layers + 2)
        kr = self.sample_src_in_chunks_khop(roots, neg, fanout, layers, allowed_offset, equal_root_time,
                                            keep_root_time, sample_type, seed=self._seed + query_index,
                                            _defer=live[: 3 * layers])
        arrays = [roots.roots, neg.roots] + [h.neighbors for h in kr.hops]
        lens = [None, None] + [h.counts[1:2] for h in kr.hops]
        return self._remap_arrays(roots, neg, kr, arrays, lens, live, reset=(op != "f"))

    def _remap_arrays(self, roots, neg, kr, arrays, lens, live, reset):
        hp, L = self._hp, len(kr.hops)
        if self._state is None:
            self._state = hp.remap_state(self._n)
            self._unique = None
        local, uniq, _ = hp.unique_compact(arrays, _abi.UNIQUE_GROUPED, self._state, reset, lens_dev=lens,
                                           finalize=False, U_out=live[3 * L:])
        vals = hp.be.tolist(live)
        if reset and (vals[3 * L] == POISON or (L and vals[2] >= POISON)):
            # a block of a single-launch kernel gave up its bounded wait: the sampler call is re-issued through the
            # launch-per-hop route and the numbering in separate launches, on a state initialised again.  Only a
            # query that opens an epoch can afford that; one that continues an epoch raises below.
            if getattr(kr, "_recover", None) is not None and vals[2] >= POISON:
                kr._recover()
                kr._recover = None
            self._state = hp.remap_state(self._n)
            hp.recoveries += 1
            local, uniq, _ = hp.unique_compact(arrays, _abi.UNIQUE_GROUPED | _abi.UNIQUE_MULTI_LAUNCH, self._state, reset,
                                               lens_dev=lens, finalize=False, U_out=live[3 * L:])
            vals = hp.be.tolist(live)
        kr.finalize(vals[: 3 * L])
        total, before = vals[3 * L], vals[3 * L + 1]
        check_unique_total(total)
        self._unique = uniq[:total] if (reset or self._unique is None) else torch.cat([self._unique[:before],
                                                                                        uniq[before:total]])
        res = TemporalResult(TemporalRoot(local[0], roots.ts_ptr, roots.ts, roots.q_ptr, roots.q_eid),
                             NegativeRoot(local[1], neg.ts), [TemporalNeighbor(h) for h in kr.hops])
        for layer, loc in zip(res.neighbors_list, local[2:]):
            layer.neighbors = loc[: layer.neighbors.numel()]
        res.nodes_remapper_id = self._unique
        torch.cuda.current_stream().synchronize()
        return res

    def remap(self, result, reset=True):
        """Remapper::insert (sample.cu.hpp:1825-1852): roots, negatives and every
        layer's neighbours become local ids, numbered per array in ascending id
        order; nodes_remapper_id is the local -> global table of the epoch."""
        hp = self._hp
        if self._state is None:
            self._state = hp.remap_state(self._n)
            self._unique = None
        arrays = [result.roots.roots, result.neg_roots.roots] + [l.neighbors for l in result.neighbors_list]
        local, uniq, (total, before) = hp.unique_compact(arrays, _abi.UNIQUE_GROUPED, self._state, reset)
        if reset or self._unique is None:
            self._unique = uniq[:total]
        else:
            self._unique = torch.cat([self._unique[:before], uniq[before:total]])
        result.roots = TemporalRoot(local[0], result.roots.ts_ptr, result.roots.ts, result.roots.q_ptr,
                                    result.roots.q_eid)
        result.neg_roots = NegativeRoot(local[1], result.neg_roots.ts)
        for layer, loc in zip(result.neighbors_list, local[2:]):
            layer.neighbors = loc
        result.nodes_remapper_id = self._unique
        torch.cuda.current_stream().synchronize()
        return result

    def _empty_neg(self):
        e = torch.empty(0, dtype=torch.int64, device=self._hp.be.device)
        return NegativeRoot(e, e)


class _Future:
    def __init__(self):
        self._ev, self._val, self._exc = threading.Event(), None, None

    def set_result(self, v):
        self._val = v
        self._ev.set()

    def set_exception(self, e):
        self._exc = e
        self._ev.set()

    def result(self):
        self._ev.wait()
        if self._exc is not None:
            raise self._exc
        return self._val


def from_edge_index(n, chunk_size, src, dst, ts, eid, mapper=None, stream=0, rank=0, hop_hint=True):
    """Build the T-CSR on device `rank` (export.cu:229-250).  Raises
    RuntimeError-family exceptions for non-int64 input and out-of-range ids
    (sample.cu.hpp:1001-1020, 1043-1062).  `hop_hint` (not in the reference): also build the
    next-hop index (8 bytes per edge) that spares the sampler the searches of hops >= 1."""
    device = torch.device("cuda", int(rank))
    hp = hot_path(device)
    n, chunk_size = int(n), int(chunk_size)
    src, dst, ts = (_i64(t, device, nm) for t, nm in ((src, "src"), (dst, "dst"), (ts, "ts")))
    eid = None if eid is None else _i64(eid, device, "eid")
    if not (src.numel() == dst.numel() == ts.numel()) or (eid is not None and eid.numel() != src.numel()):
        raise RuntimeError("src, dst, ts and eid must have the same length")
    if mapper is not None:
        if mapper.numel() != n:
            raise RuntimeError("row_chunk_mapper must have one entry per node")
        if n > 0 and (int(mapper.min()) < 0 or int(mapper.max()) >= max(chunk_size, 1)):
            raise IndexError("row_chunk_mapper names a chunk outside [0, chunk_size)")   # sample.cu.hpp:1059-1062
    with torch.cuda.device(device):
        g = hp.tcsr_build(n, src, dst, ts, eid)
        if hop_hint:
            hp.build_hop_hint(g)
    return CUDAGraph(hp, g, chunk_size, mapper, stream if isinstance(stream, torch.cuda.Stream) else None)


class ShardTensor:
    """A logical [rows, ...] tensor made of shards appended in row order, each either in this GPU's memory
    (`target_device` = the GPU's index) or in pinned host memory read in place by the gather kernel
    (`target_device` < 0); `st[indices]` gathers rows into a new device tensor.  The interface of the
    reference's ShardTensor (csrc/include/starrygl/feature.cu.hpp:236-297 append, :298-422 operator[],
    :713-750 bindings) on one GPU: shards on other GPUs, IPC sharing and NCCL exchange are not part of it."""

    def __init__(self, device, ctx=None):
        self._device = int(device.index if isinstance(device, torch.device) else device)
        self._hp = hot_path(torch.device("cuda", self._device))
        self._shards, self._where = [], []
        self._tail_shape, self._dtype, self._cache = None, None, None

    def append(self, tensor, target_device):
        if not isinstance(tensor, torch.Tensor) or tensor.is_cuda:
            raise RuntimeError("ShardTensor.append expects a CPU tensor")        # CHECK_CPU, feature.cu.hpp:238
        if target_device >= 0 and int(target_device) != self._device:
            raise RuntimeError(f"this build serves one GPU: a shard can live on device {self._device} or on the host (-1)")
        t = tensor.contiguous()
        if self._tail_shape is None:
            self._tail_shape, self._dtype = tuple(t.shape[1:]), t.dtype
        elif tuple(t.shape[1:]) != self._tail_shape or t.dtype != self._dtype:
            raise RuntimeError("ShardTensor.append: shards differ in row shape or dtype")
        if (t.numel() // max(t.shape[0], 1)) * t.element_size() % 4 != 0:
            raise RuntimeError("ShardTensor: the row size must be a multiple of 4 bytes")
        self._shards.append(t.to(self._hp.be.device) if target_device >= 0 else (t if t.is_pinned() else t.pin_memory()))
        self._where.append(int(target_device))
        self._cache = None

    def _build(self):
        dev = self._hp.be.device
        rows = [int(s.shape[0]) for s in self._shards]
        total = sum(rows)
        row_elems = 1
        for d in self._tail_shape:
            row_elems *= int(d)
        host = [s.reshape(s.shape[0], row_elems) for s, w in zip(self._shards, self._where) if w < 0]
        devs = [s.reshape(s.shape[0], row_elems) for s, w in zip(self._shards, self._where) if w >= 0]
        n_host = sum(int(s.shape[0]) for s in host)
        # local row space: host rows first (their rows of the cold table), then the device rows
        g2l = torch.empty(total, dtype=torch.int64)
        h_off, d_off, lo = 0, n_host, 0
        for r, w in zip(rows, self._where):
            if w < 0:
                g2l[lo: lo + r] = torch.arange(h_off, h_off + r)
                h_off += r
            else:
                g2l[lo: lo + r] = torch.arange(d_off, d_off + r)
                d_off += r
            lo += r
        slot = torch.full((total,), -1, dtype=torch.int32)
        slot[n_host:] = torch.arange(total - n_host, dtype=torch.int32)
        cold = None
        if host:
            cold = host[0] if len(host) == 1 else torch.cat(host).pin_memory()
        if not devs:      # (one placeholder row: the cache wants a device table)
            hot = torch.zeros((1, row_elems), dtype=self._dtype, device=dev)
        else:
            hot = torch.cat(devs) if len(devs) != 1 else devs[0]
        self._keep = (hot, cold)
        self._cache = self._hp.cache(row_elems * self._shards[0].element_size(), hot, rows=total, cold=cold,
                                     hot_slot=slot.to(dev) if cold is not None else None,
                                     g2l=g2l.to(dev) if cold is not None else None)
        self._rows, self._row_elems = total, row_elems

    def __getitem__(self, indices):
        if not self._shards:
            raise RuntimeError("ShardTensor is empty")
        if self._cache is None:
            self._build()
        ids = _i64(indices, self._hp.be.device, "indices").reshape(-1)
        out = torch.empty((ids.numel(), self._row_elems), dtype=self._dtype, device=self._hp.be.device)
        if ids.numel():
            self._hp.gather(self._cache, ids, out)
        return out.reshape((ids.numel(),) + self._tail_shape)

    def shape(self):
        return [sum(int(s.shape[0]) for s in self._shards)] + list(self._tail_shape or ())

    def size(self, dim):
        return self.shape()[dim]

    def numel(self):
        n = 1
        for d in self.shape():
            n *= d
        return n

    def stride(self, dim):
        st = 1
        for d in self.shape()[dim + 1:]:
            st *= d
        return st

    def device(self):
        return self._device

    def device_count(self):
        return len(self._shards)

    def unregister(self, tensor=None):
        """Drop the shards (the reference un-registers its zero-copy host mappings here)."""
        self._shards, self._where, self._cache, self._keep = [], [], None, None

    def share_ipc(self):
        raise NotImplementedError("sharing shards between processes is part of the multi-GPU exchange, which this "
                                  "one-GPU build does not contain")
