"""Array-level driver of the C ABI in include/sgl_hot.h.

`HotPath(lib, backend)` marshals arrays into the structs of the ABI, sizes the
outputs and the workspace, and narrows ragged results.  The backend decides
where arrays live: `TorchBackend` (device tensors, current HIP stream) is what
the package uses; anything else that offers the same five methods can drive a
library with the same ABI on host memory.
"""
import contextlib
import ctypes as C
import gc
import os

from . import _abi
from ._abi import (TCSR, Cache, GatherSeg, HopOut, SampleParams, SeedQuery, WindowParams, check, i64, vp)


def _itemsize(a):
    return a.element_size() if hasattr(a, "element_size") else a.itemsize


def _byte_strides(a):
    """strides in bytes of a torch tensor or a numpy array"""
    if hasattr(a, "element_size"):
        return tuple(int(x) * a.element_size() for x in a.stride())
    return tuple(int(x) for x in a.strides)


def _address(a):
    """address of the first element (the array may be a strided view)"""
    return a.data_ptr() if hasattr(a, "data_ptr") else a.ctypes.data


class TorchBackend:
    """Device memory and stream plumbing through PyTorch-ROCm."""

    def __init__(self, device):
        import torch
        self.torch = torch
        self.device = torch.device(device)
        self._one_gpu = self.device.type == "cuda" and torch.cuda.device_count() == 1
        self._dt = {"i64": torch.int64, "i32": torch.int32, "f32": torch.float32,
                    "u8": torch.uint8, "bf16": torch.bfloat16, "f16": torch.float16}

    def empty(self, shape, dtype="i64"):
        return self.torch.empty(shape, dtype=self._dt[dtype], device=self.device)

    def zeros(self, shape, dtype="i64"):
        return self.torch.zeros(shape, dtype=self._dt[dtype], device=self.device)

    def asarray(self, a, dtype="i64"):
        t = self.torch.as_tensor(a, dtype=self._dt[dtype])
        return t.to(self.device).contiguous()

    def ptr(self, a):
        return None if a is None else a.data_ptr()

    def stream(self):
        if self.device.type != "cuda":
            return None
        return self.torch.cuda.current_stream(self.device).cuda_stream

    def tolist(self, a):
        return a.cpu().tolist()

    def nbytes(self, a):
        return a.numel() * a.element_size()

    def check(self, a, dtype, name):
        """The ABI takes raw pointers: an array of another dtype, a strided view or pageable host
        memory would be read as something it is not."""
        if a.dtype is self._dt[dtype] and a.is_cuda and a.is_contiguous() and self._one_gpu:
            return a                 # the common case, kept cheap: this runs on every call
        if a.dtype != self._dt[dtype]:
            raise TypeError(f"{name} must be {dtype}, got {a.dtype}")
        here = a.device.type == self.device.type and (self.device.index is None or a.device.index == self.device.index)
        if not here and not (a.device.type == "cpu" and a.is_pinned()):
            raise ValueError(f"{name} must live on {self.device}, got {a.device}")
        if not a.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
        return a


class TCSRArrays:
    """Owner of the four T-CSR arrays plus the ABI view of them."""

    def __init__(self, backend, n, row_ptr, col, ts, eid, hop_hint=None, rec=None):
        self.n, self.m = int(n), int(col.shape[0])
        self.row_ptr, self.col, self.ts, self.eid, self.hop_hint, self.rec = row_ptr, col, ts, eid, hop_hint, rec
        self.view = TCSR(self.n, self.m, backend.ptr(row_ptr), backend.ptr(col),
                         backend.ptr(ts), backend.ptr(eid), backend.ptr(hop_hint), backend.ptr(rec))


class HopResult:
    """One hop's ragged output.  Arrays are over-allocated to the worst case;
    `finalize(S, E)` narrows them once the device counts are known."""

    FIELDS = ("neighbors", "neighbors_ts", "neighbors_eid", "neighbors_dt")

    def __init__(self, backend, cap_slots, cap_edges, counts=None):
        self.cap_slots, self.cap_edges = cap_slots, cap_edges
        self.root_start_ptr = backend.empty(cap_slots + 1)
        self.root_end_ptr = backend.empty(cap_slots + 1)
        for f in self.FIELDS:
            setattr(self, f, backend.empty(cap_edges))
        self.counts = backend.zeros(3) if counts is None else counts
        self.struct = HopOut(cap_slots, cap_edges, backend.ptr(self.root_start_ptr),
                             backend.ptr(self.root_end_ptr), backend.ptr(self.neighbors),
                             backend.ptr(self.neighbors_ts), backend.ptr(self.neighbors_eid),
                             backend.ptr(self.neighbors_dt), backend.ptr(self.counts))
        self.S = self.E = None

    def finalize(self, S, E, bad=0):
        check_sample_bad(bad)
        self.S, self.E = int(S), int(E)
        self.root_start_ptr = self.root_start_ptr[: self.S + 1]
        self.root_end_ptr = self.root_end_ptr[: self.S + 1]
        for f in self.FIELDS:
            setattr(self, f, getattr(self, f)[: self.E])
        return self


POISON = (1 << 63) - 1


def check_sample_bad(bad):
    """counts[2] of a hop: slots whose node lies outside [0,n); INT64_MAX when a block of the
    single-launch 2-hop sampler gave up its bounded wait (the call's outputs are void)."""
    if bad >= (1 << 63) - 1:
        raise RuntimeError("sample_khop: a block gave up waiting for the edge totals of an earlier block")
    if bad:
        raise IndexError(f"sgl status {_abi.SGL_ERANGE}: {bad} sampling slots name a node outside [0,n)")


def _marked_state(p):
    """The RemapState a SampleParams made by HotPath.marking records ids in (None otherwise)."""
    keep = getattr(p, "_keep", None)
    while isinstance(keep, tuple):
        if isinstance(keep[1], RemapState):
            return keep[1]
        keep = keep[0] if isinstance(keep[0], tuple) else None
    return None


def _check_root_hint(p, S_pos):
    if getattr(p, "_root_hint_len", S_pos) < S_pos:
        raise ValueError(f"root_hint has {p._root_hint_len} entries for {S_pos} positive root slots")


def check_unique_total(u_total):
    """The id count of a unique_compact call is INT64_MAX when a numbering pass gave up waiting for
    an earlier tile (bounded wait): the result is void and the remap state has to be re-initialised."""
    if u_total == (1 << 63) - 1:
        raise RuntimeError("unique_compact: the result is void (a numbering pass gave up waiting, or a hashed state's "
                           "capacity was exceeded); re-initialise the remap state (HotPath.remap_reinit)")


class HotPath:
    def __init__(self, lib, backend):
        self.lib, self.be = lib, backend
        if lib.abi_version() != _abi.ABI_VERSION:
            raise RuntimeError("sgl ABI version mismatch")
        for which, mirror in enumerate(_abi.STRUCTS):     # the ctypes mirrors must have the library's layout
            if int(lib.struct_bytes(which)) != C.sizeof(mirror):
                raise RuntimeError(f"sgl ABI struct {mirror.__name__}: the library has {int(lib.struct_bytes(which))} "
                                   f"bytes, the binding {C.sizeof(mirror)}")
        self._ws = {}
        self.recoveries = 0     # calls re-issued because a block had given up its bounded wait
        self.check_hints = os.environ.get("SGL_CHECK_HINTS", "0") not in ("", "0")   # see verify_root_hint

    # ------------------------------------------------------------ helpers
    def _workspace(self, nbytes):
        """Scratch memory for one call, kept per stream: calls ordered on one stream may share
        it, calls on different streams (the query worker's and the caller's, say) must not."""
        nbytes = max(int(nbytes), 256)
        key = self.be.stream()
        ws = self._ws.get(key)
        if ws is None or self.be.nbytes(ws) < nbytes:
            ws = self._ws[key] = self.be.empty(nbytes, "u8")
        return ws, self.be.nbytes(ws)

    def _chk(self, dtype, **arrays):
        """Validate the arrays handed to a call (dtype, placement, contiguity); None entries pass."""
        for name, a in arrays.items():
            if a is not None:
                self.be.check(a, dtype, name)

    def _ck(self, rc):
        check(self.lib, rc)

    # -------------------------------------------------------------- T-CSR
    def tcsr_build(self, n, src, dst, ts, eid=None):
        self._chk("i64", src=src, dst=dst, ts=ts, eid=eid)
        be, m = self.be, int(src.shape[0])
        row_ptr, col, cts, ceid = be.empty(n + 1), be.empty(m), be.empty(m), be.empty(m)
        ws, wsb = self._workspace(self.lib.tcsr_build_workspace_bytes(n, m))
        self._ck(self.lib.tcsr_build(n, m, be.ptr(src), be.ptr(dst), be.ptr(ts), be.ptr(eid),
                                     be.ptr(row_ptr), be.ptr(col), be.ptr(cts), be.ptr(ceid),
                                     be.ptr(ws), wsb, be.stream()))
        return TCSRArrays(be, n, row_ptr, col, cts, ceid)

    def tcsr_from_sorted(self, n, row_ptr, col, ts, eid, validate=True):
        self._chk("i64", row_ptr=row_ptr, col=col, ts=ts, eid=eid)
        g = TCSRArrays(self.be, n, row_ptr, col, ts, eid)
        if validate:
            ws, wsb = self._workspace(256)
            self._ck(self.lib.tcsr_validate(C.byref(g.view), self.be.ptr(ws), wsb, self.be.stream()))
        return g

    def build_hop_hint(self, g):
        """Attach the next-hop index to the T-CSR `g` (8 bytes per edge, one search per edge, once):
        the sampler then finds the windows of the slots of hops >= 1 without searching."""
        hint = self.be.empty(g.m)
        self._ck(self.lib.tcsr_hop_hint_build(C.byref(g.view), self.be.ptr(hint), self.be.stream()))
        g.hop_hint = hint
        g.view.hop_hint = self.be.ptr(hint)
        if g.rec is not None:        # the records carry a copy of the index
            self.build_records(g)
        return g

    def build_records(self, g):
        """Attach the interleaved edge records to the T-CSR `g` (32 bytes per edge: destination, time, edge id,
        next-hop index entry): the uniform strategy then reads one memory sector per picked edge instead of
        one per array.  Build the next-hop index first if it is wanted (it is copied into the records)."""
        rec = self.be.empty(4 * g.m)
        self._ck(self.lib.tcsr_records_build(C.byref(g.view), self.be.ptr(rec), self.be.stream()))
        g.rec = rec
        g.view.rec = self.be.ptr(rec)
        return g

    def window_end(self, g, node, t, out=None):
        """out[i] = position in row node[i] of the first edge with timestamp >= t[i] (-1 for a node
        outside [0,n)): where the strictly-before window of the slot (node[i], t[i]) ends.  A loader
        computes it once for the events it will train on and passes a batch's values as `root_hint`."""
        self._chk("i64", node=node, t=t)
        if node.shape[0] != t.shape[0]:
            raise ValueError("window_end: node and t differ in length")
        if out is None:
            out = self.be.empty(int(node.shape[0]))
        else:
            self._chk("i64", out=out)
            if out.shape[0] < node.shape[0]:
                raise ValueError("window_end: out is shorter than node")
        self._ck(self.lib.window_end(C.byref(g.view), self.be.ptr(node), self.be.ptr(t), int(node.shape[0]),
                                     self.be.ptr(out), self.be.stream()))
        return out

    def verify_root_hint(self, g, roots, ts_ptr, root_ts, p):
        """Debug check (SGL_CHECK_HINTS=1 in the environment makes the sampling calls run it, at the price of a
        window search per positive slot and one host synchronisation): every root hint that is not -1 must
        be what `window_end` finds for its slot on this graph.  The kernels clamp a hint to the root's row, so
        a stale or foreign hint cannot cause a stray access, but it silently changes that slot's sample."""
        hint = getattr(p, "_keep", (None, None))[1] if getattr(p, "_root_hint_len", None) is not None else None
        if hint is None or not hasattr(self.be, "torch"):
            return
        torch = self.be.torch
        S_pos = int(root_ts.shape[0])
        if S_pos == 0:
            return
        slots = torch.arange(S_pos, device=root_ts.device)
        node = roots[torch.searchsorted(ts_ptr, slots, right=True) - 1]
        want = self.window_end(g, node.contiguous(), root_ts)
        h = hint[:S_pos]
        bad = (h >= 0) & (h != want)
        if bool(bad.any()):
            i = int(torch.nonzero(bad)[0])
            raise ValueError(f"root_hint[{i}] = {int(h[i])}, but the window of slot {i} (node {int(node[i])}, "
                             f"time {int(root_ts[i])}) ends at {int(want[i])} on this graph")

    def with_root_hint(self, p, root_hint):
        """Copy of the sampling parameters `p` that hands the k-hop sampler the window ends of the
        positive root slots (`window_end` of (root, root_ts) per slot, -1 = search): those slots are
        then sampled without a search."""
        self._chk("i64", root_hint=root_hint)
        q = SampleParams.from_buffer_copy(p)
        q.root_hint = self.be.ptr(root_hint)
        q._keep = (getattr(p, "_keep", None), root_hint)
        q._root_hint_len = int(root_hint.shape[0])
        return q

    # ----------------------------------------------------------- sampling
    @staticmethod
    def params(sample_type, fanout, allowed_offset=-1, equal_root_time=False,
               keep_root_time=False, replace=False, hop=0, seed=0):
        if isinstance(sample_type, str):
            if sample_type not in _abi.SAMPLE_TYPES:
                # same message as sample.cu.hpp:1688-1690
                raise RuntimeError("undefined sampling strategy")
            sample_type = _abi.SAMPLE_TYPES[sample_type]
        return SampleParams(int(sample_type), int(fanout), int(allowed_offset),
                            int(bool(equal_root_time)), int(bool(keep_root_time)),
                            int(bool(replace)), int(hop), int(seed) & (2**64 - 1), None, 0, None, 0, 0)

    def set_wait_limit(self, polls):
        """Polls before a block that waits for another block's totals gives up (<= 0: default);
        returns the previous limit.  For tests of that error path."""
        return int(self.lib.set_wait_limit(int(polls)))

    def multi_launch(self, p):
        """Copy of the sampling parameters `p` that keeps a k-hop call off the single-launch route."""
        q = SampleParams.from_buffer_copy(p)
        q.flags |= _abi.SAMPLE_MULTI_LAUNCH
        q._keep = getattr(p, "_keep", None)
        if hasattr(p, "_root_hint_len"):
            q._root_hint_len = p._root_hint_len
        return q

    def _reinit_marked(self, p):
        """Initialise the remap state that the sampling parameters `p` record ids in (if any) again."""
        st = _marked_state(p)
        if st is not None:
            self._ck(self.lib.remap_init(self.be.ptr(st.buf), self.be.nbytes(st.buf), st.universe, self.be.stream()))
            st.count_bound = 0

    def marking(self, p, state):
        """Copy of the sampling parameters `p` that makes the sampler record every id it
        emits as pending in the remap `state`: the following `unique_compact(..., state,
        reset=True, premarked=True)` over the sampled arrays then skips its first pass."""
        q = SampleParams.from_buffer_copy(p)
        q.mark_state, q.mark_universe = self.be.ptr(state.buf), state.universe
        q._keep = (getattr(p, "_keep", None), state)
        return q

    def sample_hop(self, g, slot_node, slot_ts, p, S_dev=None, finalize=True):
        self._chk("i64", slot_node=slot_node, slot_ts=slot_ts, S_dev=S_dev)
        be, S = self.be, int(slot_node.shape[0])
        out = HopResult(be, S, S * p.fanout)
        ws, wsb = self._workspace(self.lib.sample_hop_workspace_bytes(S))
        self._ck(self.lib.sample_hop(C.byref(g.view), be.ptr(slot_node), be.ptr(slot_ts), S,
                                     be.ptr(S_dev), C.byref(p), C.byref(out.struct),
                                     be.ptr(ws), wsb, be.stream()))
        if finalize:
            out.finalize(*be.tolist(out.counts))
        return out

    def sample_hop_static(self, g, slot_node, slot_ts, p, out, S_dev=None):
        """`sample_hop` into the caller's `out` (a HopResult) with the hop's scratch in the library's own
        per-GPU array: the call allocates nothing.  At most STATIC_HOP_MAX_SLOTS slots; calls that overlap
        on one GPU share the array and race.  The result is not finalized."""
        self._chk("i64", slot_node=slot_node, slot_ts=slot_ts, S_dev=S_dev)
        be = self.be
        self._ck(self.lib.sample_hop_static(C.byref(g.view), be.ptr(slot_node), be.ptr(slot_ts), int(slot_node.shape[0]),
                                            be.ptr(S_dev), C.byref(p), C.byref(out.struct), be.stream()))
        return out

    def sample_window(self, g, slot_node, slot_ts, lo_offset=None, hi_offset=0, first_k=-1, edge_tag=None,
                      tag_value=0, keep_slot_time=False):
        """Every edge of each slot's window [t + lo_offset (None: unbounded), t + hi_offset), or the first
        `first_k` of them, optionally only edges whose `edge_tag` (an [m] array in T-CSR order) equals
        `tag_value`.  Two library calls: count, then fill into arrays of the counted size.  -> HopResult."""
        self._chk("i64", slot_node=slot_node, slot_ts=slot_ts, edge_tag=edge_tag)
        be, S = self.be, int(slot_node.shape[0])
        p = WindowParams(int(lo_offset or 0), int(hi_offset), int(lo_offset is not None), int(bool(keep_slot_time)),
                         int(first_k), be.ptr(edge_tag), int(tag_value))
        ws, wsb = self._workspace(self.lib.sample_window_workspace_bytes(S))
        out = HopResult(be, S, 0)
        count_only = HopOut(S, 0, be.ptr(out.root_start_ptr), be.ptr(out.root_end_ptr), None, None, None, None,
                            be.ptr(out.counts))
        self._ck(self.lib.sample_window(C.byref(g.view), be.ptr(slot_node), be.ptr(slot_ts), S, C.byref(p),
                                        C.byref(count_only), be.ptr(ws), wsb, be.stream()))
        _, E, bad = be.tolist(out.counts)
        check_sample_bad(bad)
        full = HopResult(be, S, E, counts=out.counts)
        self._ck(self.lib.sample_window(C.byref(g.view), be.ptr(slot_node), be.ptr(slot_ts), S, C.byref(p),
                                        C.byref(full.struct), be.ptr(ws), wsb, be.stream()))
        return full.finalize(*be.tolist(full.counts))

    def khop_buffers(self, S0, layers, fanout, counts=None):
        """Worst-case output buffers of a k-hop call; reusable across calls.  `counts`
        (int64[3 * layers], zeroed) may be a slice of a larger array of the caller's."""
        be = self.be
        slot_node0, slot_ts0 = be.empty(S0), be.empty(S0)
        outs, cap = [], S0
        if counts is None:
            counts = be.zeros(3 * max(layers, 1))
        for l in range(layers):
            outs.append(HopResult(be, cap, cap * fanout, counts[3 * l: 3 * l + 3]))
            cap *= fanout
        res = KHopResult(self, slot_node0, slot_ts0, outs, counts)
        res.S0, res.fanout = S0, fanout
        res.structs = (HopOut * max(layers, 1))(*[o.struct for o in outs])
        # a private workspace: calls on different buffers may overlap on different streams
        res.ws_bytes = int(self.lib.sample_khop_workspace_bytes(S0, layers, fanout))
        res.ws = be.empty(max(res.ws_bytes, 256), "u8")
        return res

    def sample_khop(self, g, roots, ts_ptr, root_ts, neg_roots, neg_ts, layers, p,
                    finalize=True, out=None):
        self._chk("i64", roots=roots, ts_ptr=ts_ptr, root_ts=root_ts, neg_roots=neg_roots, neg_ts=neg_ts)
        be = self.be
        R, S_pos, N_neg = int(roots.shape[0]), int(root_ts.shape[0]), int(neg_roots.shape[0])
        S0 = S_pos + N_neg
        _check_root_hint(p, S_pos)
        if self.check_hints:
            self.verify_root_hint(g, roots, ts_ptr, root_ts, p)
        res = out if out is not None else self.khop_buffers(S0, layers, p.fanout)
        if res.S0 < S0 or len(res.hops) != layers or res.fanout < p.fanout:
            raise MemoryError("khop buffers are smaller than this call needs")
        ws, wsb = res.ws, be.nbytes(res.ws)

        def launch(params):
            self._ck(self.lib.sample_khop(C.byref(g.view), R, be.ptr(roots), be.ptr(ts_ptr), S_pos,
                                          be.ptr(root_ts), N_neg, be.ptr(neg_roots), be.ptr(neg_ts),
                                          layers, C.byref(params), be.ptr(res.slot_node0), be.ptr(res.slot_ts0),
                                          res.structs, be.ptr(ws), wsb, be.stream()))

        launch(p)
        res.S0_live = S0
        # Should a block of the single-launch route have given up its bounded wait, reading the result
        # re-issues the call through the launch-per-hop route (which has no such wait); a remap state the
        # sampler was recording ids in is initialised again first.
        res._recover = lambda: (self._reinit_marked(p), launch(self.multi_launch(p)))
        return res.finalize() if finalize else res

    def sample_khop_multi(self, g, roots, ts_ptr, root_ts, neg_roots, neg_ts, layers, params, outs):
        """Several k-hop calls (params[q] -> outs[q], buffers of khop_buffers) over the same roots
        in one library call; a most-recent and a uniform 2-hop call share one launch.  The results
        are not finalized; they share the hop-0 slot arrays of outs[0].  The inputs must stay unchanged
        until the results have been finalized (a poisoned call is re-issued from them, see `recover` below)."""
        self._chk("i64", roots=roots, ts_ptr=ts_ptr, root_ts=root_ts, neg_roots=neg_roots, neg_ts=neg_ts)
        be, Q = self.be, len(params)
        R, S_pos, N_neg = int(roots.shape[0]), int(root_ts.shape[0]), int(neg_roots.shape[0])
        S0 = S_pos + N_neg
        fan = max(p.fanout for p in params)
        for p, res in zip(params, outs):
            _check_root_hint(p, S_pos)
            if self.check_hints:
                self.verify_root_hint(g, roots, ts_ptr, root_ts, p)
            if res.S0 < S0 or len(res.hops) != layers or res.fanout < p.fanout:
                raise MemoryError("khop buffers are smaller than this call needs")
        head = outs[0]
        need = int(self.lib.sample_khop_multi_workspace_bytes(S0, layers, fan, Q))
        if getattr(head, "ws_multi", None) is None or be.nbytes(head.ws_multi) < need:
            head.ws_multi = be.empty(max(need, 256), "u8")
        structs = (HopOut * max(Q * layers, 1))(*[o.struct for res in outs for o in res.hops])

        def launch(ps):
            pa = (_abi.SampleParams * max(Q, 1))(*ps)
            self._ck(self.lib.sample_khop_multi(C.byref(g.view), R, be.ptr(roots), be.ptr(ts_ptr), S_pos,
                                                be.ptr(root_ts), N_neg, be.ptr(neg_roots), be.ptr(neg_ts),
                                                layers, Q, pa, be.ptr(head.slot_node0), be.ptr(head.slot_ts0),
                                                structs, be.ptr(head.ws_multi), be.nbytes(head.ws_multi), be.stream()))

        launch(params)

        # Should a block of the shared single launch have given up its bounded wait, reading any of the results
        # re-issues the WHOLE call once through the launch-per-hop route (a pair shares one kernel: both queries are
        # void), after initialising the remap states that the queries were recording ids in.  The re-issue reads the
        # input arrays again: they must hold this call's batch until the results have been finalized.
        def recover():
            for res in outs:
                res._recover = None
            for p in params:
                self._reinit_marked(p)
            launch([self.multi_launch(p) for p in params])

        for res in outs:
            res.slot_node0, res.slot_ts0, res.S0_live = head.slot_node0, head.slot_ts0, S0
            res._recover = recover
            res.final = False
        return outs

    # ---------------------------------------------- several batches per call
    def khop_batched_buffers(self, S_max, B, layers, fanout, Q=1, counts=None):
        """Worst-case output buffers of `sample_khop_batched` for Q queries over up to S_max root slots in
        B batches; reusable across calls.  `counts` (int64[Q * 3 * layers], zeroed) may be the caller's."""
        be = self.be
        if counts is None:
            counts = be.zeros(Q * 3 * max(layers, 1))
        queries = []
        for q in range(Q):
            outs, cap = [], S_max
            cq = counts[q * 3 * layers: (q + 1) * 3 * layers]
            for l in range(layers):
                outs.append(HopResult(be, cap, cap * fanout, cq[3 * l: 3 * l + 3]))
                cap *= fanout
            r = KHopResult(self, None, None, outs, cq)
            r.S0, r.fanout = S_max, fanout
            queries.append(r)
        res = KHopBatched(self, queries, B, S_max, layers, fanout, counts)
        res.seg = be.zeros((Q, layers + 1, B + 1))
        res.structs = (HopOut * max(Q * layers, 1))(*[o.struct for r in queries for o in r.hops])
        res.ws_bytes = int(self.lib.sample_khop_batched_workspace_bytes(S_max, layers, fanout, Q))
        res.ws = be.empty(max(res.ws_bytes, 256), "u8")
        return res

    def sample_khop_batched(self, g, slot_node, slot_ts, batch_ptr, layers, params, out=None, slot_hint=None,
                            finalize=False):
        """The root slots of B mini-batches (slot_node/slot_ts, batch b owning [batch_ptr[b], batch_ptr[b+1]);
        batch_ptr: device int64[B+1]) sampled by one k-hop call per entry of `params`; -> KHopBatched whose
        `seg[q, l+1]` says where each batch's edges of hop l begin.  slot_hint: window ends of the slots
        (`window_end`; -1 = search)."""
        self._chk("i64", slot_node=slot_node, slot_ts=slot_ts, batch_ptr=batch_ptr, slot_hint=slot_hint)
        be, Q = self.be, len(params)
        S_max, B = int(slot_node.shape[0]), int(batch_ptr.shape[0]) - 1
        if int(slot_ts.shape[0]) != S_max or (slot_hint is not None and int(slot_hint.shape[0]) < S_max):
            raise ValueError("sample_khop_batched: slot_node, slot_ts and slot_hint differ in length")
        fan = max(p.fanout for p in params)
        res = out if out is not None else self.khop_batched_buffers(S_max, B, layers, fan, Q)
        if res.S_max < S_max or res.B != B or res.layers != layers or res.fanout < fan or len(res.queries) != Q:
            raise MemoryError("khop batched buffers do not fit this call")
        pa = (_abi.SampleParams * Q)(*params)
        self._ck(self.lib.sample_khop_batched(C.byref(g.view), B, be.ptr(batch_ptr), S_max, be.ptr(slot_node),
                                              be.ptr(slot_ts), be.ptr(slot_hint), layers, Q, pa, res.structs,
                                              be.ptr(res.seg), be.ptr(res.ws), be.nbytes(res.ws), be.stream()))
        res.slot_node, res.slot_ts, res.batch_ptr = slot_node, slot_ts, batch_ptr
        res.final = False
        for r in res.queries:
            r.slot_node0, r.slot_ts0, r.final = slot_node, slot_ts, False
        return res.finalize() if finalize else res

    def remap_batched_state(self, universe, B):
        """Remap state for `unique_compact_batched`: B copies of the id universe [0, universe)."""
        nbytes = int(self.lib.remap_batched_state_bytes(universe, B))
        if nbytes == 0:
            raise ValueError(f"remap_batched_state: universe must be positive and B in 1..{_abi.BATCH_MAX}")
        st = self.be.empty(max(nbytes, 8), "u8")
        self._ck(self.lib.remap_batched_init(self.be.ptr(st), nbytes, universe, B, self.be.stream()))
        rs = RemapState(st, universe)
        rs.B = int(B)
        return rs

    def unique_compact_batched(self, arrays, segs, state, out_arrays=None, unique_out=None, U_off=None,
                               workspace=None, finalize=True):
        """Per batch np.unique(return_inverse) over the batch's slices of `arrays` (segs[g]: device int64[B+1]
        offsets of array g, segs[g][B] = its live length).  -> (local arrays, unique_out, U_off) where batch
        b's distinct ids are unique_out[U_off[b]: U_off[b+1]]; finalize reads U_off on the host and narrows."""
        self._chk("i64", **{f"arrays[{i}]": a for i, a in enumerate(arrays)})
        self._chk("i64", **{f"segs[{i}]": a for i, a in enumerate(segs)})
        be, G, B = self.be, len(arrays), state.B
        if len(segs) != G or any(int(sg.shape[0]) != B + 1 for sg in segs):
            raise ValueError("unique_compact_batched: one segment table of B + 1 entries per array")
        len_max = (i64 * max(G, 1))(*[int(a.shape[0]) for a in arrays])
        ids = (vp * max(G, 1))(*[be.ptr(a) for a in arrays])
        sg = (vp * max(G, 1))(*[be.ptr(a) for a in segs])
        if out_arrays is None:
            out_arrays = [be.empty(int(a.shape[0])) for a in arrays]
        outs = (vp * max(G, 1))(*[be.ptr(a) for a in out_arrays])
        if unique_out is None:
            unique_out = be.empty(max(min(sum(len_max[:G]), B * state.universe), 1))
        if U_off is None:
            U_off = be.zeros(B + 1)
        need = int(self.lib.unique_batched_workspace_bytes(state.universe, B))
        ws, wsb = (workspace, be.nbytes(workspace)) if workspace is not None else self._workspace(need)
        self._ck(self.lib.unique_compact_batched(be.ptr(state.buf), state.universe, B, G, ids, len_max, sg, outs,
                                                 be.ptr(unique_out), int(unique_out.shape[0]), be.ptr(U_off),
                                                 be.ptr(ws), wsb, be.stream()))
        if not finalize:
            return out_arrays, unique_out, U_off
        off = be.tolist(U_off)
        return out_arrays, unique_out[: off[B]], off

    # ------------------------------------------------------------- unique
    def remap_state(self, universe):
        nbytes = self.lib.remap_state_bytes(universe)
        st = self.be.empty(max(nbytes, 8), "u8")
        self._ck(self.lib.remap_init(self.be.ptr(st), nbytes, universe, self.be.stream()))
        return RemapState(st, universe)

    def remap_reinit(self, state):
        """Initialise a remap state again in place (dense, hashed or batched): what a caller does after a call on
        it reported a void result - a numbering pass that gave up its bounded wait, or a hashed state whose epoch
        outgrew its capacity (that flag is sticky: every later call on the state reports it until this)."""
        be = self.be
        if isinstance(state, HashedRemapState):
            self._ck(self.lib.remap_hashed_init(be.ptr(state.buf), be.nbytes(state.buf), state.universe, be.stream()))
        elif getattr(state, "B", None) is not None:
            self._ck(self.lib.remap_batched_init(be.ptr(state.buf), be.nbytes(state.buf), state.universe, state.B, be.stream()))
        else:
            self._ck(self.lib.remap_init(be.ptr(state.buf), be.nbytes(state.buf), state.universe, be.stream()))
        state.count_bound = 0
        return state

    def remap_hashed_state(self, capacity):
        """Persistent hash-set remap state for arbitrary non-negative ids: `capacity` is the largest
        number of distinct ids one epoch may hold."""
        nbytes = self.lib.remap_hashed_state_bytes(capacity)
        st = self.be.empty(max(nbytes, 8), "u8")
        self._ck(self.lib.remap_hashed_init(self.be.ptr(st), nbytes, capacity, self.be.stream()))
        return HashedRemapState(st, capacity)

    def unique_compact(self, arrays, mode=_abi.UNIQUE_SORTED, state=None, reset=True,
                       lens_dev=None, out_arrays=None, finalize=True, unique_out=None, U_out=None,
                       premarked=False, workspace=None, _retry=False):
        self._chk("i64", **{f"arrays[{i}]": a for i, a in enumerate(arrays)})
        be, G = self.be, len(arrays)
        len_max = (i64 * max(G, 1))(*[int(a.shape[0]) for a in arrays])
        total = sum(len_max[:G])
        ids = (vp * max(G, 1))(*[be.ptr(a) for a in arrays])
        if out_arrays is None:
            out_arrays = [be.empty(int(a.shape[0])) for a in arrays]
        outs = (vp * max(G, 1))(*[be.ptr(a) for a in out_arrays])
        ldev = None
        if lens_dev is not None:
            ldev = (vp * max(G, 1))(*[be.ptr(a) for a in lens_dev])
        hashed = isinstance(state, HashedRemapState)
        if hashed and premarked:
            raise ValueError("unique_compact: premarked needs a dense remap state")
        cap = total if state is None else min(total + state.count_bound, state.universe)
        if state is not None and reset:
            cap = min(total, state.universe)
        if unique_out is not None:
            unique, cap = unique_out, int(unique_out.shape[0])
        else:
            unique = be.empty(max(cap, 1))
        U = be.zeros(2) if U_out is None else U_out
        universe = 0 if state is None else state.universe
        if hashed:
            need = self.lib.unique_hashed_workspace_bytes(universe, G, len_max)
            ws, wsb = (workspace, be.nbytes(workspace)) if workspace is not None else self._workspace(need)
            self._ck(self.lib.unique_compact_hashed(be.ptr(state.buf), universe, int(bool(reset)), int(mode),
                                                    G, ids, len_max, ldev, outs, be.ptr(unique), cap, be.ptr(U),
                                                    be.ptr(ws), wsb, be.stream()))
        else:
            need = self.lib.unique_workspace_bytes(universe, G, len_max)
            ws, wsb = (workspace, be.nbytes(workspace)) if workspace is not None else self._workspace(need)
            self._ck(self.lib.unique_compact(None if state is None else be.ptr(state.buf), universe,
                                             int(bool(reset)), int(mode) | (_abi.UNIQUE_PREMARKED if premarked else 0),
                                             G, ids, len_max, ldev, outs,
                                             be.ptr(unique), cap, be.ptr(U), be.ptr(ws), wsb,
                                             be.stream()))
        if state is not None:
            state.count_bound = cap
        if not finalize:
            return out_arrays, unique, U
        u_total, u_before = be.tolist(U)
        if (u_total == POISON and state is not None and not hashed and reset and not premarked and not _retry):
            # a tile of the single-launch numbering pass gave up its bounded wait: the state is initialised
            # again and the call re-issued with the numbering in separate launches (nothing there waits)
            self._ck(self.lib.remap_init(be.ptr(state.buf), be.nbytes(state.buf), state.universe, be.stream()))
            state.count_bound = 0
            self.recoveries += 1
            return self.unique_compact(arrays, int(mode) | _abi.UNIQUE_MULTI_LAUNCH, state, True, lens_dev=lens_dev,
                                       out_arrays=out_arrays, unique_out=unique_out, U_out=U_out, workspace=workspace,
                                       _retry=True)
        check_unique_total(u_total)
        return out_arrays, unique[:u_total], (u_total, u_before)

    # ------------------------------------------------------------- gather
    def cache(self, row_bytes, hot, rows=None, cold=None, hot_slot=None, g2l=None,
              id_mask=-1, ts_hot=None, ts_cold=None):
        """`cold` and `hot` may be row-strided views ([rows, width] with unit stride inside a row) and `ts_cold`
        a strided 1-D view: their strides travel in the struct, so a cold tier that keeps a row and its
        time in one record (see `interleaved_cold`) is read in place, and a cache over some columns of wider
        rows (the memory part of rows holding memory and features side by side) needs no copy."""
        be = self.be
        hot_rows = 0 if hot is None else int(hot.shape[0])
        if rows is None:
            rows = int(cold.shape[0]) if cold is not None else hot_rows
        cold_stride = ts_cold_stride = hot_stride = 0
        cold_ptr, ts_cold_ptr, hot_ptr = None, None, None
        if cold is not None:
            st = _byte_strides(cold)
            if len(st) == 2 and cold.shape[0] > 1 and st[0] != cold.shape[1] * st[1]:
                if st[1] != _itemsize(cold):
                    raise ValueError("cache: the cold table must have unit stride inside a row")
                cold_stride = int(st[0])
            cold_ptr = _address(cold)
        if hot is not None:       # (a column slice of wider HBM rows: the row stride travels in the struct)
            st = _byte_strides(hot)
            if len(st) == 2 and hot.shape[0] > 1 and st[0] != hot.shape[1] * st[1]:
                if st[1] != _itemsize(hot):
                    raise ValueError("cache: the hot table must have unit stride inside a row")
                hot_stride = int(st[0])
            hot_ptr = _address(hot)
        if ts_cold is not None:
            st = _byte_strides(ts_cold)
            if len(st) == 1 and ts_cold.shape[0] > 1 and st[0] != _itemsize(ts_cold):
                ts_cold_stride = int(st[0])
            ts_cold_ptr = _address(ts_cold)
        c = Cache(int(rows), int(row_bytes), int(id_mask), be.ptr(g2l),
                  0 if g2l is None else int(g2l.shape[0]), be.ptr(hot_slot), hot_ptr,
                  hot_rows, cold_ptr, be.ptr(ts_hot), ts_cold_ptr, cold_stride, ts_cold_stride, hot_stride)
        c._keep = (hot, cold, hot_slot, g2l, ts_hot, ts_cold)  # keep the arrays alive
        return c

    def interleaved_cold(self, rows, width, dtype=None, record_bytes=None):
        """Pinned host memory for a cold tier whose records hold a row and its last-update time side by
        side: -> (data [rows, width] view, ts [rows] int64 view, record buffer).  Reads over PCIe are paid
        for in whole 128-byte lines, so a time kept in a table of its own costs a line per row; in a
        record of a multiple of 128 bytes it rides in the row's last line."""
        torch = self.be.torch
        dtype = dtype or torch.float32
        item = torch.empty((), dtype=dtype).element_size()
        row_bytes = width * item
        ts_off = (row_bytes + 7) // 8 * 8
        if record_bytes is None:
            record_bytes = (ts_off + 8 + 127) // 128 * 128
        if record_bytes % 8 or record_bytes % item or record_bytes < ts_off + 8:
            raise ValueError("interleaved_cold: record size %d does not fit row + time" % record_bytes)
        buf = torch.zeros((rows, record_bytes), dtype=torch.uint8, pin_memory=self.be.device.type == "cuda")
        data = buf.view(dtype)[:, :width]
        ts = buf.view(torch.int64)[:, ts_off // 8]
        return data, ts, buf

    def gather(self, cache, ids, out, out_ts=None, stats=None, N_dev=None):
        self._chk("i64", ids=ids, out_ts=out_ts, stats=stats, N_dev=N_dev)
        be = self.be
        self._ck(self.lib.gather(C.byref(cache), be.ptr(ids), int(ids.shape[0]), be.ptr(N_dev),
                                 be.ptr(out), be.ptr(out_ts), be.ptr(stats), be.stream()))
        return out

    def gather_dedup(self, cache, ids, out, staging, out_ts=None, staging_ts=None, stats=None, N_dev=None, workspace=None):
        """`gather` with every distinct cold row of the call read from pinned host memory once (into `staging`, an
        HBM buffer of [rows, row_bytes]; `staging_ts` int64[rows] when times are gathered too) and the requests of
        cold rows served from there.  stats: optional int64[4] += {hot, cold requests, absent, distinct cold rows}."""
        self._chk("i64", ids=ids, out_ts=out_ts, stats=stats, N_dev=N_dev, staging_ts=staging_ts)
        be, N = self.be, int(ids.shape[0])
        need = int(self.lib.gather_dedup_workspace_bytes(N))
        ws, wsb = (workspace, be.nbytes(workspace)) if workspace is not None else self._workspace(need)
        self._ck(self.lib.gather_dedup(C.byref(cache), be.ptr(ids), N, be.ptr(N_dev), be.ptr(out), be.ptr(out_ts),
                                       be.ptr(stats), be.ptr(staging), be.ptr(staging_ts),
                                       0 if staging is None else int(staging.shape[0]), be.ptr(ws), wsb, be.stream()))
        return out

    def gather_plan(self, segments):
        """Pre-marshalled argument block for `gather_multi`: segments is a list of
        (cache, ids, out, out_ts or None, N_dev or None)."""
        be = self.be
        arr = (GatherSeg * len(segments))()
        for i, (c, ids, out, out_ts, n_dev) in enumerate(segments):
            arr[i] = GatherSeg(C.pointer(c), be.ptr(ids), int(ids.shape[0]), be.ptr(n_dev), be.ptr(out), be.ptr(out_ts))
        arr._keep = segments
        return arr

    def gather_multi(self, plan):
        """All segments of `plan` (from gather_plan) in one launch."""
        self._ck(self.lib.gather_multi(len(plan), plan, self.be.stream()))

    def scatter_update(self, cache, hot_rw, cold_rw, ts_hot_rw, ts_cold_rw, ids, values, ts=None):
        self._chk("i64", ids=ids, ts=ts)
        be = self.be
        addr = lambda a: None if a is None else _address(a)     # (the cold tier may be strided views of a record buffer)
        self._ck(self.lib.scatter_update(C.byref(cache), be.ptr(hot_rw), addr(cold_rw),
                                         be.ptr(ts_hot_rw), addr(ts_cold_rw), be.ptr(ids),
                                         int(ids.shape[0]), be.ptr(values), be.ptr(ts),
                                         be.stream()))

    # ------------------------------------------------------ chunks / seeds
    def chunk_index(self, n, num_chunks, node_chunk):
        """-> (chunk_ptr[num_chunks+1], chunk_nodes[n]) on the backend's device."""
        self._chk("i64", node_chunk=node_chunk)
        be = self.be
        chunk_ptr, chunk_nodes = be.empty(num_chunks + 1), be.empty(max(n, 1))
        ws, wsb = self._workspace(self.lib.chunk_index_workspace_bytes(n))
        self._ck(self.lib.chunk_index_build(n, num_chunks, be.ptr(node_chunk), be.ptr(chunk_ptr),
                                            be.ptr(chunk_nodes), be.ptr(ws), wsb, be.stream()))
        return chunk_ptr, chunk_nodes[:n]

    def seeds(self, g, chunk_ptr, chunk_nodes, chunks, cand_off, n_cand, t_begin, t_end, with_window_end=False):
        """-> (roots, ts_ptr, ts, q_ptr, q_eid).  `cand_off` is the exclusive prefix
        of the selected chunks' sizes, `n_cand` its last entry (host int).  with_window_end: a sixth
        array, per (root, timestamp) where the window strictly before it ends (the `root_hint` of
        a sampling call over these roots)."""
        self._chk("i64", chunk_ptr=chunk_ptr, chunk_nodes=chunk_nodes, chunks=chunks, cand_off=cand_off)
        be = self.be
        q = SeedQuery(be.ptr(chunk_ptr), be.ptr(chunk_nodes), int(chunks.shape[0]), be.ptr(chunks),
                      be.ptr(cand_off), int(n_cand), int(t_begin), int(t_end))
        totals = be.zeros(3)
        ws, wsb = self._workspace(self.lib.seeds_workspace_bytes(n_cand))
        self._ck(self.lib.seeds_count(C.byref(g.view), C.byref(q), be.ptr(totals), be.ptr(ws), wsb, be.stream()))
        R, S, Q = be.tolist(totals)
        roots, ts_ptr, ts, q_ptr, q_eid = be.empty(R), be.empty(R + 1), be.empty(S), be.empty(S + 1), be.empty(Q)
        w_end = be.empty(S) if with_window_end else None
        self._ck(self.lib.seeds_fill(C.byref(g.view), C.byref(q), be.ptr(totals), be.ptr(roots), be.ptr(ts_ptr),
                                     be.ptr(ts), be.ptr(q_ptr), be.ptr(q_eid), be.ptr(w_end) if with_window_end else None,
                                     be.ptr(ws), wsb, be.stream()))
        return (roots, ts_ptr, ts, q_ptr, q_eid, w_end) if with_window_end else (roots, ts_ptr, ts, q_ptr, q_eid)

    def slice(self, g, chunk_ptr, chunk_nodes, node_chunk, chunks, cand_off, n_cand, t_begin, t_end,
              full_timestamps=False):
        """Sub-graph of the selected chunks over [t_begin, t_end)
        -> (nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid)."""
        self._chk("i64", chunk_ptr=chunk_ptr, chunk_nodes=chunk_nodes, node_chunk=node_chunk, chunks=chunks, cand_off=cand_off)
        be = self.be
        q = SeedQuery(be.ptr(chunk_ptr), be.ptr(chunk_nodes), int(chunks.shape[0]), be.ptr(chunks),
                      be.ptr(cand_off), int(n_cand), int(t_begin), int(t_end))
        total_chunks, full = int(chunk_ptr.shape[0]) - 1, int(bool(full_timestamps))
        totals = be.zeros(3)
        ws, wsb = self._workspace(self.lib.slice_workspace_bytes(n_cand, total_chunks))
        self._ck(self.lib.slice_count(C.byref(g.view), C.byref(q), be.ptr(node_chunk), total_chunks, full,
                                      be.ptr(totals), be.ptr(ws), wsb, be.stream()))
        R, T, E = be.tolist(totals)
        nodes, ts_ptr, ts, edge_ptr = be.empty(R), be.empty(R + 1), be.empty(T), be.empty(T + 1)
        col, col_ts, col_eid = be.empty(E), be.empty(E), be.empty(E)
        self._ck(self.lib.slice_fill(C.byref(g.view), C.byref(q), be.ptr(node_chunk), total_chunks, full,
                                     be.ptr(totals), be.ptr(nodes), be.ptr(ts_ptr), be.ptr(ts), be.ptr(edge_ptr),
                                     be.ptr(col), be.ptr(col_ts), be.ptr(col_eid), be.ptr(ws), wsb, be.stream()))
        return nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid

    # ------------------------------------------------------------- blocks
    def block_build(self, root_start_ptr, counts, S_max, E_max, dst_offset, src_offset, with_edge_dst=False):
        be = self.be
        indptr, indices = be.empty(dst_offset + S_max + 1), be.empty(E_max)
        edge_dst = be.empty(E_max) if with_edge_dst else None
        self._ck(self.lib.block_build(be.ptr(root_start_ptr), be.ptr(counts), S_max, E_max, dst_offset,
                                      src_offset, be.ptr(indptr), be.ptr(indices), be.ptr(edge_dst), be.stream()))
        return indptr, indices, edge_dst

    # ------------------------------------------------- (id, ts) pair algebra
    def unique_pairs(self, ids, ts, N_dev=None):
        """-> (uniq_ids[U], uniq_ts[U], inverse[N]): np.unique over (id, ts) records with
        return_inverse (one synchronising read of U)."""
        self._chk("i64", ids=ids, ts=ts, N_dev=N_dev)
        be, N = self.be, int(ids.shape[0])
        uid, uts, inv, U = be.empty(max(N, 1)), be.empty(max(N, 1)), be.empty(max(N, 1)), be.zeros(1)
        ws, wsb = self._workspace(self.lib.unique_pairs_workspace_bytes(N))
        self._ck(self.lib.unique_pairs(be.ptr(ids), be.ptr(ts), N, be.ptr(N_dev), be.ptr(uid), be.ptr(uts),
                                       be.ptr(inv), be.ptr(U), be.ptr(ws), wsb, be.stream()))
        u = be.tolist(U)[0]
        n = N if N_dev is None else min(N, be.tolist(N_dev)[0])
        return uid[:u], uts[:u], inv[:n]

    def csc_from_pairs(self, dst_local, ts, num_dst, E_dev=None):
        """-> (indptr[num_dst + 1], perm[E]): the stable (dst_local, ts) edge order."""
        self._chk("i64", dst_local=dst_local, ts=ts, E_dev=E_dev)
        be, E = self.be, int(dst_local.shape[0])
        indptr, perm = be.empty(num_dst + 1), be.empty(max(E, 1))
        ws, wsb = self._workspace(self.lib.csc_from_pairs_workspace_bytes(E))
        self._ck(self.lib.csc_from_pairs(be.ptr(dst_local), be.ptr(ts), E, be.ptr(E_dev), int(num_dst),
                                         be.ptr(indptr), be.ptr(perm), be.ptr(ws), wsb, be.stream()))
        return indptr, perm[:E]

    # ------------------------------------------------------ latest by key
    def segment_max_ts(self, local, ts, U, N_dev=None, U_dev=None):
        """-> (max_ts[U], arg[U]): per dense key the largest timestamp and the first
        event index attaining it."""
        self._chk("i64", local=local, ts=ts, N_dev=N_dev, U_dev=U_dev)
        be = self.be
        max_ts, arg = be.empty(max(U, 1)), be.empty(max(U, 1))
        self._ck(self.lib.segment_max_ts(be.ptr(local), be.ptr(ts), int(local.shape[0]), be.ptr(N_dev), int(U),
                                         be.ptr(U_dev), be.ptr(max_ts), be.ptr(arg), be.stream()))
        return max_ts[:U], arg[:U]

    # -------------------------------------------------------- time encode
    def time_encode(self, dt, w, b, dt_dtype=_abi.DT_I64, out=None, N_dev=None):
        self._chk("i64" if dt_dtype == _abi.DT_I64 else "f32", dt=dt)
        self._chk("f32", w=w, b=b, out=out)
        be, N, dim = self.be, int(dt.shape[0]), int(w.shape[0])
        if out is None:
            out = be.empty((N, dim), "f32")
        self._ck(self.lib.time_encode(be.ptr(dt), dt_dtype, N, be.ptr(N_dev), be.ptr(w),
                                      be.ptr(b), dim, be.ptr(out), be.stream()))
        return out


@contextlib.contextmanager
def graph_capture(graph, stream=None):
    """`torch.cuda.graph(graph, stream=stream)` with Python's cycle collector held off.  A collection that runs
    while a stream is capturing may free a dead object that owns another CUDAGraph (a dropped pipeline, say);
    that graph's destructor calls the runtime, the runtime refuses calls of that kind from a capturing thread,
    and an error thrown from a destructor ends the process in std::terminate.  Dead cycles are collected before
    the capture starts instead (torch itself no longer does that by default)."""
    import torch
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph, stream=stream):
            yield
    finally:
        if was_enabled:
            gc.enable()


class RemapState:
    def __init__(self, buf, universe):
        self.buf, self.universe, self.count_bound = buf, int(universe), 0


class HashedRemapState(RemapState):
    """Hash-set remap state: `universe` holds its capacity in distinct ids (what bounds an epoch)."""

    def __init__(self, buf, capacity):
        super().__init__(buf, capacity)
        self.capacity = int(capacity)


class KHopResult:
    def __init__(self, hp, slot_node0, slot_ts0, hops, counts):
        self.hp, self.slot_node0, self.slot_ts0, self.hops = hp, slot_node0, slot_ts0, hops
        self.counts, self.final = counts, False

    def finalize(self, counts_host=None):
        """Read the per-hop device counts (one synchronising copy, unless the caller
        already has them on the host) and narrow."""
        if not self.final:
            c = self.hp.be.tolist(self.counts) if counts_host is None else list(counts_host)
            if self.hops and c[2] >= POISON and getattr(self, "_recover", None) is not None:
                self._recover()                      # once: the launch-per-hop route cannot give up
                self._recover = None
                self.hp.recoveries += 1
                c = self.hp.be.tolist(self.counts)
            for l, h in enumerate(self.hops):
                h.finalize(*c[3 * l: 3 * l + 3])
            S0 = getattr(self, "S0_live", None)
            if S0 is not None:
                self.slot_node0, self.slot_ts0 = self.slot_node0[:S0], self.slot_ts0[:S0]
            self.final = True
        return self


class KHopBatched:
    """Result of `HotPath.sample_khop_batched`: `queries[q]` is a KHopResult over all batches' slots;
    `seg[q, l]` (device, B + 1 entries) delimits the batches in the slots of hop l (= the edges of hop l - 1)."""

    def __init__(self, hp, queries, B, S_max, layers, fanout, counts):
        self.hp, self.queries, self.B, self.S_max, self.layers, self.fanout = hp, queries, B, S_max, layers, fanout
        self.counts, self.final, self.seg_host = counts, False, None

    def finalize(self):
        """One synchronising read of the segment table and the counts; narrows every query's arrays (for good:
        buffers that a later call is to reuse are read through `seg` and `counts` instead, without finalizing)."""
        if not self.final:
            be = self.hp.be
            self.seg_host = be.tolist(self.seg)
            c = be.tolist(self.counts)
            L = self.layers
            S = self.seg_host[0][0][self.B]
            for q, r in enumerate(self.queries):
                r.S0_live = S
                r.finalize(c[q * 3 * L: (q + 1) * 3 * L])
            self.final = True
        return self

    def batch(self, q, b):
        """Batch b of query q: [(slot range), (edge range of hop 0), ...] as python ints (after finalize)."""
        self.finalize()
        sg = self.seg_host[q]
        return [(sg[l][b], sg[l][b + 1]) for l in range(self.layers + 1)]
