"""Node state cache (TGN memory / historical embeddings) with the interface of
the reference's starrygl/cache/NodeState.py:8-82, served by the two-tier gather
of libsgl_hot.so.

Storage follows the reference: `data [loc_nums, dim] fp32` and `ts [loc_nums]`
on `device` ('cpu' = pinned host memory by default).  Added here: an optional
HBM tier (`hot_ids`): those local rows are mirrored in device memory and a
gather reads them from HBM, every other row is read in place from the pinned
host table.  `__getitem__` and `prefetch` return tensors on the GPU.

Host-resident state keeps a row and its time in ONE record of a multiple of 128
bytes (`data` and `ts` are strided views of the record buffer): the GPU pays for
reads over PCIe in whole 128-byte lines, so a time in a table of its own would
cost a line per row - a third of what a 400-byte row costs - and a second launch.
The time occupies an 8-byte slot of the record whatever `ts_dtype` is, and one
gather / one scatter launch moves rows and times together.
"""
from typing import Optional, Tuple, Union

import torch
from torch import Tensor

from ..lib import hot_path
from ..utils.context import DistributedContext
from ..utils.partition_book import DistRouteIndex, PartitionState


def _low_f32(raw: Tensor) -> Tensor:
    """float32 view of the low halves of a (possibly strided) int64 array"""
    n = raw.shape[0]
    base = torch.as_strided(raw, (n, 1), (raw.stride(0), 1)) if n else raw.reshape(0, 1)
    return base.view(torch.float32)[:, 0]


class DistNodeState:
    def __init__(self, state: PartitionState, dim: int, device: Union[str, torch.device] = "cpu",
                 pinned: bool = True, hot_ids: Optional[Tensor] = None, ts_dtype: torch.dtype = torch.float32,
                 gpu: Optional[Union[str, torch.device]] = None):
        self.state = state
        self.node_mapper = state.node_mapper
        self.loc_nums = self.node_mapper.loc_nums
        self.dim = dim
        self.device = torch.device(device)
        self.gpu = torch.device(gpu) if gpu is not None else (
            self.device if self.device.type == "cuda" else DistributedContext.get_default_context().device)
        if ts_dtype not in (torch.float32, torch.int64):
            raise TypeError("ts_dtype must be torch.float32 (reference layout) or torch.int64")
        if self.device.type == "cpu":
            if not pinned:
                raise ValueError("host-resident node state must be pinned: the GPU reads it in place")
            self._alloc_host(ts_dtype)
        else:
            self.data = torch.zeros(self.loc_nums, dim, dtype=torch.float32, device=self.device)
            self.ts = torch.zeros(self.loc_nums, dtype=ts_dtype, device=self.device)
        self._hot_ids = None
        self._build_tiers(hot_ids)

    def _alloc_host(self, ts_dtype):
        """record buffer in pinned memory; `data`, `ts` and the 8-byte time slots (`_ts_raw`) are views of it"""
        hp = hot_path(self.gpu)
        self.data, self._ts_raw, self._rec = hp.interleaved_cold(self.loc_nums, self.dim, torch.float32)
        self.ts = self._as_ts(self._ts_raw, ts_dtype)

    @staticmethod
    def _as_ts(raw: Tensor, ts_dtype) -> Tensor:
        """the times held in a strided array of 8-byte slots, as a view of dtype ts_dtype"""
        if ts_dtype == torch.int64:
            return raw
        return _low_f32(raw)

    @staticmethod
    def _raw_ts(t: Tensor) -> Tensor:
        """times of either dtype as contiguous 8-byte slots (a float sits in the low half, the rest is zero)"""
        if t.dtype == torch.int64:
            return t.contiguous()
        raw = torch.zeros(t.numel(), dtype=torch.int64, device=t.device)
        raw.view(torch.float32)[::2] = t.reshape(-1)
        return raw

    # ------------------------------------------------------------ tiers
    def _build_tiers(self, hot_ids):
        hp = hot_path(self.gpu)
        self._hp = hp
        self.hot_data = self.hot_ts = self.hot_slot = self._hot_ts_raw = None
        if self.device.type == "cuda" or hot_ids is None:
            hot_ids = None
        self._hot_ids = hot_ids
        if hot_ids is not None:
            hot_ids = hot_ids.to(torch.int64).cpu()
            slot = torch.full((self.loc_nums,), -1, dtype=torch.int32)
            slot[hot_ids] = torch.arange(hot_ids.numel(), dtype=torch.int32)
            self.hot_slot = slot.to(self.gpu)
            self.hot_data = self.data[hot_ids].to(self.gpu)
            self._hot_ts_raw = self._ts_raw[hot_ids].to(self.gpu)
            self.hot_ts = self._as_ts(self._hot_ts_raw, self.ts.dtype)
        m = self.node_mapper
        g2l, mask = None, -1
        if m.mode == "map":
            g2l = m._g2l_map.to(self.gpu)
        elif m.mode == "dist_route_index":
            mask = DistRouteIndex.LOC_MASK
        self._g2l, self._mask = g2l, mask
        self._offset = m.offset if m.mode == "offset" else 0
        es = self.ts.element_size()
        if self.device.type == "cuda":      # single tier: the table itself is the hot tier
            self._c_data = hp.cache(self.dim * 4, self.data, g2l=g2l, id_mask=mask)
            self._c_ts = hp.cache(es, self.ts, g2l=g2l, id_mask=mask)
        else:                               # rows and times in one cache: one launch moves both
            self._c_data = hp.cache(self.dim * 4, self.hot_data, rows=self.loc_nums, cold=self.data,
                                    hot_slot=self._slot_or_all_cold(), g2l=g2l, id_mask=mask,
                                    ts_hot=self._hot_ts_raw, ts_cold=self._ts_raw)
            self._c_ts = None

    def _slot_or_all_cold(self):
        if self.hot_slot is None:
            self.hot_slot = torch.full((self.loc_nums,), -1, dtype=torch.int32, device=self.gpu)
        return self.hot_slot

    def _keys(self, key):
        ids = key.dist if isinstance(key, DistRouteIndex) else key
        ids = ids.to(self.gpu, torch.int64).contiguous()
        if isinstance(key, DistRouteIndex) and self._mask == -1:
            ids = ids & DistRouteIndex.LOC_MASK
        if self._offset:
            ids = ids - self._offset
        return ids

    # -------------------------------------------------------------- API
    def __getitem__(self, key: Union[Tensor, DistRouteIndex]) -> Tuple[Tensor, Tensor]:
        """(data rows, ts) of the given global ids / DistRouteIndex; ids that are
        not stored here yield zero rows."""
        ids = self._keys(key)
        n = ids.numel()
        out = torch.empty((n, self.dim), dtype=torch.float32, device=self.gpu)
        if self._c_ts is None:
            raw = torch.empty((n,), dtype=torch.int64, device=self.gpu)
            self._hp.gather(self._c_data, ids, out, out_ts=raw)
            return out, self._as_ts(raw, self.ts.dtype)
        out_ts = torch.empty((n,), dtype=self.ts.dtype, device=self.gpu)
        self._hp.gather(self._c_data, ids, out)
        self._hp.gather(self._c_ts, ids, out_ts)
        return out, out_ts

    def update(self, gids: Tensor, values: Tensor, ts: Optional[Tensor] = None, check_unique: bool = False):
        """Overwrite the rows of the given ids (ids not stored here are skipped).
        Ids must be unique within one call: with a repeated id the row that wins is unspecified (the
        reference's index_put keeps the last one); check_unique=True verifies it (one host synchronisation).
        Rows of the HBM tier are written there only: `.data` / `.ts` show them after flush()."""
        ids = self._keys(gids)
        if check_unique and torch.unique(ids).numel() != ids.numel():
            raise ValueError("DistNodeState.update: ids repeat within one call")
        vals = values.to(self.gpu, torch.float32).contiguous()
        if self.device.type == "cpu":
            raw = None if ts is None else self._raw_ts(ts.to(self.gpu, self.ts.dtype).reshape(-1))
            self._hp.scatter_update(self._c_data, self.hot_data, self.data, self._hot_ts_raw, self._ts_raw, ids, vals, ts=raw)
            torch.cuda.current_stream(self.gpu).synchronize()   # host-visible before the caller reads .data
            return
        self._hp.scatter_update(self._c_data, self.data, None, None, None, ids, vals)
        if ts is not None:
            t = ts.to(self.gpu, self.ts.dtype).reshape(-1).contiguous()
            self._hp.scatter_update(self._c_ts, self.ts, None, None, None, ids, t)

    def flush(self):
        """Fold the rows of the HBM tier back into `.data` / `.ts` (the tensors of the reference's layout, which
        callers read and checkpoint): until then those tensors hold the hot rows as of the last flush."""
        if self.hot_data is not None:
            torch.cuda.current_stream(self.gpu).synchronize()
            self.data[self._hot_ids] = self.hot_data.cpu()
            self.ts[self._hot_ids] = self.hot_ts.cpu()
        return self

    def state_dict(self):
        """{'data', 'ts'} with the HBM tier folded in."""
        self.flush()
        return {"data": self.data, "ts": self.ts}

    def to(self, device: Union[str, torch.device]):
        new_device = torch.device(device)
        if new_device != self.device:
            self.flush()                     # fold the HBM tier back before moving
            data, ts = self.data, self.ts
            if new_device.type == "cpu":
                self._alloc_host(ts.dtype)
                self.data.copy_(data)
                self.ts.copy_(ts)
            else:
                self.data, self.ts = data.to(new_device), ts.to(new_device)
                self._ts_raw = self._rec = None
            self.device = new_device
            if new_device.type == "cuda":
                self.gpu = new_device
            self._build_tiers(self._hot_ids)
        return self

    def reset(self):
        self.data.fill_(0)
        self.ts.fill_(0)
        if self.hot_data is not None:
            self.hot_data.fill_(0)
            self.hot_ts.fill_(0)

    def prefetch(self, gids: Tensor, stream: Optional[torch.cuda.Stream] = None):
        """The same gather issued on `stream` (a side stream overlaps it with compute)."""
        if stream is None:
            return self[gids]
        with torch.cuda.stream(stream):
            return self[gids]
