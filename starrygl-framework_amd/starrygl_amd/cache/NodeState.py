"""Node state cache (TGN memory / historical embeddings) with the interface of
the reference's starrygl/cache/NodeState.py:8-82, served by the two-tier gather
of libsgl_hot.so.

Storage follows the reference: `data [loc_nums, dim] fp32` and `ts [loc_nums]`
on `device` ('cpu' = pinned host memory by default).  Added here: an optional
HBM tier (`hot_ids`): those local rows are mirrored in device memory and a
gather reads them from HBM, every other row is read in place from the pinned
host table.  `__getitem__` and `prefetch` return tensors on the GPU.
"""
from typing import Optional, Tuple, Union

import torch
from torch import Tensor

from ..lib import hot_path
from ..utils.context import DistributedContext
from ..utils.partition_book import DistRouteIndex, PartitionState


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
        self.data = torch.zeros(self.loc_nums, dim, dtype=torch.float32, device=self.device)
        self.ts = torch.zeros(self.loc_nums, dtype=ts_dtype, device=self.device)
        if self.device.type == "cpu":
            if not pinned:
                raise ValueError("host-resident node state must be pinned: the GPU reads it in place")
            self.data, self.ts = self.data.pin_memory(), self.ts.pin_memory()
        self._hot_ids = None
        self._build_tiers(hot_ids)

    # ------------------------------------------------------------ tiers
    def _build_tiers(self, hot_ids):
        hp = hot_path(self.gpu)
        self._hp = hp
        self.hot_data = self.hot_ts = self.hot_slot = None
        if self.device.type == "cuda" or hot_ids is None:
            hot_ids = None
        self._hot_ids = hot_ids
        if hot_ids is not None:
            hot_ids = hot_ids.to(torch.int64).cpu()
            slot = torch.full((self.loc_nums,), -1, dtype=torch.int32)
            slot[hot_ids] = torch.arange(hot_ids.numel(), dtype=torch.int32)
            self.hot_slot = slot.to(self.gpu)
            self.hot_data = self.data[hot_ids].to(self.gpu)
            self.hot_ts = self.ts[hot_ids].to(self.gpu)
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
        else:
            self._c_data = hp.cache(self.dim * 4, self.hot_data, rows=self.loc_nums, cold=self.data,
                                    hot_slot=self._slot_or_all_cold(), g2l=g2l, id_mask=mask)
            self._c_ts = hp.cache(es, self.hot_ts, rows=self.loc_nums, cold=self.ts,
                                  hot_slot=self._slot_or_all_cold(), g2l=g2l, id_mask=mask)

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
        hot_rw = self.hot_data if self.hot_data is not None else (self.data if self.device.type == "cuda" else None)
        cold_rw = self.data if self.device.type == "cpu" else None
        self._hp.scatter_update(self._c_data, hot_rw, cold_rw, None, None, ids, vals)
        if ts is not None:
            t = ts.to(self.gpu, self.ts.dtype).reshape(-1).contiguous()
            hot_t = self.hot_ts if self.hot_ts is not None else (self.ts if self.device.type == "cuda" else None)
            cold_t = self.ts if self.device.type == "cpu" else None
            self._hp.scatter_update(self._c_ts, hot_t, cold_t, None, None, ids, t)
        if self.device.type == "cpu":
            torch.cuda.current_stream(self.gpu).synchronize()   # host-visible before the caller reads .data

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
            self.data, self.ts = self.data.to(new_device), self.ts.to(new_device)
            if new_device.type == "cpu":
                self.data, self.ts = self.data.pin_memory(), self.ts.pin_memory()
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
