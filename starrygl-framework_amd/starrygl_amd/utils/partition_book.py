"""Id codecs and local/global id mapping with the class names and methods of
the reference's starrygl/utils/partition_book.py (DistRouteIndex :7-52,
IDMapper :56-176, PartitionState :179-276).

The lookup `to_local` is plain tensor indexing here; the fused form (id mask ->
g2l table -> hot slot -> row copy in one kernel) is `sgl_gather`, which
`DistNodeState` drives with the tables these classes own.
"""
from typing import Optional, Union

import torch
from torch import Tensor


class DistRouteIndex:
    """64-bit id: bit 62 shared flag, bits 48-61 partition, bits 0-47 local index."""
    PART_SHIFT = 48
    SHARED_BIT = 62
    LOC_MASK = 0xFFFFFFFFFFFF
    PART_MASK = 0x3FFF

    def __init__(self, index: Tensor, part_ids: Optional[Tensor] = None) -> None:
        index = index.long()
        if part_ids is None:
            self._data = index
        else:
            part_ids = part_ids.long().to(index.device)
            self._data = (index & self.LOC_MASK) | ((part_ids & self.PART_MASK) << self.PART_SHIFT)

    @property
    def loc(self) -> Tensor:
        return self._data & self.LOC_MASK

    @property
    def part(self) -> Tensor:
        return (self._data >> self.PART_SHIFT) & self.PART_MASK

    def set_shared(self, indx):
        self._data[indx] |= (1 << self.SHARED_BIT)

    @property
    def is_shared(self) -> Tensor:
        return ((self._data >> self.SHARED_BIT) & 1).to(torch.bool)

    @property
    def dist(self) -> Tensor:
        return self._data

    @property
    def device(self):
        return self._data.device

    @property
    def shape(self):
        return self._data.shape

    def to(self, device):
        return DistRouteIndex(self._data.to(device))


class IDMapper:
    """Local / global / dist id conversion and master test for one entity kind
    (nodes or edges).  mode: 'identity' | 'offset' | 'map' | 'dist_route_index'."""

    def __init__(self, loc_ids: Tensor, num_master: int, mode: str = "identity",
                 dist_mapper: Optional[Tensor] = None, replica_table=None, offset: int = 0, global_num: int = 0):
        if mode not in ("identity", "offset", "map", "dist_route_index"):
            raise ValueError(f"unknown IDMapper mode {mode!r}")
        self.loc_ids = loc_ids
        self._num_master = num_master
        self.mode = mode
        self.dist_mapper = dist_mapper
        self.offset = offset
        self._replica_table = replica_table
        self._global_num = global_num
        self._g2l_map: Optional[Tensor] = None
        if mode == "map":
            self.build_g2l_map()

    @property
    def loc_nums(self):
        return self.loc_ids.size(0)

    @property
    def num_master(self):
        return self._num_master

    @property
    def global_nums(self):
        return self._global_num

    @property
    def replica_table(self):
        return self._replica_table

    @property
    def device(self):
        return self.loc_ids.device if self.loc_ids is not None else torch.device("cpu")

    def build_g2l_map(self):
        """Dense global -> local table of global_nums + 1 entries, -1 = not stored here."""
        if self.mode == "map" and self.loc_ids is not None:
            size = max(int(self.global_nums), int(self.loc_ids.max()) if self.loc_ids.numel() else 0) + 1
            g2l = torch.full((size,), -1, dtype=torch.long, device=self.device)
            g2l[self.loc_ids] = torch.arange(self.loc_ids.size(0), dtype=torch.long, device=self.device)
            self._g2l_map = g2l

    def to_local(self, gids: Union[Tensor, DistRouteIndex], device: torch.device = None) -> Tensor:
        if device is None:
            device = self.device
        raw = gids
        if isinstance(gids, DistRouteIndex):
            raw = gids.loc
        elif self.mode == "dist_route_index" and isinstance(gids, Tensor):
            raw = DistRouteIndex(gids).loc
        if isinstance(raw, Tensor) and raw.device != device:
            raw = raw.to(device)
        if self.mode == "offset":
            return raw - self.offset
        if self.mode == "map":
            if self._g2l_map is None:
                raise RuntimeError("G2L Map not built! Call build_g2l_map() first.")
            return self._g2l_map[raw.to(self._g2l_map.device)].to(device)
        return raw  # identity / dist_route_index

    def to_dist(self, local_idx: Tensor) -> Tensor:
        table = self.dist_mapper if self.dist_mapper is not None else self.loc_ids
        return table[local_idx.to(table.device)].to(local_idx.device)

    def gid_to_dist_route_index(self, local_idx: Tensor) -> DistRouteIndex:
        assert self.dist_mapper is not None, "dist_mapper is required for DistRouteIndex conversion"
        return DistRouteIndex(self.dist_mapper[local_idx.to(self.dist_mapper.device)].to(local_idx.device))

    def get_master_part_by_dist(self, dist_idx: DistRouteIndex) -> Tensor:
        assert isinstance(dist_idx, DistRouteIndex), "dist_idx must be DistRouteIndex"
        return dist_idx.part

    def get_master_part_by_global(self, gid: Tensor) -> Tensor:
        d = self.dist_mapper[gid.to(self.dist_mapper.device)]
        return DistRouteIndex(d.to(gid.device)).part

    def is_master_by_local(self, local_idx: Tensor) -> Tensor:
        return (local_idx >= 0) & (local_idx < self._num_master)

    def _local_of(self, global_idx: Tensor) -> Tensor:
        return global_idx if self.mode == "identity" else self.to_local(global_idx, device=global_idx.device)

    def is_remote_ids(self, global_idx: Tensor) -> Tensor:
        loc = self._local_of(global_idx)
        return (loc < 0) | (loc >= self._num_master)

    def is_store_local(self, global_idx: Tensor) -> Tensor:
        return self._local_of(global_idx) >= 0


class PartitionState:
    def __init__(self, loc_ids: Tensor, num_master_nums: int, dist_nid_mapper: Optional[Tensor] = None,
                 node_mode: str = "identity", node_replica_table=None, loc_eids: Optional[Tensor] = None,
                 num_master_edges: int = 0, dist_eid_mapper: Optional[Tensor] = None, edge_mode: str = "identity",
                 edge_replica_table=None, num_nodes: int = 0, num_edges: int = 0):
        self.node_mapper = IDMapper(loc_ids, num_master_nums, node_mode, dist_nid_mapper, node_replica_table,
                                    global_num=num_nodes)
        self.edge_mapper = None
        if loc_eids is not None:
            self.edge_mapper = IDMapper(loc_eids, num_master_edges, edge_mode, dist_eid_mapper, edge_replica_table,
                                        global_num=num_edges)

    def build_g2l_maps(self):
        self.node_mapper.build_g2l_map()
        if self.edge_mapper:
            self.edge_mapper.build_g2l_map()

    # nodes
    def to_local_nid(self, gids, device: torch.device = None):
        return self.node_mapper.to_local(gids, device)

    def get_dist_nid(self, local_idx: Tensor):
        return self.node_mapper.to_dist(local_idx)

    def get_node_part_by_dist(self, global_idx: DistRouteIndex):
        return self.node_mapper.get_master_part_by_dist(global_idx)

    def is_master_node_by_local(self, local_idx: Tensor) -> Tensor:
        return self.node_mapper.is_master_by_local(local_idx)

    def is_master_node_by_global(self, gid: Tensor) -> Tensor:
        return self.is_master_node_by_local(self.to_local_nid(gid))

    # edges
    def _check_edge(self):
        if self.edge_mapper is None:
            raise RuntimeError("Edge data not initialized in PartitionState")

    def to_local_eid(self, gids, device: torch.device = None):
        self._check_edge()
        return self.edge_mapper.to_local(gids, device)

    def get_dist_eid(self, local_idx: Tensor):
        self._check_edge()
        return self.edge_mapper.to_dist(local_idx)

    def get_edge_part_by_dist(self, global_idx: DistRouteIndex):
        self._check_edge()
        return self.edge_mapper.get_master_part_by_dist(global_idx)

    def is_master_edge_by_local(self, local_idx: Tensor) -> Tensor:
        self._check_edge()
        return self.edge_mapper.is_master_by_local(local_idx)
