"""Id codecs and local/global id mapping behind the class and method names of
the reference's starrygl/utils/partition_book.py (DistRouteIndex :7-52,
IDMapper :56-176, PartitionState :179-276).

Everything here is table driven: the 64-bit id layout is one field table, an
IDMapper's behaviour per mode is one decode function, and PartitionState
forwards to its node and edge mappers through generated methods.  The lookup
`to_local` is plain tensor indexing; the fused form (id mask -> g2l table ->
hot slot -> row copy in one kernel) is `sgl_gather`, which `DistNodeState`
drives with the tables these classes own.
"""
from typing import Optional, Union

import torch
from torch import Tensor

# field -> (lowest bit, width) of the packed 64-bit id
_FIELDS = {"loc": (0, 48), "part": (48, 14), "shared": (62, 1)}


def _field(data: Tensor, name: str) -> Tensor:
    low, width = _FIELDS[name]
    return (data >> low) & ((1 << width) - 1)


def _packed(index: Tensor, part: Tensor) -> Tensor:
    (l0, lw), (p0, pw) = _FIELDS["loc"], _FIELDS["part"]
    return ((index >> l0) & ((1 << lw) - 1)) | ((part & ((1 << pw) - 1)) << p0)


class DistRouteIndex:
    """Packed id of a row somewhere in the partitioned graph: local index in the
    low 48 bits, owning partition in the next 14, bit 62 set for shared rows."""

    LOC_MASK = (1 << _FIELDS["loc"][1]) - 1          # what sgl_cache.id_mask takes for packed ids
    PART_SHIFT, PART_MASK = _FIELDS["part"][0], (1 << _FIELDS["part"][1]) - 1
    SHARED_BIT = _FIELDS["shared"][0]

    def __init__(self, index: Tensor, part_ids: Optional[Tensor] = None) -> None:
        data = index.long()
        self._data = data if part_ids is None else _packed(data, part_ids.long().to(data.device))

    loc = property(lambda self: _field(self._data, "loc"), doc="local index (bits 0-47)")
    part = property(lambda self: _field(self._data, "part"), doc="owning partition (bits 48-61)")
    is_shared = property(lambda self: _field(self._data, "shared").to(torch.bool), doc="bit 62")
    dist = property(lambda self: self._data, doc="the packed int64 tensor itself")
    device = property(lambda self: self._data.device)
    shape = property(lambda self: self._data.shape)

    def set_shared(self, indx):
        self._data[indx] |= 1 << _FIELDS["shared"][0]

    def to(self, device):
        return DistRouteIndex(self._data.to(device))


_MODES = ("identity", "offset", "map", "dist_route_index")


class IDMapper:
    """Local / global / dist id conversion and master test for one entity kind
    (nodes or edges).  The first `num_master` local rows are the ones this
    partition owns; `mode` says how a global id becomes a local row:
      identity          the id is the row,
      offset            row = id - offset,
      map               dense table of global_num + 1 entries, -1 = not stored here,
      dist_route_index  row = low 48 bits of the packed id."""

    def __init__(self, loc_ids: Tensor, num_master: int, mode: str = "identity",
                 dist_mapper: Optional[Tensor] = None, replica_table=None, offset: int = 0, global_num: int = 0):
        if mode not in _MODES:
            raise ValueError(f"unknown IDMapper mode {mode!r}")
        self.loc_ids, self.mode, self.dist_mapper, self.offset = loc_ids, mode, dist_mapper, offset
        self._owned, self._replicas, self._universe = num_master, replica_table, global_num
        self._g2l_map: Optional[Tensor] = None
        self.build_g2l_map()

    loc_nums = property(lambda self: self.loc_ids.size(0))
    num_master = property(lambda self: self._owned)
    global_nums = property(lambda self: self._universe)
    replica_table = property(lambda self: self._replicas)

    @property
    def device(self):
        return torch.device("cpu") if self.loc_ids is None else self.loc_ids.device

    def build_g2l_map(self):
        """(Re)build the dense global -> local table; only the 'map' mode has one."""
        if self.mode != "map" or self.loc_ids is None:
            return
        rows = self.loc_ids.size(0)
        top = int(self.loc_ids.max()) if rows else 0
        table = torch.full((max(int(self._universe), top) + 1,), -1, dtype=torch.long, device=self.device)
        table[self.loc_ids] = torch.arange(rows, dtype=torch.long, device=self.device)
        self._g2l_map = table

    def to_local(self, gids: Union[Tensor, DistRouteIndex], device: torch.device = None) -> Tensor:
        target = self.device if device is None else device
        if isinstance(gids, DistRouteIndex):
            ids = gids.loc
        elif self.mode == "dist_route_index":
            ids = _field(gids.long(), "loc")
        else:
            ids = gids
        if ids.device != target:
            ids = ids.to(target)
        if self.mode == "map":
            if self._g2l_map is None:
                raise RuntimeError("G2L Map not built! Call build_g2l_map() first.")
            return self._g2l_map[ids.to(self._g2l_map.device)].to(target)
        return ids - self.offset if self.mode == "offset" else ids

    def _dist_rows(self, local_idx: Tensor, table: Tensor) -> Tensor:
        return table[local_idx.to(table.device)].to(local_idx.device)

    def to_dist(self, local_idx: Tensor) -> Tensor:
        return self._dist_rows(local_idx, self.loc_ids if self.dist_mapper is None else self.dist_mapper)

    def gid_to_dist_route_index(self, local_idx: Tensor) -> DistRouteIndex:
        assert self.dist_mapper is not None, "dist_mapper is required for DistRouteIndex conversion"
        return DistRouteIndex(self._dist_rows(local_idx, self.dist_mapper))

    def get_master_part_by_dist(self, dist_idx: DistRouteIndex) -> Tensor:
        assert isinstance(dist_idx, DistRouteIndex), "dist_idx must be DistRouteIndex"
        return dist_idx.part

    def get_master_part_by_global(self, gid: Tensor) -> Tensor:
        return _field(self._dist_rows(gid, self.dist_mapper), "part")

    def is_master_by_local(self, local_idx: Tensor) -> Tensor:
        return (local_idx >= 0) & (local_idx < self._owned)

    def _rows_of(self, global_idx: Tensor) -> Tensor:
        return global_idx if self.mode == "identity" else self.to_local(global_idx, device=global_idx.device)

    def is_remote_ids(self, global_idx: Tensor) -> Tensor:
        return ~self.is_master_by_local(self._rows_of(global_idx))

    def is_store_local(self, global_idx: Tensor) -> Tensor:
        return self._rows_of(global_idx) >= 0


def _forward(mapper_attr: str, method: str, needs_edges: bool):
    """A PartitionState method that calls `method` of its node or edge mapper."""
    def call(self, *args, **kwargs):
        mapper = getattr(self, mapper_attr)
        if needs_edges and mapper is None:
            raise RuntimeError("Edge data not initialized in PartitionState")
        return getattr(mapper, method)(*args, **kwargs)
    call.__name__ = method
    return call


class PartitionState:
    """The node mapper and (optionally) the edge mapper of one partition, with the
    reference's method names: to_local_nid / to_local_eid, get_dist_nid /
    get_dist_eid, get_node_part_by_dist / get_edge_part_by_dist,
    is_master_node_by_local / is_master_edge_by_local, is_master_node_by_global."""

    def __init__(self, loc_ids: Tensor, num_master_nums: int, dist_nid_mapper: Optional[Tensor] = None,
                 node_mode: str = "identity", node_replica_table=None, loc_eids: Optional[Tensor] = None,
                 num_master_edges: int = 0, dist_eid_mapper: Optional[Tensor] = None, edge_mode: str = "identity",
                 edge_replica_table=None, num_nodes: int = 0, num_edges: int = 0):
        self.node_mapper = IDMapper(loc_ids, num_master_nums, node_mode, dist_nid_mapper, node_replica_table,
                                    global_num=num_nodes)
        self.edge_mapper = None if loc_eids is None else IDMapper(
            loc_eids, num_master_edges, edge_mode, dist_eid_mapper, edge_replica_table, global_num=num_edges)

    def build_g2l_maps(self):
        for mapper in (self.node_mapper, self.edge_mapper):
            if mapper is not None:
                mapper.build_g2l_map()

    def is_master_node_by_global(self, gid: Tensor) -> Tensor:
        return self.node_mapper.is_master_by_local(self.node_mapper.to_local(gid))


for _kind, _attr, _edges in (("n", "node_mapper", False), ("e", "edge_mapper", True)):
    _noun = "node" if _kind == "n" else "edge"
    for _name, _method in ((f"to_local_{_kind}id", "to_local"), (f"get_dist_{_kind}id", "to_dist"),
                           (f"get_{_noun}_part_by_dist", "get_master_part_by_dist"),
                           (f"is_master_{_noun}_by_local", "is_master_by_local")):
        setattr(PartitionState, _name, _forward(_attr, _method, _edges))
del _kind, _attr, _edges, _noun, _name, _method
