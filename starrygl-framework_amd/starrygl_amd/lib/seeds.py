"""Host side of seed extraction (Graph::get_seeds_in_chunks,
csrc/include/starrygl/sample.cu.hpp:1303-1449): which chunks are selected and
how many candidate nodes they hold is decided on the host from a host copy of
chunk_ptr; the per-candidate work runs in libsgl_hot.so."""
import numpy as np
import torch


def _chunk_index(graph):
    """Lazily build (chunk_ptr, chunk_nodes) on the device + a host chunk_ptr."""
    if graph._chunk_index is None:
        hp, n, C = graph._hp, graph._n, max(graph._chunks, 1)
        dev = hp.be.device
        mapper = graph._mapper
        if mapper is None:   # no mapper: every node in chunk 0
            mapper = torch.zeros(n, dtype=torch.int64)
        node_chunk = mapper.to(dev, torch.int64).contiguous()
        chunk_ptr, chunk_nodes = hp.chunk_index(n, C, node_chunk)
        graph._chunk_index = (chunk_ptr, chunk_nodes, chunk_ptr.cpu().numpy(), node_chunk)
    return graph._chunk_index


def _candidates(graph, chunks):
    """-> (device chunk ids, device exclusive prefix of their sizes, candidate count)."""
    dev = graph._hp.be.device
    chunk_ptr_h = _chunk_index(graph)[2]
    if not isinstance(chunks, torch.Tensor):
        raise TypeError("chunks must be a torch.Tensor")
    chunks_h = chunks.detach().cpu().to(torch.int64).numpy().reshape(-1)
    C = chunk_ptr_h.shape[0] - 1
    if chunks_h.size and (chunks_h.min() < 0 or chunks_h.max() >= C):
        raise IndexError("chunk id outside [0, chunk_size)")
    # training loops ask for the same few chunk lists over and over: their device copies are kept
    # (two small host-to-device copies cost more host time than the whole query costs GPU time)
    cache = graph.__dict__.setdefault("_cand_cache", {})
    key = chunks_h.tobytes()
    hit = cache.get(key)
    if hit is not None:
        return hit
    sizes = chunk_ptr_h[chunks_h + 1] - chunk_ptr_h[chunks_h] if chunks_h.size else np.zeros(0, np.int64)
    cand_off = np.zeros(chunks_h.size + 1, dtype=np.int64)
    np.cumsum(sizes, out=cand_off[1:])
    packed = torch.from_numpy(np.concatenate([chunks_h, cand_off])).to(dev)      # one copy for both
    out = (packed[: chunks_h.size], packed[chunks_h.size:], int(cand_off[-1]))
    if len(cache) >= 64:
        cache.clear()
    cache[key] = out
    return out


def seeds_in_chunks(graph, chunks, t_begin, t_end, full_timestamps=False):
    """`full_timestamps`: every root lists all integers of [t_begin, t_end) as its timestamps
    (discrete-time snapshots; filter_seeds_kernel, sample.cu.hpp:575-578) instead of the distinct
    timestamps of its events."""
    from .libstarrygl_comm import TemporalRoot
    chunk_ptr, chunk_nodes = _chunk_index(graph)[:2]
    d_chunks, d_off, n_cand = _candidates(graph, chunks)
    if full_timestamps:
        nodes, ts_ptr, ts, q_ptr, _, _, q_eid = graph._hp.slice(graph._g, chunk_ptr, chunk_nodes, None, d_chunks, d_off,
                                                                n_cand, t_begin, t_end, True)
        return TemporalRoot(nodes, ts_ptr, ts, q_ptr, q_eid)
    out = graph._hp.seeds(graph._g, chunk_ptr, chunk_nodes, d_chunks, d_off, n_cand, t_begin, t_end,
                          with_window_end=True)
    return TemporalRoot(*out)


def slice_in_chunks(graph, chunks, t_begin, t_end, full_timestamps):
    """Graph::slice_by_chunk_ts (sample.cu.hpp:1189-1299): the selected chunks'
    nodes with edges in [t_begin, t_end) as roots (one timestamp list per node)
    and, as the single neighbour layer, the window edges whose destination lies
    in a selected chunk; `root_start_ptr` indexes them per (node, timestamp)."""
    from .libstarrygl_comm import NegativeRoot, TemporalNeighbor, TemporalResult, TemporalRoot
    chunk_ptr, chunk_nodes, _, node_chunk = _chunk_index(graph)
    d_chunks, d_off, n_cand = _candidates(graph, chunks)
    nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid = graph._hp.slice(
        graph._g, chunk_ptr, chunk_nodes, node_chunk, d_chunks, d_off, n_cand, t_begin, t_end, full_timestamps)
    e = nodes.new_empty(0)
    layer = TemporalNeighbor.from_arrays(edge_ptr, torch.cat([edge_ptr[1:], edge_ptr[-1:]]), col, col_ts, col_eid, e)
    return TemporalResult(TemporalRoot(nodes, ts_ptr, ts), NegativeRoot(e, e), [layer])
