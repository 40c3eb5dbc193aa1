// Sub-graph slice of a chunk set over a time window ("cluster" loading) for
// gfx950.
//
// Candidates are the nodes of the selected chunks in chunk-list order, as for
// the seeds.  A group of G lanes owns one candidate: it finds the window
// [t_begin, t_end) on the candidate's row, then walks the window G edges at a
// time; two ballots per step (timestamp changes, destination in a selected
// chunk) give the counts in `count` and the output positions in `fill`.
// Three device-wide exclusive scans between the two turn per-candidate counts
// into offsets, so the output order (chunk-list order, ascending node id,
// storage order of the edges) does not depend on the launch geometry.
//
// Replaces mark_chunks_exists_kernel / count_edges_kernel / write_edges_kernel
// and Graph::slice_by_chunk_ts (csrc/include/starrygl/sample.cu.hpp:115-120,
// 299-515, 1189-1299).
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int G = 16;               // lanes per candidate
constexpr int CPB = BLOCK / G;      // candidates per block

struct SliceWs {
    int64_t* node;    // [n_cand]
    int64_t* lo;      // [n_cand]
    int64_t* hi;      // [n_cand]
    int64_t* off_r;   // [n_cand] has-window flag -> offset in nodes[]
    int64_t* off_s;   // [n_cand] timestamp entries -> offset in ts[]
    int64_t* off_e;   // [n_cand] kept edges -> offset in col[]
    uint8_t* member;  // [total_chunks] 1 = chunk selected
    void* scan_ws;
    size_t scan_ws_bytes;
};

size_t slice_ws_bytes(int64_t n_cand, int64_t total_chunks) {
    return 6 * align_up((size_t)(n_cand + 1) * 8) + align_up((size_t)total_chunks + 8) +
           exclusive_scan_workspace_bytes(n_cand) + 4096;
}

bool carve(void* ws, size_t bytes, int64_t n_cand, int64_t total_chunks, SliceWs* out) {
    Arena ar(ws, bytes);
    out->node = ar.take<int64_t>(n_cand + 1);
    out->lo = ar.take<int64_t>(n_cand + 1);
    out->hi = ar.take<int64_t>(n_cand + 1);
    out->off_r = ar.take<int64_t>(n_cand + 1);
    out->off_s = ar.take<int64_t>(n_cand + 1);
    out->off_e = ar.take<int64_t>(n_cand + 1);
    out->member = ar.take<uint8_t>(total_chunks + 8);
    out->scan_ws_bytes = exclusive_scan_workspace_bytes(n_cand);
    out->scan_ws = ar.take<char>(out->scan_ws_bytes);
    return ar.ok();
}

__global__ __launch_bounds__(BLOCK) void clear_member_kernel(uint8_t* member, int64_t total_chunks) {
    for (int64_t c = (int64_t)blockIdx.x * BLOCK + threadIdx.x; c < total_chunks; c += (int64_t)gridDim.x * BLOCK)
        member[c] = 0;
}

__global__ __launch_bounds__(BLOCK) void mark_member_kernel(const int64_t* chunks, int64_t num_chunks, uint8_t* member,
                                                            int64_t total_chunks) {
    const int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= num_chunks) return;
    const int64_t c = chunks[i];
    if (c >= 0 && c < total_chunks) member[c] = 1;
}

__device__ __forceinline__ int64_t lower_bound_i64(const int64_t* __restrict__ a, int64_t lo, int64_t hi, int64_t key) {
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (a[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// candidate j -> its node (position of j in the flattened selected chunks)
__device__ __forceinline__ int64_t candidate_node(const sgl_seed_query& q, int64_t j) {
    int64_t a = 0, b = q.num_chunks;
    while (b - a > 1) {
        const int64_t mid = a + ((b - a) >> 1);
        if (q.cand_off[mid] <= j) a = mid; else b = mid;
    }
    return q.chunk_nodes[q.chunk_ptr[q.chunks[a]] + (j - q.cand_off[a])];
}

// 1 when the chunk of node `dst` is selected; chunk ids outside the table count as not selected
__device__ __forceinline__ bool dst_selected(const SliceWs& w, const int64_t* __restrict__ node_chunk, int64_t total_chunks,
                                             int64_t dst) {
    if (node_chunk == nullptr) return true;          // no destination filter
    const int64_t c = node_chunk[dst];
    return c >= 0 && c < total_chunks && w.member[c] != 0;
}

__global__ __launch_bounds__(BLOCK) void slice_count_kernel(sgl_tcsr g, sgl_seed_query q, const int64_t* __restrict__ node_chunk,
                                                            int64_t total_chunks, int32_t full, SliceWs w) {
    const int lig = threadIdx.x % G, wlane = threadIdx.x % WAVE;
    const int gshift = wlane / G * G;
    const int64_t j = (int64_t)blockIdx.x * CPB + threadIdx.x / G;
    const bool valid = j < q.n_cand;
    int64_t v = 0, lo = 0, hi = 0;
    if (valid) {   // every lane of the group runs the same searches: the loads are broadcasts
        v = candidate_node(q, j);
        const int64_t rs = g.row_ptr[v], re = g.row_ptr[v + 1];
        lo = lower_bound_i64(g.ts, rs, re, q.t_begin);
        hi = lower_bound_i64(g.ts, lo, re, q.t_end);
    }
    int64_t n_ts = 0, n_keep = 0;
    for (int64_t base = lo; __any(base < hi); base += G) {
        const int64_t e = base + lig;
        bool fresh = false, keep = false;
        if (e < hi) {
            fresh = e == lo || g.ts[e] != g.ts[e - 1];
            keep = dst_selected(w, node_chunk, total_chunks, g.col[e]);
        }
        n_ts += __popcll(group_ballot<G>(fresh, gshift));
        n_keep += __popcll(group_ballot<G>(keep, gshift));
    }
    if (valid && lig == 0) {
        w.node[j] = v;
        w.lo[j] = lo;
        w.hi[j] = hi;
        w.off_r[j] = hi > lo ? 1 : 0;
        w.off_s[j] = hi > lo ? (full ? q.t_end - q.t_begin : n_ts) : 0;
        w.off_e[j] = n_keep;
    }
}

__global__ __launch_bounds__(BLOCK) void slice_fill_kernel(sgl_tcsr g, sgl_seed_query q, const int64_t* __restrict__ node_chunk,
                                                           int64_t total_chunks, int32_t full, SliceWs w, const int64_t* totals, int64_t* nodes,
                                                           int64_t* ts_ptr, int64_t* ts, int64_t* edge_ptr, int64_t* col,
                                                           int64_t* col_ts, int64_t* col_eid) {
    const int lig = threadIdx.x % G, wlane = threadIdx.x % WAVE;
    const int gshift = wlane / G * G;
    const int64_t j = (int64_t)blockIdx.x * CPB + threadIdx.x / G;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        ts_ptr[totals[0]] = totals[1];
        edge_ptr[totals[1]] = totals[2];
    }
    const bool valid = j < q.n_cand;
    int64_t lo = 0, hi = 0, s0 = 0, e0 = 0;
    if (valid) {
        lo = w.lo[j];
        hi = w.hi[j];
        s0 = w.off_s[j];
        e0 = w.off_e[j];
        if (hi > lo && lig == 0) {
            const int64_t r = w.off_r[j];
            nodes[r] = w.node[j];
            ts_ptr[r] = s0;
        }
    }
    const uint64_t below = (1ull << lig) - 1ull;
    int64_t seen_ts = 0, kept = 0;    // timestamp entries / kept edges before `base`
    for (int64_t base = lo; __any(base < hi); base += G) {
        const int64_t e = base + lig;
        bool fresh = false, keep = false;
        int64_t t = 0, prev = 0;
        if (e < hi) {
            t = g.ts[e];
            prev = e == lo ? q.t_begin - 1 : g.ts[e - 1];
            fresh = t != prev;
            keep = dst_selected(w, node_chunk, total_chunks, g.col[e]);
        }
        const uint64_t bf = group_ballot<G>(fresh, gshift), bk = group_ballot<G>(keep, gshift);
        const int64_t kept_before = e0 + kept + __popcll(bk & below);
        if (fresh) {
            if (full) {   // every integer in (prev, t] starts at this edge
                for (int64_t x = prev + 1; x <= t; ++x) edge_ptr[s0 + (x - q.t_begin)] = kept_before;
            } else {
                const int64_t s = s0 + seen_ts + __popcll(bf & below);
                ts[s] = t;
                edge_ptr[s] = kept_before;
            }
        }
        if (keep) {
            col[kept_before] = g.col[e];
            col_ts[kept_before] = t;
            col_eid[kept_before] = g.eid[e];
        }
        seen_ts += __popcll(bf);
        kept += __popcll(bk);
    }
    if (full && valid && hi > lo) {
        // the integers after the last window timestamp own nothing; all of them are listed
        const int64_t last = g.ts[hi - 1];
        for (int64_t x = last + 1 + lig; x < q.t_end; x += G) edge_ptr[s0 + (x - q.t_begin)] = e0 + kept;
        for (int64_t x = q.t_begin + lig; x < q.t_end; x += G) ts[s0 + (x - q.t_begin)] = x;
    }
}

__global__ void empty_slice_kernel(int64_t* totals) { totals[0] = totals[1] = totals[2] = 0; }

int32_t check(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk, int64_t total_chunks, int32_t full) {
    if (!g || !q) return fail(SGL_EINVAL, "slice: NULL graph or query");
    if (q->num_chunks < 0 || q->n_cand < 0 || total_chunks < 0) return fail(SGL_EINVAL, "slice: negative size");
    if (q->n_cand > 0 && (!q->chunk_ptr || !q->chunk_nodes || !q->chunks || !q->cand_off || !g->row_ptr))
        return fail(SGL_EINVAL, "slice: NULL array");
    if (full && q->t_end < q->t_begin) return fail(SGL_EINVAL, "slice: t_end < t_begin");
    if (ceil_div<int64_t>(q->n_cand + 1, CPB) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "slice: too many candidates");
    return SGL_OK;
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_slice_workspace_bytes(int64_t n_cand, int64_t total_chunks) {
    return slice_ws_bytes(n_cand < 0 ? 0 : n_cand, total_chunks < 0 ? 0 : total_chunks);
}

extern "C" int32_t sgl_slice_count(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk,
                                   int64_t total_chunks, int32_t full_timestamps, int64_t* totals, void* ws,
                                   size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check(g, q, node_chunk, total_chunks, full_timestamps)) != SGL_OK) return rc;
    if (!totals) return fail(SGL_EINVAL, "slice_count: totals is NULL");
    hipStream_t st = as_stream(stream);
    if (q->n_cand == 0) {
        hipLaunchKernelGGL(empty_slice_kernel, dim3(1), dim3(1), 0, st, totals);
        SGL_LAUNCH_CHECK();
        return SGL_OK;
    }
    SliceWs w;
    if (!ws || ws_bytes < slice_ws_bytes(q->n_cand, total_chunks) || !carve(ws, ws_bytes, q->n_cand, total_chunks, &w))
        return fail(SGL_ENOMEM, "slice_count: workspace %zu < %zu bytes", ws_bytes, slice_ws_bytes(q->n_cand, total_chunks));
    int64_t cb = ceil_div<int64_t>(total_chunks > 0 ? total_chunks : 1, BLOCK);
    hipLaunchKernelGGL(clear_member_kernel, dim3((unsigned)(cb > 1024 ? 1024 : cb)), dim3(BLOCK), 0, st, w.member, total_chunks);
    SGL_LAUNCH_CHECK();
    if (q->num_chunks > 0) {
        hipLaunchKernelGGL(mark_member_kernel, dim3((unsigned)ceil_div<int64_t>(q->num_chunks, BLOCK)), dim3(BLOCK), 0, st,
                           q->chunks, q->num_chunks, w.member, total_chunks);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(slice_count_kernel, dim3((unsigned)ceil_div<int64_t>(q->n_cand, CPB)), dim3(BLOCK), 0, st, *g, *q,
                       node_chunk, total_chunks, full_timestamps, w);
    SGL_LAUNCH_CHECK();
    if ((rc = exclusive_scan_i64(w.off_r, w.off_r, q->n_cand, totals + 0, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    if ((rc = exclusive_scan_i64(w.off_s, w.off_s, q->n_cand, totals + 1, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    if ((rc = exclusive_scan_i64(w.off_e, w.off_e, q->n_cand, totals + 2, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    return SGL_OK;
}

extern "C" int32_t sgl_slice_fill(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk,
                                  int64_t total_chunks, int32_t full_timestamps, const int64_t* totals, int64_t* nodes,
                                  int64_t* ts_ptr, int64_t* ts, int64_t* edge_ptr, int64_t* col, int64_t* col_ts,
                                  int64_t* col_eid, void* ws, size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check(g, q, node_chunk, total_chunks, full_timestamps)) != SGL_OK) return rc;
    if (!totals || !ts_ptr || !edge_ptr) return fail(SGL_EINVAL, "slice_fill: totals/ts_ptr/edge_ptr is NULL");
    hipStream_t st = as_stream(stream);
    SliceWs w{};
    if (q->n_cand > 0 &&
        (!ws || ws_bytes < slice_ws_bytes(q->n_cand, total_chunks) || !carve(ws, ws_bytes, q->n_cand, total_chunks, &w)))
        return fail(SGL_ENOMEM, "slice_fill: workspace %zu < %zu bytes", ws_bytes, slice_ws_bytes(q->n_cand, total_chunks));
    hipLaunchKernelGGL(slice_fill_kernel, dim3((unsigned)ceil_div<int64_t>(q->n_cand + 1, CPB)), dim3(BLOCK), 0, st, *g, *q,
                       node_chunk, total_chunks, full_timestamps, w, totals, nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
