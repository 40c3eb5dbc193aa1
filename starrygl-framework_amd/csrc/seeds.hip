// Seed (root) extraction per chunk and time window, and CSC block assembly, for
// gfx950.
//
// Seeds: the candidates are the nodes of the selected chunks, flattened in
// chunk-list order.  `count` finds each candidate's window [t_begin, t_end) on
// its row (two binary searches), the number of distinct timestamps and of
// events in it; three device-wide exclusive scans turn the per-candidate counts
// into output offsets; `fill` writes roots / ts_ptr / ts / q_ptr / q_eid.  The
// output order (chunk-list order, ascending node id, ascending time) does not
// depend on the launch geometry.
//
// Replaces filter_seeds_kernel / collect_seeds_kernel and get_seeds_in_chunks
// (csrc/include/starrygl/sample.cu.hpp:517-705, 1303-1449).
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;

__device__ __forceinline__ int64_t lower_bound_i64(const int64_t* __restrict__ a, int64_t lo, int64_t hi, int64_t key) {
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (a[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

struct SeedWs {
    int64_t* node;   // [n_cand]
    int64_t* lo;     // [n_cand]
    int64_t* hi;     // [n_cand]
    int64_t* off_r;  // [n_cand] is-root flag -> exclusive offset
    int64_t* off_s;  // [n_cand] distinct timestamps -> offset
    int64_t* off_q;  // [n_cand] events -> offset
    void* scan_ws;
    size_t scan_ws_bytes;
};

size_t seeds_ws_bytes(int64_t n_cand) {
    return 6 * align_up((size_t)(n_cand + 1) * 8) + exclusive_scan_workspace_bytes(n_cand) + 2048;
}

bool carve(void* ws, size_t bytes, int64_t n_cand, SeedWs* out) {
    Arena ar(ws, bytes);
    out->node = ar.take<int64_t>(n_cand + 1);
    out->lo = ar.take<int64_t>(n_cand + 1);
    out->hi = ar.take<int64_t>(n_cand + 1);
    out->off_r = ar.take<int64_t>(n_cand + 1);
    out->off_s = ar.take<int64_t>(n_cand + 1);
    out->off_q = ar.take<int64_t>(n_cand + 1);
    out->scan_ws_bytes = exclusive_scan_workspace_bytes(n_cand);
    out->scan_ws = ar.take<char>(out->scan_ws_bytes);
    return ar.ok();
}

__global__ __launch_bounds__(BLOCK) void seeds_count_kernel(sgl_tcsr g, sgl_seed_query q, SeedWs w) {
    const int64_t j = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (j >= q.n_cand) return;
    // selected-chunk position p with cand_off[p] <= j < cand_off[p+1]
    int64_t a = 0, b = q.num_chunks;
    while (b - a > 1) {
        const int64_t mid = a + ((b - a) >> 1);
        if (q.cand_off[mid] <= j) a = mid; else b = mid;
    }
    const int64_t c = q.chunks[a];
    const int64_t v = q.chunk_nodes[q.chunk_ptr[c] + (j - q.cand_off[a])];
    const int64_t rs = g.row_ptr[v], re = g.row_ptr[v + 1];
    const int64_t lo = lower_bound_i64(g.ts, rs, re, q.t_begin);
    const int64_t hi = lower_bound_i64(g.ts, lo, re, q.t_end);
    int64_t n_ts = 0;
    for (int64_t e = lo; e < hi; ++e) n_ts += (e == lo || g.ts[e] != g.ts[e - 1]) ? 1 : 0;
    w.node[j] = v;
    w.lo[j] = lo;
    w.hi[j] = hi;
    w.off_r[j] = hi > lo ? 1 : 0;
    w.off_s[j] = n_ts;
    w.off_q[j] = hi - lo;
}

__global__ __launch_bounds__(BLOCK) void seeds_fill_kernel(sgl_tcsr g, sgl_seed_query q, SeedWs w,
                                                           const int64_t* totals, int64_t* roots, int64_t* ts_ptr,
                                                           int64_t* ts, int64_t* q_ptr, int64_t* q_eid) {
    const int64_t j = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (j == 0) {
        ts_ptr[totals[0]] = totals[1];
        q_ptr[totals[1]] = totals[2];
    }
    if (j >= q.n_cand) return;
    const int64_t lo = w.lo[j], hi = w.hi[j];
    if (hi <= lo) return;
    const int64_t r = w.off_r[j], q0 = w.off_q[j];
    int64_t s = w.off_s[j];
    roots[r] = w.node[j];
    ts_ptr[r] = s;
    for (int64_t e = lo; e < hi; ++e) {
        const int64_t t = g.ts[e];
        if (e == lo || t != g.ts[e - 1]) {
            ts[s] = t;
            q_ptr[s] = q0 + (e - lo);
            ++s;
        }
        q_eid[q0 + (e - lo)] = g.eid[e];
    }
}

__global__ void empty_seed_ptrs_kernel(int64_t* totals) { totals[0] = totals[1] = totals[2] = 0; }

__global__ __launch_bounds__(BLOCK) void block_build_kernel(const int64_t* __restrict__ root_start_ptr,
                                                            const int64_t* counts, int64_t S_max, int64_t E_max,
                                                            int64_t dst_offset, int64_t src_offset,
                                                            int64_t* __restrict__ indptr, int64_t* __restrict__ indices,
                                                            int64_t* __restrict__ edge_dst) {
    int64_t S = counts[0], E = counts[1];
    S = S > S_max ? S_max : S;
    E = E > E_max ? E_max : E;
    const int64_t t = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    // indptr: dst_offset zeros, then the S+1 prefix entries
    if (t < dst_offset) indptr[t] = 0;
    else if (t <= dst_offset + S) indptr[t] = root_start_ptr[t - dst_offset];
    if (t < E) {
        indices[t] = src_offset + t;
        if (edge_dst != nullptr) {  // slot s with root_start_ptr[s] <= t < root_start_ptr[s+1]
            int64_t a = 0, b = S;
            while (b - a > 1) {
                const int64_t mid = a + ((b - a) >> 1);
                if (root_start_ptr[mid] <= t) a = mid; else b = mid;
            }
            edge_dst[t] = dst_offset + a;
        }
    }
}

int32_t check_query(const sgl_tcsr* g, const sgl_seed_query* q) {
    if (!g || !q) return fail(SGL_EINVAL, "seeds: NULL graph or query");
    if (q->num_chunks < 0 || q->n_cand < 0) return fail(SGL_EINVAL, "seeds: negative size");
    if (q->n_cand > 0 && (!q->chunk_ptr || !q->chunk_nodes || !q->chunks || !q->cand_off || !g->row_ptr))
        return fail(SGL_EINVAL, "seeds: NULL array");
    if (ceil_div<int64_t>(q->n_cand + 1, BLOCK) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "seeds: too many candidates");
    return SGL_OK;
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_seeds_workspace_bytes(int64_t n_cand) { return seeds_ws_bytes(n_cand < 0 ? 0 : n_cand); }

extern "C" int32_t sgl_seeds_count(const sgl_tcsr* g, const sgl_seed_query* q, int64_t* totals, void* ws,
                                   size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_query(g, q)) != SGL_OK) return rc;
    if (!totals) return fail(SGL_EINVAL, "seeds_count: totals is NULL");
    hipStream_t st = as_stream(stream);
    if (q->n_cand == 0) {
        hipLaunchKernelGGL(empty_seed_ptrs_kernel, dim3(1), dim3(1), 0, st, totals);
        SGL_LAUNCH_CHECK();
        return SGL_OK;
    }
    SeedWs w;
    if (!ws || ws_bytes < seeds_ws_bytes(q->n_cand) || !carve(ws, ws_bytes, q->n_cand, &w))
        return fail(SGL_ENOMEM, "seeds_count: workspace %zu < %zu bytes", ws_bytes, seeds_ws_bytes(q->n_cand));
    hipLaunchKernelGGL(seeds_count_kernel, dim3((unsigned)ceil_div<int64_t>(q->n_cand, BLOCK)), dim3(BLOCK), 0, st, *g, *q, w);
    SGL_LAUNCH_CHECK();
    if ((rc = exclusive_scan_i64(w.off_r, w.off_r, q->n_cand, totals + 0, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    if ((rc = exclusive_scan_i64(w.off_s, w.off_s, q->n_cand, totals + 1, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    if ((rc = exclusive_scan_i64(w.off_q, w.off_q, q->n_cand, totals + 2, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    return SGL_OK;
}

extern "C" int32_t sgl_seeds_fill(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* totals,
                                  int64_t* roots, int64_t* ts_ptr, int64_t* ts, int64_t* q_ptr, int64_t* q_eid,
                                  void* ws, size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_query(g, q)) != SGL_OK) return rc;
    if (!totals || !ts_ptr || !q_ptr) return fail(SGL_EINVAL, "seeds_fill: totals/ts_ptr/q_ptr is NULL");
    hipStream_t st = as_stream(stream);
    SeedWs w{};
    if (q->n_cand > 0 && (!ws || ws_bytes < seeds_ws_bytes(q->n_cand) || !carve(ws, ws_bytes, q->n_cand, &w)))
        return fail(SGL_ENOMEM, "seeds_fill: workspace %zu < %zu bytes", ws_bytes, seeds_ws_bytes(q->n_cand));
    hipLaunchKernelGGL(seeds_fill_kernel, dim3((unsigned)ceil_div<int64_t>(q->n_cand + 1, BLOCK)), dim3(BLOCK), 0, st, *g, *q, w,
                       totals, roots, ts_ptr, ts, q_ptr, q_eid);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" int32_t sgl_block_build(const int64_t* root_start_ptr, const int64_t* counts, int64_t S_max,
                                   int64_t E_max, int64_t dst_offset, int64_t src_offset, int64_t* indptr,
                                   int64_t* indices, int64_t* edge_dst, void* stream) {
    if (S_max < 0 || E_max < 0 || dst_offset < 0 || src_offset < 0) return fail(SGL_EINVAL, "block_build: negative size");
    if (!root_start_ptr || !counts || !indptr || (E_max > 0 && !indices)) return fail(SGL_EINVAL, "block_build: NULL array");
    const int64_t threads = (dst_offset + S_max + 1) > E_max ? (dst_offset + S_max + 1) : E_max;
    if (ceil_div<int64_t>(threads, BLOCK) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "block_build: too large");
    hipLaunchKernelGGL(block_build_kernel, dim3((unsigned)ceil_div<int64_t>(threads, BLOCK)), dim3(BLOCK), 0,
                       as_stream(stream), root_start_ptr, counts, S_max, E_max, dst_offset, src_offset, indptr, indices,
                       edge_dst);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

// ---- latest event per node (mailbox update reduce) ---------------------------
namespace sgl {
namespace {

__global__ void segmax_init_kernel(int64_t U_max, const int64_t* U_dev, int64_t* max_ts, int64_t* arg) {
    const int64_t U = live_count(U_dev, U_max);
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < U; u += (int64_t)gridDim.x * blockDim.x) {
        max_ts[u] = INT64_MIN;
        arg[u] = INT64_MAX;
    }
}

// pass 1: max_ts[u] = max ts (atomics spread over the keys)
__global__ void segmax_max_kernel(const int64_t* __restrict__ local, const int64_t* __restrict__ ts, int64_t N_max,
                                  const int64_t* N_dev, int64_t U_max, const int64_t* U_dev, int64_t* max_ts) {
    const int64_t N = live_count(N_dev, N_max), U = live_count(U_dev, U_max);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t u = local[i];
        if (u >= 0 && u < U) atomicMax(reinterpret_cast<long long*>(&max_ts[u]), (long long)ts[i]);
    }
}

// pass 2: arg[u] = smallest i with ts[i] == max_ts[u]
__global__ void segmax_arg_kernel(const int64_t* __restrict__ local, const int64_t* __restrict__ ts, int64_t N_max,
                                  const int64_t* N_dev, int64_t U_max, const int64_t* U_dev,
                                  const int64_t* __restrict__ max_ts, int64_t* arg) {
    const int64_t N = live_count(N_dev, N_max), U = live_count(U_dev, U_max);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t u = local[i];
        if (u >= 0 && u < U && ts[i] == max_ts[u]) atomicMin(reinterpret_cast<long long*>(&arg[u]), (long long)i);
    }
}

__global__ void segmax_fix_kernel(int64_t U_max, const int64_t* U_dev, int64_t* arg) {
    const int64_t U = live_count(U_dev, U_max);
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < U; u += (int64_t)gridDim.x * blockDim.x)
        if (arg[u] == INT64_MAX) arg[u] = -1;
}

}  // namespace
}  // namespace sgl

extern "C" int32_t sgl_segment_max_ts(const int64_t* local, const int64_t* ts, int64_t N_max, const int64_t* N_dev,
                                      int64_t U_max, const int64_t* U_dev, int64_t* max_ts, int64_t* arg,
                                      void* stream) {
    if (N_max < 0 || U_max < 0) return fail(SGL_EINVAL, "segment_max_ts: negative size");
    if ((N_max > 0 && (!local || !ts)) || (U_max > 0 && (!max_ts || !arg))) return fail(SGL_EINVAL, "segment_max_ts: NULL array");
    if (U_max == 0) return SGL_OK;
    hipStream_t st = as_stream(stream);
    auto grid = [](int64_t n) { int64_t b = ceil_div<int64_t>(n > 0 ? n : 1, BLOCK); return dim3((unsigned)(b > 2048 ? 2048 : b)); };
    hipLaunchKernelGGL(segmax_init_kernel, grid(U_max), dim3(BLOCK), 0, st, U_max, U_dev, max_ts, arg);
    SGL_LAUNCH_CHECK();
    if (N_max > 0) {
        hipLaunchKernelGGL(segmax_max_kernel, grid(N_max), dim3(BLOCK), 0, st, local, ts, N_max, N_dev, U_max, U_dev, max_ts);
        SGL_LAUNCH_CHECK();
        hipLaunchKernelGGL(segmax_arg_kernel, grid(N_max), dim3(BLOCK), 0, st, local, ts, N_max, N_dev, U_max, U_dev, max_ts, arg);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(segmax_fix_kernel, grid(U_max), dim3(BLOCK), 0, st, U_max, U_dev, arg);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
