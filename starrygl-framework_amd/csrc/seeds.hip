// Seed (root) extraction per chunk and time window, and CSC block assembly, for
// gfx950.
//
// Seeds: the candidates are the nodes of the selected chunks, flattened in
// chunk-list order.  `count` finds each candidate's window [t_begin, t_end) on
// its row (two binary searches), the number of distinct timestamps and of
// events in it, and leaves per-tile sums of the three counters; one block scans
// the tile sums; `fill` redoes the scan inside each tile and writes roots /
// ts_ptr / ts / q_ptr / q_eid.  A candidate with more than a handful of events
// in the window is walked by its whole wavefront, 64 events per step, in both
// kernels (a hub node of a skewed graph holds a few percent of every window: one
// thread looping over its events would be the launch's critical path).  The
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

constexpr int SEED_ROUNDS = 4;                  // candidates per thread
constexpr int SEED_TILE = BLOCK * SEED_ROUNDS;  // candidates per block
constexpr int SEED_LIGHT = 4;                   // up to this many window events a candidate is walked by its own thread
constexpr int SEED_SCAN_BLOCK = 1024;

struct SeedWs {
    int64_t* node;   // [n_cand]
    int64_t* lo;     // [n_cand] window on the row
    int64_t* hi;     // [n_cand]
    int64_t* n_ts;   // [n_cand] distinct timestamps in the window
    int64_t* tile;   // [3][nt + 1] per-tile sums of (roots, timestamps, events) -> exclusive offsets
    int64_t nt;
};

int64_t seed_tiles(int64_t n_cand) { return ceil_div<int64_t>(n_cand > 0 ? n_cand : 1, SEED_TILE); }

size_t seeds_ws_bytes(int64_t n_cand) {
    return 4 * align_up((size_t)(n_cand + 1) * 8) + align_up((size_t)(3 * (seed_tiles(n_cand) + 1)) * 8) + 1024;
}

bool carve(void* ws, size_t bytes, int64_t n_cand, SeedWs* out) {
    Arena ar(ws, bytes);
    out->nt = seed_tiles(n_cand);
    out->node = ar.take<int64_t>(n_cand + 1);
    out->lo = ar.take<int64_t>(n_cand + 1);
    out->hi = ar.take<int64_t>(n_cand + 1);
    out->n_ts = ar.take<int64_t>(n_cand + 1);
    out->tile = ar.take<int64_t>(3 * (out->nt + 1));
    return ar.ok();
}

// Sum over the block of three counters; every thread gets the totals.
__device__ __forceinline__ void block_sum3(int64_t& a, int64_t& b, int64_t& c, int64_t (*s_w)[3]) {
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    for (int d = WAVE / 2; d > 0; d >>= 1) {
        a += shfl_i64(a, lane ^ d);
        b += shfl_i64(b, lane ^ d);
        c += shfl_i64(c, lane ^ d);
    }
    __syncthreads();
    if (lane == 0) { s_w[wid][0] = a; s_w[wid][1] = b; s_w[wid][2] = c; }
    __syncthreads();
    a = b = c = 0;
    for (int w = 0; w < BLOCK / WAVE; ++w) { a += s_w[w][0]; b += s_w[w][1]; c += s_w[w][2]; }
}

// Exclusive prefix over the block of three counters (in place); tot* = block totals.
__device__ __forceinline__ void block_excl_scan3(int64_t& a, int64_t& b, int64_t& c, int64_t& ta, int64_t& tb,
                                                 int64_t& tc, int64_t (*s_w)[3]) {
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    int64_t ia = a, ib = b, ic = c;
    for (int d = 1; d < WAVE; d <<= 1) {
        const int from = lane >= d ? lane - d : lane;
        const int64_t xa = shfl_i64(ia, from), xb = shfl_i64(ib, from), xc = shfl_i64(ic, from);
        if (lane >= d) { ia += xa; ib += xb; ic += xc; }
    }
    __syncthreads();
    if (lane == WAVE - 1) { s_w[wid][0] = ia; s_w[wid][1] = ib; s_w[wid][2] = ic; }
    __syncthreads();
    int64_t oa = 0, ob = 0, oc = 0;
    ta = tb = tc = 0;
    for (int w = 0; w < BLOCK / WAVE; ++w) {
        if (w < wid) { oa += s_w[w][0]; ob += s_w[w][1]; oc += s_w[w][2]; }
        ta += s_w[w][0]; tb += s_w[w][1]; tc += s_w[w][2];
    }
    a = oa + ia - a;
    b = ob + ib - b;
    c = oc + ic - c;
}

// node, window and distinct timestamps of candidate j (workspace), tile sums of the three counters
__global__ __launch_bounds__(BLOCK) void seeds_count_kernel(sgl_tcsr g, sgl_seed_query q, SeedWs w) {
    __shared__ int64_t s_w[BLOCK / WAVE][3];
    const int lane = threadIdx.x % WAVE;
    int64_t sum_r = 0, sum_s = 0, sum_q = 0;
    for (int r = 0; r < SEED_ROUNDS; ++r) {
        const int64_t j = (int64_t)blockIdx.x * SEED_TILE + r * BLOCK + threadIdx.x;
        const bool valid = j < q.n_cand;
        int64_t v = 0, lo = 0, hi = 0, n_ts = 0;
        if (valid) {
            // selected-chunk position p with cand_off[p] <= j < cand_off[p+1]
            int64_t a = 0, b = q.num_chunks;
            while (b - a > 1) {
                const int64_t mid = a + ((b - a) >> 1);
                if (q.cand_off[mid] <= j) a = mid; else b = mid;
            }
            const int64_t c = q.chunks[a];
            v = q.chunk_nodes[q.chunk_ptr[c] + (j - q.cand_off[a])];
            const int64_t rs = g.row_ptr[v], re = g.row_ptr[v + 1];
            lo = lower_bound_i64(g.ts, rs, re, q.t_begin);
            hi = lower_bound_i64(g.ts, lo, re, q.t_end);
        }
        const bool heavy = hi - lo > SEED_LIGHT;
        if (!heavy)
            for (int64_t e = lo; e < hi; ++e) n_ts += (e == lo || g.ts[e] != g.ts[e - 1]) ? 1 : 0;
        for (uint64_t hm = __ballot(heavy); hm != 0; hm &= hm - 1) {   // the wave walks one heavy window at a time
            const int src = __ffsll((unsigned long long)hm) - 1;
            const int64_t l = shfl_i64(lo, src), h = shfl_i64(hi, src);
            int64_t heads = 0;
            for (int64_t e0 = l; e0 < h; e0 += WAVE) {
                const int64_t e = e0 + lane;
                const bool head = e < h && (e == l || g.ts[e] != g.ts[e - 1]);
                heads += __popcll(__ballot(head));
            }
            if (lane == src) n_ts = heads;
        }
        if (valid) {
            w.node[j] = v;
            w.lo[j] = lo;
            w.hi[j] = hi;
            w.n_ts[j] = n_ts;
            sum_r += hi > lo ? 1 : 0;
            sum_s += n_ts;
            sum_q += hi - lo;
        }
    }
    block_sum3(sum_r, sum_s, sum_q, s_w);
    if (threadIdx.x == 0) {
        w.tile[blockIdx.x] = sum_r;
        w.tile[(w.nt + 1) + blockIdx.x] = sum_s;
        w.tile[2 * (w.nt + 1) + blockIdx.x] = sum_q;
    }
}

// one block: exclusive scan of the three tile arrays in place, grand totals -> totals[0..2]
__global__ __launch_bounds__(SEED_SCAN_BLOCK) void seeds_scan_kernel(SeedWs w, int64_t* totals) {
    __shared__ int64_t s_part[SEED_SCAN_BLOCK];
    const int64_t per = ceil_div<int64_t>(w.nt, SEED_SCAN_BLOCK);
    const int64_t b0 = (int64_t)threadIdx.x * per;
    const int64_t b1 = b0 + per < w.nt ? b0 + per : w.nt;
    for (int k = 0; k < 3; ++k) {
        int64_t* t = w.tile + (int64_t)k * (w.nt + 1);
        int64_t sum = 0;
        for (int64_t b = b0; b < b1; ++b) sum += t[b];
        __syncthreads();
        s_part[threadIdx.x] = sum;
        __syncthreads();
        for (int d = 1; d < SEED_SCAN_BLOCK; d <<= 1) {
            int64_t x = 0;
            if ((int)threadIdx.x >= d) x = s_part[threadIdx.x - d];
            __syncthreads();
            s_part[threadIdx.x] += x;
            __syncthreads();
        }
        int64_t run = s_part[threadIdx.x] - sum;
        for (int64_t b = b0; b < b1; ++b) {
            const int64_t x = t[b];
            t[b] = run;
            run += x;
        }
        if (threadIdx.x == SEED_SCAN_BLOCK - 1) totals[k] = s_part[SEED_SCAN_BLOCK - 1];
    }
}

__global__ __launch_bounds__(BLOCK) void seeds_fill_kernel(sgl_tcsr g, sgl_seed_query q, SeedWs w,
                                                           const int64_t* totals, int64_t* roots, int64_t* ts_ptr,
                                                           int64_t* ts, int64_t* q_ptr, int64_t* q_eid,
                                                           int64_t* window_end) {
    __shared__ int64_t s_w[BLOCK / WAVE][3];
    const int lane = threadIdx.x % WAVE;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        ts_ptr[totals[0]] = totals[1];
        q_ptr[totals[1]] = totals[2];
    }
    int64_t run_r = w.tile[blockIdx.x], run_s = w.tile[(w.nt + 1) + blockIdx.x], run_q = w.tile[2 * (w.nt + 1) + blockIdx.x];
    for (int r = 0; r < SEED_ROUNDS; ++r) {
        const int64_t j = (int64_t)blockIdx.x * SEED_TILE + r * BLOCK + threadIdx.x;
        const bool valid = j < q.n_cand;
        const int64_t lo = valid ? w.lo[j] : 0, hi = valid ? w.hi[j] : 0;
        int64_t pr = hi > lo ? 1 : 0, ps = valid ? w.n_ts[j] : 0, pq = hi - lo, tr, tsum, tq;
        block_excl_scan3(pr, ps, pq, tr, tsum, tq, s_w);
        const int64_t r0 = run_r + pr, s0 = run_s + ps, q0 = run_q + pq;
        run_r += tr; run_s += tsum; run_q += tq;
        if (hi > lo) {
            roots[r0] = w.node[j];
            ts_ptr[r0] = s0;
        }
        const bool heavy = hi - lo > SEED_LIGHT;
        if (!heavy) {
            int64_t s = s0;
            for (int64_t e = lo; e < hi; ++e) {
                const int64_t t = g.ts[e];
                if (e == lo || t != g.ts[e - 1]) {
                    ts[s] = t;
                    q_ptr[s] = q0 + (e - lo);
                    // the first edge of the row at this time: where the window strictly before it ends
                    if (window_end != nullptr) window_end[s] = e;
                    ++s;
                }
                q_eid[q0 + (e - lo)] = g.eid[e];
            }
        }
        for (uint64_t hm = __ballot(heavy); hm != 0; hm &= hm - 1) {
            const int src = __ffsll((unsigned long long)hm) - 1;
            const int64_t l = shfl_i64(lo, src), h = shfl_i64(hi, src), qb = shfl_i64(q0, src);
            int64_t s = shfl_i64(s0, src);
            const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
            for (int64_t e0 = l; e0 < h; e0 += WAVE) {
                const int64_t e = e0 + lane;
                const bool in = e < h;
                const int64_t t = in ? g.ts[e] : 0;
                const bool head = in && (e == l || t != g.ts[e - 1]);
                const uint64_t hb = __ballot(head);
                if (head) {
                    const int64_t si = s + __popcll(hb & lt);
                    ts[si] = t;
                    q_ptr[si] = qb + (e - l);
                    if (window_end != nullptr) window_end[si] = e;
                }
                if (in) q_eid[qb + (e - l)] = g.eid[e];
                s += __popcll(hb);
            }
        }
    }
}

__global__ void empty_seed_ptrs_kernel(int64_t* totals) { totals[0] = totals[1] = totals[2] = 0; }

__global__ void seeds_close_kernel(const int64_t* totals, int64_t* ts_ptr, int64_t* q_ptr) {
    ts_ptr[totals[0]] = totals[1];
    q_ptr[totals[1]] = totals[2];
}

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
    hipLaunchKernelGGL(seeds_count_kernel, dim3((unsigned)w.nt), dim3(BLOCK), 0, st, *g, *q, w);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(seeds_scan_kernel, dim3(1), dim3(SEED_SCAN_BLOCK), 0, st, w, totals);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" int32_t sgl_seeds_fill(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* totals,
                                  int64_t* roots, int64_t* ts_ptr, int64_t* ts, int64_t* q_ptr, int64_t* q_eid,
                                  int64_t* window_end, void* ws, size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_query(g, q)) != SGL_OK) return rc;
    if (!totals || !ts_ptr || !q_ptr) return fail(SGL_EINVAL, "seeds_fill: totals/ts_ptr/q_ptr is NULL");
    hipStream_t st = as_stream(stream);
    SeedWs w{};
    if (q->n_cand > 0 && (!ws || ws_bytes < seeds_ws_bytes(q->n_cand) || !carve(ws, ws_bytes, q->n_cand, &w)))
        return fail(SGL_ENOMEM, "seeds_fill: workspace %zu < %zu bytes", ws_bytes, seeds_ws_bytes(q->n_cand));
    if (q->n_cand == 0) {     // nothing but the closing pointers (totals are all zero)
        hipLaunchKernelGGL(seeds_close_kernel, dim3(1), dim3(1), 0, st, totals, ts_ptr, q_ptr);
        SGL_LAUNCH_CHECK();
        return SGL_OK;
    }
    hipLaunchKernelGGL(seeds_fill_kernel, dim3((unsigned)w.nt), dim3(BLOCK), 0, st, *g, *q, w, totals, roots, ts_ptr, ts, q_ptr,
                       q_eid, window_end);
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
