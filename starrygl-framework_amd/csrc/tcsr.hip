// T-CSR validation and construction for gfx950.
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;

// flag bits: 1 row_ptr ends, 2 row_ptr not monotone, 4 col out of range, 8 ts not ascending
__global__ void validate_rows_kernel(sgl_tcsr g, int32_t* flag) {
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v == 0 && (g.row_ptr[0] != 0 || g.row_ptr[g.n] != g.m)) atomicOr(flag, 1);
    if (v < g.n && g.row_ptr[v + 1] < g.row_ptr[v]) atomicOr(flag, 2);
}

__global__ void validate_edges_kernel(sgl_tcsr g, int32_t* flag) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= g.m) return;
    const int64_t c = g.col[e];
    if (c < 0 || c >= g.n) atomicOr(flag, 4);
    if (e + 1 < g.m && g.ts[e + 1] < g.ts[e]) {
        // a descent is legal only across a row boundary: find the row of e
        int64_t lo = 0, hi = g.n;  // last v with row_ptr[v] <= e
        while (hi - lo > 1) {
            const int64_t mid = lo + ((hi - lo) >> 1);
            if (g.row_ptr[mid] <= e) lo = mid; else hi = mid;
        }
        if (g.row_ptr[lo + 1] > e + 1) atomicOr(flag, 8);
    }
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" int32_t sgl_tcsr_validate(const sgl_tcsr* g, void* ws, size_t ws_bytes, void* stream) {
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "tcsr_validate: NULL graph");
    if (g->m > 0 && (!g->col || !g->ts || !g->eid)) return fail(SGL_EINVAL, "tcsr_validate: NULL array");
    if (!ws || ws_bytes < 8) return fail(SGL_ENOMEM, "tcsr_validate: workspace < 8 bytes");
    hipStream_t st = as_stream(stream);
    int32_t* flag = static_cast<int32_t*>(ws);
    SGL_HIP_TRY(hipMemsetAsync(flag, 0, 8, st));
    hipLaunchKernelGGL(validate_rows_kernel, dim3((unsigned)ceil_div<int64_t>(g->n + 1, BLOCK)), dim3(BLOCK), 0, st, *g, flag);
    SGL_LAUNCH_CHECK();
    if (g->m > 0) {
        hipLaunchKernelGGL(validate_edges_kernel, dim3((unsigned)ceil_div<int64_t>(g->m, BLOCK)), dim3(BLOCK), 0, st, *g, flag);
        SGL_LAUNCH_CHECK();
    }
    int32_t h = 0;
    SGL_HIP_TRY(hipMemcpyAsync(&h, flag, 4, hipMemcpyDeviceToHost, st));
    SGL_HIP_TRY(hipStreamSynchronize(st));
    if (h & 1) return fail(SGL_ERANGE, "tcsr_validate: row_ptr[0] != 0 or row_ptr[n] != m");
    if (h & 2) return fail(SGL_ERANGE, "tcsr_validate: row_ptr not monotone");
    if (h & 4) return fail(SGL_ERANGE, "tcsr_validate: col outside [0,n)");
    if (h & 8) return fail(SGL_ERANGE, "tcsr_validate: ts not ascending in row");
    return SGL_OK;
}

namespace sgl {
namespace {

struct BuildStats {
    long long ts_min, ts_max, eid_max;
    int32_t flags;  // bit0 src/dst out of range, bit1 not (src,ts,eid)-sorted, bit2 not (ts,eid)-sorted,
                    // bit3 eid not strictly ascending, bit4 negative eid
    int32_t pad;
};

__global__ void stats_init_kernel(BuildStats* st) {
    st->ts_min = INT64_MAX;
    st->ts_max = INT64_MIN;
    st->eid_max = 0;
    st->flags = 0;
}

__global__ __launch_bounds__(BLOCK) void stats_kernel(int64_t n, int64_t m, const int64_t* __restrict__ src,
                                                      const int64_t* __restrict__ dst,
                                                      const int64_t* __restrict__ ts,
                                                      const int64_t* __restrict__ eid, BuildStats* st) {
    __shared__ long long s_min[BLOCK / WAVE], s_max[BLOCK / WAVE], s_emax[BLOCK / WAVE];
    __shared__ int32_t s_flags[BLOCK / WAVE];
    long long tmin = INT64_MAX, tmax = INT64_MIN, emax = 0;
    int32_t f = 0;
    // grid-stride: a block ends with four atomics on the same four words, so there must be few blocks
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < m; i += (int64_t)gridDim.x * BLOCK) {
        const int64_t s = src[i], d = dst[i], t = ts[i], e = eid ? eid[i] : i;
        if (s < 0 || s >= n || d < 0 || d >= n) f |= 1;
        if (e < 0) f |= 16;
        tmin = t < tmin ? t : tmin;
        tmax = t > tmax ? t : tmax;
        emax = e > emax ? e : emax;
        if (i > 0) {
            const int64_t ps = src[i - 1], pt = ts[i - 1], pe = eid ? eid[i - 1] : i - 1;
            const bool te_le = (pt < t) || (pt == t && pe <= e);
            if (!((ps < s) || (ps == s && te_le))) f |= 2;
            if (!te_le) f |= 4;
            if (!(pe < e)) f |= 8;
        }
    }
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    for (int d = WAVE / 2; d > 0; d >>= 1) {
        const long long a = shfl_i64(tmin, lane ^ d), b = shfl_i64(tmax, lane ^ d), c = shfl_i64(emax, lane ^ d);
        tmin = a < tmin ? a : tmin;
        tmax = b > tmax ? b : tmax;
        emax = c > emax ? c : emax;
        f |= __shfl(f, lane ^ d);
    }
    if (lane == 0) { s_min[wid] = tmin; s_max[wid] = tmax; s_emax[wid] = emax; s_flags[wid] = f; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < BLOCK / WAVE; ++w) {
            tmin = s_min[w] < tmin ? s_min[w] : tmin;
            tmax = s_max[w] > tmax ? s_max[w] : tmax;
            emax = s_emax[w] > emax ? s_emax[w] : emax;
            f |= s_flags[w];
        }
        if (tmin != INT64_MAX) atomicMin(&st->ts_min, tmin);
        if (tmax != INT64_MIN) atomicMax(&st->ts_max, tmax);
        atomicMax(&st->eid_max, emax);
        if (f) atomicOr(&st->flags, f);
    }
}

__global__ void iota_kernel(int64_t* p, int64_t m) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m) p[i] = i;
}

// key[i] = arr[perm[i]] - bias  (arr == nullptr: the identity array)
__global__ void gather_key_kernel(const int64_t* __restrict__ arr, const int64_t* __restrict__ perm, int64_t bias,
                                  int64_t m, uint64_t* __restrict__ key) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m) {
        const int64_t p = perm[i];
        key[i] = (uint64_t)((arr ? arr[p] : p) - bias);
    }
}

// row_ptr from the sorted source keys: position i opens every row in (key[i-1], key[i]]
__global__ void row_ptr_kernel(const uint64_t* __restrict__ skey, int64_t n, int64_t m, int64_t* __restrict__ row_ptr) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i > m) return;
    const int64_t prev = (i == 0) ? -1 : (int64_t)skey[i - 1];
    const int64_t cur = (i == m) ? n : (int64_t)skey[i];
    for (int64_t v = prev + 1; v <= cur; ++v) row_ptr[v] = i;
}

__global__ void permute_out_kernel(const int64_t* __restrict__ perm, const int64_t* __restrict__ dst,
                                   const int64_t* __restrict__ ts, const int64_t* __restrict__ eid, int64_t m,
                                   int64_t* __restrict__ col, int64_t* __restrict__ col_ts,
                                   int64_t* __restrict__ col_eid) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m) {
        const int64_t p = perm[i];
        col[i] = dst[p];
        col_ts[i] = ts[p];
        col_eid[i] = eid ? eid[p] : p;
    }
}

int bits_of(uint64_t x) {
    int b = 0;
    while (x) { ++b; x >>= 1; }
    return b;
}

}  // namespace
}  // namespace sgl

extern "C" size_t sgl_tcsr_build_workspace_bytes(int64_t n, int64_t m) {
    (void)n;
    if (m < 0) m = 0;
    return 4 * align_up((size_t)(m + 1) * 8) + radix_sort_workspace_bytes(m) + 1024;
}

extern "C" int32_t sgl_tcsr_build(int64_t n, int64_t m, const int64_t* src, const int64_t* dst,
                                  const int64_t* ts, const int64_t* eid, int64_t* row_ptr, int64_t* col,
                                  int64_t* col_ts, int64_t* col_eid, void* ws, size_t ws_bytes,
                                  void* stream) {
    if (n < 0 || m < 0 || !row_ptr) return fail(SGL_EINVAL, "tcsr_build: negative size or NULL row_ptr");
    if (m > 0 && (!src || !dst || !ts || !col || !col_ts || !col_eid)) return fail(SGL_EINVAL, "tcsr_build: NULL array");
    if (!ws || ws_bytes < sgl_tcsr_build_workspace_bytes(n, m))
        return fail(SGL_ENOMEM, "tcsr_build: workspace %zu < %zu bytes", ws_bytes, sgl_tcsr_build_workspace_bytes(n, m));
    if (ceil_div<int64_t>(m + 1, BLOCK) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "tcsr_build: too many edges");
    hipStream_t st = as_stream(stream);
    Arena ar(ws, ws_bytes);
    BuildStats* d_stats = ar.take<BuildStats>(1);
    uint64_t* key_a = ar.take<uint64_t>(m + 1);
    uint64_t* key_b = ar.take<uint64_t>(m + 1);
    int64_t* perm_a = ar.take<int64_t>(m + 1);
    int64_t* perm_b = ar.take<int64_t>(m + 1);
    const size_t rws_bytes = radix_sort_workspace_bytes(m);
    void* rws = ar.take<char>(rws_bytes);
    if (!ar.ok()) return fail(SGL_ENOMEM, "tcsr_build: workspace too small");
    const unsigned eb = (unsigned)ceil_div<int64_t>(m > 0 ? m : 1, BLOCK);

    hipLaunchKernelGGL(stats_init_kernel, dim3(1), dim3(1), 0, st, d_stats);
    SGL_LAUNCH_CHECK();
    if (m > 0) {
        hipLaunchKernelGGL(stats_kernel, dim3(eb < 4096u ? eb : 4096u), dim3(BLOCK), 0, st, n, m, src, dst, ts, eid, d_stats);
        SGL_LAUNCH_CHECK();
    }
    BuildStats h;
    SGL_HIP_TRY(hipMemcpyAsync(&h, d_stats, sizeof h, hipMemcpyDeviceToHost, st));
    SGL_HIP_TRY(hipStreamSynchronize(st));
    if (h.flags & 1) return fail(SGL_ERANGE, "tcsr_build: src/dst outside [0,n)");
    if (h.flags & 16) return fail(SGL_ERANGE, "tcsr_build: negative edge id");

    int64_t* perm = perm_a;
    hipLaunchKernelGGL(iota_kernel, dim3(eb), dim3(BLOCK), 0, st, perm_a, m);
    SGL_LAUNCH_CHECK();
    const bool sorted_all = !(h.flags & 2), sorted_te = !(h.flags & 4), sorted_e = !(h.flags & 8);
    // LSD order: eid, then ts, then src; a pass whose key is already in order is skipped
    struct Pass { const int64_t* arr; int64_t bias; int bits; bool run; };
    const Pass passes[3] = {
        {eid, 0, bits_of((uint64_t)h.eid_max), m > 0 && !sorted_all && !sorted_te && !sorted_e},
        {ts, h.ts_min, m > 0 ? bits_of((uint64_t)h.ts_max - (uint64_t)h.ts_min) : 0, m > 0 && !sorted_all && !sorted_te},
        {src, 0, bits_of((uint64_t)(n > 0 ? n - 1 : 0)), m > 0 && !sorted_all},
    };
    const uint64_t* skey = nullptr;
    for (int q = 0; q < 3; ++q) {
        if (!passes[q].run) continue;
        int64_t* other = (perm == perm_a) ? perm_b : perm_a;
        hipLaunchKernelGGL(gather_key_kernel, dim3(eb), dim3(BLOCK), 0, st, (q == 0 && !eid) ? nullptr : passes[q].arr,
                           perm, passes[q].bias, m, key_a);
        SGL_LAUNCH_CHECK();
        int in_b = 0;
        // sort (key_a, perm) using (key_b, other) as the ping-pong partner
        int32_t rc = radix_sort_pairs(key_a, perm, key_b, other, m, nullptr, 0, passes[q].bits, &in_b, rws, rws_bytes, st);
        if (rc != SGL_OK) return rc;
        if (in_b) perm = other;
        if (q == 2) skey = in_b ? key_b : key_a;
    }
    if (skey == nullptr) {  // the src pass was skipped: keys are the sources in input order
        hipLaunchKernelGGL(gather_key_kernel, dim3(eb), dim3(BLOCK), 0, st, src, perm, (int64_t)0, m, key_a);
        SGL_LAUNCH_CHECK();
        skey = key_a;
    }
    hipLaunchKernelGGL(row_ptr_kernel, dim3((unsigned)ceil_div<int64_t>(m + 1, BLOCK)), dim3(BLOCK), 0, st, skey, n, m, row_ptr);
    SGL_LAUNCH_CHECK();
    if (m > 0) {
        hipLaunchKernelGGL(permute_out_kernel, dim3(eb), dim3(BLOCK), 0, st, perm, dst, ts, eid, m, col, col_ts, col_eid);
        SGL_LAUNCH_CHECK();
    }
    SGL_HIP_TRY(hipStreamSynchronize(st));
    return SGL_OK;
}

namespace sgl {
namespace {
__global__ void chunk_range_kernel(const int64_t* __restrict__ node_chunk, int64_t n, int64_t num_chunks, int32_t* flag) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && (node_chunk[i] < 0 || node_chunk[i] >= num_chunks)) atomicOr(flag, 1);
}
}  // namespace
}  // namespace sgl

extern "C" size_t sgl_chunk_index_workspace_bytes(int64_t n) {
    if (n < 0) n = 0;
    return 3 * align_up((size_t)(n + 1) * 8) + radix_sort_workspace_bytes(n) + 2048;
}

extern "C" int32_t sgl_chunk_index_build(int64_t n, int64_t num_chunks, const int64_t* node_chunk,
                                         int64_t* chunk_ptr, int64_t* chunk_nodes, void* ws, size_t ws_bytes,
                                         void* stream) {
    if (n < 0 || num_chunks < 0 || !chunk_ptr) return fail(SGL_EINVAL, "chunk_index_build: negative size or NULL chunk_ptr");
    if (n > 0 && (!node_chunk || !chunk_nodes)) return fail(SGL_EINVAL, "chunk_index_build: NULL array");
    if (!ws || ws_bytes < sgl_chunk_index_workspace_bytes(n)) return fail(SGL_ENOMEM, "chunk_index_build: workspace too small");
    if (ceil_div<int64_t>((n > num_chunks ? n : num_chunks) + 1, BLOCK) > 0x7FFFFFFFll)
        return fail(SGL_ENOTSUP, "chunk_index_build: too many nodes");
    hipStream_t st = as_stream(stream);
    Arena ar(ws, ws_bytes);
    int32_t* flag = ar.take<int32_t>(2);
    uint64_t* key_a = ar.take<uint64_t>(n + 1);
    uint64_t* key_b = ar.take<uint64_t>(n + 1);
    int64_t* val_b = ar.take<int64_t>(n + 1);
    const size_t rws_bytes = radix_sort_workspace_bytes(n);
    void* rws = ar.take<char>(rws_bytes);
    if (!ar.ok()) return fail(SGL_ENOMEM, "chunk_index_build: workspace too small");
    const unsigned nb = (unsigned)ceil_div<int64_t>(n > 0 ? n : 1, BLOCK);
    SGL_HIP_TRY(hipMemsetAsync(flag, 0, 8, st));
    const uint64_t* skey = key_a;
    if (n > 0) {
        hipLaunchKernelGGL(chunk_range_kernel, dim3(nb), dim3(BLOCK), 0, st, node_chunk, n, num_chunks, flag);
        SGL_LAUNCH_CHECK();
        int32_t h = 0;
        SGL_HIP_TRY(hipMemcpyAsync(&h, flag, 4, hipMemcpyDeviceToHost, st));
        SGL_HIP_TRY(hipStreamSynchronize(st));
        if (h) return fail(SGL_ERANGE, "chunk_index_build: chunk id outside [0, num_chunks)");
        hipLaunchKernelGGL(iota_kernel, dim3(nb), dim3(BLOCK), 0, st, chunk_nodes, n);
        SGL_LAUNCH_CHECK();
        hipLaunchKernelGGL(gather_key_kernel, dim3(nb), dim3(BLOCK), 0, st, node_chunk, chunk_nodes, (int64_t)0, n, key_a);
        SGL_LAUNCH_CHECK();
        int in_b = 0;
        int32_t rc = radix_sort_pairs(key_a, chunk_nodes, key_b, val_b, n, nullptr, 0,
                                      bits_of((uint64_t)(num_chunks > 0 ? num_chunks - 1 : 0)), &in_b, rws, rws_bytes, st);
        if (rc != SGL_OK) return rc;
        if (in_b) {
            SGL_HIP_TRY(hipMemcpyAsync(chunk_nodes, val_b, (size_t)n * 8, hipMemcpyDeviceToDevice, st));
            skey = key_b;
        }
    }
    hipLaunchKernelGGL(row_ptr_kernel, dim3((unsigned)ceil_div<int64_t>(n + 1, BLOCK)), dim3(BLOCK), 0, st, skey, num_chunks, n, chunk_ptr);
    SGL_LAUNCH_CHECK();
    SGL_HIP_TRY(hipStreamSynchronize(st));
    return SGL_OK;
}

namespace sgl {
namespace {

// out[i] = first position in row node[i] whose timestamp is >= t[i] (-1: node outside [0,n)).
// With node = col and t = ts (N = m) this is the next-hop index.
__global__ __launch_bounds__(BLOCK) void window_end_kernel(sgl_tcsr g, const int64_t* __restrict__ node,
                                                           const int64_t* __restrict__ t_of, int64_t N,
                                                           int64_t* __restrict__ out) {
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < N; i += (int64_t)gridDim.x * BLOCK) {
        const int64_t v = node[i], t = t_of[i];
        int64_t lo = -1;
        if (v >= 0 && v < g.n) {
            lo = g.row_ptr[v];
            int64_t hi = g.row_ptr[v + 1];
            while (lo < hi) {
                const int64_t mid = lo + ((hi - lo) >> 1);
                if (g.ts[mid] < t) lo = mid + 1; else hi = mid;
            }
        }
        out[i] = lo;
    }
}

int32_t launch_window_end(const sgl_tcsr* g, const int64_t* node, const int64_t* t, int64_t N, int64_t* out,
                          void* stream) {
    int64_t blocks = ceil_div<int64_t>(N, BLOCK);
    if (blocks > (1 << 20)) blocks = 1 << 20;
    hipLaunchKernelGGL(window_end_kernel, dim3((unsigned)blocks), dim3(BLOCK), 0, as_stream(stream), *g, node, t, N, out);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

}  // namespace
}  // namespace sgl

namespace sgl {
namespace {
__global__ __launch_bounds__(BLOCK) void records_kernel(sgl_tcsr g, int64_t* __restrict__ rec) {
    for (int64_t e = (int64_t)blockIdx.x * BLOCK + threadIdx.x; e < g.m; e += (int64_t)gridDim.x * BLOCK) {
        longlong2 a, b;
        a.x = g.col[e];
        a.y = g.ts[e];
        b.x = g.eid[e];
        int64_t h = g.hop_hint != nullptr ? g.hop_hint[e] : -1;
        // with the window's length (hint_pack): the entry lies in row col[e], whose start the row pointers give
        if (h >= 0 && g.m <= HINT_POS_MASK && a.x >= 0 && a.x < g.n) {
            const int64_t len = h - g.row_ptr[a.x];
            if (len >= 0) h = hint_pack(h, len);
        }
        b.y = h;
        reinterpret_cast<longlong2*>(rec)[2 * e] = a;
        reinterpret_cast<longlong2*>(rec)[2 * e + 1] = b;
    }
}
}  // namespace
}  // namespace sgl

extern "C" int32_t sgl_tcsr_records_build(const sgl_tcsr* g, int64_t* rec, void* stream) {
    if (!g || g->n < 0 || g->m < 0) return fail(SGL_EINVAL, "tcsr_records_build: NULL graph");
    if (g->m == 0) return SGL_OK;
    if (!g->col || !g->ts || !g->eid || !rec || (g->hop_hint && !g->row_ptr)) return fail(SGL_EINVAL, "tcsr_records_build: NULL array");
    if (reinterpret_cast<uintptr_t>(rec) % 32 != 0) return fail(SGL_EINVAL, "tcsr_records_build: rec must be 32-byte aligned");
    int64_t blocks = ceil_div<int64_t>(g->m, BLOCK);
    if (blocks > (1 << 20)) blocks = 1 << 20;
    hipLaunchKernelGGL(records_kernel, dim3((unsigned)blocks), dim3(BLOCK), 0, as_stream(stream), *g, rec);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" int32_t sgl_tcsr_hop_hint_build(const sgl_tcsr* g, int64_t* hop_hint, void* stream) {
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "tcsr_hop_hint_build: NULL graph");
    if (g->m == 0) return SGL_OK;
    if (!g->col || !g->ts || !hop_hint) return fail(SGL_EINVAL, "tcsr_hop_hint_build: NULL array");
    return launch_window_end(g, g->col, g->ts, g->m, hop_hint, stream);
}

extern "C" int32_t sgl_window_end(const sgl_tcsr* g, const int64_t* node, const int64_t* t, int64_t N,
                                  int64_t* out, void* stream) {
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "window_end: NULL graph");
    if (N < 0) return fail(SGL_EINVAL, "window_end: N < 0");
    if (N == 0) return SGL_OK;
    if (!node || !t || !out || (g->m > 0 && !g->ts)) return fail(SGL_EINVAL, "window_end: NULL array");
    return launch_window_end(g, node, t, N, out, stream);
}
