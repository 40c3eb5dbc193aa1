// Batch materialisation helpers for gfx950: unique over (id, timestamp) pairs
// with inverse map, and the stable (destination, timestamp) edge order with its
// CSC pointer array.  Both are two stable LSD radix sorts (secondary key first)
// over (key, position) pairs followed by one flag / scan / scatter pass.
//
// Replaces _get_unique_pairs / _merge_and_map_nodes (np.unique over structured
// (id, ts) records, prepare_sample.py:205-213, 231-246) and
// _build_csc_from_pairs (np.lexsort((ts, dst)) + counts, prepare_sample.py:215-229).
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int MAX_GRID = 4096;
constexpr uint64_t SIGN = 1ull << 63;   // signed order -> unsigned order

unsigned grid_for(int64_t n) {
    const int64_t b = ceil_div<int64_t>(n > 0 ? n : 1, BLOCK);
    return (unsigned)(b > MAX_GRID ? MAX_GRID : b);
}

struct PairWs {
    uint64_t *ka, *kb;
    int64_t *va, *vb, *head;
    void* sort_ws;
    size_t sort_ws_bytes;
    void* scan_ws;
    size_t scan_ws_bytes;
};

size_t pair_ws_bytes(int64_t n) {
    return 5 * align_up((size_t)(n + 1) * 8) + radix_sort_workspace_bytes(n) + exclusive_scan_workspace_bytes(n) + 4096;
}

bool carve(void* ws, size_t bytes, int64_t n, PairWs* w) {
    Arena ar(ws, bytes);
    w->ka = ar.take<uint64_t>(n + 1);
    w->kb = ar.take<uint64_t>(n + 1);
    w->va = ar.take<int64_t>(n + 1);
    w->vb = ar.take<int64_t>(n + 1);
    w->head = ar.take<int64_t>(n + 1);
    w->sort_ws_bytes = radix_sort_workspace_bytes(n);
    w->sort_ws = ar.take<char>(w->sort_ws_bytes);
    w->scan_ws_bytes = exclusive_scan_workspace_bytes(n);
    w->scan_ws = ar.take<char>(w->scan_ws_bytes);
    return ar.ok();
}

// keys[i] = key[i] in unsigned order, vals[i] = i
__global__ __launch_bounds__(BLOCK) void load_keys_kernel(const int64_t* __restrict__ key, int64_t n_max, const int64_t* n_dev,
                                                          uint64_t* keys, int64_t* vals) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
        keys[i] = (uint64_t)key[i] ^ SIGN;
        vals[i] = i;
    }
}

// keys[i] = key[vals[i]]: the primary key in the order the secondary sort produced
__global__ __launch_bounds__(BLOCK) void regather_keys_kernel(const int64_t* __restrict__ key, const int64_t* __restrict__ vals,
                                                              int64_t n_max, const int64_t* n_dev, uint64_t* keys) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK)
        keys[i] = (uint64_t)key[vals[i]] ^ SIGN;
}

// perm = stable order of positions by (primary, secondary); the sorted primary keys end in *keys_out
int32_t sort_two_keys(const int64_t* primary, int primary_bits, const int64_t* secondary, int64_t n_max,
                      const int64_t* n_dev, PairWs& w, uint64_t** keys_out, int64_t** perm_out, hipStream_t st) {
    hipLaunchKernelGGL(load_keys_kernel, dim3(grid_for(n_max)), dim3(BLOCK), 0, st, secondary, n_max, n_dev, w.ka, w.va);
    SGL_LAUNCH_CHECK();
    int in_b = 0;
    int32_t rc = radix_sort_pairs(w.ka, w.va, w.kb, w.vb, n_max, n_dev, 0, 64, &in_b, w.sort_ws, w.sort_ws_bytes, st);
    if (rc != SGL_OK) return rc;
    uint64_t* k0 = in_b ? w.kb : w.ka; int64_t* v0 = in_b ? w.vb : w.va;
    uint64_t* k1 = in_b ? w.ka : w.kb; int64_t* v1 = in_b ? w.va : w.vb;
    hipLaunchKernelGGL(regather_keys_kernel, dim3(grid_for(n_max)), dim3(BLOCK), 0, st, primary, v0, n_max, n_dev, k0);
    SGL_LAUNCH_CHECK();
    // non-negative primary keys below 2^primary_bits all carry the flipped sign bit: the low bits order them
    rc = radix_sort_pairs(k0, v0, k1, v1, n_max, n_dev, 0, primary_bits, &in_b, w.sort_ws, w.sort_ws_bytes, st);
    if (rc != SGL_OK) return rc;
    *keys_out = in_b ? k1 : k0;
    *perm_out = in_b ? v1 : v0;
    return SGL_OK;
}

__global__ __launch_bounds__(BLOCK) void pair_heads_kernel(const uint64_t* __restrict__ keys, const int64_t* __restrict__ perm,
                                                           const int64_t* __restrict__ ts, int64_t n_max, const int64_t* n_dev,
                                                           int64_t* head) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK)
        head[i] = (i == 0 || keys[i] != keys[i - 1] || ts[perm[i]] != ts[perm[i - 1]]) ? 1 : 0;
}

// rank[i] = exclusive prefix of the head flags; a head's rank is its place in the unique list
__global__ __launch_bounds__(BLOCK) void pair_emit_kernel(const uint64_t* __restrict__ keys, const int64_t* __restrict__ perm,
                                                          const int64_t* __restrict__ ts, const int64_t* __restrict__ rank,
                                                          int64_t n_max, const int64_t* n_dev, int64_t* uniq_ids,
                                                          int64_t* uniq_ts, int64_t* inverse, int64_t* U_dev) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
        const int64_t p = perm[i], t = ts[p];
        const bool head = i == 0 || keys[i] != keys[i - 1] || t != ts[perm[i - 1]];
        const int64_t r = rank[i] - (head ? 0 : 1);      // exclusive prefix counts this head only from i + 1 on
        if (head) {
            uniq_ids[r] = (int64_t)(keys[i] ^ SIGN);
            uniq_ts[r] = t;
        }
        inverse[p] = r;
        if (i == n - 1) U_dev[0] = r + 1;
    }
}

__global__ void zero_total_kernel(int64_t* total) { total[0] = 0; }

// indptr[d] = number of sorted keys below d (keys are dst ^ SIGN, ascending)
__global__ __launch_bounds__(BLOCK) void indptr_kernel(const uint64_t* __restrict__ keys, int64_t n_max, const int64_t* n_dev,
                                                       int64_t num_dst, int64_t* indptr) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t d = (int64_t)blockIdx.x * BLOCK + threadIdx.x; d <= num_dst; d += (int64_t)gridDim.x * BLOCK) {
        const uint64_t key = (uint64_t)d ^ SIGN;
        int64_t lo = 0, hi = n;
        while (lo < hi) {
            const int64_t mid = lo + ((hi - lo) >> 1);
            if (keys[mid] < key) lo = mid + 1; else hi = mid;
        }
        indptr[d] = lo;
    }
}

__global__ __launch_bounds__(BLOCK) void copy_perm_kernel(const int64_t* __restrict__ src, int64_t n_max, const int64_t* n_dev,
                                                          int64_t* dst) {
    const int64_t n = live_count(n_dev, n_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) dst[i] = src[i];
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_unique_pairs_workspace_bytes(int64_t N_max) { return pair_ws_bytes(N_max < 0 ? 0 : N_max); }

extern "C" int32_t sgl_unique_pairs(const int64_t* ids, const int64_t* ts, int64_t N_max, const int64_t* N_dev,
                                    int64_t* uniq_ids, int64_t* uniq_ts, int64_t* inverse, int64_t* U_dev, void* ws,
                                    size_t ws_bytes, void* stream) {
    if (N_max < 0) return fail(SGL_EINVAL, "unique_pairs: N_max < 0");
    if (!U_dev || (N_max > 0 && (!ids || !ts || !uniq_ids || !uniq_ts || !inverse)))
        return fail(SGL_EINVAL, "unique_pairs: NULL array");
    hipStream_t st = as_stream(stream);
    if (N_max == 0) {
        hipLaunchKernelGGL(zero_total_kernel, dim3(1), dim3(1), 0, st, U_dev);
        SGL_LAUNCH_CHECK();
        return SGL_OK;
    }
    PairWs w;
    if (!ws || ws_bytes < pair_ws_bytes(N_max) || !carve(ws, ws_bytes, N_max, &w))
        return fail(SGL_ENOMEM, "unique_pairs: workspace %zu < %zu bytes", ws_bytes, pair_ws_bytes(N_max));
    uint64_t* keys; int64_t* perm;
    int32_t rc = sort_two_keys(ids, 64, ts, N_max, N_dev, w, &keys, &perm, st);
    if (rc != SGL_OK) return rc;
    hipLaunchKernelGGL(pair_heads_kernel, dim3(grid_for(N_max)), dim3(BLOCK), 0, st, keys, perm, ts, N_max, N_dev, w.head);
    SGL_LAUNCH_CHECK();
    // entries of the flag array beyond the live length are never read back
    if ((rc = exclusive_scan_i64(w.head, w.head, N_max, nullptr, w.scan_ws, w.scan_ws_bytes, st)) != SGL_OK) return rc;
    hipLaunchKernelGGL(zero_total_kernel, dim3(1), dim3(1), 0, st, U_dev);   // stays 0 when the live length is 0
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(pair_emit_kernel, dim3(grid_for(N_max)), dim3(BLOCK), 0, st, keys, perm, ts, w.head, N_max, N_dev,
                       uniq_ids, uniq_ts, inverse, U_dev);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" size_t sgl_csc_from_pairs_workspace_bytes(int64_t E_max) { return pair_ws_bytes(E_max < 0 ? 0 : E_max); }

extern "C" int32_t sgl_csc_from_pairs(const int64_t* dst_local, const int64_t* ts, int64_t E_max, const int64_t* E_dev,
                                      int64_t num_dst, int64_t* indptr, int64_t* perm_out, void* ws, size_t ws_bytes,
                                      void* stream) {
    if (E_max < 0 || num_dst < 0) return fail(SGL_EINVAL, "csc_from_pairs: negative size");
    if (!indptr || (E_max > 0 && (!dst_local || !ts || !perm_out))) return fail(SGL_EINVAL, "csc_from_pairs: NULL array");
    hipStream_t st = as_stream(stream);
    PairWs w{};
    uint64_t* keys = nullptr; int64_t* perm = nullptr;
    if (E_max > 0) {
        if (!ws || ws_bytes < pair_ws_bytes(E_max) || !carve(ws, ws_bytes, E_max, &w))
            return fail(SGL_ENOMEM, "csc_from_pairs: workspace %zu < %zu bytes", ws_bytes, pair_ws_bytes(E_max));
        int bits = 8;
        while (bits < 64 && (num_dst >> bits) != 0) bits += 8;
        int32_t rc = sort_two_keys(dst_local, bits, ts, E_max, E_dev, w, &keys, &perm, st);
        if (rc != SGL_OK) return rc;
        hipLaunchKernelGGL(copy_perm_kernel, dim3(grid_for(E_max)), dim3(BLOCK), 0, st, perm, E_max, E_dev, perm_out);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(indptr_kernel, dim3(grid_for(num_dst + 1)), dim3(BLOCK), 0, st, keys, E_max, E_dev, num_dst, indptr);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
