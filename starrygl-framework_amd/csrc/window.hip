// Whole-window sampling for gfx950: every edge of a slot's time window, or the first k of them,
// optionally only the edges that carry a given tag (the event's cluster id).
//
// These are the layer types of the reference's offline sampler that the k-hop sampler does not cover
// (_jit_sample_kernel, prepare_sample.py:32-172): 'full' and 'cluster' of a continuous-time graph (all
// edges before the cut), and the discrete-time branch ('uniform' = the first `fanout` edges of the
// snapshot window, 'full' = all of them, 'cluster' = those of one cluster; the edge time reported is the
// target's).  The result has no a-priori bound, so a call is made twice: without neighbour arrays it only
// counts (root_*_ptr and counts are written), then the caller allocates counts[1] edges and calls again.
//
// One wavefront per slot: lane 0 finds the window with two binary searches, the lanes stride over it.
// Without a tag the count is the window length; with one, matches are counted by ballot and, in the fill
// pass, placed in storage order by a running popcount.
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int SPB = BLOCK / WAVE;     // slots per block
constexpr int MAX_GRID = 8192;

struct WinArgs {
    sgl_tcsr g;
    const int64_t* slot_node;
    const int64_t* slot_ts;
    int64_t S;
    sgl_window_params p;
    int64_t* cnt;        // [S] edges taken per slot
    int64_t* off;        // [S] their exclusive prefix
    int64_t* total;      // [1]
    unsigned long long* bad;   // [1] slots whose node is outside [0,n)
    sgl_hop_out out;
};

__device__ __forceinline__ int64_t lower_bound(const int64_t* __restrict__ ts, int64_t lo, int64_t hi, int64_t key) {
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (ts[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// window [lo, hi) of slot s, found by lane 0 and broadcast; false for a node outside [0,n)
__device__ __forceinline__ bool window_of(const WinArgs& a, int64_t s, int lane, int64_t* lo_out, int64_t* hi_out, int64_t* t_out) {
    int64_t lo = 0, hi = 0, t = 0;
    int ok = 0;
    if (lane == 0) {
        const int64_t v = a.slot_node[s];
        t = a.slot_ts[s];
        if (v >= 0 && v < a.g.n) {
            ok = 1;
            const int64_t rs = a.g.row_ptr[v], re = a.g.row_ptr[v + 1];
            hi = lower_bound(a.g.ts, rs, re, t + a.p.hi_offset);
            lo = a.p.bounded_below ? lower_bound(a.g.ts, rs, hi, t + a.p.lo_offset) : rs;
            if (lo > hi) lo = hi;
        }
    }
    *lo_out = shfl_i64(lo, 0);
    *hi_out = shfl_i64(hi, 0);
    *t_out = shfl_i64(t, 0);
    return __shfl(ok, 0) != 0;
}

__global__ void window_prep_kernel(WinArgs a) { *a.bad = 0ull; }

__global__ __launch_bounds__(BLOCK) void window_count_kernel(WinArgs a) {
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    for (int64_t s = (int64_t)blockIdx.x * SPB + wid; s < a.S; s += (int64_t)gridDim.x * SPB) {
        int64_t lo, hi, t;
        const bool ok = window_of(a, s, lane, &lo, &hi, &t);
        int64_t c = hi - lo;
        if (a.p.edge_tag != nullptr) {
            c = 0;
            for (int64_t e0 = lo; e0 < hi; e0 += WAVE) {
                const int64_t e = e0 + lane;
                c += __popcll(__ballot(e < hi && a.p.edge_tag[e] == a.p.tag_value));
            }
        }
        if (a.p.first_k >= 0 && c > a.p.first_k) c = a.p.first_k;
        if (lane == 0) {
            a.cnt[s] = ok ? c : 0;
            if (!ok) atomicAdd(a.bad, 1ull);
        }
    }
}

__global__ void window_publish_kernel(WinArgs a) {
    a.out.counts[0] = a.S;
    a.out.counts[1] = *a.total;
    a.out.counts[2] = (int64_t)*a.bad;
    a.out.root_start_ptr[a.S] = *a.total;
    a.out.root_end_ptr[a.S] = *a.total;
}

// FILL: also copy the edges (second call); otherwise only the pointer arrays are written
template <bool FILL>
__global__ __launch_bounds__(BLOCK) void window_fill_kernel(WinArgs a) {
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    for (int64_t s = (int64_t)blockIdx.x * SPB + wid; s < a.S; s += (int64_t)gridDim.x * SPB) {
        const int64_t off = a.off[s], c = a.cnt[s];
        if (lane == 0) {
            a.out.root_start_ptr[s] = off;
            a.out.root_end_ptr[s] = off + c;
        }
        if (!FILL || c == 0) continue;
        if (off + c > a.out.capacity_edges) {     // the caller's arrays are smaller than the count says: void result
            if (lane == 0) atomicMax(reinterpret_cast<long long*>(&a.out.counts[2]), (long long)INT64_MAX);
            continue;
        }
        int64_t lo, hi, t;
        window_of(a, s, lane, &lo, &hi, &t);
        auto emit = [&](int64_t e, int64_t place) {
            const int64_t ets = a.g.ts[e];
            a.out.neighbors[off + place] = a.g.col[e];
            a.out.neighbors_ts[off + place] = a.p.keep_slot_time ? t : ets;
            a.out.neighbors_eid[off + place] = a.g.eid[e];
            a.out.neighbors_dt[off + place] = ets - t;
        };
        if (a.p.edge_tag == nullptr) {
            for (int64_t j = lane; j < c; j += WAVE) emit(lo + j, j);
        } else {
            int64_t placed = 0;
            for (int64_t e0 = lo; e0 < hi && placed < c; e0 += WAVE) {
                const int64_t e = e0 + lane;
                const bool hit = e < hi && a.p.edge_tag[e] == a.p.tag_value;
                const uint64_t m = __ballot(hit);
                const int64_t place = placed + __popcll(m & ((lane == 0) ? 0ull : (~0ull >> (64 - lane))));
                if (hit && place < c) emit(e, place);
                placed += __popcll(m);
            }
        }
    }
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_sample_window_workspace_bytes(int64_t S) {
    const int64_t s = S < 0 ? 0 : S;
    return 2 * align_up((size_t)(s + 1) * 8) + exclusive_scan_workspace_bytes(s) + 1024;
}

extern "C" int32_t sgl_sample_window(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts, int64_t S,
                                     const sgl_window_params* p, const sgl_hop_out* out, void* ws, size_t ws_bytes,
                                     void* stream) {
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr || (g->m > 0 && (!g->col || !g->ts || !g->eid)))
        return fail(SGL_EINVAL, "sample_window: graph is NULL or incomplete");
    if (!p || !out) return fail(SGL_EINVAL, "sample_window: params/out is NULL");
    if (S < 0) return fail(SGL_EINVAL, "sample_window: S < 0");
    if (S > 0 && (!slot_node || !slot_ts)) return fail(SGL_EINVAL, "sample_window: slot array is NULL");
    if (out->capacity_slots < S || !out->root_start_ptr || !out->root_end_ptr || !out->counts)
        return fail(SGL_EINVAL, "sample_window: pointer arrays / counts missing or shorter than S + 1");
    const bool fill = out->neighbors != nullptr;
    if (fill && (!out->neighbors_ts || !out->neighbors_eid || !out->neighbors_dt || out->capacity_edges < 0))
        return fail(SGL_EINVAL, "sample_window: neighbour arrays incomplete");
    if (!ws || ws_bytes < sgl_sample_window_workspace_bytes(S))
        return fail(SGL_ENOMEM, "sample_window: workspace %zu < %zu bytes", ws_bytes, sgl_sample_window_workspace_bytes(S));
    Arena ar(ws, ws_bytes);
    WinArgs a{};
    a.g = *g; a.slot_node = slot_node; a.slot_ts = slot_ts; a.S = S; a.p = *p; a.out = *out;
    a.cnt = ar.take<int64_t>(S + 1);
    a.off = ar.take<int64_t>(S + 1);
    a.total = ar.take<int64_t>(1);
    a.bad = reinterpret_cast<unsigned long long*>(ar.take<int64_t>(1));
    const size_t scan_bytes = exclusive_scan_workspace_bytes(S);
    void* scan_ws = ar.take<char>(scan_bytes);
    if (!ar.ok()) return fail(SGL_ENOMEM, "sample_window: workspace too small");
    hipStream_t st = as_stream(stream);
    int64_t blocks = ceil_div<int64_t>(S > 0 ? S : 1, SPB);
    if (blocks > MAX_GRID) blocks = MAX_GRID;
    hipLaunchKernelGGL(window_prep_kernel, dim3(1), dim3(1), 0, st, a);
    SGL_LAUNCH_CHECK();
    if (S > 0) {
        hipLaunchKernelGGL(window_count_kernel, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
        SGL_LAUNCH_CHECK();
    }
    const int32_t rc = exclusive_scan_i64(a.cnt, a.off, S, a.total, scan_ws, scan_bytes, st);
    if (rc != SGL_OK) return rc;
    hipLaunchKernelGGL(window_publish_kernel, dim3(1), dim3(1), 0, st, a);
    SGL_LAUNCH_CHECK();
    if (S > 0) {
        if (fill) hipLaunchKernelGGL(window_fill_kernel<true>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
        else hipLaunchKernelGGL(window_fill_kernel<false>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
        SGL_LAUNCH_CHECK();
    }
    return SGL_OK;
}
