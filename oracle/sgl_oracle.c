/*
 * sgl_oracle.c -- CPU restatement of StarryGL's temporal mini-batch hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP library is
 * compared against and the CPU baseline the benchmark times; nothing in the
 * shipped library links, loads or falls back to it.
 *
 * Every function mirrors one entry point of include/sgl_hot.h (prefix `sglo_`
 * instead of `sgl_`), takes HOST pointers, ignores `stream` and `workspace`,
 * and follows the reference source cited above it (paths relative to the
 * StarryGL tree).  Where the reference disagrees with itself the rule that is
 * implemented is written next to the citation.
 *
 * What pins each function (tests/test_oracle.py, tests/test_facade_cpu.py):
 *   window / recent      np.searchsorted + brute-force list comprehension
 *   next-hop index,      np.searchsorted(side='left') on the row slice, a
 *   window ends          brute-force count of the row's earlier edges
 *   uniform              Philox4x32-10 known-answer vectors (Random123),
 *                        subset invariants, chi-square over seeds
 *   unique               np.unique(return_inverse), np.setdiff1d per group
 *   gather / scatter     numpy fancy indexing
 *   time encode          float64 closed form
 *   t-csr build          np.lexsort((eid, ts, src)) + bincount/cumsum
 *   seeds / block /      brute-force python loops on tiny graphs,
 *   slice / chunk index  np.argsort(kind='stable')
 *   pair unique / CSC    np.unique over (id, ts) records, np.lexsort((ts, dst))
 *   latest event / node  per-key maximum and first arg-maximum in numpy
 *
 * Build:  make -C oracle      (gcc -O2 -fopenmp -ffp-contract=off)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "../include/sgl_hot.h"

static __thread char g_err[256];
static int g_threads = 1;

static int32_t fail(int32_t code, const char* msg) {
    snprintf(g_err, sizeof g_err, "%s", msg);
    return code;
}

const char* sglo_last_error_string(void) { return g_err; }
int32_t     sglo_abi_version(void) { return SGL_ABI_VERSION; }
size_t      sglo_struct_bytes(int32_t which) {
    switch (which) {
        case 0: return sizeof(sgl_tcsr);
        case 1: return sizeof(sgl_sample_params);
        case 2: return sizeof(sgl_hop_out);
        case 3: return sizeof(sgl_cache);
        case 4: return sizeof(sgl_gather_seg);
        case 5: return sizeof(sgl_seed_query);
        case 6: return sizeof(sgl_window_params);
        default: return 0;
    }
}

/* The oracle has no kernels that wait for each other: the limit is kept and returned only. */
static int32_t g_wait_limit = 1 << 20;
int32_t sglo_set_wait_limit(int32_t polls) {
    int32_t prev = g_wait_limit;
    g_wait_limit = polls > 0 ? polls : (1 << 20);
    return prev;
}

/* Number of OpenMP threads the sampler loops use (1 = the scalar port).  The
 * reference runs its sampler loops under numba.prange
 * (prepare_sample.py:31,44,91) / at::parallel_for (graph.cpu.hpp:270,293). */
void sglo_set_num_threads(int32_t t) { g_threads = t < 1 ? 1 : t; }
int32_t sglo_get_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ T-CSR */

typedef struct { int64_t src, ts, eid, dst; } edge_rec;

static int edge_cmp(const void* a, const void* b) {
    const edge_rec* x = (const edge_rec*)a;
    const edge_rec* y = (const edge_rec*)b;
    if (x->src != y->src) return x->src < y->src ? -1 : 1;
    if (x->ts != y->ts) return x->ts < y->ts ? -1 : 1;
    if (x->eid != y->eid) return x->eid < y->eid ? -1 : 1;
    return 0;
}

size_t sglo_tcsr_build_workspace_bytes(int64_t n, int64_t m) {
    (void)n; (void)m;
    return 0;
}

/* T-CSR build.  Reference: Graph::Graph sorts Edge records with
 * EdgeComparator and scatters them (sample.cu.hpp:51-63, 985-1185); the CPU
 * twin sorts with np.lexsort((ts, dst)) keyed by the row node
 * (prepare_sample.py:192-203).  Rule implemented: rows by source node,
 * inside a row ascending (ts, eid); row_ptr = cumsum(bincount(src)). */
int32_t sglo_tcsr_build(int64_t n, int64_t m, const int64_t* src,
                        const int64_t* dst, const int64_t* ts,
                        const int64_t* eid, int64_t* row_ptr, int64_t* col,
                        int64_t* col_ts, int64_t* col_eid, void* ws,
                        size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (n < 0 || m < 0 || !row_ptr) return fail(SGL_EINVAL, "tcsr_build: bad sizes");
    if (m > 0 && (!src || !dst || !ts || !col || !col_ts || !col_eid))
        return fail(SGL_EINVAL, "tcsr_build: null array");
    for (int64_t i = 0; i < m; ++i)
        if (src[i] < 0 || src[i] >= n || dst[i] < 0 || dst[i] >= n)
            return fail(SGL_ERANGE, "tcsr_build: src/dst outside [0,n)");
    edge_rec* e = (edge_rec*)malloc((size_t)(m > 0 ? m : 1) * sizeof *e);
    if (!e) return fail(SGL_ENOMEM, "tcsr_build: malloc");
    for (int64_t i = 0; i < m; ++i) {
        e[i].src = src[i]; e[i].ts = ts[i];
        e[i].eid = eid ? eid[i] : i; e[i].dst = dst[i];
    }
    qsort(e, (size_t)m, sizeof *e, edge_cmp);
    memset(row_ptr, 0, (size_t)(n + 1) * sizeof(int64_t));
    for (int64_t i = 0; i < m; ++i) {
        row_ptr[e[i].src + 1]++;
        col[i] = e[i].dst; col_ts[i] = e[i].ts; col_eid[i] = e[i].eid;
    }
    for (int64_t v = 0; v < n; ++v) row_ptr[v + 1] += row_ptr[v];
    free(e);
    return SGL_OK;
}

int32_t sglo_tcsr_validate(const sgl_tcsr* g, void* ws, size_t ws_bytes,
                           void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "tcsr_validate: null");
    if (g->row_ptr[0] != 0 || g->row_ptr[g->n] != g->m)
        return fail(SGL_ERANGE, "tcsr_validate: row_ptr ends");
    for (int64_t v = 0; v < g->n; ++v) {
        int64_t a = g->row_ptr[v], b = g->row_ptr[v + 1];
        if (b < a) return fail(SGL_ERANGE, "tcsr_validate: row_ptr not monotone");
        for (int64_t e = a; e < b; ++e) {
            if (g->col[e] < 0 || g->col[e] >= g->n)
                return fail(SGL_ERANGE, "tcsr_validate: col outside [0,n)");
            if (e > a && g->ts[e] < g->ts[e - 1])
                return fail(SGL_ERANGE, "tcsr_validate: ts not ascending in row");
        }
    }
    return SGL_OK;
}

/* --------------------------------------------------------------- sampling */

/* first index in [lo,hi) whose ts >= key (np.searchsorted side='left',
 * prepare_sample.py:50-51; std::lower_bound, graph.cpu.hpp:301). */
static int64_t lower_bound_ts(const int64_t* ts, int64_t lo, int64_t hi, int64_t key) {
    while (lo < hi) {
        int64_t mid = lo + ((hi - lo) >> 1);
        if (ts[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

/* The next-hop index is an accelerator of the kernels; the oracle samples by
 * searching (hop_hint of the graph is ignored) and only restates the index's
 * definition so that the built array can be checked. */
int32_t sglo_tcsr_hop_hint_build(const sgl_tcsr* g, int64_t* hop_hint, void* stream) {
    (void)stream;
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "tcsr_hop_hint_build: null");
    if (g->m > 0 && (!g->col || !g->ts || !hop_hint)) return fail(SGL_EINVAL, "tcsr_hop_hint_build: null array");
    for (int64_t e = 0; e < g->m; ++e) {
        int64_t v = g->col[e], p = -1;
        if (v >= 0 && v < g->n) p = lower_bound_ts(g->ts, g->row_ptr[v], g->row_ptr[v + 1], g->ts[e]);
        hop_hint[e] = p;
    }
    return SGL_OK;
}

/* The interleaved records are an accelerator of the kernels as well: the oracle samples from the
 * separate arrays and only restates the layout so that the built array can be checked.  Fourth field: the
 * edge's next-hop index entry p (bits 0..39) with the length of the window it ends, p - row_ptr[col[e]], as
 * length + 1 in bits 40..62 (saturating at 2^23 - 1; 0 = not recorded: graphs beyond 2^40 edges, destinations
 * outside [0, n)); -1 without the index. */
int32_t sglo_tcsr_records_build(const sgl_tcsr* g, int64_t* rec, void* stream) {
    (void)stream;
    if (!g || g->n < 0 || g->m < 0) return fail(SGL_EINVAL, "tcsr_records_build: null");
    if (g->m > 0 && (!g->col || !g->ts || !g->eid || !rec || (g->hop_hint && !g->row_ptr)))
        return fail(SGL_EINVAL, "tcsr_records_build: null array");
    const int64_t pos_mask = (1ll << 40) - 1, sat = (1ll << 23) - 1;
    for (int64_t e = 0; e < g->m; ++e) {
        rec[4 * e] = g->col[e]; rec[4 * e + 1] = g->ts[e]; rec[4 * e + 2] = g->eid[e];
        int64_t h = g->hop_hint ? g->hop_hint[e] : -1;
        const int64_t v = g->col[e];
        if (h >= 0 && g->m <= pos_mask && v >= 0 && v < g->n) {
            const int64_t len = h - g->row_ptr[v];
            if (len >= 0) h |= (len + 1 < sat ? len + 1 : sat) << 40;
        }
        rec[4 * e + 3] = h;
    }
    return SGL_OK;
}

/* Where the strictly-before window of (node[i], t[i]) ends: the upper end of
 * find_time_range (sample.cu.hpp:264-295) for a batch of slots. */
int32_t sglo_window_end(const sgl_tcsr* g, const int64_t* node, const int64_t* t, int64_t N, int64_t* out,
                        void* stream) {
    (void)stream;
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr || N < 0) return fail(SGL_EINVAL, "window_end: null/negative");
    if (N > 0 && (!node || !t || !out || (g->m > 0 && !g->ts))) return fail(SGL_EINVAL, "window_end: null array");
    for (int64_t i = 0; i < N; ++i) {
        int64_t v = node[i];
        out[i] = (v >= 0 && v < g->n) ? lower_bound_ts(g->ts, g->row_ptr[v], g->row_ptr[v + 1], t[i]) : -1;
    }
    return SGL_OK;
}

/* Candidate window of a slot.  Reference: find_time_range
 * (sample.cu.hpp:264-295) called with (ts - allowed_offset or 0,
 * ts + equal_root_time) at :723-724; numba cut_idx/start_idx
 * (prepare_sample.py:50-55).  Rule implemented: strictly before t unless
 * equal_root_time, lower bound only when allowed_offset >= 0. */
static void window(const sgl_tcsr* g, int64_t v, int64_t t, int64_t allowed_offset,
                   int32_t equal_root_time, int64_t* lo_out, int64_t* hi_out) {
    int64_t rs = g->row_ptr[v], re = g->row_ptr[v + 1];
    int64_t t_hi = t + (equal_root_time ? 1 : 0);
    int64_t hi = lower_bound_ts(g->ts, rs, re, t_hi);
    int64_t lo = rs;
    if (allowed_offset >= 0) lo = lower_bound_ts(g->ts, rs, re, t - allowed_offset);
    if (lo > hi) lo = hi;
    *lo_out = lo; *hi_out = hi;
}

/* Philox4x32-10 (Salmon et al., SC'11; Random123 v1.x philox.h).  Replaces
 * curand_init(1317, threadIdx.x, 0) + curand_uniform (sample.cu.hpp:791-816)
 * with a counter-based generator so that a draw depends only on
 * (seed, hop, slot, draw index). */
static void philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

void sglo_philox4x32_10(const uint32_t* ctr, const uint32_t* key, uint32_t* out) {
    philox4x32_10(ctr, key, out);
}

/* 64 random bits of draw j of slot s in hop h: counter = (j, s_lo, s_hi, h),
 * key = (seed_lo, seed_hi); bits = x0 | x1 << 32. */
static uint64_t draw_bits(uint64_t seed, int32_t hop, int64_t slot, int32_t j) {
    uint32_t ctr[4] = {(uint32_t)j, (uint32_t)((uint64_t)slot & 0xFFFFFFFFu),
                       (uint32_t)((uint64_t)slot >> 32), (uint32_t)hop};
    uint32_t key[2] = {(uint32_t)(seed & 0xFFFFFFFFu), (uint32_t)(seed >> 32)};
    uint32_t x[4];
    philox4x32_10(ctr, key, x);
    return (uint64_t)x[0] | ((uint64_t)x[1] << 32);
}

/* floor(bits * range / 2^64): a value in [0, range). */
static int64_t bounded(uint64_t bits, int64_t range) {
    return (int64_t)(((unsigned __int128)bits * (uint64_t)range) >> 64);
}

uint64_t sglo_draw_bits(uint64_t seed, int32_t hop, int64_t slot, int32_t j) {
    return draw_bits(seed, hop, slot, j);
}
int64_t sglo_bounded(uint64_t bits, int64_t range) { return bounded(bits, range); }

/* k distinct offsets in [0,cnt), ascending (Floyd's subset sampling; the
 * reference draws np.random.choice(cut_idx, fanout, replace=False) then
 * sorts, prepare_sample.py:124-125). */
static void floyd_subset(uint64_t seed, int32_t hop, int64_t slot, int64_t cnt,
                         int32_t k, int64_t* sel) {
    for (int32_t j = 0; j < k; ++j) {
        int64_t i = cnt - k + j;
        int64_t t = bounded(draw_bits(seed, hop, slot, j), i + 1);
        int dup = 0;
        for (int32_t q = 0; q < j; ++q) if (sel[q] == t) { dup = 1; break; }
        sel[j] = dup ? i : t;
    }
    for (int32_t a = 1; a < k; ++a) { /* insertion sort, k is small */
        int64_t x = sel[a]; int32_t b = a - 1;
        while (b >= 0 && sel[b] > x) { sel[b + 1] = sel[b]; --b; }
        sel[b + 1] = x;
    }
}

size_t sglo_sample_hop_workspace_bytes(int64_t S_max) { (void)S_max; return 0; }


/* One hop: count pass -> prefix sum -> fill pass, parallel over slots.
 * Reference: _jit_sample_kernel (prepare_sample.py:43-78 count, :80-82
 * prefix, :91-145 fill; recent :117-119, uniform :120-134);
 * static_recent_neighbor_num / recent_sample_single_hop_kernel and
 * static_neighbor_num / uniform_sample_single_hop_kernel
 * (sample.cu.hpp:706-827); sample_kernel (graph.cpu.hpp:256-310). */
/* slot_hint / hint_out: only for the indexed CPU baseline (sglo_sample_khop_indexed below).  slot_hint[s] >= 0
 * is taken as the end of slot s's strictly-before window instead of searching for it; hint_out receives the
 * graph's next-hop index entry of every emitted edge. */
static int32_t hop_impl(const sgl_tcsr* g, const int64_t* slot_node,
                        const int64_t* slot_ts, int64_t S_max,
                        const int64_t* S_dev, const sgl_sample_params* p,
                        const sgl_hop_out* out, const int64_t* slot_hint, int64_t* hint_out) {
    if (!g || !p || !out || S_max < 0) return fail(SGL_EINVAL, "sample_hop: null/negative");
    if (p->type != SGL_SAMPLE_RECENT && p->type != SGL_SAMPLE_UNIFORM)
        return fail(SGL_ENOTSUP, "undefined sampling strategy");
    if (p->fanout < 0) return fail(SGL_EINVAL, "sample_hop: fanout < 0");
    if (p->type == SGL_SAMPLE_UNIFORM && p->fanout > SGL_UNIFORM_MAX_FANOUT)
        return fail(SGL_ENOTSUP, "uniform fanout > SGL_UNIFORM_MAX_FANOUT");
    if (p->type == SGL_SAMPLE_RECENT && p->fanout > SGL_RECENT_MAX_FANOUT)
        return fail(SGL_ENOTSUP, "recent fanout > SGL_RECENT_MAX_FANOUT");
    int64_t S = S_dev ? *S_dev : S_max;
    if (S > S_max || S > out->capacity_slots) return fail(SGL_ENOMEM, "sample_hop: slots > capacity");
    if (out->capacity_edges < out->capacity_slots * (int64_t)p->fanout)
        return fail(SGL_ENOMEM, "sample_hop: capacity_edges < capacity_slots*fanout");
    const int32_t k = p->fanout;
    int64_t* cnt = (int64_t*)malloc((size_t)(S + 1) * sizeof(int64_t));
    int64_t* wlo = (int64_t*)malloc((size_t)(S + 1) * sizeof(int64_t));
    int64_t* whi = (int64_t*)malloc((size_t)(S + 1) * sizeof(int64_t));
    if (!cnt || !wlo || !whi) { free(cnt); free(wlo); free(whi); return fail(SGL_ENOMEM, "malloc"); }
    int64_t bad = 0;
    /* pass 1: count */
#pragma omp parallel for schedule(dynamic, 256) num_threads(g_threads) reduction(+ : bad)
    for (int64_t s = 0; s < S; ++s) {
        int64_t v = slot_node[s];
        if (v < 0 || v >= g->n) { cnt[s] = 0; wlo[s] = whi[s] = 0; bad++; continue; }
        int64_t lo, hi;
        if (slot_hint && slot_hint[s] >= 0 && !p->equal_root_time) {
            const int64_t rs = g->row_ptr[v], re = g->row_ptr[v + 1];
            hi = slot_hint[s] < rs ? rs : (slot_hint[s] > re ? re : slot_hint[s]);
            lo = rs;
            if (p->allowed_offset >= 0) lo = lower_bound_ts(g->ts, rs, hi, slot_ts[s] - p->allowed_offset);
        } else {
            window(g, v, slot_ts[s], p->allowed_offset, p->equal_root_time, &lo, &hi);
        }
        wlo[s] = lo; whi[s] = hi;
        int64_t c = hi - lo;
        cnt[s] = c < k ? c : k;
    }
    /* prefix */
    int64_t acc = 0;
    for (int64_t s = 0; s < S; ++s) { out->root_start_ptr[s] = acc; acc += cnt[s]; out->root_end_ptr[s] = acc; }
    out->root_start_ptr[S] = acc; out->root_end_ptr[S] = acc;
    /* pass 2: fill */
#pragma omp parallel for schedule(dynamic, 256) num_threads(g_threads)
    for (int64_t s = 0; s < S; ++s) {
        int64_t c = cnt[s];
        if (c == 0) continue;
        int64_t off = out->root_start_ptr[s], t = slot_ts[s];
        int64_t lo = wlo[s], hi = whi[s], len = hi - lo;
        if (p->type == SGL_SAMPLE_RECENT || len <= k) {
            int64_t b = (p->type == SGL_SAMPLE_RECENT) ? hi - c : lo;
            for (int64_t j = 0; j < c; ++j) {
                int64_t e = b + j;
                out->neighbors[off + j] = g->col[e];
                out->neighbors_ts[off + j] =
                    (p->type == SGL_SAMPLE_UNIFORM && p->keep_root_time) ? t : g->ts[e];
                out->neighbors_eid[off + j] = g->eid[e];
                out->neighbors_dt[off + j] = g->ts[e] - t;
                if (hint_out) hint_out[off + j] = g->hop_hint[e];
            }
        } else {
            int64_t sel[SGL_UNIFORM_MAX_FANOUT];      /* 8 KB of stack per thread */
            if (p->replace) {
                for (int32_t j = 0; j < k; ++j)
                    sel[j] = bounded(draw_bits(p->seed, p->hop, s, j), len);
            } else {
                floyd_subset(p->seed, p->hop, s, len, k, sel);
            }
            for (int32_t j = 0; j < k; ++j) {
                int64_t e = lo + sel[j];
                out->neighbors[off + j] = g->col[e];
                out->neighbors_ts[off + j] = p->keep_root_time ? t : g->ts[e];
                out->neighbors_eid[off + j] = g->eid[e];
                out->neighbors_dt[off + j] = g->ts[e] - t;
                if (hint_out) hint_out[off + j] = g->hop_hint[e];
            }
        }
    }
    out->counts[0] = S; out->counts[1] = acc; out->counts[2] = bad;
    free(cnt); free(wlo); free(whi);
    return SGL_OK;
}

int32_t sglo_sample_hop(const sgl_tcsr* g, const int64_t* slot_node,
                        const int64_t* slot_ts, int64_t S_max,
                        const int64_t* S_dev, const sgl_sample_params* p,
                        const sgl_hop_out* out, void* ws, size_t ws_bytes,
                        void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    return hop_impl(g, slot_node, slot_ts, S_max, S_dev, p, out, NULL, NULL);
}

/* The workspace-free variant of the hop: the oracle never uses a workspace, so
 * it is the same function (kept so that the oracle mirrors every entry point of
 * include/sgl_hot.h; it has no counterpart in the reference). */
int32_t sglo_sample_hop_static(const sgl_tcsr* g, const int64_t* slot_node,
                               const int64_t* slot_ts, int64_t S_max,
                               const int64_t* S_dev, const sgl_sample_params* p,
                               const sgl_hop_out* out, void* stream) {
    if (S_max > SGL_STATIC_HOP_MAX_SLOTS) return fail(SGL_ENOMEM, "sample_hop_static: slots exceed the limit");
    return sglo_sample_hop(g, slot_node, slot_ts, S_max, S_dev, p, out, NULL, 0, stream);
}


/* Whole-window sampling.  Reference: _jit_sample_kernel (prepare_sample.py:32-172): cut_idx / start_idx
 * = np.searchsorted (side='left') of t + end_offset / t + start_offset on the target's time-sorted edges
 * (:50-55), 'cluster' and 'full' of a continuous graph take [0, cut_idx) (:62, :112-113, :131-132); the
 * discrete branch takes [start_idx, cut_idx): every edge ('full'), the first `fanout` ('uniform', :68-70,
 * :159-170) or the edges of one cluster (:65-67, :148-158), and reports the target's time as the edge time. */
size_t sglo_sample_window_workspace_bytes(int64_t S) { (void)S; return 0; }

int32_t sglo_sample_window(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts, int64_t S,
                           const sgl_window_params* p, const sgl_hop_out* out, void* ws, size_t ws_bytes,
                           void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!g || !p || !out || S < 0) return fail(SGL_EINVAL, "sample_window: null/negative");
    if (out->capacity_slots < S) return fail(SGL_EINVAL, "sample_window: capacity_slots < S");
    const int fill = out->neighbors != NULL;
    int64_t acc = 0, bad = 0, overflow = 0;
    for (int64_t s = 0; s < S; ++s) {
        out->root_start_ptr[s] = acc;
        int64_t v = slot_node[s], t = slot_ts[s];
        if (v < 0 || v >= g->n) { bad++; out->root_end_ptr[s] = acc; continue; }
        int64_t rs = g->row_ptr[v], re = g->row_ptr[v + 1];
        int64_t hi = lower_bound_ts(g->ts, rs, re, t + p->hi_offset);
        int64_t lo = p->bounded_below ? lower_bound_ts(g->ts, rs, hi, t + p->lo_offset) : rs;
        if (lo > hi) lo = hi;
        int64_t taken = 0;
        for (int64_t e = lo; e < hi; ++e) {
            if (p->edge_tag && p->edge_tag[e] != p->tag_value) continue;
            if (p->first_k >= 0 && taken >= p->first_k) break;
            if (fill) {
                if (acc + taken >= out->capacity_edges) { overflow = 1; }
                else {
                    out->neighbors[acc + taken] = g->col[e];
                    out->neighbors_ts[acc + taken] = p->keep_slot_time ? t : g->ts[e];
                    out->neighbors_eid[acc + taken] = g->eid[e];
                    out->neighbors_dt[acc + taken] = g->ts[e] - t;
                }
            }
            taken++;
        }
        acc += taken;
        out->root_end_ptr[s] = acc;
    }
    out->root_start_ptr[S] = acc; out->root_end_ptr[S] = acc;
    out->counts[0] = S; out->counts[1] = acc; out->counts[2] = overflow ? INT64_MAX : bad;
    return SGL_OK;
}

size_t sglo_sample_khop_workspace_bytes(int64_t S0, int32_t layers, int32_t fanout) {
    (void)S0; (void)layers; (void)fanout;
    return 0;
}

/* k-hop driver.  Reference: sample_src_in_chunks_khop
 * (sample.cu.hpp:1532-1716): roots = concat(seeds, negatives) (:1545-1547),
 * next hop roots = neighbors, ts = neighbors_ts, one slot each (:1692-1702). */
int32_t sglo_sample_khop(const sgl_tcsr* g, int64_t R, const int64_t* roots,
                         const int64_t* ts_ptr, int64_t S_pos,
                         const int64_t* root_ts, int64_t N_neg,
                         const int64_t* neg_roots, const int64_t* neg_ts,
                         int32_t layers, const sgl_sample_params* p,
                         int64_t* slot_node0, int64_t* slot_ts0,
                         const sgl_hop_out* outs, void* ws, size_t ws_bytes,
                         void* stream) {
    if (!g || !p || !outs || R < 0 || S_pos < 0 || N_neg < 0 || layers < 1)
        return fail(SGL_EINVAL, "sample_khop: null/negative");
    for (int64_t r = 0; r < R; ++r) {
        if (ts_ptr[r] > ts_ptr[r + 1] || ts_ptr[r] < 0 || ts_ptr[r + 1] > S_pos)
            return fail(SGL_EINVAL, "sample_khop: ts_ptr not a prefix array over root_ts");
        for (int64_t s = ts_ptr[r]; s < ts_ptr[r + 1]; ++s) {
            slot_node0[s] = roots[r]; slot_ts0[s] = root_ts[s];
        }
    }
    if (R > 0 && (ts_ptr[0] != 0 || ts_ptr[R] != S_pos))
        return fail(SGL_EINVAL, "sample_khop: ts_ptr ends");
    for (int64_t i = 0; i < N_neg; ++i) {
        slot_node0[S_pos + i] = neg_roots[i]; slot_ts0[S_pos + i] = neg_ts[i];
    }
    /* root_hint is an accelerator of the kernels: the oracle searches, and as the checker it
     * refuses a hint that is not the window end it finds itself */
    if (p->root_hint && !p->equal_root_time)
        for (int64_t s = 0; s < S_pos; ++s) {
            int64_t v = slot_node0[s], h = p->root_hint[s];
            if (h < 0 || v < 0 || v >= g->n) continue;
            if (h != lower_bound_ts(g->ts, g->row_ptr[v], g->row_ptr[v + 1], slot_ts0[s]))
                return fail(SGL_EINVAL, "sample_khop: a root_hint entry is not the window end");
        }
    const int64_t* sn = slot_node0; const int64_t* st = slot_ts0;
    int64_t S = S_pos + N_neg;
    for (int32_t l = 0; l < layers; ++l) {
        sgl_sample_params pl = *p; pl.hop = l;
        int32_t rc = sglo_sample_hop(g, sn, st, S, NULL, &pl, &outs[l], ws, ws_bytes, stream);
        if (rc != SGL_OK) return rc;
        sn = outs[l].neighbors; st = outs[l].neighbors_ts; S = outs[l].counts[1];
    }
    return SGL_OK;
}

/* The k-hop driver given the same two indexes as the HIP library's fastest route: positive roots
 * take their window end from p->root_hint (negatives are searched), the slots of hops >= 1 from
 * the graph's next-hop index (g->hop_hint) - no search for them.  NOT part of the checker (the
 * oracle proper always searches): this is the CPU side of an equal-work timing, and the tests
 * hold it against sglo_sample_khop on the same inputs.  Same arguments as sglo_sample_khop. */
int32_t sglo_sample_khop_indexed(const sgl_tcsr* g, int64_t R, const int64_t* roots,
                                 const int64_t* ts_ptr, int64_t S_pos,
                                 const int64_t* root_ts, int64_t N_neg,
                                 const int64_t* neg_roots, const int64_t* neg_ts,
                                 int32_t layers, const sgl_sample_params* p,
                                 int64_t* slot_node0, int64_t* slot_ts0,
                                 const sgl_hop_out* outs, void* ws, size_t ws_bytes,
                                 void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!g || !p || !outs || R < 0 || S_pos < 0 || N_neg < 0 || layers < 1)
        return fail(SGL_EINVAL, "sample_khop_indexed: null/negative");
    for (int64_t r = 0; r < R; ++r)
        for (int64_t s = ts_ptr[r]; s < ts_ptr[r + 1]; ++s) { slot_node0[s] = roots[r]; slot_ts0[s] = root_ts[s]; }
    for (int64_t i = 0; i < N_neg; ++i) { slot_node0[S_pos + i] = neg_roots[i]; slot_ts0[S_pos + i] = neg_ts[i]; }
    const int carry = g->hop_hint != NULL && !p->equal_root_time && !(p->type == SGL_SAMPLE_UNIFORM && p->keep_root_time);
    int64_t S = S_pos + N_neg;
    int64_t* hint = (int64_t*)malloc((size_t)(S + 1) * sizeof(int64_t));
    if (!hint) return fail(SGL_ENOMEM, "malloc");
    for (int64_t s = 0; s < S; ++s) hint[s] = (p->root_hint && s < S_pos) ? p->root_hint[s] : -1;
    const int64_t* sn = slot_node0; const int64_t* st = slot_ts0;
    for (int32_t l = 0; l < layers; ++l) {
        sgl_sample_params pl = *p; pl.hop = l;
        int64_t* next = NULL;
        if (carry && l + 1 < layers) {
            next = (int64_t*)malloc((size_t)(S * (int64_t)p->fanout + 1) * sizeof(int64_t));
            if (!next) { free(hint); return fail(SGL_ENOMEM, "malloc"); }
        }
        int32_t rc = hop_impl(g, sn, st, S, NULL, &pl, &outs[l], hint, next);
        free(hint);
        hint = next;
        if (rc != SGL_OK) { free(hint); return rc; }
        sn = outs[l].neighbors; st = outs[l].neighbors_ts; S = outs[l].counts[1];
    }
    free(hint);
    return SGL_OK;
}

/* Several k-hop calls over the same roots: by definition the calls one after
 * the other (the reference submits one query per policy, graph.py:274-293). */
size_t sglo_sample_khop_multi_workspace_bytes(int64_t S0, int32_t layers, int32_t fanout, int32_t Q) {
    (void)S0; (void)layers; (void)fanout; (void)Q;
    return 0;
}

int32_t sglo_sample_khop_multi(const sgl_tcsr* g, int64_t R, const int64_t* roots,
                               const int64_t* ts_ptr, int64_t S_pos,
                               const int64_t* root_ts, int64_t N_neg,
                               const int64_t* neg_roots, const int64_t* neg_ts,
                               int32_t layers, int32_t Q, const sgl_sample_params* p,
                               int64_t* slot_node0, int64_t* slot_ts0,
                               const sgl_hop_out* outs, void* ws, size_t ws_bytes,
                               void* stream) {
    if (Q < 0 || layers < 1 || (Q > 0 && (!p || !outs)))
        return fail(SGL_EINVAL, "sample_khop_multi: bad Q, layers or NULL argument");
    for (int32_t q = 0; q < Q; ++q) {
        int32_t rc = sglo_sample_khop(g, R, roots, ts_ptr, S_pos, root_ts, N_neg, neg_roots, neg_ts,
                                      layers, &p[q], slot_node0, slot_ts0,
                                      outs + (size_t)q * layers, ws, ws_bytes, stream);
        if (rc != SGL_OK) return rc;
    }
    return SGL_OK;
}

/* B mini-batches in one call.  The reference queues one query per window and runs them one after the other
 * (AsyncGraphBlob, graph.py:274-293; submit_query, sample.cu.hpp:1990-2020); by definition the batched call
 * is the k-hop driver (sample.cu.hpp:1532-1716) over the concatenated root slots, plus the table that says
 * where each batch's edges begin in every hop.  slot_hint is an accelerator of the kernels: the oracle
 * searches, and refuses a hint that is not the window end it finds itself. */
size_t sglo_sample_khop_batched_workspace_bytes(int64_t S_max, int32_t layers, int32_t fanout, int32_t Q) {
    (void)S_max; (void)layers; (void)fanout; (void)Q;
    return 0;
}

int32_t sglo_sample_khop_batched(const sgl_tcsr* g, int32_t B, const int64_t* batch_ptr, int64_t S_max,
                                 const int64_t* slot_node, const int64_t* slot_ts, const int64_t* slot_hint,
                                 int32_t layers, int32_t Q, const sgl_sample_params* p, const sgl_hop_out* outs,
                                 int64_t* seg, void* ws, size_t ws_bytes, void* stream) {
    if (!g || B < 1 || !batch_ptr || S_max < 0 || layers < 1 || Q < 1 || !p || !outs || !seg)
        return fail(SGL_EINVAL, "sample_khop_batched: bad argument");
    const int64_t S = batch_ptr[B];
    if (S < 0 || S > S_max) return fail(SGL_EINVAL, "sample_khop_batched: batch_ptr[B] outside [0, S_max]");
    for (int32_t b = 0; b < B; ++b)
        if (batch_ptr[b] < 0 || batch_ptr[b] > batch_ptr[b + 1])
            return fail(SGL_EINVAL, "sample_khop_batched: batch_ptr does not ascend");
    for (int32_t q = 0; q < Q; ++q) {
        if (p[q].mark_state) return fail(SGL_EINVAL, "sample_khop_batched: mark_state is not supported");
        if (slot_hint && !p[q].equal_root_time)
            for (int64_t s = 0; s < S; ++s) {
                int64_t v = slot_node[s], h = slot_hint[s];
                if (h < 0 || v < 0 || v >= g->n) continue;
                if (h != lower_bound_ts(g->ts, g->row_ptr[v], g->row_ptr[v + 1], slot_ts[s]))
                    return fail(SGL_EINVAL, "sample_khop_batched: a slot_hint entry is not the window end");
            }
        const sgl_hop_out* oq = outs + (size_t)q * layers;
        const int64_t* sn = slot_node; const int64_t* st = slot_ts;
        int64_t Sl = S;
        for (int32_t l = 0; l < layers; ++l) {
            sgl_sample_params pl = p[q]; pl.hop = l;
            int32_t rc = sglo_sample_hop(g, sn, st, Sl, NULL, &pl, &oq[l], ws, ws_bytes, stream);
            if (rc != SGL_OK) return rc;
            sn = oq[l].neighbors; st = oq[l].neighbors_ts; Sl = oq[l].counts[1];
        }
        int64_t* sq = seg + (size_t)q * (layers + 1) * (B + 1);
        for (int32_t b = 0; b <= B; ++b) {
            int64_t x = batch_ptr[b];
            sq[b] = x;
            for (int32_t l = 0; l < layers; ++l) {
                x = oq[l].root_start_ptr[x];
                sq[(size_t)(l + 1) * (B + 1) + b] = x;
            }
        }
    }
    return SGL_OK;
}

/* ----------------------------------------------------- unique / compaction */

/* state layout: int64 header[3] = {epoch, id_count, universe}; then
 * int64 table[universe] holding the local id of the current epoch or -1. */
size_t sglo_remap_state_bytes(int64_t universe) {
    return (size_t)(universe + 3) * sizeof(int64_t);
}

int32_t sglo_remap_init(void* state, size_t bytes, int64_t universe, void* stream) {
    (void)stream;
    if (!state || universe < 0 || bytes < sglo_remap_state_bytes(universe))
        return fail(SGL_EINVAL, "remap_init: state too small");
    int64_t* h = (int64_t*)state;
    h[0] = 1; h[1] = 0; h[2] = universe;
    for (int64_t i = 0; i < universe; ++i) h[3 + i] = -1;
    return SGL_OK;
}

static int i64_cmp(const void* a, const void* b) {
    int64_t x = *(const int64_t*)a, y = *(const int64_t*)b;
    return x < y ? -1 : (x > y ? 1 : 0);
}

typedef struct { int64_t id, local; } seen_rec;
static int seen_cmp(const void* a, const void* b) {
    return i64_cmp(&((const seen_rec*)a)->id, &((const seen_rec*)b)->id);
}
static int64_t seen_find(const seen_rec* s, int64_t n, int64_t id) {
    int64_t lo = 0, hi = n;
    while (lo < hi) { int64_t mid = (lo + hi) >> 1; if (s[mid].id < id) lo = mid + 1; else hi = mid; }
    return (lo < n && s[lo].id == id) ? s[lo].local : -1;
}

size_t sglo_unique_workspace_bytes(int64_t universe, int32_t G, const int64_t* len_max) {
    (void)universe; (void)G; (void)len_max;
    return 0;
}

/* unique + compaction.  Reference: Remapper::insert -> remapper per array:
 * mark ids already mapped in this epoch, copy_if the rest, sort, unique,
 * number consecutively from id_counts, scatter into id_mapper, patch
 * (sample.cu.hpp:1764-1852); sorted mode == np.unique(return_inverse=True)
 * (prepare_sample.py:205-213).  Rule implemented for the epoch flag: reset=1
 * restarts numbering, reset=0 continues it (the comment at
 * sample.cu.hpp:1874, and graph.py:291).  Ids that are negative, or outside
 * the state's universe, map to -1 and are never numbered. */
static int32_t unique_core(void* state, int64_t universe_arg, seen_rec* known, int64_t* n_known_io, int64_t known_capacity,
                           int32_t reset, int32_t mode, int32_t G,
                           const int64_t* const* ids, const int64_t* len_max,
                           const int64_t* const* len_dev,
                           int64_t* const* local_out, int64_t* unique_out,
                           int64_t unique_capacity, int64_t* U_dev) {
    if (G < 0 || (G > 0 && (!ids || !len_max || !local_out)) || !U_dev)
        return fail(SGL_EINVAL, "unique_compact: null");
    /* PREMARKED only tells the HIP library that the sampler already did its first pass; the
     * result is defined by the arrays alone, so the restatement just numbers them. */
    mode &= ~SGL_UNIQUE_MULTI_LAUNCH;      /* a launch-structure choice of the HIP library, no meaning here */
    if ((mode & SGL_UNIQUE_PREMARKED) && ((mode & ~SGL_UNIQUE_PREMARKED) != SGL_UNIQUE_SORTED || !reset || !state))
        return fail(SGL_EINVAL, "unique_compact: PREMARKED needs the dense state, SORTED mode and reset = 1");
    mode &= ~SGL_UNIQUE_PREMARKED;
    if (mode != SGL_UNIQUE_SORTED && mode != SGL_UNIQUE_GROUPED)
        return fail(SGL_EINVAL, "unique_compact: bad mode");
    if (!state && !known && !reset) return fail(SGL_ENOTSUP, "unique_compact: hash path needs reset=1");
    int64_t* hdr = (int64_t*)state;
    int64_t* table = state ? hdr + 3 : NULL;
    const int64_t universe = state ? hdr[2] : INT64_MAX;
    if (state && universe_arg != hdr[2]) return fail(SGL_EINVAL, "unique_compact: universe differs from remap_init");
    int64_t total = 0;
    for (int32_t g = 0; g < G; ++g) {
        int64_t L = (len_dev && len_dev[g]) ? *len_dev[g] : len_max[g];
        if (L < 0 || L > len_max[g]) return fail(SGL_EINVAL, "unique_compact: bad length");
        total += L;
    }
    int64_t id_count = 0;
    if (state) {
        if (reset) {
            hdr[0] += 1; hdr[1] = 0;
            for (int64_t i = 0; i < universe; ++i) table[i] = -1;
        }
        id_count = hdr[1];
    }
    /* hashed state: the ids of the epoch so far, sorted by id, with their local ids */
    int64_t n_known = 0;
    if (known) {
        if (reset) *n_known_io = 0;
        n_known = *n_known_io;
        id_count = n_known;
    }
    const int64_t U_before = id_count;
    /* `seen` = ids numbered by this call, kept sorted by id. */
    seen_rec* seen = (seen_rec*)malloc((size_t)(total + 1) * sizeof *seen);
    int64_t n_seen = 0;
    int64_t* tmp = (int64_t*)malloc((size_t)(total + 1) * sizeof(int64_t));
    if (!seen || !tmp) { free(seen); free(tmp); return fail(SGL_ENOMEM, "malloc"); }
    const int32_t n_groups = (mode == SGL_UNIQUE_SORTED) ? 1 : G;
    for (int32_t grp = 0; grp < n_groups; ++grp) {
        int64_t nt = 0;
        for (int32_t g = 0; g < G; ++g) {
            if (mode == SGL_UNIQUE_GROUPED && g != grp) continue;
            int64_t L = (len_dev && len_dev[g]) ? *len_dev[g] : len_max[g];
            for (int64_t i = 0; i < L; ++i) {
                int64_t id = ids[g][i];
                if (id < 0 || id >= universe) continue;
                tmp[nt++] = id;
            }
        }
        qsort(tmp, (size_t)nt, sizeof(int64_t), i64_cmp);
        const int64_t n_prev = n_seen;
        for (int64_t i = 0; i < nt; ++i) {
            if (i > 0 && tmp[i] == tmp[i - 1]) continue;
            int64_t id = tmp[i];
            if (state && table[id] >= 0) continue;            /* earlier call, same epoch */
            if (known && seen_find(known, n_known, id) >= 0) continue;
            if (seen_find(seen, n_prev, id) >= 0) continue;   /* earlier group, this call */
            if (known && id_count >= known_capacity) {       /* the epoch outgrows the hashed state: void result */
                U_dev[0] = INT64_MAX; U_dev[1] = U_before;
                free(seen); free(tmp);
                return SGL_OK;
            }
            if (id_count >= unique_capacity) { free(seen); free(tmp); return fail(SGL_ENOMEM, "unique_out too small"); }
            seen[n_seen].id = id; seen[n_seen].local = id_count; n_seen++;
            unique_out[id_count] = id;
            id_count++;
        }
        qsort(seen, (size_t)n_seen, sizeof *seen, seen_cmp);
    }
    for (int32_t g = 0; g < G; ++g) {
        int64_t L = (len_dev && len_dev[g]) ? *len_dev[g] : len_max[g];
        for (int64_t i = 0; i < L; ++i) {
            int64_t id = ids[g][i];
            int64_t loc = -1;
            if (id >= 0 && id < universe) {
                loc = seen_find(seen, n_seen, id);
                if (loc < 0 && state) loc = table[id];
                if (loc < 0 && known) loc = seen_find(known, n_known, id);
            }
            local_out[g][i] = loc;
        }
    }
    if (state) {
        for (int64_t i = 0; i < n_seen; ++i) table[seen[i].id] = seen[i].local;
        hdr[1] = id_count;
    }
    if (known) {
        for (int64_t i = 0; i < n_seen; ++i) known[n_known + i] = seen[i];
        *n_known_io = n_known + n_seen;
        qsort(known, (size_t)*n_known_io, sizeof *known, seen_cmp);
    }
    U_dev[0] = id_count; U_dev[1] = U_before;
    free(seen); free(tmp);
    return SGL_OK;
}

int32_t sglo_unique_compact(void* state, int64_t universe_arg, int32_t reset, int32_t mode, int32_t G,
                            const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev,
                            int64_t* const* local_out, int64_t* unique_out,
                            int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    return unique_core(state, universe_arg, NULL, NULL, 0, reset, mode, G, ids, len_max, len_dev, local_out,
                       unique_out, unique_capacity, U_dev);
}

/* Hashed state of the oracle: int64 header {capacity, ids of the epoch, void flag}, then the
 * epoch's (id, local id) records sorted by id.  Same numbering rule as above
 * (Remapper::insert, sample.cu.hpp:1825-1852) for ids of any non-negative value. */
size_t sglo_remap_hashed_state_bytes(int64_t capacity) {
    return 3 * sizeof(int64_t) + (size_t)(capacity > 0 ? capacity : 0) * sizeof(seen_rec);
}

int32_t sglo_remap_hashed_init(void* state, size_t bytes, int64_t capacity, void* stream) {
    (void)stream;
    if (!state || capacity < 1 || bytes < sglo_remap_hashed_state_bytes(capacity))
        return fail(SGL_EINVAL, "remap_hashed_init: bad state");
    int64_t* h = (int64_t*)state;
    h[0] = capacity; h[1] = 0; h[2] = 0;
    return SGL_OK;
}

size_t sglo_unique_hashed_workspace_bytes(int64_t capacity, int32_t G, const int64_t* len_max) {
    (void)capacity; (void)G; (void)len_max;
    return 0;
}

int32_t sglo_unique_compact_hashed(void* state, int64_t capacity, int32_t reset, int32_t mode, int32_t G,
                                   const int64_t* const* ids, const int64_t* len_max,
                                   const int64_t* const* len_dev,
                                   int64_t* const* local_out, int64_t* unique_out,
                                   int64_t unique_capacity, int64_t* U_dev, void* ws,
                                   size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!state) return fail(SGL_EINVAL, "unique_compact_hashed: state is NULL");
    int64_t* h = (int64_t*)state;
    if (capacity != h[0]) return fail(SGL_EINVAL, "unique_compact_hashed: capacity differs from remap_hashed_init");
    if (mode & SGL_UNIQUE_PREMARKED) return fail(SGL_EINVAL, "unique_compact_hashed: bad mode");
    int32_t rc = unique_core(NULL, 0, (seen_rec*)(h + 3), &h[1], capacity, reset, mode, G, ids, len_max, len_dev,
                             local_out, unique_out, unique_capacity, U_dev);
    if (rc == SGL_OK && U_dev[0] == INT64_MAX) h[2] = 1;
    if (rc == SGL_OK && h[2]) U_dev[0] = INT64_MAX;      /* sticky */
    return rc;
}

/* B independent unique problems: per batch np.unique(return_inverse) over the batch's slices of the arrays
 * (_get_unique_pairs, prepare_sample.py:205-213; Remapper::insert with a fresh epoch per batch,
 * sample.cu.hpp:1825-1852).  State: int64 header {universe, B}. */
size_t sglo_remap_batched_state_bytes(int64_t universe, int32_t B) {
    if (universe <= 0 || B < 1 || B > SGL_BATCH_MAX) return 0;
    return 2 * sizeof(int64_t);
}

int32_t sglo_remap_batched_init(void* state, size_t bytes, int64_t universe, int32_t B, void* stream) {
    (void)stream;
    if (!state || universe <= 0 || B < 1 || B > SGL_BATCH_MAX || bytes < 2 * sizeof(int64_t))
        return fail(SGL_EINVAL, "remap_batched_init: bad argument");
    ((int64_t*)state)[0] = universe; ((int64_t*)state)[1] = B;
    return SGL_OK;
}

size_t sglo_unique_batched_workspace_bytes(int64_t universe, int32_t B) { (void)universe; (void)B; return 0; }

int32_t sglo_unique_compact_batched(void* state, int64_t universe, int32_t B, int32_t G,
                                    const int64_t* const* ids, const int64_t* len_max,
                                    const int64_t* const* seg, int64_t* const* local_out,
                                    int64_t* unique_out, int64_t unique_capacity, int64_t* U_off,
                                    void* ws, size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!state || G < 1 || !ids || !len_max || !seg || !local_out || !U_off)
        return fail(SGL_EINVAL, "unique_compact_batched: null");
    const int64_t* h = (const int64_t*)state;
    if (h[0] != universe || h[1] != B) return fail(SGL_EINVAL, "unique_compact_batched: universe / B differ from remap_batched_init");
    int64_t total = 0;
    for (int32_t g = 0; g < G; ++g) {
        if (seg[g][B] < 0 || seg[g][B] > len_max[g]) return fail(SGL_EINVAL, "unique_compact_batched: bad live length");
        for (int32_t b = 0; b < B; ++b)
            if (seg[g][b] < 0 || seg[g][b] > seg[g][b + 1]) return fail(SGL_EINVAL, "unique_compact_batched: seg does not ascend");
        total += seg[g][B];
    }
    int64_t* tmp = (int64_t*)malloc((size_t)(total + 1) * sizeof(int64_t));
    if (!tmp) return fail(SGL_ENOMEM, "malloc");
    int64_t count = 0;
    for (int32_t b = 0; b < B; ++b) {
        U_off[b] = count;
        int64_t nt = 0;
        for (int32_t g = 0; g < G; ++g)
            for (int64_t i = seg[g][b]; i < seg[g][b + 1]; ++i) {
                int64_t id = ids[g][i];
                if (id >= 0 && id < universe) tmp[nt++] = id;
            }
        qsort(tmp, (size_t)nt, sizeof(int64_t), i64_cmp);
        int64_t nu = 0;
        for (int64_t i = 0; i < nt; ++i)
            if (i == 0 || tmp[i] != tmp[i - 1]) tmp[nu++] = tmp[i];
        if (count + nu > unique_capacity) { free(tmp); return fail(SGL_ENOMEM, "unique_out too small"); }
        for (int64_t i = 0; i < nu; ++i) unique_out[count + i] = tmp[i];
        for (int32_t g = 0; g < G; ++g)
            for (int64_t i = seg[g][b]; i < seg[g][b + 1]; ++i) {
                int64_t id = ids[g][i], loc = -1;
                if (id >= 0 && id < universe) {
                    int64_t lo = 0, hi = nu;
                    while (lo < hi) { int64_t mid = (lo + hi) >> 1; if (tmp[mid] < id) lo = mid + 1; else hi = mid; }
                    loc = lo;
                }
                local_out[g][i] = loc;
            }
        count += nu;
    }
    U_off[B] = count;
    free(tmp);
    return SGL_OK;
}

/* ------------------------------------------------------------ cache gather */

/* cold rows and their times may sit at a stride of their own (0 = packed) */
static int64_t cold_stride(const sgl_cache* c) { return c->cold_stride ? c->cold_stride : c->row_bytes; }
static int64_t hot_stride(const sgl_cache* c) { return c->hot_stride ? c->hot_stride : c->row_bytes; }
static int64_t* cold_ts_at(const sgl_cache* c, const int64_t* base, int64_t loc) {
    return (int64_t*)((char*)base + loc * (c->ts_cold_stride ? c->ts_cold_stride : 8));
}

static int64_t cache_loc(const sgl_cache* c, int64_t id) {
    int64_t key = id & c->id_mask;
    if (id < 0) return -1;
    if (c->g2l) {
        if (key < 0 || key >= c->g2l_len) return -1;
        key = c->g2l[key];
    }
    if (key < 0 || key >= c->rows) return -1;
    return key;
}

/* Reference: IDMapper.to_local (partition_book.py:106-133) then
 * data[loc], ts[loc] (NodeState.py:36-44); tensor_gather row copy
 * (feature.cu.hpp:42-88); DistRouteIndex.loc = id & 0xFFFFFFFFFFFF
 * (partition_book.py:14-31). */
int32_t sglo_gather(const sgl_cache* c, const int64_t* ids, int64_t N_max,
                    const int64_t* N_dev, void* out, int64_t* out_ts,
                    int64_t* stats, void* stream) {
    (void)stream;
    if (!c || N_max < 0 || (N_max > 0 && (!ids || !out))) return fail(SGL_EINVAL, "gather: null");
    if (c->row_bytes <= 0 || c->row_bytes % 4) return fail(SGL_EINVAL, "gather: row_bytes must be a positive multiple of 4");
    int64_t N = N_dev ? *N_dev : N_max;
    if (N > N_max) return fail(SGL_EINVAL, "gather: N > N_max");
    int64_t hit = 0, cold = 0, absent = 0;
    for (int64_t i = 0; i < N; ++i) {
        char* dst = (char*)out + i * c->row_bytes;
        int64_t loc = cache_loc(c, ids[i]);
        if (loc < 0) {
            memset(dst, 0, (size_t)c->row_bytes);
            if (out_ts) out_ts[i] = 0;
            absent++;
            continue;
        }
        int64_t slot = c->hot_slot ? (int64_t)c->hot_slot[loc] : loc;
        if (slot >= 0) {
            memcpy(dst, (const char*)c->hot + slot * hot_stride(c), (size_t)c->row_bytes);
            if (out_ts) out_ts[i] = c->ts_hot ? c->ts_hot[slot] : 0;
            hit++;
        } else {
            memcpy(dst, (const char*)c->cold + loc * cold_stride(c), (size_t)c->row_bytes);
            if (out_ts) out_ts[i] = c->ts_cold ? *cold_ts_at(c, c->ts_cold, loc) : 0;
            cold++;
        }
    }
    if (stats) { stats[0] += hit; stats[1] += cold; stats[2] += absent; }
    return SGL_OK;
}

/* The gather with each distinct cold row fetched once: by definition the rows sglo_gather yields; the fourth
 * statistic counts the distinct local rows of the cold tier among the requests (np.unique of their locs). */
size_t sglo_gather_dedup_workspace_bytes(int64_t N_max) { (void)N_max; return 0; }

int32_t sglo_gather_dedup(const sgl_cache* c, const int64_t* ids, int64_t N_max, const int64_t* N_dev,
                          void* out, int64_t* out_ts, int64_t* stats, void* staging, int64_t* staging_ts,
                          int64_t staging_rows, void* ws, size_t ws_bytes, void* stream) {
    (void)staging; (void)staging_ts; (void)staging_rows; (void)ws; (void)ws_bytes;
    int32_t rc = sglo_gather(c, ids, N_max, N_dev, out, out_ts, stats, stream);
    if (rc != SGL_OK || !stats) return rc;
    int64_t N = N_dev ? *N_dev : N_max;
    int64_t* locs = (int64_t*)malloc((size_t)(N + 1) * sizeof(int64_t));
    if (!locs) return fail(SGL_ENOMEM, "malloc");
    int64_t nc = 0;
    for (int64_t i = 0; i < N; ++i) {
        int64_t loc = cache_loc(c, ids[i]);
        if (loc >= 0 && c->hot_slot && c->hot_slot[loc] < 0) locs[nc++] = loc;
    }
    qsort(locs, (size_t)nc, sizeof(int64_t), i64_cmp);
    int64_t distinct = 0;
    for (int64_t i = 0; i < nc; ++i) if (i == 0 || locs[i] != locs[i - 1]) distinct++;
    stats[3] += distinct;
    free(locs);
    return SGL_OK;
}

/* Reference: DistNodeState.update (NodeState.py:46-61): loc = to_local(gids),
 * rows with loc >= 0 are overwritten, ts likewise. */
int32_t sglo_scatter_update(const sgl_cache* c, void* hot_rw, void* cold_rw,
                            int64_t* ts_hot_rw, int64_t* ts_cold_rw,
                            const int64_t* ids, int64_t N, const void* values,
                            const int64_t* ts, void* stream) {
    (void)stream;
    if (!c || N < 0 || (N > 0 && (!ids || !values))) return fail(SGL_EINVAL, "scatter_update: null");
    for (int64_t i = 0; i < N; ++i) {
        int64_t loc = cache_loc(c, ids[i]);
        if (loc < 0) continue;
        int64_t slot = c->hot_slot ? (int64_t)c->hot_slot[loc] : loc;
        const char* srcp = (const char*)values + i * c->row_bytes;
        if (slot >= 0) {
            memcpy((char*)hot_rw + slot * hot_stride(c), srcp, (size_t)c->row_bytes);
            if (ts && ts_hot_rw) ts_hot_rw[slot] = ts[i];
        } else {
            memcpy((char*)cold_rw + loc * cold_stride(c), srcp, (size_t)c->row_bytes);
            if (ts && ts_cold_rw) *cold_ts_at(c, ts_cold_rw, loc) = ts[i];
        }
    }
    return SGL_OK;
}

/* ----------------------------------------------------------- time encoding */

/* Reference: TimeEncoder.forward = cos(Linear(1,dim)(t.float()))
 * (time_encoder.py:29-31); Linear computes x*W^T + b.  Rule implemented:
 * x = (float)dt (round to nearest even), a = fl32(fl32(w*x) + b) with a
 * separately rounded multiply and add, y = (float)cos((double)a). */
int32_t sglo_time_encode(const void* dt, int32_t dt_dtype, int64_t N_max,
                         const int64_t* N_dev, const float* w, const float* b,
                         int32_t dim, float* out, void* stream) {
    (void)stream;
    if (N_max < 0 || dim <= 0 || !w || !b || (N_max > 0 && (!dt || !out)))
        return fail(SGL_EINVAL, "time_encode: null");
    if (dt_dtype != SGL_DT_I64 && dt_dtype != SGL_DT_F32) return fail(SGL_EINVAL, "time_encode: dtype");
    int64_t N = N_dev ? *N_dev : N_max;
    for (int64_t i = 0; i < N; ++i) {
        volatile float x = dt_dtype == SGL_DT_I64 ? (float)((const int64_t*)dt)[i]
                                                  : ((const float*)dt)[i];
        for (int32_t j = 0; j < dim; ++j) {
            volatile float prod = w[j] * x;
            volatile float a = prod + b[j];
            out[i * (int64_t)dim + j] = (float)cos((double)a);
        }
    }
    return SGL_OK;
}

/* ------------------------------------------------------- chunks and seeds */

size_t sglo_chunk_index_workspace_bytes(int64_t n) { (void)n; return 0; }

/* Reference: Graph::Graph computes each edge's source chunk from
 * row_chunk_mapper, sorts by it first and derives chunk_ptr_/row_idx_
 * (sample.cu.hpp:1053-1065, 1135-1146).  Rule implemented: nodes grouped by
 * chunk id, ascending node id inside a chunk (a counting sort). */
int32_t sglo_chunk_index_build(int64_t n, int64_t num_chunks, const int64_t* node_chunk,
                               int64_t* chunk_ptr, int64_t* chunk_nodes, void* ws,
                               size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (n < 0 || num_chunks < 0 || !chunk_ptr) return fail(SGL_EINVAL, "chunk_index_build: bad sizes");
    for (int64_t v = 0; v < n; ++v)
        if (node_chunk[v] < 0 || node_chunk[v] >= num_chunks)
            return fail(SGL_ERANGE, "chunk_index_build: chunk id outside [0, num_chunks)");
    for (int64_t c = 0; c <= num_chunks; ++c) chunk_ptr[c] = 0;
    for (int64_t v = 0; v < n; ++v) chunk_ptr[node_chunk[v] + 1]++;
    for (int64_t c = 0; c < num_chunks; ++c) chunk_ptr[c + 1] += chunk_ptr[c];
    int64_t* fill = (int64_t*)malloc((size_t)(num_chunks + 1) * sizeof(int64_t));
    if (!fill) return fail(SGL_ENOMEM, "malloc");
    memcpy(fill, chunk_ptr, (size_t)(num_chunks + 1) * sizeof(int64_t));
    for (int64_t v = 0; v < n; ++v) chunk_nodes[fill[node_chunk[v]]++] = v;
    free(fill);
    return SGL_OK;
}

size_t sglo_seeds_workspace_bytes(int64_t n_cand) { (void)n_cand; return 0; }

/* Walks the candidates in output order and either counts (roots == NULL) or
 * writes.  Reference: filter_seeds_kernel / collect_seeds_kernel
 * (sample.cu.hpp:517-705): a node of a selected chunk is a root when
 * find_time_range gives a non-empty edge range; its timestamps are the
 * distinct ts of that range ("prefix_different_timestamp", :944-952,
 * 1147-1162), q_ptr/q_eid list the events per (node, timestamp).  Rule
 * implemented for the window: t_begin <= ts < t_end (the early-exit tests of
 * find_time_range, :273, 279). */
static int32_t seeds_walk(const sgl_tcsr* g, const sgl_seed_query* q, int64_t* totals,
                          int64_t* roots, int64_t* ts_ptr, int64_t* ts, int64_t* q_ptr, int64_t* q_eid,
                          int64_t* window_end) {
    int64_t R = 0, S = 0, Q = 0;
    for (int64_t p = 0; p < q->num_chunks; ++p) {
        const int64_t c = q->chunks[p];
        const int64_t a = q->chunk_ptr[c], b = q->chunk_ptr[c + 1];
        if (q->cand_off[p + 1] - q->cand_off[p] != b - a)
            return fail(SGL_EINVAL, "seeds: cand_off is not the prefix of the selected chunk sizes");
        for (int64_t x = a; x < b; ++x) {
            const int64_t v = q->chunk_nodes[x];
            const int64_t rs = g->row_ptr[v], re = g->row_ptr[v + 1];
            const int64_t lo = lower_bound_ts(g->ts, rs, re, q->t_begin);
            const int64_t hi = lower_bound_ts(g->ts, lo, re, q->t_end);
            if (hi <= lo) continue;
            if (roots) { roots[R] = v; ts_ptr[R] = S; }
            for (int64_t e = lo; e < hi; ++e) {
                if (e == lo || g->ts[e] != g->ts[e - 1]) {
                    if (roots) { ts[S] = g->ts[e]; q_ptr[S] = Q; }
                    /* by definition, not by position: the first edge of the row with ts >= this time */
                    if (roots && window_end) window_end[S] = lower_bound_ts(g->ts, rs, re, g->ts[e]);
                    ++S;
                }
                if (roots) q_eid[Q] = g->eid[e];
                ++Q;
            }
            ++R;
        }
    }
    if (roots) { ts_ptr[R] = S; q_ptr[S] = Q; }
    if (totals) { totals[0] = R; totals[1] = S; totals[2] = Q; }
    return SGL_OK;
}

int32_t sglo_seeds_count(const sgl_tcsr* g, const sgl_seed_query* q, int64_t* totals, void* ws,
                         size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!g || !q || !totals) return fail(SGL_EINVAL, "seeds_count: null");
    return seeds_walk(g, q, totals, NULL, NULL, NULL, NULL, NULL, NULL);
}

int32_t sglo_seeds_fill(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* totals,
                        int64_t* roots, int64_t* ts_ptr, int64_t* ts, int64_t* q_ptr, int64_t* q_eid,
                        int64_t* window_end, void* ws, size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream; (void)totals;
    if (!g || !q || !ts_ptr || !q_ptr) return fail(SGL_EINVAL, "seeds_fill: null");
    int64_t dummy;
    if (!roots) roots = &dummy; /* R == 0 */
    return seeds_walk(g, q, NULL, roots, ts_ptr, ts, q_ptr, q_eid, window_end);
}

/* ------------------------------------------- sub-graph slice ("cluster" mode) */

size_t sglo_slice_workspace_bytes(int64_t n_cand, int64_t total_chunks) { (void)n_cand; (void)total_chunks; return 0; }

/* Walks the candidates in output order and counts (nodes == NULL) or writes.
 * Reference: count_edges_kernel / write_edges_kernel (sample.cu.hpp:299-515):
 * per chunk, per node of the chunk, the edge range of the time window
 * (lower_bound / upper_bound, :347-348); the node is listed when the range is
 * not empty (:349-351); timestamps are counted where col_ts changes (:358-366)
 * or, with use_full_timestamps, as t_end - t_begin per node (:352-355); an edge
 * is written when the chunk of its destination is selected (:370-377, 497-503);
 * out_ts_ptr holds, per listed timestamp, the offset of its first written edge
 * (:487-491; every integer of a gap maps to the next edge's offset, :462-470).
 * The window is t_begin <= ts < t_end as for the seeds. */
static int32_t slice_walk(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk,
                          int64_t total_chunks, int32_t full, int64_t* totals, int64_t* nodes,
                          int64_t* ts_ptr, int64_t* ts, int64_t* edge_ptr, int64_t* col, int64_t* col_ts,
                          int64_t* col_eid) {
    uint8_t* member = (uint8_t*)calloc((size_t)total_chunks + 1, 1);
    if (!member) return fail(SGL_ENOMEM, "malloc");
    for (int64_t p = 0; p < q->num_chunks; ++p)
        if (q->chunks[p] >= 0 && q->chunks[p] < total_chunks) member[q->chunks[p]] = 1;
    int64_t R = 0, T = 0, E = 0;
    const int write = ts_ptr != NULL;
    for (int64_t p = 0; p < q->num_chunks; ++p) {
        const int64_t c = q->chunks[p];
        const int64_t a = q->chunk_ptr[c], b = q->chunk_ptr[c + 1];
        if (q->cand_off[p + 1] - q->cand_off[p] != b - a) {
            free(member);
            return fail(SGL_EINVAL, "slice: cand_off is not the prefix of the selected chunk sizes");
        }
        for (int64_t x = a; x < b; ++x) {
            const int64_t v = q->chunk_nodes[x];
            const int64_t rs = g->row_ptr[v], re = g->row_ptr[v + 1];
            const int64_t lo = lower_bound_ts(g->ts, rs, re, q->t_begin);
            const int64_t hi = lower_bound_ts(g->ts, lo, re, q->t_end);
            if (hi <= lo) continue;
            if (write) { nodes[R] = v; ts_ptr[R] = T; }
            int64_t next_t = q->t_begin;      /* full mode: first integer not yet listed */
            for (int64_t e = lo; e < hi; ++e) {
                const int64_t t = g->ts[e];
                if (full) {
                    for (; next_t <= t; ++next_t) {
                        if (write) { ts[T] = next_t; edge_ptr[T] = E; }
                        ++T;
                    }
                } else if (e == lo || t != g->ts[e - 1]) {
                    if (write) { ts[T] = t; edge_ptr[T] = E; }
                    ++T;
                }
                const int64_t dc = node_chunk ? node_chunk[g->col[e]] : -1;
                if (!node_chunk || (dc >= 0 && dc < total_chunks && member[dc])) {
                    if (write) { col[E] = g->col[e]; col_ts[E] = t; col_eid[E] = g->eid[e]; }
                    ++E;
                }
            }
            if (full)
                for (; next_t < q->t_end; ++next_t) {
                    if (write) { ts[T] = next_t; edge_ptr[T] = E; }
                    ++T;
                }
            ++R;
        }
    }
    free(member);
    if (write) { ts_ptr[R] = T; edge_ptr[T] = E; }
    if (totals) { totals[0] = R; totals[1] = T; totals[2] = E; }
    return SGL_OK;
}

int32_t sglo_slice_count(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk,
                         int64_t total_chunks, int32_t full_timestamps, int64_t* totals, void* ws,
                         size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (!g || !q || !totals || total_chunks < 0) return fail(SGL_EINVAL, "slice_count: null");
    if (full_timestamps && q->t_end < q->t_begin) return fail(SGL_EINVAL, "slice: t_end < t_begin");
    return slice_walk(g, q, node_chunk, total_chunks, full_timestamps, totals, NULL, NULL, NULL, NULL, NULL, NULL, NULL);
}

int32_t sglo_slice_fill(const sgl_tcsr* g, const sgl_seed_query* q, const int64_t* node_chunk,
                        int64_t total_chunks, int32_t full_timestamps, const int64_t* totals, int64_t* nodes,
                        int64_t* ts_ptr, int64_t* ts, int64_t* edge_ptr, int64_t* col, int64_t* col_ts,
                        int64_t* col_eid, void* ws, size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream; (void)totals;
    if (!g || !q || !ts_ptr || !edge_ptr || total_chunks < 0) return fail(SGL_EINVAL, "slice_fill: null");
    return slice_walk(g, q, node_chunk, total_chunks, full_timestamps, NULL, nodes, ts_ptr, ts, edge_ptr, col, col_ts, col_eid);
}

/* ------------------------------------------------ batch materialisation */

typedef struct { int64_t a, b, pos; } rec3;

static int rec3_cmp(const void* x, const void* y) {
    const rec3* p = (const rec3*)x; const rec3* q = (const rec3*)y;
    if (p->a != q->a) return p->a < q->a ? -1 : 1;
    if (p->b != q->b) return p->b < q->b ? -1 : 1;
    return p->pos < q->pos ? -1 : (p->pos > q->pos ? 1 : 0);
}

size_t sglo_unique_pairs_workspace_bytes(int64_t N_max) { (void)N_max; return 0; }

/* Reference: _get_unique_pairs (prepare_sample.py:205-213): np.unique of
 * records (id, ts) with return_inverse - records ascend by id, then ts. */
int32_t sglo_unique_pairs(const int64_t* ids, const int64_t* ts, int64_t N_max, const int64_t* N_dev,
                          int64_t* uniq_ids, int64_t* uniq_ts, int64_t* inverse, int64_t* U_dev, void* ws,
                          size_t ws_bytes, void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (N_max < 0 || !U_dev) return fail(SGL_EINVAL, "unique_pairs: bad argument");
    const int64_t N = N_dev ? (*N_dev < N_max ? *N_dev : N_max) : N_max;
    rec3* r = (rec3*)malloc((size_t)(N > 0 ? N : 1) * sizeof(rec3));
    if (!r) return fail(SGL_ENOMEM, "malloc");
    for (int64_t i = 0; i < N; ++i) { r[i].a = ids[i]; r[i].b = ts[i]; r[i].pos = i; }
    qsort(r, (size_t)N, sizeof(rec3), rec3_cmp);
    int64_t U = 0;
    for (int64_t i = 0; i < N; ++i) {
        if (i == 0 || r[i].a != r[i - 1].a || r[i].b != r[i - 1].b) {
            uniq_ids[U] = r[i].a; uniq_ts[U] = r[i].b; ++U;
        }
        inverse[r[i].pos] = U - 1;
    }
    free(r);
    U_dev[0] = U;
    return SGL_OK;
}

size_t sglo_csc_from_pairs_workspace_bytes(int64_t E_max) { (void)E_max; return 0; }

/* Reference: _build_csc_from_pairs (prepare_sample.py:215-229): perm =
 * np.lexsort((ts, dst_local)) (stable), indptr = cumsum of the per-destination
 * counts. */
int32_t sglo_csc_from_pairs(const int64_t* dst_local, const int64_t* ts, int64_t E_max, const int64_t* E_dev,
                            int64_t num_dst, int64_t* indptr, int64_t* perm, void* ws, size_t ws_bytes,
                            void* stream) {
    (void)ws; (void)ws_bytes; (void)stream;
    if (E_max < 0 || num_dst < 0 || !indptr) return fail(SGL_EINVAL, "csc_from_pairs: bad argument");
    const int64_t E = E_dev ? (*E_dev < E_max ? *E_dev : E_max) : E_max;
    rec3* r = (rec3*)malloc((size_t)(E > 0 ? E : 1) * sizeof(rec3));
    if (!r) return fail(SGL_ENOMEM, "malloc");
    for (int64_t d = 0; d <= num_dst; ++d) indptr[d] = 0;
    for (int64_t i = 0; i < E; ++i) {
        r[i].a = dst_local[i]; r[i].b = ts[i]; r[i].pos = i;
        if (dst_local[i] < 0 || dst_local[i] >= num_dst) { free(r); return fail(SGL_ERANGE, "csc_from_pairs: destination outside [0, num_dst)"); }
        indptr[dst_local[i] + 1] += 1;
    }
    qsort(r, (size_t)E, sizeof(rec3), rec3_cmp);
    for (int64_t i = 0; i < E; ++i) perm[i] = r[i].pos;
    for (int64_t d = 0; d < num_dst; ++d) indptr[d + 1] += indptr[d];
    free(r);
    return SGL_OK;
}

/* --------------------------------------------------------- block building */

/* Reference: AsyncBlock.to_block builds ('csc', (indptr, indices, [])) with
 * indices = arange(E) + number of self-loop sources (graph.py:186-197,
 * 228-241); _build_csc_from_pairs builds indptr by bincount + cumsum
 * (prepare_sample.py:220-227). */
int32_t sglo_block_build(const int64_t* root_start_ptr, const int64_t* counts, int64_t S_max,
                         int64_t E_max, int64_t dst_offset, int64_t src_offset, int64_t* indptr,
                         int64_t* indices, int64_t* edge_dst, void* stream) {
    (void)stream;
    if (!root_start_ptr || !counts || !indptr) return fail(SGL_EINVAL, "block_build: null");
    int64_t S = counts[0] < S_max ? counts[0] : S_max, E = counts[1] < E_max ? counts[1] : E_max;
    for (int64_t d = 0; d < dst_offset; ++d) indptr[d] = 0;
    for (int64_t s = 0; s <= S; ++s) indptr[dst_offset + s] = root_start_ptr[s];
    for (int64_t s = 0; s < S; ++s)
        for (int64_t e = root_start_ptr[s]; e < root_start_ptr[s + 1] && e < E; ++e) {
            indices[e] = src_offset + e;
            if (edge_dst) edge_dst[e] = dst_offset + s;
        }
    return SGL_OK;
}

/* -------------------------------------------------- latest event per node */

/* Reference: unq, inv = index.unique(return_inverse=True);
 * max_ts, idx = torch_scatter.scatter_max(mail_ts, inv, 0)
 * (starrygl/nn/memory/mailbox.py:78-83).  Ties: the first event wins. */
int32_t sglo_segment_max_ts(const int64_t* local, const int64_t* ts, int64_t N_max,
                            const int64_t* N_dev, int64_t U_max, const int64_t* U_dev,
                            int64_t* max_ts, int64_t* arg, void* stream) {
    (void)stream;
    if (N_max < 0 || U_max < 0 || (N_max > 0 && (!local || !ts)) || (U_max > 0 && (!max_ts || !arg)))
        return fail(SGL_EINVAL, "segment_max_ts: null");
    int64_t N = N_dev ? *N_dev : N_max, U = U_dev ? *U_dev : U_max;
    if (N > N_max) N = N_max;
    if (U > U_max) U = U_max;
    for (int64_t u = 0; u < U; ++u) { max_ts[u] = INT64_MIN; arg[u] = -1; }
    for (int64_t i = 0; i < N; ++i) {
        int64_t u = local[i];
        if (u < 0 || u >= U) continue;
        if (arg[u] < 0 || ts[i] > max_ts[u]) { max_ts[u] = ts[i]; arg[u] = i; }
    }
    return SGL_OK;
}

/* Several gathers at once: by definition the same as one sglo_gather per segment. */
int32_t sglo_gather_multi(int32_t T, const sgl_gather_seg* segs, void* stream) {
    if (T < 0 || (T > 0 && !segs)) return fail(SGL_EINVAL, "gather_multi: bad segment list");
    if (T > SGL_GATHER_MAX_SEGMENTS) return fail(SGL_ENOTSUP, "gather_multi: too many segments");
    for (int32_t t = 0; t < T; ++t) {
        int32_t rc = sglo_gather(segs[t].cache, segs[t].ids, segs[t].N_max, segs[t].N_dev, segs[t].out,
                                 segs[t].out_ts, NULL, stream);
        if (rc != SGL_OK) return rc;
    }
    return SGL_OK;
}
