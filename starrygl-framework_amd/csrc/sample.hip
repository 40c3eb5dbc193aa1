// Temporal neighbour sampling over a T-CSR for gfx950.
//
// One hop = three launches on the caller's stream, no host synchronisation:
//   count : a group of G lanes owns one (node, t) slot; the group finds the
//           slot's candidate window with a (G+1)-ary cooperative search on the
//           row's timestamp slice (ballot + popcount per step) and records the
//           window start / length; the block writes the sum of its slot counts;
//   scan  : one block turns the per-block sums into exclusive block offsets and
//           publishes S, E and the number of out-of-range slots;
//   fill  : the same grid copies (recent) or draws (uniform) the slot's edges
//           into the ragged outputs with group-coalesced 8-byte accesses.
// The slot count of hop l+1 is hop l's E, read from device memory, so a k-hop
// call is a fixed launch sequence sized for the worst case.
//
// Replaces static_recent_neighbor_num / recent_sample_single_hop_kernel /
// static_neighbor_num / uniform_sample_single_hop_kernel and the thrust calls
// between them (csrc/include/starrygl/sample.cu.hpp:706-827, 1532-1716).
#include "common.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int SCAN_BLOCK = 1024;

struct HopArgs {
    // graph
    int64_t n;
    const int64_t* row_ptr;
    const int64_t* col;
    const int64_t* ts;
    const int64_t* eid;
    // slots
    const int64_t* slot_node;
    const int64_t* slot_ts;
    int64_t S_max;
    const int64_t* S_dev;
    // params
    int32_t type, k;
    int64_t allowed_offset;
    int32_t equal_root_time, keep_root_time, replace, hop;
    uint64_t seed;
    // workspace
    int64_t* w_start;    // [S_max] first candidate position (recent: first copied edge)
    int64_t* w_len;      // [S_max] window length
    int64_t* block_sum;  // [blocks] -> exclusive block offsets after the scan
    int32_t* block_bad;  // [blocks]
    // outputs
    int64_t* root_start_ptr;
    int64_t* root_end_ptr;
    int64_t* nbr;
    int64_t* nbr_ts;
    int64_t* nbr_eid;
    int64_t* nbr_dt;
    int64_t* counts;
};

// First index in [lo, hi) with ts[idx] >= key, found by the G lanes of a group
// together.  Every lane of the wave must call this (ballots are wave-wide);
// groups with active == false idle through the loop.
template <int G>
__device__ __forceinline__ int64_t group_lower_bound(const int64_t* __restrict__ ts, int64_t lo,
                                                     int64_t hi, int64_t key, int lig, int gshift,
                                                     bool active) {
    bool done = !active || lo >= hi;
    while (!__all(done)) {
        const int64_t len = hi - lo;
        const bool last = len <= G;
        bool pred = false;
        if (!done) {
            if (last) {
                if (lig < len) pred = ts[lo + lig] < key;
            } else {
                pred = ts[lo + ((int64_t)(lig + 1) * len) / (G + 1)] < key;
            }
        }
        const int c = __popcll(group_ballot<G>(pred, gshift));
        if (!done) {
            if (last) {
                lo += c;
                hi = lo;
                done = true;
            } else {
                // probes p_i = lo + (i+1)*len/(G+1) ascend strictly; c of them are < key
                const int64_t nlo = (c == 0) ? lo : lo + ((int64_t)c * len) / (G + 1) + 1;
                const int64_t nhi = (c == G) ? hi : lo + ((int64_t)(c + 1) * len) / (G + 1);
                lo = nlo;
                hi = nhi;
                done = lo >= hi;
            }
        }
    }
    return lo;
}

template <int G>
__global__ __launch_bounds__(BLOCK) void count_kernel(HopArgs a) {
    constexpr int SPB = BLOCK / G;  // slots per block
    __shared__ int32_t s_cnt[SPB];
    __shared__ int32_t s_bad[SPB];
    const int64_t S = live_count(a.S_dev, a.S_max);
    const int gib = threadIdx.x / G;             // group in block
    const int lig = threadIdx.x % G;             // lane in group
    const int gshift = (threadIdx.x % WAVE) / G * G;
    const int64_t slot = (int64_t)blockIdx.x * SPB + gib;
    if ((int64_t)blockIdx.x * SPB >= S) return;  // whole block past the live slots
    bool active = slot < S;
    int64_t v = 0, t = 0;
    if (active) {
        v = a.slot_node[slot];
        t = a.slot_ts[slot];
    }
    const bool bad = active && (v < 0 || v >= a.n);
    active = active && !bad;
    int64_t rs = 0, re = 0;
    if (active) {
        rs = a.row_ptr[v];
        re = a.row_ptr[v + 1];
    }
    const int64_t t_hi = t + (a.equal_root_time ? 1 : 0);
    const int64_t hi = group_lower_bound<G>(a.ts, rs, re, t_hi, lig, gshift, active);
    int64_t lo = rs;
    if (a.allowed_offset >= 0)  // kernel argument: uniform across the wave
        lo = group_lower_bound<G>(a.ts, rs, hi, t - a.allowed_offset, lig, gshift, active);
    const int64_t len = hi - lo;
    const int32_t c = (int32_t)(len < a.k ? len : a.k);
    if (lig == 0) {
        s_cnt[gib] = active ? c : 0;
        s_bad[gib] = bad ? 1 : 0;
        if (slot < S) {
            a.w_start[slot] = (a.type == SGL_SAMPLE_RECENT) ? hi - c : lo;
            a.w_len[slot] = active ? len : 0;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t sum = 0;
        int32_t nbad = 0;
#pragma unroll
        for (int i = 0; i < SPB; ++i) {
            sum += s_cnt[i];
            nbad += s_bad[i];
        }
        a.block_sum[blockIdx.x] = sum;
        a.block_bad[blockIdx.x] = nbad;
    }
}

// Exclusive scan of the live block sums by one block; publishes the counts and
// the terminating entries of the two pointer arrays.
__global__ __launch_bounds__(SCAN_BLOCK) void scan_kernel(HopArgs a, int spb) {
    __shared__ int64_t s_part[SCAN_BLOCK];
    __shared__ int32_t s_badp[SCAN_BLOCK];
    const int64_t S = live_count(a.S_dev, a.S_max);
    const int64_t nb = ceil_div<int64_t>(S, spb);
    const int64_t per = ceil_div<int64_t>(nb, SCAN_BLOCK);
    const int64_t b0 = (int64_t)threadIdx.x * per;
    const int64_t b1 = b0 + per < nb ? b0 + per : nb;
    int64_t sum = 0;
    int32_t bad = 0;
    for (int64_t b = b0; b < b1; ++b) {
        sum += a.block_sum[b];
        bad += a.block_bad[b];
    }
    s_part[threadIdx.x] = sum;
    s_badp[threadIdx.x] = bad;
    __syncthreads();
    // Hillis-Steele inclusive scan over the 1024 partials
    for (int d = 1; d < SCAN_BLOCK; d <<= 1) {
        int64_t x = 0;
        int32_t y = 0;
        if ((int)threadIdx.x >= d) {
            x = s_part[threadIdx.x - d];
            y = s_badp[threadIdx.x - d];
        }
        __syncthreads();
        s_part[threadIdx.x] += x;
        s_badp[threadIdx.x] += y;
        __syncthreads();
    }
    int64_t run = s_part[threadIdx.x] - sum;  // exclusive prefix of this thread's chunk
    for (int64_t b = b0; b < b1; ++b) {
        const int64_t x = a.block_sum[b];
        a.block_sum[b] = run;
        run += x;
    }
    if (threadIdx.x == SCAN_BLOCK - 1) {
        const int64_t E = s_part[SCAN_BLOCK - 1];
        a.counts[0] = S;
        a.counts[1] = E;
        a.counts[2] = s_badp[SCAN_BLOCK - 1];
        a.root_start_ptr[S] = E;
        a.root_end_ptr[S] = E;
    }
}

// Philox4x32-10, counter (draw, slot_lo, slot_hi, hop), key (seed_lo, seed_hi);
// returns x0 | x1 << 32.
__device__ __forceinline__ uint64_t draw_bits(uint64_t seed, int32_t hop, int64_t slot, int32_t j) {
    uint32_t c0 = (uint32_t)j, c1 = (uint32_t)((uint64_t)slot & 0xFFFFFFFFu),
             c2 = (uint32_t)((uint64_t)slot >> 32), c3 = (uint32_t)hop;
    uint32_t k0 = (uint32_t)(seed & 0xFFFFFFFFu), k1 = (uint32_t)(seed >> 32);
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t h0 = __umulhi(0xD2511F53u, c0), l0 = 0xD2511F53u * c0;
        const uint32_t h1 = __umulhi(0xCD9E8D57u, c2), l1 = 0xCD9E8D57u * c2;
        const uint32_t n0 = h1 ^ c1 ^ k0, n2 = h0 ^ c3 ^ k1;
        c0 = n0; c1 = l1; c2 = n2; c3 = l0;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    return (uint64_t)c0 | ((uint64_t)c1 << 32);
}

__device__ __forceinline__ int64_t bounded(uint64_t bits, int64_t range) {
    return (int64_t)__umul64hi(bits, (uint64_t)range);
}

template <int G>
__global__ __launch_bounds__(BLOCK) void fill_kernel(HopArgs a) {
    constexpr int SPB = BLOCK / G;
    __shared__ int64_t s_off[SPB];
    const int64_t S = live_count(a.S_dev, a.S_max);
    const int gib = threadIdx.x / G;
    const int lig = threadIdx.x % G;
    const int gshift = (threadIdx.x % WAVE) / G * G;
    const int wlane = threadIdx.x % WAVE;
    const int64_t slot = (int64_t)blockIdx.x * SPB + gib;
    if ((int64_t)blockIdx.x * SPB >= S) return;
    const bool active = slot < S;
    int64_t start = 0, len = 0, t = 0;
    if (active) {
        start = a.w_start[slot];
        len = a.w_len[slot];
        t = a.slot_ts[slot];
    }
    const int32_t k = a.k;
    const int32_t c = (int32_t)(len < k ? len : k);
    // exclusive prefix of c over the block's slots
    if (lig == 0) s_off[gib] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t run = a.block_sum[blockIdx.x];
#pragma unroll
        for (int i = 0; i < SPB; ++i) {
            const int64_t x = s_off[i];
            s_off[i] = run;
            run += x;
        }
    }
    __syncthreads();
    const int64_t off = s_off[gib];
    if (active && lig == 0) {
        a.root_start_ptr[slot] = off;
        a.root_end_ptr[slot] = off + c;
    }
    if (a.type == SGL_SAMPLE_RECENT) {
        if (active) {
            for (int32_t j = lig; j < c; j += G) {
                const int64_t e = start + j;
                const int64_t ets = a.ts[e];
                a.nbr[off + j] = a.col[e];
                a.nbr_ts[off + j] = ets;
                a.nbr_eid[off + j] = a.eid[e];
                a.nbr_dt[off + j] = ets - t;
            }
        }
        return;
    }
    // ---- uniform: needs k <= G (checked on the host) ------------------------
    const bool draw = active && len > k;  // uniform inside the group
    int64_t sel = lig;                    // offset inside the window; copy path: identity
    int32_t rank = lig;
    const bool any_draw = __any(draw);
    if (any_draw) {                       // wave-uniform branch
        int64_t tj = 0;
        if (draw && lig < k) {
            const uint64_t bits = draw_bits(a.seed, a.hop, slot, lig);
            tj = a.replace ? bounded(bits, len) : bounded(bits, len - k + lig + 1);
        }
        if (a.replace) {
            if (draw) sel = tj;  // draw order is kept
        } else {
            // Floyd: step j picks t_j from [0, len-k+j]; a repeat is replaced by len-k+j
            int64_t mine = -1;
            for (int32_t j = 0; j < k; ++j) {
                const int64_t cand = shfl_i64(tj, (wlane - lig) + j);
                const bool dup = group_ballot<G>(draw && lig < j && mine == cand, gshift) != 0;
                if (lig == j) mine = dup ? (len - k + j) : cand;
            }
            // rank among the k picks (all distinct) = output position
            int32_t r = 0;
            for (int32_t j = 0; j < k; ++j) {
                const int64_t other = shfl_i64(mine, (wlane - lig) + j);
                r += (other < mine) ? 1 : 0;
            }
            if (draw) {
                sel = mine;
                rank = r;
            }
        }
    }
    if (active && lig < c) {
        const int64_t e = start + sel;
        const int64_t ets = a.ts[e];
        a.nbr[off + rank] = a.col[e];
        a.nbr_ts[off + rank] = a.keep_root_time ? t : ets;
        a.nbr_eid[off + rank] = a.eid[e];
        a.nbr_dt[off + rank] = ets - t;
    }
}

// Hop-0 slots: positives expanded over their timestamp lists, then negatives.
__global__ void expand_roots_kernel(int64_t R, const int64_t* __restrict__ roots,
                                    const int64_t* __restrict__ ts_ptr, int64_t S_pos,
                                    const int64_t* __restrict__ root_ts, int64_t N_neg,
                                    const int64_t* __restrict__ neg_roots,
                                    const int64_t* __restrict__ neg_ts, int64_t* slot_node,
                                    int64_t* slot_ts) {
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (s < S_pos) {
        // last r with ts_ptr[r] <= s
        int64_t lo = 0, hi = R;  // answer in [lo, hi)
        while (hi - lo > 1) {
            const int64_t mid = lo + ((hi - lo) >> 1);
            if (ts_ptr[mid] <= s) lo = mid; else hi = mid;
        }
        slot_node[s] = roots[lo];
        slot_ts[s] = root_ts[s];
    } else if (s < S_pos + N_neg) {
        slot_node[s] = neg_roots[s - S_pos];
        slot_ts[s] = neg_ts[s - S_pos];
    }
}

int pick_group(const sgl_sample_params* p) {
    if (p->type == SGL_SAMPLE_UNIFORM) {
        if (p->fanout <= 16) return 16;
        if (p->fanout <= 32) return 32;
        return 64;
    }
    return 16;
}

size_t hop_workspace_bytes(int64_t S_max) {
    // sized for the largest block grid: 64-lane groups, 4 slots per block
    const int64_t blocks = ceil_div<int64_t>(S_max > 0 ? S_max : 1, BLOCK / 64);
    size_t b = 0;
    b += align_up((size_t)(S_max + 1) * 8) * 2;
    b += align_up((size_t)blocks * 8);
    b += align_up((size_t)blocks * 4);
    return b + 1024;
}

int32_t check_params(const sgl_sample_params* p) {
    if (!p) return fail(SGL_EINVAL, "sample: params is NULL");
    if (p->type != SGL_SAMPLE_RECENT && p->type != SGL_SAMPLE_UNIFORM)
        return fail(SGL_ENOTSUP, "undefined sampling strategy");
    if (p->fanout < 0) return fail(SGL_EINVAL, "sample: fanout < 0");
    if (p->type == SGL_SAMPLE_UNIFORM && p->fanout > SGL_UNIFORM_MAX_FANOUT)
        return fail(SGL_ENOTSUP, "uniform fanout %d > %d", p->fanout, SGL_UNIFORM_MAX_FANOUT);
    return SGL_OK;
}

int32_t check_graph(const sgl_tcsr* g) {
    if (!g) return fail(SGL_EINVAL, "sample: graph is NULL");
    if (g->n < 0 || g->m < 0) return fail(SGL_EINVAL, "sample: negative graph size");
    if (!g->row_ptr || (g->m > 0 && (!g->col || !g->ts || !g->eid)))
        return fail(SGL_EINVAL, "sample: graph array is NULL");
    return SGL_OK;
}

int32_t check_out(const sgl_hop_out* o, int64_t S_max, int32_t k) {
    if (!o) return fail(SGL_EINVAL, "sample: out is NULL");
    if (o->capacity_slots < S_max)
        return fail(SGL_ENOMEM, "sample: capacity_slots %lld < %lld slots", (long long)o->capacity_slots,
                    (long long)S_max);
    if (o->capacity_edges < S_max * (int64_t)k)
        return fail(SGL_ENOMEM, "sample: capacity_edges %lld < slots*fanout %lld",
                    (long long)o->capacity_edges, (long long)(S_max * (int64_t)k));
    if (!o->root_start_ptr || !o->root_end_ptr || !o->counts)
        return fail(SGL_EINVAL, "sample: out pointer array is NULL");
    if (S_max * (int64_t)k > 0 && (!o->neighbors || !o->neighbors_ts || !o->neighbors_eid || !o->neighbors_dt))
        return fail(SGL_EINVAL, "sample: out neighbour array is NULL");
    return SGL_OK;
}

template <int G>
int32_t launch_hop(const HopArgs& a, hipStream_t st) {
    constexpr int SPB = BLOCK / G;
    const int64_t blocks64 = ceil_div<int64_t>(a.S_max > 0 ? a.S_max : 1, SPB);
    if (blocks64 > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "sample: too many slots for one launch");
    const unsigned blocks = (unsigned)blocks64;
    if (a.S_max > 0) {
        hipLaunchKernelGGL(count_kernel<G>, dim3(blocks), dim3(BLOCK), 0, st, a);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, a, SPB);
    SGL_LAUNCH_CHECK();
    if (a.S_max > 0 && a.k > 0) {
        hipLaunchKernelGGL(fill_kernel<G>, dim3(blocks), dim3(BLOCK), 0, st, a);
        SGL_LAUNCH_CHECK();
    }
    return SGL_OK;
}

int32_t run_hop(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts, int64_t S_max,
                const int64_t* S_dev, const sgl_sample_params* p, const sgl_hop_out* out, void* ws,
                size_t ws_bytes, hipStream_t st) {
    if (S_max > 0 && (!slot_node || !slot_ts)) return fail(SGL_EINVAL, "sample: slot array is NULL");
    if (ws_bytes < hop_workspace_bytes(S_max) || !ws)
        return fail(SGL_ENOMEM, "sample: workspace %zu < %zu bytes", ws_bytes, hop_workspace_bytes(S_max));
    Arena ar(ws, ws_bytes);
    HopArgs a;
    a.n = g->n; a.row_ptr = g->row_ptr; a.col = g->col; a.ts = g->ts; a.eid = g->eid;
    a.slot_node = slot_node; a.slot_ts = slot_ts; a.S_max = S_max; a.S_dev = S_dev;
    a.type = p->type; a.k = p->fanout; a.allowed_offset = p->allowed_offset;
    a.equal_root_time = p->equal_root_time; a.keep_root_time = p->keep_root_time;
    a.replace = p->replace; a.hop = p->hop; a.seed = p->seed;
    const int64_t max_blocks = ceil_div<int64_t>(S_max > 0 ? S_max : 1, BLOCK / 64);
    a.w_start = ar.take<int64_t>(S_max + 1);
    a.w_len = ar.take<int64_t>(S_max + 1);
    a.block_sum = ar.take<int64_t>(max_blocks);
    a.block_bad = ar.take<int32_t>(max_blocks);
    if (!ar.ok()) return fail(SGL_ENOMEM, "sample: workspace too small");
    a.root_start_ptr = out->root_start_ptr; a.root_end_ptr = out->root_end_ptr;
    a.nbr = out->neighbors; a.nbr_ts = out->neighbors_ts; a.nbr_eid = out->neighbors_eid;
    a.nbr_dt = out->neighbors_dt; a.counts = out->counts;
    switch (pick_group(p)) {
        case 16: return launch_hop<16>(a, st);
        case 32: return launch_hop<32>(a, st);
        default: return launch_hop<64>(a, st);
    }
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_sample_hop_workspace_bytes(int64_t S_max) {
    return hop_workspace_bytes(S_max < 0 ? 0 : S_max);
}

extern "C" int32_t sgl_sample_hop(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts,
                                  int64_t S_max, const int64_t* S_dev, const sgl_sample_params* p,
                                  const sgl_hop_out* out, void* ws, size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_graph(g)) != SGL_OK) return rc;
    if ((rc = check_params(p)) != SGL_OK) return rc;
    if (S_max < 0) return fail(SGL_EINVAL, "sample_hop: S_max < 0");
    if ((rc = check_out(out, S_max, p->fanout)) != SGL_OK) return rc;
    return run_hop(g, slot_node, slot_ts, S_max, S_dev, p, out, ws, ws_bytes, as_stream(stream));
}

static int64_t worst_slots(int64_t S0, int32_t layer, int32_t k) {
    int64_t s = S0;
    for (int32_t l = 0; l < layer; ++l) {
        if (k != 0 && s > INT64_MAX / (k > 0 ? k : 1)) return INT64_MAX;
        s *= k;
    }
    return s;
}

extern "C" size_t sgl_sample_khop_workspace_bytes(int64_t S0, int32_t layers, int32_t fanout) {
    if (S0 < 0 || layers <= 0 || fanout < 0) return hop_workspace_bytes(0);
    int64_t worst = S0;
    for (int32_t l = 0; l < layers; ++l) {
        const int64_t s = worst_slots(S0, l, fanout);
        if (s > worst) worst = s;
    }
    return hop_workspace_bytes(worst);
}

extern "C" int32_t sgl_sample_khop(const sgl_tcsr* g, int64_t R, const int64_t* roots,
                                   const int64_t* ts_ptr, int64_t S_pos, const int64_t* root_ts,
                                   int64_t N_neg, const int64_t* neg_roots, const int64_t* neg_ts,
                                   int32_t layers, const sgl_sample_params* p, int64_t* slot_node0,
                                   int64_t* slot_ts0, const sgl_hop_out* outs, void* ws,
                                   size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_graph(g)) != SGL_OK) return rc;
    if ((rc = check_params(p)) != SGL_OK) return rc;
    if (R < 0 || S_pos < 0 || N_neg < 0 || layers < 0) return fail(SGL_EINVAL, "sample_khop: negative size");
    if (S_pos > 0 && (R == 0 || !roots || !ts_ptr || !root_ts))
        return fail(SGL_EINVAL, "sample_khop: positive root array is NULL");
    if (N_neg > 0 && (!neg_roots || !neg_ts)) return fail(SGL_EINVAL, "sample_khop: negative root array is NULL");
    if (layers > 0 && !outs) return fail(SGL_EINVAL, "sample_khop: outs is NULL");
    const int64_t S0 = S_pos + N_neg;
    if (S0 > 0 && (!slot_node0 || !slot_ts0)) return fail(SGL_EINVAL, "sample_khop: slot_node0/slot_ts0 is NULL");
    for (int32_t l = 0; l < layers; ++l) {
        const int64_t s = worst_slots(S0, l, p->fanout);
        if (s == INT64_MAX) return fail(SGL_ENOTSUP, "sample_khop: worst-case slot count overflows");
        if ((rc = check_out(&outs[l], s, p->fanout)) != SGL_OK) return rc;
    }
    hipStream_t st = as_stream(stream);
    if (S0 > 0) {
        const unsigned blocks = (unsigned)ceil_div<int64_t>(S0, 256);
        hipLaunchKernelGGL(expand_roots_kernel, dim3(blocks), dim3(256), 0, st, R, roots, ts_ptr, S_pos,
                           root_ts, N_neg, neg_roots, neg_ts, slot_node0, slot_ts0);
        SGL_LAUNCH_CHECK();
    }
    const int64_t* sn = slot_node0;
    const int64_t* stt = slot_ts0;
    const int64_t* S_dev = nullptr;
    for (int32_t l = 0; l < layers; ++l) {
        sgl_sample_params pl = *p;
        pl.hop = l;
        const int64_t s_max = worst_slots(S0, l, p->fanout);
        rc = run_hop(g, sn, stt, s_max, S_dev, &pl, &outs[l], ws, ws_bytes, st);
        if (rc != SGL_OK) return rc;
        sn = outs[l].neighbors;
        stt = outs[l].neighbors_ts;
        S_dev = outs[l].counts + 1;
    }
    return SGL_OK;
}
