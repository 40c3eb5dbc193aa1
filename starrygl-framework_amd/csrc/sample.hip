// Temporal neighbour sampling over a T-CSR for gfx950.
//
// One hop = two (large hops: three) launches on the caller's stream, no host
// synchronisation:
//   count : a group of G lanes owns one (node, t) slot; the group finds the
//           slot's candidate window with a (G+1)-ary cooperative search on the
//           row's timestamp slice (ballot + popcount per step; G = 1, a plain
//           binary search per lane, for very large hops) and records the
//           window start / length; a block walks a contiguous run of slots, G
//           lanes per slot, BLOCK/G slots at a time, and writes the sum of its
//           slot counts.  For hop 0 the slots are derived on the fly from the
//           positive roots (expanded over their timestamp lists) and the
//           negative roots, and written out for the caller;
//   fill  : the same grid; a block first adds up the sums of the blocks before
//           it (no inter-block waiting; beyond FUSED_PREFIX_MAX blocks a
//           one-block scan kernel runs in between instead), then copies
//           (recent) or draws (uniform) its slots' edges into the ragged
//           outputs with group-coalesced 8-byte accesses.  The last block (or
//           the scan kernel) publishes S, E and the number of bad slots.
// The grid is capped at MAX_BLOCKS; the run length per block is derived on the
// device from the live slot count, which for hop l+1 is hop l's E read from
// device memory, so a k-hop call is a fixed launch sequence sized for the worst
// case.
//
// 2-hop calls of at most 32768 root slots and fanout <= 16 - a training mini-batch -
// take a different route: one kernel does both hops (see fused2_kernel below).
//
// Replaces static_recent_neighbor_num / recent_sample_single_hop_kernel /
// static_neighbor_num / uniform_sample_single_hop_kernel and the thrust calls
// between them (csrc/include/starrygl/sample.cu.hpp:706-827, 1532-1716).
#include <mutex>

#include "common.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;          // 4 waves: 16 slots per block iteration at 16 lanes per slot
constexpr int NWAVE = BLOCK / WAVE;
constexpr int MAX_BLOCKS = 8192;   // grid cap of count/fill
constexpr int FUSED_PREFIX_MAX = 1024;  // up to this many blocks a fill block adds up the sums before it itself
constexpr int SCAN_BLOCK = 1024;

struct HopArgs {
    // graph
    int64_t n, m;
    const int64_t* row_ptr;
    const int64_t* col;
    const int64_t* ts;
    const int64_t* eid;
    const int64_t* hint; // next-hop index of the graph (sgl_tcsr.hop_hint), or nullptr
    const int64_t* rec;  // interleaved edge records of the graph (sgl_tcsr.rec), or nullptr
    const int64_t* slot_hint;  // per explicit slot: where its window ends (the index entry of the edge the slot
                               // came from), or nullptr: search
    int32_t hint_optional;     // 1: slot_hint comes from a caller (the root slots of a batched call) and an entry
                               // of -1 means "search"; 0: every entry is an index entry of the graph
    int64_t* hint_out;   // per emitted edge: its index entry, for the next hop's slots; or nullptr
    const int64_t* root_hint;  // derived slots only: per positive slot, where its window ends according to the
                               // caller (sgl_sample_params.root_hint; -1: search), or nullptr
    // slots: explicit (slot_node/slot_ts), or - when roots != nullptr - derived from
    // R positive roots over ts_ptr/root_ts followed by N_neg negatives, and then
    // written to slot_node_out/slot_ts_out
    const int64_t* slot_node;
    const int64_t* slot_ts;
    int64_t S_max;
    const int64_t* S_dev;
    const int64_t* roots;
    const int64_t* ts_ptr;
    const int64_t* root_ts;
    const int64_t* neg_roots;
    const int64_t* neg_ts;
    int64_t R, S_pos;
    int32_t derive;      // 1: slots come from roots/negatives
    int32_t lean;        // 1: slots whose index entry carries the window's length keep their window in that entry only
                         //    (count_lane_kernel does not write w_start / w_len for them, the flat fill kernels read the entry)
    int32_t scanned;     // 1: scan_kernel wrote chunk_off and published the counts
    int32_t align;       // a block's run of slots is a multiple of this (both kernels of a hop agree on it)
    int64_t* slot_node_out;
    int64_t* slot_ts_out;
    // params
    int32_t type, k;
    int64_t allowed_offset;
    int32_t equal_root_time, keep_root_time, replace, hop;
    uint64_t seed;
    void* mark;          // pending-id flags of a remap state, or nullptr
    int64_t mark_universe;
    int32_t mark_bytes;  // 1: a flag byte per id, 0: a bit per id
    // workspace
    int64_t* w_start;    // [S_max] first candidate position (the window's first edge, whatever the strategy)
    int64_t* w_len;      // [S_max] window length
    int64_t* block_sum;  // [gridDim] edges counted by each block
    int32_t* block_bad;  // [gridDim] out-of-range slots seen by each block
    int64_t* chunk_off;  // [SCAN_BLOCK] written by scan_kernel: edges counted before each chunk of blocks
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
        int c;
        if constexpr (G == 1) {
            c = pred ? 1 : 0;     // one lane per slot: plain binary search, no exchange between lanes
        } else {
            c = __popcll(group_ballot<G>(pred, gshift));
        }
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

// One edge for the uniform strategy, whose picks are scattered over a window: from the graph's interleaved
// records when it has them (one 32-byte access), else from the four arrays (a memory sector each).
struct Edge {
    int64_t col, ts, eid, hint;
};
__device__ __forceinline__ Edge load_picked_edge(const HopArgs& a, int64_t e) {
    Edge r;
    if (a.rec != nullptr) {     // kernel argument: uniform across the launch
        const longlong2* p = reinterpret_cast<const longlong2*>(a.rec) + 2 * e;
        const longlong2 x = p[0], y = p[1];
        r.col = x.x; r.ts = x.y; r.eid = y.x; r.hint = y.y;
    } else {
        r.ts = a.ts[e];
        r.col = a.col[e];
        r.eid = a.eid[e];
        r.hint = a.hint != nullptr ? a.hint[e] : -1;
    }
    return r;
}

// Records `id` as pending in the remap state (as unique.hip's mark pass does)
__device__ __forceinline__ void mark_id(const HopArgs& a, int64_t id) {
    if (id >= 0 && id < a.mark_universe) remap_set_pending(a.mark, a.mark_bytes, id);
}

// Slots [first, first + run) belong to block b; run is a multiple of `spb`, itself a
// multiple of the slots either kernel of the hop handles per block iteration, so that
// iterations never straddle two blocks and both kernels see the same partition.
__device__ __forceinline__ void block_run(int64_t S, int spb, int64_t* first, int64_t* run, unsigned bid = blockIdx.x,
                                          unsigned nblk = gridDim.x) {
    int64_t r = ceil_div<int64_t>(S, (int64_t)nblk);
    r = ceil_div<int64_t>(r, spb) * spb;
    if (r < spb) r = spb;
    *run = r;
    *first = (int64_t)bid * r;
}

// (node, t) of slot s
__device__ __forceinline__ void load_slot(const HopArgs& a, int64_t s, int64_t* v, int64_t* t) {
    if (!a.derive) {
        *v = a.slot_node[s];
        *t = a.slot_ts[s];
        return;
    }
    if (s >= a.S_pos) {
        *v = a.neg_roots[s - a.S_pos];
        *t = a.neg_ts[s - a.S_pos];
        return;
    }
    *t = a.root_ts[s];
    // root r with ts_ptr[r] <= s < ts_ptr[r+1].  One timestamp per root is the common
    // case (ts_ptr[s] == s): the root is loaded speculatively beside the two pointers.
    if (s < a.R) {
        const int64_t p0 = a.ts_ptr[s], p1 = a.ts_ptr[s + 1], guess = a.roots[s];
        if (p0 == s && p1 == s + 1) {
            *v = guess;
            return;
        }
    }
    int64_t lo = 0, hi = a.R;
    while (hi - lo > 1) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (a.ts_ptr[mid] <= s) lo = mid; else hi = mid;
    }
    *v = a.roots[lo];
}

// Where the window of derived slot s ends according to the caller, or -1 (search)
__device__ __forceinline__ int64_t root_hint_of(const HopArgs& a, int64_t s) {
    return (a.root_hint != nullptr && s < a.S_pos) ? a.root_hint[s] : -1;
}

// A caller's window end, kept inside the row [rs, re]
__device__ __forceinline__ int64_t clamp_to_row(int64_t h, int64_t rs, int64_t re) {
    h = hint_pos(h);        // (an entry that came out of an edge record carries the window's length above the position)
    return h < rs ? rs : (h > re ? re : h);
}

// Slots of a deeper hop whose index entries may carry their windows' lengths (entries out of edge records): for such
// an entry the window is [position - length, position) and neither the slot nor a row pointer is read.
__device__ __forceinline__ bool whole_window_hop(const HopArgs& a) {      // kernel arguments: uniform across the launch
    return a.slot_hint != nullptr && !a.hint_optional && !a.derive && a.allowed_offset < 0 && !a.equal_root_time;
}
__device__ __forceinline__ bool whole_window(const HopArgs& a, int64_t h, int64_t* start, int64_t* len) {
    const int64_t l = hint_len(h), pos = hint_pos(h);
    if (l < 0 || l > pos || pos > a.m) return false;
    *start = pos - l;
    *len = l;
    return true;
}
// (start, length) of slot's window for the fill kernels: out of the slot's entry in a lean hop, else what the counting
// kernel stored
__device__ __forceinline__ void slot_window(const HopArgs& a, int64_t slot, int64_t* start, int64_t* len) {
    if (a.lean && whole_window_hop(a) && whole_window(a, a.slot_hint[slot], start, len)) return;
    *start = a.w_start[slot];
    *len = a.w_len[slot];
}

template <int G>
__global__ __launch_bounds__(BLOCK) void count_kernel(HopArgs a) {
    constexpr int SPB = BLOCK / G;  // slots per block iteration
    __shared__ int32_t s_cnt[NWAVE];
    __shared__ int32_t s_bad[NWAVE];
    const int gib = threadIdx.x / G;             // group in block
    const int lig = threadIdx.x % G;             // lane in group
    const int wlane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int gshift = wlane / G * G;
    // When the grid is not capped every block owns exactly SPB slots whatever the live
    // count is: the slot can be loaded before the live count has arrived (one dependent
    // memory round trip less).  Slots in [S, S_max) are allocated, their content is unused.
    const bool fixed = a.align == SPB && (int64_t)gridDim.x * SPB >= a.S_max;
    int64_t v0 = 0, t0 = 0, h0 = -1;
    const int64_t slot0 = (int64_t)blockIdx.x * SPB + gib;
    if (fixed && slot0 < a.S_max) {
        load_slot(a, slot0, &v0, &t0);
        h0 = root_hint_of(a, slot0);
    }
    const int64_t S = live_count(a.S_dev, a.S_max);
    int64_t first, run;
    block_run(S, a.align, &first, &run);
    int32_t sum = 0, nbad = 0;                   // per-wave partials, kept by lane 0 of each wave
    for (int64_t it = first; it < first + run && it < S; it += SPB) {
        const int64_t slot = it + gib;
        bool active = slot < S;
        int64_t v = v0, t = t0, rh = h0;
        if (!fixed || it != first) {
            v = t = 0;
            rh = -1;
            if (active) {
                load_slot(a, slot, &v, &t);
                rh = root_hint_of(a, slot);
            }
        }
        const bool bad = active && (v < 0 || v >= a.n);
        active = active && !bad;
        int64_t rs = 0, re = 0;
        if (active) {
            rs = a.row_ptr[v];
            re = a.row_ptr[v + 1];
        }
        const int64_t t_hi = t + (a.equal_root_time ? 1 : 0);
        int64_t hi;
        if (a.slot_hint != nullptr && !a.hint_optional) {     // kernel arguments: uniform across the wave
            // the slot is (destination, time) of an edge whose index entry says where the window ends;
            // an entry of -1 belongs to a destination outside [0,n), which is a bad slot anyway
            const int64_t h = active ? a.slot_hint[slot] : 0;
            hi = clamp_to_row(h, rs, re);     // an index that does not belong to this graph cannot lead outside the row
        } else {
            // positive roots whose window end the caller knows are not searched
            if (a.slot_hint != nullptr && active) rh = a.slot_hint[slot];     // (explicit root slots of a batched call)
            const bool told = active && rh >= 0;
            hi = group_lower_bound<G>(a.ts, rs, re, t_hi, lig, gshift, active && !told);
            if (told) hi = clamp_to_row(rh, rs, re);
        }
        int64_t lo = rs;
        if (a.allowed_offset >= 0)  // kernel argument: uniform across the wave
            lo = group_lower_bound<G>(a.ts, rs, hi, t - a.allowed_offset, lig, gshift, active);
        const int64_t len = hi - lo;
        const int32_t c = (int32_t)(len < a.k ? len : a.k);
        if (lig == 0 && slot < S) {
            a.w_start[slot] = lo;
            a.w_len[slot] = active ? len : 0;
            if (a.derive) {
                a.slot_node_out[slot] = v;
                a.slot_ts_out[slot] = t;
                if (a.mark != nullptr) mark_id(a, v);
            }
        }
        // wave totals of c and of the bad flags (one contribution per group)
        int32_t wc = (lig == 0 && active) ? c : 0;
        int32_t wb = (lig == 0 && bad) ? 1 : 0;
        for (int d = WAVE / 2; d > 0; d >>= 1) {
            wc += __shfl(wc, wlane ^ d);
            wb += __shfl(wb, wlane ^ d);
        }
        sum += wc;
        nbad += wb;
    }
    if (wlane == 0) {
        s_cnt[wid] = sum;
        s_bad[wid] = nbad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t tot = 0;
        int32_t totb = 0;
#pragma unroll
        for (int i = 0; i < NWAVE; ++i) {
            tot += s_cnt[i];
            totb += s_bad[i];
        }
        a.block_sum[blockIdx.x] = tot;
        a.block_bad[blockIdx.x] = totb;
    }
}

// First index in [lo, hi) with ts[idx] >= key, by one lane.  (Wider searches - 8-ary per lane,
// several probes per lane in the group search - were measured slower here: the searches are
// bound by the number of scattered loads, not by the number of rounds.)
__device__ __forceinline__ int64_t lane_lower_bound(const int64_t* __restrict__ ts, int64_t lo, int64_t hi, int64_t key) {
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (ts[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// The counting pass with one lane per slot and a plain binary search per lane, for hops of so many slots that the
// number of loads and of wavefronts in flight, not the length of one slot's chain, bound the launch.  (Several
// slots per lane with their searches stepping together were measured slower: 116 and 122 us against 114 us per
// 192 000-root two-hop call at two and four slots per lane; so was ending every bisection at 16 entries that are
// loaded side by side and counted, 124 us: more loads cost more than fewer dependent rounds save.)
__device__ __forceinline__ void count_lane_body(const HopArgs& a, unsigned bid, unsigned nblk) {
    __shared__ int32_t s_cnt[NWAVE];
    __shared__ int32_t s_bad[NWAVE];
    const int wlane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int64_t S = live_count(a.S_dev, a.S_max);
    int64_t first, run;
    block_run(S, a.align, &first, &run, bid, nblk);
    const int64_t end = first + run < S ? first + run : S;
    const int64_t eq = a.equal_root_time ? 1 : 0;
    int32_t sum = 0, nbad = 0;
    // slots of a deeper hop whose index entries carry their windows' lengths (entries out of edge records): the
    // window is [position - length, position), no row pointer and no slot is read
    const bool whole = whole_window_hop(a);
    for (int64_t slot = first + threadIdx.x; slot < end; slot += BLOCK) {
        if (whole) {
            int64_t st, len;
            if (whole_window(a, a.slot_hint[slot], &st, &len)) {
                if (!a.lean) {
                    a.w_start[slot] = st;
                    a.w_len[slot] = len;
                }
                sum += (int32_t)(len < a.k ? len : a.k);
                continue;
            }
        }
        int64_t v, t;
        load_slot(a, slot, &v, &t);
        const int64_t rh = a.slot_hint != nullptr ? a.slot_hint[slot] : root_hint_of(a, slot);
        if (v < 0 || v >= a.n) {
            ++nbad;
            a.w_start[slot] = 0;
            a.w_len[slot] = 0;
        } else {
            const int64_t rs = a.row_ptr[v], re = a.row_ptr[v + 1];
            // where the window ends: told by an index entry of the graph (every slot of a deeper hop), by the
            // caller (an entry >= 0), or searched
            const bool told = rh >= 0 || (a.slot_hint != nullptr && !a.hint_optional);
            const int64_t hi = told ? clamp_to_row(rh, rs, re) : lane_lower_bound(a.ts, rs, re, t + eq);
            const int64_t lo = a.allowed_offset >= 0 ? lane_lower_bound(a.ts, rs, hi, t - a.allowed_offset) : rs;
            const int64_t len = hi - lo;
            a.w_start[slot] = lo;
            a.w_len[slot] = len;
            sum += (int32_t)(len < a.k ? len : a.k);
        }
        if (a.derive) {
            a.slot_node_out[slot] = v;
            a.slot_ts_out[slot] = t;
            if (a.mark != nullptr) mark_id(a, v);
        }
    }
    for (int d = WAVE / 2; d > 0; d >>= 1) {
        sum += __shfl(sum, wlane ^ d);
        nbad += __shfl(nbad, wlane ^ d);
    }
    if (wlane == 0) {
        s_cnt[wid] = sum;
        s_bad[wid] = nbad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t tot = 0;
        int32_t totb = 0;
#pragma unroll
        for (int i = 0; i < NWAVE; ++i) {
            tot += s_cnt[i];
            totb += s_bad[i];
        }
        a.block_sum[bid] = tot;
        a.block_bad[bid] = totb;
    }
}

__global__ __launch_bounds__(BLOCK) void count_lane_kernel(HopArgs a) { count_lane_body(a, blockIdx.x, gridDim.x); }

// Two hops' kernels in one launch (the same hop of two queries over grids of the same size: a most-recent and a
// uniform query of a batched call): the blocks of the two take turns in the grid, so that both kinds are spread over
// all CUs and run beside each other - each of these kernels alone leaves a chip of 256 CUs waiting on its dependent
// loads, and two launches one after the other pay two ramps and two tails.
__global__ __launch_bounds__(BLOCK) void count_lane_dual_kernel(HopArgs a, HopArgs b) {
    const unsigned bid = blockIdx.x >> 1, nblk = gridDim.x >> 1;
    if (blockIdx.x & 1) count_lane_body(b, bid, nblk);
    else count_lane_body(a, bid, nblk);
}

// Prefix of the block sums at a granularity of CHUNK blocks, by one block (only
// for grids beyond FUSED_PREFIX_MAX): chunk_off[c] = sum of block_sum[0 .. c*CHUNK).
// Loads are coalesced and staged in LDS, thread t then owns the CHUNK consecutive
// sums of chunk t, so a single shuffle scan over the thread totals suffices.  A
// fill block adds the < CHUNK sums of its own chunk (one cache line) itself.
// Publishes the counts and the terminating pointer entries.
constexpr int CHUNK = MAX_BLOCKS / SCAN_BLOCK;
__device__ __forceinline__ void scan_body(const HopArgs& a, int nb) {
    constexpr int NW = SCAN_BLOCK / WAVE;
    __shared__ int32_t s_v[MAX_BLOCKS];
    __shared__ int64_t s_w[NW];
    __shared__ int32_t s_wb[NW];
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    int32_t bad = 0;
#pragma unroll
    for (int r = 0; r < CHUNK; ++r) {
        const int b = r * SCAN_BLOCK + threadIdx.x;
        s_v[b] = b < nb ? (int32_t)a.block_sum[b] : 0;   // a block counts at most BLOCK/16 * fanout edges
        if (b < nb) bad += a.block_bad[b];
    }
    const int64_t S = live_count(a.S_dev, a.S_max);
    __syncthreads();
    int64_t sum = 0;
#pragma unroll
    for (int q = 0; q < CHUNK; ++q) sum += s_v[threadIdx.x * CHUNK + q];
    int64_t inc = sum;
    for (int d = 1; d < WAVE; d <<= 1) {
        const int64_t y = shfl_i64(inc, lane >= d ? lane - d : lane);
        if (lane >= d) inc += y;
    }
    for (int d = WAVE / 2; d > 0; d >>= 1) bad += __shfl(bad, lane ^ d);
    if (lane == WAVE - 1) s_w[wid] = inc;
    if (lane == 0) s_wb[wid] = bad;
    __syncthreads();
    int64_t off = inc - sum, total = 0;
    int32_t bad_total = 0;
#pragma unroll
    for (int q = 0; q < NW; ++q) {
        if (q < wid) off += s_w[q];
        total += s_w[q];
        bad_total += s_wb[q];
    }
    a.chunk_off[threadIdx.x] = off;
    if (threadIdx.x == 0) {
        a.counts[0] = S;
        a.counts[1] = total;
        a.counts[2] = bad_total;
        a.root_start_ptr[S] = total;
        a.root_end_ptr[S] = total;
    }
}
__global__ __launch_bounds__(SCAN_BLOCK) void scan_kernel(HopArgs a, int nb) { scan_body(a, nb); }
__global__ __launch_bounds__(SCAN_BLOCK) void scan_dual_kernel(HopArgs a, HopArgs b, int nb) {     // two blocks
    if (blockIdx.x) scan_body(b, nb);
    else scan_body(a, nb);
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

// x of lane j of every G-lane group of the wave, handed to the group's lanes (j is wave-uniform): lane reads
// into scalar registers and a select per group instead of a trip through the LDS crossbar.
template <int G>
__device__ __forceinline__ int32_t group_bcast(int32_t x, int j, int wlane) {
    int32_t r = __builtin_amdgcn_readlane(x, j);
#pragma unroll
    for (int g = 1; g < WAVE / G; ++g) {
        const int32_t y = __builtin_amdgcn_readlane(x, g * G + j);
        r = wlane >= g * G ? y : r;
    }
    return r;
}

// Floyd's subset of k of [0, len) for every drawing group of the wave (draw is uniform inside a group; lane
// lig < k holds draw tj from [0, len - k + lig]): step j keeps its draw unless an earlier step holds the same
// value, then it takes len - k + j.  -> the lane's pick and its rank among the k picks (all distinct).
// Two draws of a group collide only in windows of a few thousand edges or fewer: the ranks are counted on the raw
// draws first, and the sequential construction runs only in waves where some group saw two equal draws.  Counting
// goes through LDS: every lane parks its draw, then reads its group's draws four at a time (lanes of a group read
// the same words: a broadcast) - a fifth of the instructions of handing the draws round lane by lane, and this
// part is what the uniform kernels spend their issue slots on.  The groups never leave their wavefront, whose LDS
// accesses are served in program order.  Windows close to 2^31 edges and more take the 64-bit variant.
template <int G>
__device__ __forceinline__ void floyd_subset(bool draw, int lig, int wlane, int gshift, int32_t k, int64_t len, int64_t tj,
                                             int64_t* pick, int32_t* rank) {
    __shared__ __attribute__((aligned(16))) int32_t s_draw[BLOCK];
    const bool mine_on = draw && lig < k;
    if (__all(!draw || len < (int64_t)INT32_MAX - WAVE)) {          // wave-uniform
        const int gbase = (int)threadIdx.x - lig;                     // (a multiple of G >= 16: 16-byte aligned words)
        int32_t v = mine_on ? (int32_t)tj : INT32_MAX - lig;          // (idle lanes hold distinct values above every draw)
        // rank of v among the group's values = how many are smaller; eq = how many are equal (itself included)
        auto count = [&](int32_t* smaller, int32_t* equal) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            s_draw[threadIdx.x] = v;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            int32_t r = 0, e = 0;
            for (int32_t j = 0; j < k; j += 4) {                      // (k <= G, G a multiple of 4: inside the group's words)
                const int4 o = *reinterpret_cast<const int4*>(&s_draw[gbase + j]);
                r += (o.x < v ? 1 : 0) + (o.y < v ? 1 : 0) + (o.z < v ? 1 : 0) + (o.w < v ? 1 : 0);
                e += (o.x == v ? 1 : 0) + (o.y == v ? 1 : 0) + (o.z == v ? 1 : 0) + (o.w == v ? 1 : 0);
            }
            *smaller = r;
            *equal = e;
        };
        int32_t r, e;
        count(&r, &e);
        if (__any(mine_on && e > 1)) {
            int32_t m = -1;
            for (int32_t j = 0; j < k; ++j) {
                const int32_t cand = group_bcast<G>(v, j, wlane);
                const bool hit = group_ballot<G>(draw && lig < j && m == cand, gshift) != 0;
                if (lig == j) m = hit ? (int32_t)(len - k + j) : cand;
            }
            v = mine_on ? m : INT32_MAX - lig;
            count(&r, &e);
        }
        if (draw) {
            *pick = (int64_t)v;
            *rank = r;
        }
        return;
    }
    int64_t mine = -1;
    for (int32_t j = 0; j < k; ++j) {
        const int64_t cand = shfl_i64(tj, (wlane - lig) + j);
        const bool hit = group_ballot<G>(draw && lig < j && mine == cand, gshift) != 0;
        if (lig == j) mine = hit ? (len - k + j) : cand;
    }
    int32_t r = 0;
    for (int32_t j = 0; j < k; ++j) {
        const int64_t other = shfl_i64(mine, (wlane - lig) + j);
        r += (other < mine) ? 1 : 0;
    }
    if (draw) {
        *pick = mine;
        *rank = r;
    }
}

// Uniform picks with a wavefront per slot, for fanouts beyond 32 (G = WAVE is the only instantiation; smaller
// fanouts take fill_uniform_flat_kernel): the block walks its run one iteration's slots at a time.
template <int G>
__global__ __launch_bounds__(BLOCK) void fill_kernel(HopArgs a) {
    static_assert(G == WAVE, "a wavefront per slot");
    constexpr int SPB = BLOCK / G;
    __shared__ int64_t s_red[NWAVE];
    __shared__ int32_t s_redb[NWAVE];
    __shared__ int32_t s_wtot[2][NWAVE];  // per-wave edge totals of an iteration, double buffered
    const int gib = threadIdx.x / G;
    const int lig = threadIdx.x % G;
    const int wlane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int gshift = wlane / G * G;
    const int32_t k = a.k;
    // first iteration's slot data: loaded before the live count arrives when the grid is
    // not capped (see count_kernel), and before the prefix sum, so the loads overlap both
    const bool fixed = a.align == SPB && (int64_t)gridDim.x * SPB >= a.S_max;
    int64_t slot = (int64_t)blockIdx.x * SPB + gib;
    int64_t start = 0, len = 0, t = 0;
    if (fixed && slot < a.S_max) {
        start = a.w_start[slot];
        len = a.w_len[slot];
        t = a.derive ? a.slot_ts_out[slot] : a.slot_ts[slot];
    }
    const int64_t S = live_count(a.S_dev, a.S_max);
    int64_t first, run;
    block_run(S, a.align, &first, &run);
    bool active = first < S && first + gib < S;
    if (!fixed) {
        slot = first + gib;
        if (active) {
            start = a.w_start[slot];
            len = a.w_len[slot];
            t = a.derive ? a.slot_ts_out[slot] : a.slot_ts[slot];
        }
    }
    if (!active) start = len = t = 0;   // speculative loads of slots beyond the live count
    // exclusive prefix of this block: read it (scan_kernel ran) or add up the sums of
    // the blocks before it
    int64_t run_off = 0;
    if (a.scanned) {
        constexpr int CH = MAX_BLOCKS / SCAN_BLOCK;
        const int c0 = (int)blockIdx.x / CH * CH;
        run_off = a.chunk_off[blockIdx.x / CH];
#pragma unroll
        for (int q = 0; q < CH - 1; ++q)
            if (c0 + q < (int)blockIdx.x) run_off += a.block_sum[c0 + q];
    } else {
        int64_t part = 0;
        int32_t partb = 0;
        const bool last = blockIdx.x == gridDim.x - 1;
        for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += BLOCK) {
            part += a.block_sum[b];
            if (last) partb += a.block_bad[b];
        }
        for (int d = WAVE / 2; d > 0; d >>= 1) {
            part += shfl_i64(part, wlane ^ d);
            partb += __shfl(partb, wlane ^ d);
        }
        if (wlane == 0) {
            s_red[wid] = part;
            s_redb[wid] = partb;
        }
        __syncthreads();
        int32_t bad_total = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            run_off += s_red[q];
            bad_total += s_redb[q];
        }
        if (last && threadIdx.x == 0) {
            const int64_t E = run_off + a.block_sum[blockIdx.x];
            a.counts[0] = S;
            a.counts[1] = E;
            a.counts[2] = bad_total + a.block_bad[blockIdx.x];
            a.root_start_ptr[S] = E;
            a.root_end_ptr[S] = E;
        }
    }
    // one slot of the hop: its two offsets, then its edges (copied, or picked and copied)
    auto emit_slot = [&](int64_t slot, bool active, int64_t start, int64_t len, int64_t t, int32_t c, int64_t off) {
            if (active && lig == 0) {
                a.root_start_ptr[slot] = off;
                a.root_end_ptr[slot] = off + c;
            }
            if (G == WAVE && k > G) {
                // ---- uniform with a fanout beyond one wavefront (a wave per slot, picks in dynamic LDS) ----
                // Block-uniform control flow (the loops run to k for every wave, idle waves skip the work),
                // so that block barriers order the LDS accesses of the sequential subset construction.
                extern __shared__ int64_t s_wide[];
                int64_t* pk = s_wide + (size_t)wid * k;
                const bool draw = active && len > k;
                auto emit = [&](int64_t sel, int64_t place) {
                    const Edge ed = load_picked_edge(a, start + sel);
                    a.nbr[off + place] = ed.col;
                    if (a.mark != nullptr) mark_id(a, ed.col);
                    a.nbr_ts[off + place] = a.keep_root_time ? t : ed.ts;
                    a.nbr_eid[off + place] = ed.eid;
                    a.nbr_dt[off + place] = ed.ts - t;
                    if (a.hint_out != nullptr) a.hint_out[off + place] = ed.hint;
                };
                if (active && !draw)                      // the whole window, in storage order
                    for (int32_t j = lig; j < c; j += G) emit(j, j);
                if (draw)
                    for (int32_t j = lig; j < k; j += G) {
                        const uint64_t bits = draw_bits(a.seed, a.hop, slot, j);
                        pk[j] = a.replace ? bounded(bits, len) : bounded(bits, len - k + j + 1);
                    }
                __syncthreads();
                if (a.replace) {                          // kernel argument: uniform; draw order is kept
                    if (draw)
                        for (int32_t j = lig; j < k; j += G) emit(pk[j], j);
                } else {
                    // Floyd: step j keeps its draw unless an earlier step holds the same value, then it takes len-k+j
                    for (int32_t j = 1; j < k; ++j) {
                        bool dup = false;
                        if (draw) {
                            const int64_t cand = pk[j];
                            for (int32_t i = lig; i < j; i += G) dup |= pk[i] == cand;
                        }
                        dup = __any(dup);
                        __syncthreads();
                        if (draw && dup && lig == 0) pk[j] = len - k + j;
                        __syncthreads();
                    }
                    // ascending: the place of a pick is the number of smaller picks (all distinct)
                    if (draw)
                        for (int32_t j = lig; j < k; j += G) {
                            const int64_t mine = pk[j];
                            int32_t r = 0;
                            for (int32_t i = 0; i < k; ++i) r += pk[i] < mine ? 1 : 0;
                            emit(mine, r);
                        }
                }
                __syncthreads();                          // the picks are reused by the next iteration
            } else {
                // ---- uniform: k <= G ----------------------------------------------------
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
                        // Floyd: step j picks t_j from [0, len-k+j]; a repeat is replaced by len-k+j; rank among
                        // the k picks (all distinct) = output position
                        floyd_subset<G>(draw, lig, wlane, gshift, k, len, tj, &sel, &rank);
                    }
                }
                if (active && lig < c) {
                    const Edge ed = load_picked_edge(a, start + sel);
                    a.nbr[off + rank] = ed.col;
                    if (a.mark != nullptr) mark_id(a, ed.col);
                    a.nbr_ts[off + rank] = a.keep_root_time ? t : ed.ts;
                    a.nbr_eid[off + rank] = ed.eid;
                    a.nbr_dt[off + rank] = ed.ts - t;
                    if (a.hint_out != nullptr) a.hint_out[off + rank] = ed.hint;
                }
            }
    };
    int par = 0;
    for (int64_t it = first; it < first + run && it < S; it += SPB, par ^= 1) {
        // the next iteration's slot is loaded now, so that its latency runs beside this iteration's picks and copies
        const int64_t nslot = it + SPB + gib;
        const bool nactive = it + SPB < first + run && nslot < S;
        int64_t nstart = 0, nlen = 0, nt = 0;
        if (nactive) {
            nstart = a.w_start[nslot];
            nlen = a.w_len[nslot];
            nt = a.derive ? a.slot_ts_out[nslot] : a.slot_ts[nslot];
        }
        const int32_t c = (int32_t)(len < k ? len : k);
        // exclusive prefix of c over the iteration's slots: scan inside the wave (one
        // contribution per group), then add the totals of the waves before this one
        int32_t inc = (lig == 0) ? c : 0;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int32_t x = __shfl_up(inc, d);
            if (wlane >= d) inc += x;
        }
        if (wlane == WAVE - 1) s_wtot[par][wid] = inc;
        // exclusive prefix at the group's first lane, broadcast to the group
        const int32_t excl = __shfl(inc - ((lig == 0) ? c : 0), wlane - lig);
        __syncthreads();
        int32_t wave_off = 0, iter_total = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            const int32_t x = s_wtot[par][q];
            if (q < wid) wave_off += x;
            iter_total += x;
        }
        const int64_t off = run_off + wave_off + excl;
        run_off += iter_total;
        emit_slot(slot, active, start, len, t, c, off);
        slot = nslot;
        active = nactive;
        start = nstart;
        len = nlen;
        t = nt;
    }
}


// Most-recent copy with a lane per EDGE instead of a group of lanes per slot.  A block takes its run in chunks of
// FLAT_SLOTS slots: their counts are scanned into LDS (with the slots' window starts and times), then the chunk's
// edges are walked flat - edge x of the chunk belongs to the slot whose offsets enclose x (a 9-step search in LDS),
// comes from start + (x - offset) and goes to run offset + x.  Every lane has an edge whatever the slots hold
// (slots of deeper hops hold two edges on average on a power-law graph: a group of 8 lanes per slot left six idle),
// and the stores of a block-iteration are one contiguous piece per output array.
constexpr int FLAT_SLOTS = 2 * BLOCK;
static_assert((int64_t)FLAT_SLOTS * SGL_RECENT_MAX_FANOUT <= INT32_MAX, "a chunk's edge offsets are 32-bit");
struct FlatLds {      // the LDS of one block of the most-recent copy
    int64_t red[NWAVE];
    int64_t start[FLAT_SLOTS], t[FLAT_SLOTS];
    int32_t redb[NWAVE];
    int32_t w[NWAVE];
    int32_t off[FLAT_SLOTS + 1];
};
__device__ __forceinline__ void fill_flat_body(const HopArgs& a, unsigned bid, unsigned nblk, FlatLds& lds) {
    int64_t* const s_red = lds.red;
    int32_t* const s_redb = lds.redb;
    int32_t* const s_w = lds.w;
    int32_t* const s_off = lds.off;
    int64_t* const s_start = lds.start;
    int64_t* const s_t = lds.t;
    const int wlane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int32_t k = a.k;
    // Runs of up to 16 edges come from the graph's interleaved records when it has them: a run then lies in one
    // stretch of memory instead of one per array (slots of a deeper hop hold a few edges: three 64-byte sectors for
    // 16 useful bytes each become one or two); longer runs read fewer bytes from the arrays.
    const bool use_rec = a.rec != nullptr && k <= 16;
    const int64_t S = live_count(a.S_dev, a.S_max);
    int64_t first, run;
    block_run(S, a.align, &first, &run, bid, nblk);
    const int64_t run_end = first + run < S ? first + run : S;
    // the first chunk's slots (two consecutive ones per thread): loaded beside the block's offset
    constexpr int SPT = FLAT_SLOTS / BLOCK;      // consecutive slots per thread
    int64_t st[SPT], ln[SPT], tt[SPT];
    auto load_slots = [&](int64_t chunk0) {
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            const int64_t slot = chunk0 + SPT * threadIdx.x + q;
            st[q] = ln[q] = tt[q] = 0;
            if (slot < run_end) {
                slot_window(a, slot, &st[q], &ln[q]);
                st[q] += ln[q] > k ? ln[q] - k : 0;       // the last min(len, k) edges of the window
                tt[q] = a.derive ? a.slot_ts_out[slot] : a.slot_ts[slot];
            }
        }
    };
    load_slots(first);
    int64_t run_off = 0;
    if (a.scanned) {
        constexpr int CH = MAX_BLOCKS / SCAN_BLOCK;
        const int c0 = (int)bid / CH * CH;
        run_off = a.chunk_off[bid / CH];
#pragma unroll
        for (int q = 0; q < CH - 1; ++q)
            if (c0 + q < (int)bid) run_off += a.block_sum[c0 + q];
    } else {
        int64_t part = 0;
        int32_t partb = 0;
        const bool last = bid == nblk - 1;
        for (int64_t b = threadIdx.x; b < (int64_t)bid; b += BLOCK) {
            part += a.block_sum[b];
            if (last) partb += a.block_bad[b];
        }
        for (int d = WAVE / 2; d > 0; d >>= 1) {
            part += shfl_i64(part, wlane ^ d);
            partb += __shfl(partb, wlane ^ d);
        }
        if (wlane == 0) {
            s_red[wid] = part;
            s_redb[wid] = partb;
        }
        __syncthreads();
        int32_t bad_total = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            run_off += s_red[q];
            bad_total += s_redb[q];
        }
        if (last && threadIdx.x == 0) {
            const int64_t E = run_off + a.block_sum[bid];
            a.counts[0] = S;
            a.counts[1] = E;
            a.counts[2] = bad_total + a.block_bad[bid];
            a.root_start_ptr[S] = E;
            a.root_end_ptr[S] = E;
        }
    }
    for (int64_t chunk0 = first; chunk0 < run_end; chunk0 += FLAT_SLOTS) {      // block-uniform
        if (chunk0 != first) load_slots(chunk0);
        // exclusive prefix of the chunk's counts
        int32_t c[SPT], sum = 0;
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            c[q] = (int32_t)(ln[q] < k ? ln[q] : k);
            sum += c[q];
        }
        int32_t inc = sum;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int32_t y = __shfl_up(inc, d);
            if (wlane >= d) inc += y;
        }
        if (wlane == WAVE - 1) s_w[wid] = inc;
        __syncthreads();                 // (also: the previous chunk's edges are done with the LDS arrays)
        int32_t excl = inc - sum, total = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            const int32_t y = s_w[q];
            if (q < wid) excl += y;
            total += y;
        }
        if (threadIdx.x == 0) s_off[FLAT_SLOTS] = total;
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            const int j = SPT * threadIdx.x + q;
            s_off[j] = excl;
            s_start[j] = st[q];
            s_t[j] = tt[q];
            const int64_t slot = chunk0 + j;
            if (slot < run_end) {
                a.root_start_ptr[slot] = run_off + excl;
                a.root_end_ptr[slot] = run_off + excl + c[q];
            }
            excl += c[q];
        }
        __syncthreads();
        // the chunk's edges, flat: up to ROUNDS per lane, every load issued before the first store
        constexpr int ROUNDS = 4;
        for (int32_t x0 = threadIdx.x; x0 < total; x0 += ROUNDS * BLOCK) {
            int64_t ets[ROUNDS], dst[ROUNDS], id[ROUNDS], hnt[ROUNDS], tslot[ROUNDS];
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r) {
                const int32_t x = x0 + r * BLOCK;
                ets[r] = dst[r] = id[r] = hnt[r] = tslot[r] = 0;
                if (x < total) {
                    // the slot of edge x: the last one whose offset is <= x (empty slots share the offset of the
                    // slot after them, so the last one is the one that holds x)
                    int lo = 0;
#pragma unroll
                    for (int step = FLAT_SLOTS / 2; step > 0; step >>= 1)
                        lo += s_off[lo + step] <= x ? step : 0;
                    const int64_t e = s_start[lo] + (x - s_off[lo]);
                    tslot[r] = s_t[lo];
                    if (use_rec) {       // kernel argument: uniform across the launch
                        const Edge ed = load_picked_edge(a, e);
                        ets[r] = ed.ts; dst[r] = ed.col; id[r] = ed.eid; hnt[r] = ed.hint;
                    } else {
                        ets[r] = a.ts[e];
                        dst[r] = a.col[e];
                        id[r] = a.eid[e];
                        // (the entry out of the records when the graph has them: it carries the next window's length)
                        if (a.hint_out != nullptr) hnt[r] = a.rec != nullptr ? a.rec[4 * e + 3] : a.hint[e];
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r) {
                const int32_t x = x0 + r * BLOCK;
                if (x < total) {
                    const int64_t o = run_off + x;
                    a.nbr[o] = dst[r];
                    if (a.mark != nullptr) mark_id(a, dst[r]);
                    a.nbr_ts[o] = ets[r];
                    a.nbr_eid[o] = id[r];
                    a.nbr_dt[o] = ets[r] - tslot[r];
                    if (a.hint_out != nullptr) a.hint_out[o] = hnt[r];
                }
            }
        }
        run_off += total;
    }
}
__global__ __launch_bounds__(BLOCK) void fill_flat_kernel(HopArgs a) {
    __shared__ FlatLds lds;
    fill_flat_body(a, blockIdx.x, gridDim.x, lds);
}

// Uniform picks with a lane per PICK.  As fill_flat_kernel a block takes its run in chunks of SLOTS slots and walks
// the chunk's output edges flat; what differs is where an edge comes from.  A slot whose window holds at most k edges
// copies it whole.  For the others ("drawing" slots, listed compactly in LDS) the block first makes the k raw draws
// of every such slot, one (slot, draw) pair per lane - the generator is most of the cost, and with a group of lanes
// per slot the lanes of slots that do not draw (most slots of a deeper hop hold a handful of edges) idle through it
// - then a group of KP lanes turns a slot's draws into its ascending picks in place: rank = number of smaller draws;
// only in wavefronts where two draws of a slot are equal do the groups replay Floyd's construction first, stepping
// together (step j keeps its draw unless an earlier step holds that value, then it takes len - k + j; with 20 picks
// from windows of a few hundred edges most slots see such a pair, and one lane replaying it alone took three times
// as long as the whole rest of the hop).  Picks are kept as 32-bit offsets into the window; a window of 2^32 edges or
// more (no row of a graph this library can hold today) is picked by one lane into the slot's own output stretch.
// The k picks of one slot whose window has 2^32 edges or more, by one lane, into `row` (global memory: the slot's
// own k entries of an output array, which the copy that follows overwrites): Floyd's construction and an insertion
// sort, or the draws in their order when drawing with replacement.
__device__ __forceinline__ void huge_window_picks(const HopArgs& a, int64_t slot, int64_t len, int64_t* row) {
    const int32_t k = a.k;
    for (int32_t j = 0; j < k; ++j) {
        const uint64_t bits = draw_bits(a.seed, a.hop, slot, j);
        int64_t pj = a.replace ? bounded(bits, len) : bounded(bits, len - k + j + 1);
        if (!a.replace) {
            bool dup = false;
            for (int32_t i = 0; i < j; ++i) dup |= row[i] == pj;
            if (dup) pj = len - k + j;
        }
        row[j] = pj;
    }
    if (a.replace) return;
    for (int32_t x = 1; x < k; ++x) {
        const int64_t v = row[x];
        int32_t y = x - 1;
        while (y >= 0 && row[y] > v) {
            row[y + 1] = row[y];
            --y;
        }
        row[y + 1] = v;
    }
}

template <int SLOTS>
struct UniformFlatLds {      // the static LDS of one block of the uniform picks (the picks themselves are dynamic LDS)
    int64_t red[NWAVE];
    int64_t start[SLOTS], t[SLOTS], len[SLOTS];
    int32_t redb[NWAVE];
    int32_t w[NWAVE];
    int32_t off[SLOTS + 1];
    int32_t dl[SLOTS];
    int32_t didx[SLOTS];
};
template <int KP, int SLOTS, int ROUNDS>
__device__ __forceinline__ void fill_uniform_flat_body(const HopArgs& a, unsigned bid, unsigned nblk, UniformFlatLds<SLOTS>& lds) {
    static_assert(SLOTS % BLOCK == 0 && BLOCK % KP == 0 && KP % 4 == 0 && KP < WAVE, "chunk layout");
    constexpr int SPT = SLOTS / BLOCK;
    int64_t* const s_red = lds.red;
    int32_t* const s_redb = lds.redb;
    int32_t* const s_w = lds.w;
    int32_t* const s_off = lds.off;
    int64_t* const s_start = lds.start;
    int64_t* const s_t = lds.t;
    int64_t* const s_len = lds.len;
    int32_t* const s_dl = lds.dl;            // chunk-local index of the q-th drawing slot
    int32_t* const s_didx = lds.didx;        // slot -> its place in s_dl, -1: copies its window, -2: window >= 2^32 edges
    // a drawing slot's picks: rows of kp = fanout rounded up to 4 entries (16-byte rows), SLOTS rows, sized at the launch
    // (uniform_flat_lds): with rows of KP entries a block of the fanout-20 kernel held 41 KB of LDS and three blocks shared a CU
    extern __shared__ __attribute__((aligned(16))) uint32_t s_pick[];
    const int wlane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int32_t k = a.k;
    const int32_t kp = (k + 3) & ~3;
    const int64_t S = live_count(a.S_dev, a.S_max);
    int64_t first, run;
    block_run(S, a.align, &first, &run, bid, nblk);
    const int64_t run_end = first + run < S ? first + run : S;
    int64_t st[SPT], ln[SPT], tt[SPT];
    auto load_slots = [&](int64_t chunk0) {
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            const int64_t slot = chunk0 + SPT * threadIdx.x + q;
            st[q] = ln[q] = tt[q] = 0;
            if (slot < run_end) {
                slot_window(a, slot, &st[q], &ln[q]);
                tt[q] = a.derive ? a.slot_ts_out[slot] : a.slot_ts[slot];
            }
        }
    };
    load_slots(first);
    int64_t run_off = 0;
    if (a.scanned) {
        constexpr int CH = MAX_BLOCKS / SCAN_BLOCK;
        const int c0 = (int)bid / CH * CH;
        run_off = a.chunk_off[bid / CH];
#pragma unroll
        for (int q = 0; q < CH - 1; ++q)
            if (c0 + q < (int)bid) run_off += a.block_sum[c0 + q];
    } else {
        int64_t part = 0;
        int32_t partb = 0;
        const bool last = bid == nblk - 1;
        for (int64_t b = threadIdx.x; b < (int64_t)bid; b += BLOCK) {
            part += a.block_sum[b];
            if (last) partb += a.block_bad[b];
        }
        for (int d = WAVE / 2; d > 0; d >>= 1) {
            part += shfl_i64(part, wlane ^ d);
            partb += __shfl(partb, wlane ^ d);
        }
        if (wlane == 0) {
            s_red[wid] = part;
            s_redb[wid] = partb;
        }
        __syncthreads();
        int32_t bad_total = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            run_off += s_red[q];
            bad_total += s_redb[q];
        }
        if (last && threadIdx.x == 0) {
            const int64_t E = run_off + a.block_sum[bid];
            a.counts[0] = S;
            a.counts[1] = E;
            a.counts[2] = bad_total + a.block_bad[bid];
            a.root_start_ptr[S] = E;
            a.root_end_ptr[S] = E;
        }
    }
    constexpr int DSH = 20;                      // packed scan: edges in the low 20 bits (<= SLOTS * 64), drawing slots above
    for (int64_t chunk0 = first; chunk0 < run_end; chunk0 += SLOTS) {      // block-uniform
        if (chunk0 != first) load_slots(chunk0);
        int32_t c[SPT], sum = 0;
        bool dr[SPT];
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            c[q] = (int32_t)(ln[q] < k ? ln[q] : k);
            dr[q] = ln[q] > k;
            sum += c[q] + (dr[q] ? (1 << DSH) : 0);
        }
        int32_t inc = sum;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int32_t y = __shfl_up(inc, d);
            if (wlane >= d) inc += y;
        }
        if (wlane == WAVE - 1) s_w[wid] = inc;
        __syncthreads();                 // (also: the previous chunk's edges are done with the LDS arrays)
        int32_t excl = inc - sum, all = 0;
#pragma unroll
        for (int q = 0; q < NWAVE; ++q) {
            const int32_t y = s_w[q];
            if (q < wid) excl += y;
            all += y;
        }
        const int32_t total = all & ((1 << DSH) - 1), nd = all >> DSH;
        if (threadIdx.x == 0) s_off[SLOTS] = total;
#pragma unroll
        for (int q = 0; q < SPT; ++q) {
            const int j = SPT * threadIdx.x + q;
            const int32_t eoff = excl & ((1 << DSH) - 1), dpos = excl >> DSH;
            s_off[j] = eoff;
            s_start[j] = st[q];
            s_t[j] = tt[q];
            s_len[j] = ln[q];
            const bool huge = dr[q] && (ln[q] >> 32) != 0;
            s_didx[j] = dr[q] ? (huge ? -2 : dpos) : -1;
            if (dr[q]) s_dl[dpos] = huge ? -1 : j;
            const int64_t slot = chunk0 + j;
            if (slot < run_end) {
                a.root_start_ptr[slot] = run_off + eoff;
                a.root_end_ptr[slot] = run_off + eoff + c[q];
            }
            excl += c[q] + (dr[q] ? (1 << DSH) : 0);
        }
        __syncthreads();
        if (nd > 0) {                    // block-uniform
            // the raw draws, one (drawing slot, draw) pair per lane
            for (int32_t x = threadIdx.x; x < nd * k; x += BLOCK) {
                const int32_t di = x / k, d = x - di * k;
                const int j = s_dl[di];
                if (j >= 0) {
                    const int64_t len = s_len[j];
                    const uint64_t bits = draw_bits(a.seed, a.hop, chunk0 + j, d);
                    s_pick[di * kp + d] = (uint32_t)(a.replace ? bounded(bits, len) : bounded(bits, len - k + d + 1));
                }
            }
            // (windows of 2^32 edges or more: 64-bit picks, parked in the slot's own stretch of the output)
            for (int j = threadIdx.x; j < SLOTS; j += BLOCK)
                if (s_didx[j] == -2) huge_window_picks(a, chunk0 + j, s_len[j], &a.nbr_dt[run_off + s_off[j]]);
            __syncthreads();
            if (!a.replace) {
                // ascending picks in place, a group of KP lanes per drawing slot (all inside one wavefront, whose LDS
                // accesses are served in program order: the group reads its row, then writes it)
                const int lig = threadIdx.x % KP;
                const int gsh = wlane / KP * KP;
                // rank of `v` among the k values of row `di` (how many are smaller), and how many equal it
                auto count = [&](int32_t di, uint32_t v, int32_t* smaller, int32_t* equal) {
                    int32_t r = 0, e = 0;
                    for (int32_t q = 0; q < k; q += 4) {
                        const uint4 o = *reinterpret_cast<const uint4*>(&s_pick[di * kp + q]);
                        r += (o.x < v ? 1 : 0) + ((q + 1 < k && o.y < v) ? 1 : 0) + ((q + 2 < k && o.z < v) ? 1 : 0) +
                             ((q + 3 < k && o.w < v) ? 1 : 0);
                        e += (o.x == v ? 1 : 0) + ((q + 1 < k && o.y == v) ? 1 : 0) + ((q + 2 < k && o.z == v) ? 1 : 0) +
                             ((q + 3 < k && o.w == v) ? 1 : 0);
                    }
                    *smaller = r;
                    *equal = e;
                };
                auto wave_sync = [] {          // orders this wavefront's LDS accesses before and after
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                };
                for (int32_t di0 = 0; di0 < nd; di0 += BLOCK / KP) {           // block-uniform trip count
                    const int32_t di = di0 + (int)threadIdx.x / KP;
                    const bool on = di < nd && s_dl[di < nd ? di : 0] >= 0;
                    const bool mine_on = on && lig < k;
                    uint32_t m = mine_on ? s_pick[di * kp + lig] : 0xFFFFFFFFu;
                    int32_t r = 0, e = 0;
                    if (on) count(di, m, &r, &e);
                    if (__any(mine_on && e > 1)) {
                        // two equal draws somewhere in the wavefront: Floyd's construction, the groups stepping together -
                        // step j keeps its draw unless an earlier step holds that value, then it takes len - k + j
                        const int64_t len = on ? s_len[s_dl[di]] : 0;
                        for (int32_t jj = 1; jj < k; ++jj) {
                            const uint32_t cand = (uint32_t)__shfl((int)m, gsh + jj);
                            const bool hit = group_ballot<KP>(mine_on && lig < jj && m == cand, gsh) != 0;
                            if (mine_on && lig == jj && hit) m = (uint32_t)(len - k + jj);
                        }
                        wave_sync();
                        if (mine_on) s_pick[di * kp + lig] = m;
                        wave_sync();
                        if (on) count(di, m, &r, &e);
                    }
                    wave_sync();
                    if (mine_on) s_pick[di * kp + r] = m;      // (all distinct now: the rank is the place)
                }
            }
            __syncthreads();
        }
        // the chunk's edges, flat: up to ROUNDS per lane, every load issued before the first store (a chunk of
        // a deeper hop holds about as many edges as the block has lanes: more rounds only cost registers)
        for (int32_t x0 = threadIdx.x; x0 < total; x0 += ROUNDS * BLOCK) {
            Edge ed[ROUNDS];
            int64_t tslot[ROUNDS];
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r) {
                const int32_t x = x0 + r * BLOCK;
                ed[r] = Edge{0, 0, 0, -1};
                tslot[r] = 0;
                if (x < total) {
                    int lo = 0;
#pragma unroll
                    for (int step = SLOTS / 2; step > 0; step >>= 1)
                        lo += s_off[lo + step] <= x ? step : 0;
                    const int32_t j = x - s_off[lo], di = s_didx[lo];
                    int64_t sel = j;
                    if (di >= 0) {
                        sel = (int64_t)s_pick[di * kp + j];
                    } else if (di == -2) {
                        sel = a.nbr_dt[run_off + x];      // parked there by huge_window_picks (this lane overwrites it below)
                    }
                    tslot[r] = s_t[lo];
                    ed[r] = load_picked_edge(a, s_start[lo] + sel);
                }
            }
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r) {
                const int32_t x = x0 + r * BLOCK;
                if (x < total) {
                    const int64_t o = run_off + x;
                    a.nbr[o] = ed[r].col;
                    if (a.mark != nullptr) mark_id(a, ed[r].col);
                    a.nbr_ts[o] = a.keep_root_time ? tslot[r] : ed[r].ts;
                    a.nbr_eid[o] = ed[r].eid;
                    a.nbr_dt[o] = ed[r].ts - tslot[r];
                    if (a.hint_out != nullptr) a.hint_out[o] = ed[r].hint;
                }
            }
        }
        run_off += total;
    }
}
template <int KP, int SLOTS, int ROUNDS>
__global__ __launch_bounds__(BLOCK) void fill_uniform_flat_kernel(HopArgs a) {
    __shared__ UniformFlatLds<SLOTS> lds;
    fill_uniform_flat_body<KP, SLOTS, ROUNDS>(a, blockIdx.x, gridDim.x, lds);
}
// A most-recent and a uniform fill of the same hop over grids of the same size in one launch (see count_lane_dual_kernel):
// even blocks copy windows for `r`, odd blocks pick for `u`.
template <int KP, int SLOTS, int ROUNDS>
__global__ __launch_bounds__(BLOCK) void fill_dual_kernel(HopArgs r, HopArgs u) {
    __shared__ union {       // a block runs one of the two
        FlatLds r;
        UniformFlatLds<SLOTS> u;
    } lds;
    const unsigned bid = blockIdx.x >> 1, nblk = gridDim.x >> 1;
    if (blockIdx.x & 1) fill_uniform_flat_body<KP, SLOTS, ROUNDS>(u, bid, nblk, lds.u);
    else fill_flat_body(r, bid, nblk, lds.r);
}

// Lanes per slot of the uniform strategy's draws (fanout <= G: one lane per draw).  The most-recent strategy
// copies with a lane per edge (fill_flat_kernel); the figure returned for it only steers the group of its
// window search (pick_search_group) and the alignment of the blocks' runs.
int pick_group(const sgl_sample_params* p, int64_t S_max) {
    if (p->type == SGL_SAMPLE_UNIFORM) {
        if (p->fanout <= 16) return 16;
        if (p->fanout <= 32) return 32;
        return 64;
    }
    return S_max >= 32768 ? 8 : 16;
}

// Lanes per slot of the window search.  A hop that fits a few wave-residency rounds is
// bound by the length of one slot's chain of dependent loads: the G lanes of the copy
// group search together, (G+1)-ary.  A hop of several hundred thousand slots is bound by
// the number of loads in flight and by their count: one lane per slot (plain binary
// search) keeps 8x the slots in flight and issues ~2.5x fewer loads than 8 lanes do
// (857k slots over rows of up to 1M edges: 187 us against 330 us).
int pick_search_group(int Gf, int64_t S_max) {
    if (S_max >= 131072) return 1;
    if (S_max >= 32768 && Gf > 8) return 8;   // as the recent strategy: one wave-residency round for the search
    return Gf;
}

constexpr size_t hop_workspace_bytes(int64_t S_max) {
    size_t b = 0;
    b += align_up((size_t)(S_max + 1) * 8) * 2;
    b += align_up((size_t)MAX_BLOCKS * 8);
    b += align_up((size_t)MAX_BLOCKS * 4);
    b += align_up((size_t)SCAN_BLOCK * 8);
    return b + 1024;
}

int32_t check_params(const sgl_sample_params* p) {
    if (!p) return fail(SGL_EINVAL, "sample: params is NULL");
    if (p->type != SGL_SAMPLE_RECENT && p->type != SGL_SAMPLE_UNIFORM)
        return fail(SGL_ENOTSUP, "undefined sampling strategy");
    if (p->fanout < 0) return fail(SGL_EINVAL, "sample: fanout < 0");
    if (p->mark_state && (p->mark_universe < 0 || p->mark_universe > 0xFFFFFFFFll))
        return fail(SGL_EINVAL, "sample: bad mark_universe");
    if (p->type == SGL_SAMPLE_UNIFORM && p->fanout > SGL_UNIFORM_MAX_FANOUT)
        return fail(SGL_ENOTSUP, "uniform fanout %d > %d", p->fanout, SGL_UNIFORM_MAX_FANOUT);
    // (fill_flat_kernel keeps the edge offsets of a chunk of FLAT_SLOTS slots in 32 bits)
    if (p->type == SGL_SAMPLE_RECENT && p->fanout > SGL_RECENT_MAX_FANOUT)
        return fail(SGL_ENOTSUP, "recent fanout %d > %d", p->fanout, SGL_RECENT_MAX_FANOUT);
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

using HopKernel = void (*)(HopArgs);

// dynamic LDS of fill_uniform_flat_kernel: UFLAT_SLOTS rows of the fanout rounded up to 4 picks
constexpr int UFLAT_SLOTS = 256;
inline size_t uniform_flat_lds(int32_t k) { return (size_t)UFLAT_SLOTS * ((k + 3) & ~3) * sizeof(uint32_t); }


HopKernel count_fn(int G) {
    switch (G) {
        case 1: return count_lane_kernel;
        case 2: return count_kernel<2>;
        case 4: return count_kernel<4>;
        case 8: return count_kernel<8>;
        case 16: return count_kernel<16>;
        case 32: return count_kernel<32>;
        default: return count_kernel<64>;
    }
}

HopKernel fill_fn(int G, bool uniform) {
    if (uniform) {
        switch (G) {
            case 16: return fill_uniform_flat_kernel<16, UFLAT_SLOTS, 2>;
            case 32: return fill_uniform_flat_kernel<32, UFLAT_SLOTS, 4>;
            default: return fill_kernel<64>;      // fanouts beyond 32: a wavefront per slot
        }
    }
    return fill_flat_kernel;
}

// Gc lanes per slot search, Gf lanes per slot copy or draw.  do_count / do_fill: the two halves of a hop; a second
// query over the same slots with the same window rule and fanout runs only the fill, on the first query's
// window arrays and block sums (same grid and run alignment: hop_grid).
constexpr int64_t LANE_MAX_BLOCKS = 2048;
struct HopGrid {
    int32_t align;
    int64_t blocks;
};
HopGrid hop_grid(int64_t S_max, int Gc, int Gf) {
    HopGrid hg;
    hg.align = BLOCK / (Gc < Gf ? Gc : Gf);
    hg.blocks = ceil_div<int64_t>(S_max > 0 ? S_max : 1, hg.align);
    if (hg.blocks > MAX_BLOCKS) hg.blocks = MAX_BLOCKS;
    // hops of the lane-per-slot kernels: eight blocks per CU, each walking its run in several trips (the two hop-2
    // counting kernels of a 16-batch pass 17.7 -> 9.2 us, the fills 2-5 % shorter, against a block per 256 slots of capacity)
    if (Gc == 1 && hg.blocks > LANE_MAX_BLOCKS) hg.blocks = LANE_MAX_BLOCKS;
    return hg;
}

int32_t launch_hop(HopArgs a, hipStream_t st, int Gc, int Gf, bool do_count = true, bool do_fill = true) {
    const HopGrid hg = hop_grid(a.S_max, Gc, Gf);
    a.align = hg.align;
    const int64_t blocks = hg.blocks;
    // a block counts the edges of its run of slots in 32 bits (count_kernel's partial sums, scan_kernel's staging)
    const int64_t run = ceil_div<int64_t>(ceil_div<int64_t>(a.S_max > 0 ? a.S_max : 1, blocks), a.align) * a.align;
    if (a.k > 0 && run > (int64_t)INT32_MAX / a.k)
        return fail(SGL_ENOTSUP, "sample: %lld slots x fanout %d exceed what a block counts in 32 bits", (long long)a.S_max, a.k);
    a.scanned = blocks > FUSED_PREFIX_MAX ? 1 : 0;
    a.lean = (a.type == SGL_SAMPLE_UNIFORM && Gf > 32) ? 0 : 1;      // the flat fill kernels read a window through slot_window
    if (do_count) {
        hipLaunchKernelGGL(count_fn(Gc), dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
        SGL_LAUNCH_CHECK();
        if (a.scanned) {
            hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, a, (int)blocks);
            SGL_LAUNCH_CHECK();
        }
    }
    if (!do_fill) return SGL_OK;
    // a uniform fanout beyond one wavefront keeps a slot's picks in LDS (one wave per slot)
    size_t wide_lds = (a.type == SGL_SAMPLE_UNIFORM && a.k > WAVE) ? (size_t)NWAVE * a.k * sizeof(int64_t) : 0;
    if (a.type == SGL_SAMPLE_UNIFORM && Gf <= 32) wide_lds = uniform_flat_lds(a.k);
    hipLaunchKernelGGL(fill_fn(Gf, a.type == SGL_SAMPLE_UNIFORM), dim3((unsigned)blocks), dim3(BLOCK), wide_lds, st, a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}


// ---------------------------------------------------------------------------------------
// Two hops in one launch, for the latency regime (a few thousand to
// 32768 root slots, fanout <= 16): the multi-launch path spends most of such a call on launch
// floors and on re-reading what the previous kernel just wrote.
//
// A group of 16 lanes owns one root slot.  The group finds the root's window together and
// takes its c <= k edges, one per lane; lane j then finds the window of "its" hop-2 slot
// (neighbour j at its timestamp) with a plain binary search, so a root and all its hop-2
// slots are counted without leaving registers.  Output offsets need the number of edges of
// all earlier slots: the block publishes its totals in a 64-bit descriptor right after its
// searches and adds up the descriptors of all blocks before it as they appear (a block waits
// only for blocks with a smaller index, which the dispatcher started no later than itself,
// and for nothing those blocks wait for).  The wait is bounded: after `spin_limit` polls
// a lane gives up and counts[2] of hop 0 is poisoned, so every wave exits whatever happens.  Then the group writes
// hop 1 (one edge per lane) and copies each hop-2 slot's edges with all its lanes.
//
// Descriptor: published flag (2 bits) | bad root slots (16) | hop-1 edges (22) | hop-2 edges (24);
// the fields cannot overflow for <= 32768 slots and fanout <= 16, so packed values add.
constexpr int FG = 16;
constexpr int FSPB = BLOCK / FG;
constexpr int64_t FUSED_MAX_SLOTS = 32768;
constexpr uint64_t ST_AGG = 1ull << 62, ST_MASK = 3ull << 62;
constexpr int SH_E0 = 24, SH_BAD = 46;
constexpr uint64_t M_E1 = (1ull << 24) - 1, M_E0 = (1ull << 22) - 1, M_BAD = (1ull << 16) - 1;

struct Fused2Args {
    HopArgs h;            // graph, roots, parameters, hop-0 outputs
    int64_t* rsp1;        // hop-1 outputs
    int64_t* rep1;
    int64_t* nbr1;
    int64_t* nbr_ts1;
    int64_t* nbr_eid1;
    int64_t* nbr_dt1;
    int64_t* counts1;
    unsigned long long* desc;   // [gridDim] zeroed by fused_clear_kernel
    int32_t spin_limit;         // polls of one descriptor before a lane gives up
};

// Zeroes the block descriptors and the two error counts of a call (of both calls of a pair):
// counts0[2] takes atomic maxima (bad root slots from the last block, the poison value from any
// block that gave up its wait - in either order the poison stays), counts1[2] atomic adds.
__global__ void fused_clear_kernel(unsigned long long* desc, int n, int64_t* counts0, int64_t* counts1,
                                   int64_t* counts0_b, int64_t* counts1_b) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) desc[i] = 0ull;
    if (i == 0) {
        counts0[2] = 0;
        counts1[2] = 0;
        if (counts0_b != nullptr) counts0_b[2] = 0;
        if (counts1_b != nullptr) counts1_b[2] = 0;
    }
}

// What a lane carries from the counting half of the single-launch sampler (fused2_count: windows and
// counts of its root and of its hop-2 slot, the block's totals published) to the writing half
// (fused2_write: offsets from the totals of the blocks before, then the outputs).
struct F2Lane {
    int64_t v, t;                    // the root slot
    int64_t lo, hi;                  // its window (the two strategies of a pair share it)
    int64_t nbr, ets, id, t2;        // lane j's hop-1 edge and the time its hop-2 slot asks about
    int64_t start2, len2;            // that slot's window
    uint64_t gpre, btotal;           // packed counts: the groups of the block before this one, the whole block
    int32_t c, c2, inc2;
    bool in_range, e_on;
};

// `window`: the state the other strategy of a pair left for the same slot, when both ask for the same window
// (then the slot is not read and its row not searched again), else nullptr.
template <bool UNIFORM>
__device__ __forceinline__ void fused2_count(const Fused2Args& f, const int64_t b, F2Lane& s, const F2Lane* window) {
    const HopArgs& a = f.h;
    __shared__ uint64_t s_grp[FSPB];
    const int gib = threadIdx.x / FG, lig = threadIdx.x % FG;
    const int wlane = threadIdx.x % WAVE;
    const int gshift = wlane / FG * FG, gbase = wlane - lig;
    const int32_t k = a.k;
    const int64_t S = a.S_max;
    const int64_t slot = b * FSPB + gib;
    const bool in_range = slot < S;
    int64_t v = 0, t = 0, rh = -1;
    if (window != nullptr) {             // the other strategy of a pair has read the slot and found its window
        v = window->v;
        t = window->t;
    } else if (in_range) {
        load_slot(a, slot, &v, &t);
        rh = root_hint_of(a, slot);
    }
    const bool bad = in_range && (v < 0 || v >= a.n);
    const bool active = in_range && !bad;
    if (in_range && lig == 0) {
        a.slot_node_out[slot] = v;
        a.slot_ts_out[slot] = t;
        if (a.mark != nullptr) mark_id(a, v);
    }
    // ---- hop 1: the root's window, one edge per lane
    const int64_t eq = a.equal_root_time ? 1 : 0;
    int64_t lo = 0, hi = 0;
    if (window != nullptr) {
        lo = window->lo;
        hi = window->hi;
    } else {
        int64_t rs = 0, re = 0;
        if (active) {
            rs = a.row_ptr[v];
            re = a.row_ptr[v + 1];
        }
        // positive roots whose window end the caller knows are not searched
        const bool told = active && rh >= 0;
        hi = group_lower_bound<FG>(a.ts, rs, re, t + eq, lig, gshift, active && !told);
        if (told) hi = clamp_to_row(rh, rs, re);
        lo = rs;
        if (a.allowed_offset >= 0) lo = group_lower_bound<FG>(a.ts, rs, hi, t - a.allowed_offset, lig, gshift, active);
    }
    const int64_t len = hi - lo;
    const int32_t c = active ? (int32_t)(len < k ? len : k) : 0;
    const bool e_on = lig < c;
    int64_t pos = hi - c + lig;      // recent: the last c window edges, lane j takes the j-th of them
    if constexpr (UNIFORM) {
        // as fill_kernel: lane j draws, Floyd's subset, rank = output place; then the picks are
        // handed round so that lane j holds the pick of output place j
        const bool draw = active && len > k;
        int64_t sel = lig;
        int32_t rank = lig;
        if (__any(draw)) {
            int64_t tj = 0;
            if (draw && lig < k) {
                const uint64_t bits = draw_bits(a.seed, 0, slot, lig);
                tj = a.replace ? bounded(bits, len) : bounded(bits, len - k + lig + 1);
            }
            if (a.replace) {
                if (draw) sel = tj;
            } else {
                floyd_subset<FG>(draw, lig, wlane, gshift, k, len, tj, &sel, &rank);
            }
            int64_t placed = sel;
            for (int32_t j = 0; j < k; ++j) {
                const int64_t sj = shfl_i64(sel, gbase + j);
                const int32_t rj = __shfl(rank, gbase + j);
                if (rj == lig) placed = sj;
            }
            sel = placed;
        }
        pos = lo + sel;
    }
    int64_t nbr = 0, ets = 0, id = 0, hint = -1;
    if (e_on) {
        if constexpr (UNIFORM) {
            const Edge ed = load_picked_edge(a, pos);
            nbr = ed.col; ets = ed.ts; id = ed.eid;
            if (a.hint != nullptr) hint = ed.hint;
        } else if (a.rec != nullptr) {
            // the lane's one hop-1 edge out of the graph's records: one 32-byte access instead of a sector per array,
            // and an index entry that carries the length of the hop-2 window
            const Edge ed = load_picked_edge(a, pos);
            nbr = ed.col; ets = ed.ts; id = ed.eid;
            if (a.hint != nullptr) hint = ed.hint;
        } else {
            nbr = a.col[pos];
            ets = a.ts[pos];
            id = a.eid[pos];
            if (a.hint != nullptr) hint = a.hint[pos];
        }
    }
    // ---- hop 2: lane j counts the slot (neighbour j, its timestamp - or the root's, keep_root_time)
    const int64_t t2 = (UNIFORM && a.keep_root_time) ? t : ets;
    int64_t start2 = 0, len2 = 0;
    int32_t c2 = 0;
    if (e_on) {
        if (nbr >= 0 && nbr < a.n) {
            // the window of (neighbour, its edge's time) ends where the graph's next-hop index says:
            // no search (strictly-before windows only; a uniform call that keeps the root's time asks
            // about another time and searches)
            const bool hinted = hint >= 0 && eq == 0 && t2 == ets;
            const int64_t hl = hinted ? hint_len(hint) : -1, hp = hint_pos(hint);
            int64_t lo2, hi2;
            if (hl >= 0 && hl <= hp && hp <= a.m && a.allowed_offset < 0) {
                // the entry came out of an edge record and carries the window's length: no row pointer is read
                hi2 = hp;
                lo2 = hp - hl;
            } else {
                const int64_t rs2 = a.row_ptr[nbr], re2 = a.row_ptr[nbr + 1];
                hi2 = hinted ? clamp_to_row(hint, rs2, re2) : lane_lower_bound(a.ts, rs2, re2, t2 + eq);
                lo2 = rs2;
                if (a.allowed_offset >= 0) lo2 = lane_lower_bound(a.ts, rs2, hi2, t2 - a.allowed_offset);
            }
            len2 = hi2 - lo2;
            c2 = (int32_t)(len2 < k ? len2 : k);
            start2 = UNIFORM ? lo2 : hi2 - c2;
        } else {
            atomicAdd(reinterpret_cast<unsigned long long*>(&f.counts1[2]), 1ull);
        }
    }
    // exclusive prefix of c2 inside the group, group total
    int32_t inc2 = c2;
    for (int d = 1; d < FG; d <<= 1) {
        const int32_t x = __shfl_up(inc2, d, FG);
        if (lig >= d) inc2 += x;
    }
    const int32_t C2 = __shfl(inc2, FG - 1, FG);
    if (lig == 0) s_grp[gib] = ((uint64_t)(bad ? 1 : 0) << SH_BAD) | ((uint64_t)c << SH_E0) | (uint64_t)C2;
    __syncthreads();
    uint64_t gpre = 0, btotal = 0;
#pragma unroll
    for (int q = 0; q < FSPB; ++q) {
        const uint64_t x = s_grp[q];
        if (q < gib) gpre += x;
        btotal += x;
    }
    // ---- totals of all earlier blocks: publish this block's, then add up theirs as they appear
    // (every block publishes right after its searches, so nobody waits for a chain of blocks)
    if (threadIdx.x == 0)
        __hip_atomic_store(&f.desc[b], ST_AGG | btotal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.v = v; s.t = t; s.lo = lo; s.hi = hi;
    s.nbr = nbr; s.ets = ets; s.id = id; s.t2 = t2;
    s.start2 = start2; s.len2 = len2;
    s.gpre = gpre; s.btotal = btotal;
    s.c = c; s.c2 = c2; s.inc2 = inc2;
    s.in_range = in_range; s.e_on = e_on;
}

// `b` of `nb`: the block's index among the blocks of this call (set by the kernels below)
// PRE: hop-2 slots of a most-recent call whose edges are loaded while the block waits for the
// totals of the blocks before it (6 registers per slot).  s_pick: k * BLOCK entries of dynamic LDS
// (uniform only): the draws of a hop-2 slot are made by the slot's lane; its k picks live there, pick-major.
template <bool UNIFORM, int PRE>
__device__ __forceinline__ void fused2_write(const Fused2Args& f, const int64_t b, const int64_t nb, int64_t* s_pick,
                                             const F2Lane& s) {
    const HopArgs& a = f.h;
    __shared__ uint64_t s_red[NWAVE];
    __shared__ int s_gave[NWAVE];
    const int lig = threadIdx.x % FG;
    const int wlane = threadIdx.x % WAVE;
    const int gshift = wlane / FG * FG, gbase = wlane - lig;
    const int32_t k = a.k;
    const int64_t S = a.S_max;
    const int64_t slot = b * FSPB + threadIdx.x / FG;
    const bool in_range = s.in_range, e_on = s.e_on;
    const int64_t t = s.t, nbr = s.nbr, ets = s.ets, id = s.id, t2 = s.t2, start2 = s.start2, len2 = s.len2;
    const uint64_t gpre = s.gpre, btotal = s.btotal;
    const int32_t c = s.c, c2 = s.c2, inc2 = s.inc2;
    // recent: what a hop-2 slot copies is known before its output place is, so the loads are issued
    // now (after the block has published) and are in flight while it waits for the totals of the blocks before it
    constexpr int NPRE = (UNIFORM || PRE == 0) ? 1 : PRE;
    int64_t pre_ts[NPRE], pre_col[NPRE], pre_eid[NPRE];
    if constexpr (!UNIFORM) {
#pragma unroll
        for (int j = 0; j < PRE; ++j) {
            pre_ts[j] = pre_col[j] = pre_eid[j] = 0;
            if (j < k) {
                const int64_t st2 = shfl_i64(start2, gbase + j);
                const int32_t cc = __shfl(c2, gbase + j);
                if (j < c && lig < cc) {
                    // (from the records when the graph has them: a hop-2 slot holds an edge or two, one memory sector
                    // of records against one per array)
                    const Edge ed = load_picked_edge(a, st2 + lig);
                    pre_ts[j] = ed.ts;
                    pre_col[j] = ed.col;
                    pre_eid[j] = ed.eid;
                }
            }
        }
    }
    uint64_t part = 0;
    int gave_up = 0;
    for (int64_t idx = threadIdx.x; idx < b; idx += BLOCK) {
        uint64_t d;
        int spins = 0;
        while (((d = __hip_atomic_load(&f.desc[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) & ST_MASK) == 0) {
            if (++spins > f.spin_limit) {
                gave_up = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        part += d & ~ST_MASK;
    }
    for (int dd = WAVE / 2; dd > 0; dd >>= 1) {
        part += (uint64_t)shfl_i64((int64_t)part, wlane ^ dd);
        gave_up |= __shfl(gave_up, wlane ^ dd);
    }
    if (wlane == 0) {
        s_red[threadIdx.x / WAVE] = part;
        s_gave[threadIdx.x / WAVE] = gave_up;
    }
    __syncthreads();
    uint64_t prefix = 0;
    gave_up = 0;
#pragma unroll
    for (int q = 0; q < NWAVE; ++q) {
        prefix += s_red[q];
        gave_up |= s_gave[q];
    }
    if (threadIdx.x == 0) {
        // poisoned: reading the result reports an error (a maximum, so that the last block's count
        // of bad slots cannot replace it, whichever block writes first)
        if (gave_up) {
            atomicMax(reinterpret_cast<long long*>(&a.counts[2]), (long long)INT64_MAX);
            if (a.mark != nullptr) remap_poison(a.mark, a.mark_universe);   // the ids recorded there are void too
        }
        if (b == nb - 1) {            // totals of the call
            const uint64_t tot = prefix + btotal;
            const int64_t E0 = (int64_t)((tot >> SH_E0) & M_E0), E1 = (int64_t)(tot & M_E1);
            a.counts[0] = S;
            a.counts[1] = E0;
            atomicMax(reinterpret_cast<long long*>(&a.counts[2]), (long long)((tot >> SH_BAD) & M_BAD));
            a.root_start_ptr[S] = E0;
            a.root_end_ptr[S] = E0;
            f.counts1[0] = E0;
            f.counts1[1] = E1;
            f.rsp1[E0] = E1;
            f.rep1[E0] = E1;
        }
    }
    const uint64_t P = prefix + gpre;
    const int64_t off1 = (int64_t)((P >> SH_E0) & M_E0);
    const int64_t off2 = (int64_t)(P & M_E1) + (inc2 - c2);
    // ---- hop-1 outputs
    if (in_range && lig == 0) {
        a.root_start_ptr[slot] = off1;
        a.root_end_ptr[slot] = off1 + c;
    }
    if (e_on) {
        const int64_t o = off1 + lig;
        a.nbr[o] = nbr;
        if (a.mark != nullptr) mark_id(a, nbr);
        a.nbr_ts[o] = t2;
        a.nbr_eid[o] = id;
        a.nbr_dt[o] = ets - t;
        f.rsp1[o] = off2;
        f.rep1[o] = off2 + c2;
    }
    if constexpr (UNIFORM) {
        // the draws of hop-2 slot (off1 + lig), by its lane: the slot index is the counter of the
        // generator, so they can only be made now.  Picks ascend (Floyd + insertion sort), or keep
        // the draw order when drawing with replacement.
        const bool draw2 = e_on && len2 > k;
        const uint32_t dmask = (uint32_t)group_ballot<FG>(draw2, gshift);    // the group's drawing slots
        if (__any(draw2)) {
            // 1. the raw draws of all drawing slots of the group, spread over its 16 lanes (the
            //    generator is most of the cost: a lane that drew all k of its own slot would leave
            //    the lanes of non-drawing slots idle for k rounds)
            const int nd = __popc(dmask);
            for (int d = lig; __any(d < nd * k); d += FG) {
                if (d < nd * k) {
                    const int q = d / k, j = d - q * k;
                    uint32_t mm = dmask;                 // lane of the q-th drawing slot
                    for (int i = 0; i < q; ++i) mm &= mm - 1;
                    const int owner = __ffs(mm) - 1;
                    const uint64_t bits = draw_bits(a.seed, 1, off1 + owner, j);
                    s_pick[j * BLOCK + (threadIdx.x - lig) + owner] = (int64_t)bits;
                }
            }
        }
        __syncthreads();
        if (__any(draw2)) {
            // 2. the slot's lane turns its k raw draws into picks (registers, compile-time indices)
            //    and places them by rank
            int64_t pk[FG];
#pragma unroll
            for (int j = 0; j < FG; ++j) {
                pk[j] = INT64_MAX;
                if (j < k && draw2) {
                    const uint64_t bits = (uint64_t)s_pick[j * BLOCK + threadIdx.x];
                    if (a.replace) {
                        pk[j] = bounded(bits, len2);
                    } else {
                        int64_t pj = bounded(bits, len2 - k + j + 1);
                        bool dup = false;
#pragma unroll
                        for (int i = 0; i < j; ++i) dup |= pk[i] == pj;
                        pk[j] = dup ? len2 - k + j : pj;
                    }
                }
            }
            if (draw2) {
#pragma unroll
                for (int j = 0; j < FG; ++j) {
                    if (j < k) {
                        int32_t place = j;            // with replacement: the draw order
                        if (!a.replace) {             // distinct picks: ascending
                            place = 0;
#pragma unroll
                            for (int i = 0; i < FG; ++i) place += (i != j && pk[i] < pk[j]) ? 1 : 0;
                        }
                        s_pick[place * BLOCK + threadIdx.x] = pk[j];
                    }
                }
            }
        }
        if (e_on && !draw2)
            for (int32_t j = 0; j < c2; ++j) s_pick[j * BLOCK + threadIdx.x] = j;   // the whole window, in storage order
        __syncthreads();
    }
    // ---- hop-2 outputs: slot j of the group is copied by all its lanes (c2 <= k <= 16 edges)
    if constexpr (!UNIFORM) {
#pragma unroll
        for (int j = 0; j < PRE; ++j) {
            if (j < k) {
                const int64_t o2 = shfl_i64(off2, gbase + j) + lig;
                const int64_t tt = shfl_i64(t2, gbase + j);
                const int32_t cc = __shfl(c2, gbase + j);
                if (j < c && lig < cc) {
                    f.nbr1[o2] = pre_col[j];
                    if (a.mark != nullptr) mark_id(a, pre_col[j]);
                    f.nbr_ts1[o2] = pre_ts[j];
                    f.nbr_eid1[o2] = pre_eid[j];
                    f.nbr_dt1[o2] = pre_ts[j] - tt;
                }
            }
        }
    }
    // uniform, and the slots beyond the preloaded ones: four slots per pass with every load issued
    // before the first store
    constexpr int PASS = 4;
    for (int32_t j0 = UNIFORM ? 0 : PRE; j0 < k; j0 += PASS) {
        int64_t o2[PASS], tt[PASS], ets2[PASS], dst2[PASS], id2[PASS];
        bool on[PASS];
#pragma unroll
        for (int r = 0; r < PASS; ++r) {
            const int src = gbase + ((j0 + r) & (FG - 1));
            const int64_t st2 = shfl_i64(start2, src);
            o2[r] = shfl_i64(off2, src) + lig;
            tt[r] = shfl_i64(t2, src);
            const int32_t cc = __shfl(c2, src);
            on[r] = j0 + r < c && lig < cc;
            if (on[r]) {
                if constexpr (UNIFORM) {
                    const Edge ed = load_picked_edge(a, st2 + s_pick[lig * BLOCK + (threadIdx.x - lig) + ((j0 + r) & (FG - 1))]);
                    ets2[r] = ed.ts;
                    dst2[r] = ed.col;
                    id2[r] = ed.eid;
                } else {
                    const Edge ed = load_picked_edge(a, st2 + lig);
                    ets2[r] = ed.ts;
                    dst2[r] = ed.col;
                    id2[r] = ed.eid;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < PASS; ++r) {
            if (on[r]) {
                f.nbr1[o2[r]] = dst2[r];
                if (a.mark != nullptr) mark_id(a, dst2[r]);
                f.nbr_ts1[o2[r]] = (UNIFORM && a.keep_root_time) ? tt[r] : ets2[r];
                f.nbr_eid1[o2[r]] = id2[r];
                f.nbr_dt1[o2[r]] = ets2[r] - tt[r];
            }
        }
    }
}

template <bool UNIFORM, int PRE>
__device__ __forceinline__ void fused2_body(const Fused2Args& f, const int64_t b, const int64_t nb, int64_t* s_pick) {
    F2Lane s;
    fused2_count<UNIFORM>(f, b, s, nullptr);
    fused2_write<UNIFORM, PRE>(f, b, nb, s_pick, s);
}

template <bool UNIFORM>
__global__ __launch_bounds__(BLOCK) void fused2_kernel(Fused2Args f) {
    extern __shared__ int64_t s_dyn[];
    fused2_body<UNIFORM, 8>(f, blockIdx.x, gridDim.x, s_dyn);
}

// Two calls over the same roots in one launch, a most-recent and a uniform one: a group of lanes does both for
// its root, one after the other - the counting halves first (both calls' blocks have published their totals
// before any of them waits), then the writing halves.  Half the waves of two launches (or of one launch with a
// block per call and root group), and what such a kernel costs beside other kernels is the time its waves keep
// their slots: a step with three batches in flight takes 0.114 us longer for every 1000 wave-microseconds of
// waves that do nothing.  When both calls ask for the same window (same bounds rule, same hints) the second one
// takes slot and window from the first.
__global__ __launch_bounds__(BLOCK) void fused2_pair_kernel(Fused2Args fr, Fused2Args fu, int same_window) {
    extern __shared__ int64_t s_dyn[];
    const int64_t b = blockIdx.x, nb = gridDim.x;
    F2Lane sr, su;
    fused2_count<false>(fr, b, sr, nullptr);
    if (same_window)
        fused2_count<true>(fu, b, su, &sr);
    else
        fused2_count<true>(fu, b, su, nullptr);
    fused2_write<false, 0>(fr, b, nb, s_dyn, sr);
    fused2_write<true, 0>(fu, b, nb, s_dyn, su);
}

struct RootSpec {  // hop-0 slot source of the k-hop driver
    int64_t R, S_pos;
    const int64_t *roots, *ts_ptr, *root_ts, *neg_roots, *neg_ts;
    int64_t *slot_node_out, *slot_ts_out;
};

// The kernel arguments of one hop (its scratch carved out of `ws`), and the lanes per slot its two halves use.
struct PreparedHop {
    HopArgs a;
    int Gc, Gf;
};

int32_t prepare_hop(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts, const RootSpec* derive,
                    int64_t S_max, const int64_t* S_dev, const sgl_sample_params* p, const sgl_hop_out* out, void* ws,
                    size_t ws_bytes, const int64_t* slot_hint, int64_t* hint_out, bool hint_optional, PreparedHop* ph) {
    if (!derive && S_max > 0 && (!slot_node || !slot_ts)) return fail(SGL_EINVAL, "sample: slot array is NULL");
    if (ws_bytes < hop_workspace_bytes(S_max) || !ws)
        return fail(SGL_ENOMEM, "sample: workspace %zu < %zu bytes", ws_bytes, hop_workspace_bytes(S_max));
    Arena ar(ws, ws_bytes);
    HopArgs a{};
    a.n = g->n; a.m = g->m; a.row_ptr = g->row_ptr; a.col = g->col; a.ts = g->ts; a.eid = g->eid; a.hint = g->hop_hint; a.rec = g->rec;
    a.slot_node = slot_node; a.slot_ts = slot_ts; a.S_max = S_max; a.S_dev = S_dev;
    a.slot_hint = slot_hint; a.hint_out = hint_out; a.hint_optional = hint_optional ? 1 : 0;
    a.root_hint = (derive && !p->equal_root_time) ? p->root_hint : nullptr;
    a.derive = derive ? 1 : 0;
    if (derive) {
        a.R = derive->R; a.S_pos = derive->S_pos; a.roots = derive->roots; a.ts_ptr = derive->ts_ptr;
        a.root_ts = derive->root_ts; a.neg_roots = derive->neg_roots; a.neg_ts = derive->neg_ts;
        a.slot_node_out = derive->slot_node_out; a.slot_ts_out = derive->slot_ts_out;
    }
    a.type = p->type; a.k = p->fanout; a.allowed_offset = p->allowed_offset;
    a.equal_root_time = p->equal_root_time; a.keep_root_time = p->keep_root_time;
    a.replace = p->replace; a.hop = p->hop; a.seed = p->seed;
    a.mark = p->mark_state ? remap_flags(p->mark_state, p->mark_universe) : nullptr;
    a.mark_universe = p->mark_universe;
    a.mark_bytes = remap_byte_flags(p->mark_universe) ? 1 : 0;
    a.w_start = ar.take<int64_t>(S_max + 1);
    a.w_len = ar.take<int64_t>(S_max + 1);
    a.block_sum = ar.take<int64_t>(MAX_BLOCKS);
    a.block_bad = ar.take<int32_t>(MAX_BLOCKS);
    a.chunk_off = ar.take<int64_t>(SCAN_BLOCK);
    if (!ar.ok()) return fail(SGL_ENOMEM, "sample: workspace too small");
    a.root_start_ptr = out->root_start_ptr; a.root_end_ptr = out->root_end_ptr;
    a.nbr = out->neighbors; a.nbr_ts = out->neighbors_ts; a.nbr_eid = out->neighbors_eid;
    a.nbr_dt = out->neighbors_dt; a.counts = out->counts;
    ph->a = a;
    ph->Gf = pick_group(p, S_max);
    ph->Gc = pick_search_group(ph->Gf, S_max);
    return SGL_OK;
}

int32_t run_hop(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts, const RootSpec* derive,
                int64_t S_max, const int64_t* S_dev, const sgl_sample_params* p, const sgl_hop_out* out, void* ws,
                size_t ws_bytes, hipStream_t st, const int64_t* slot_hint = nullptr, int64_t* hint_out = nullptr,
                bool hint_optional = false, bool do_count = true) {
    PreparedHop ph;
    const int32_t rc = prepare_hop(g, slot_node, slot_ts, derive, S_max, S_dev, p, out, ws, ws_bytes, slot_hint, hint_out,
                                   hint_optional, &ph);
    if (rc != SGL_OK) return rc;
    return launch_hop(ph.a, st, ph.Gc, ph.Gf, do_count, true);
}

// The same hop of a most-recent query `r` and a uniform query `u` whose grids are the same, in launches that run
// the two side by side: one counting launch (or only the fill when the two share the counting pass: `u` then reads
// r's window arrays), one scan launch of two blocks, one fill launch.  false: the pair does not fit (the caller
// launches the hops one after the other).
bool dual_hop_fits(const PreparedHop& r, const PreparedHop& u) {
    if (r.a.type != SGL_SAMPLE_RECENT || u.a.type != SGL_SAMPLE_UNIFORM) return false;
    if (r.a.S_max != u.a.S_max || r.Gc != 1 || u.Gc != 1 || (u.Gf != 16 && u.Gf != 32)) return false;
    const HopGrid gr = hop_grid(r.a.S_max, r.Gc, r.Gf), gu = hop_grid(u.a.S_max, u.Gc, u.Gf);
    if (gr.align != gu.align || gr.blocks != gu.blocks) return false;
    const int64_t run = ceil_div<int64_t>(ceil_div<int64_t>(r.a.S_max > 0 ? r.a.S_max : 1, gr.blocks), gr.align) * gr.align;
    const int32_t kmax = r.a.k > u.a.k ? r.a.k : u.a.k;
    return !(kmax > 0 && run > (int64_t)INT32_MAX / kmax);
}

int32_t launch_dual_hop(PreparedHop r, PreparedHop u, hipStream_t st, bool shared_count) {
    const HopGrid hg = hop_grid(r.a.S_max, r.Gc, r.Gf);
    r.a.align = u.a.align = hg.align;
    const unsigned blocks = (unsigned)hg.blocks;
    r.a.scanned = u.a.scanned = hg.blocks > FUSED_PREFIX_MAX ? 1 : 0;
    r.a.lean = u.a.lean = 1;
    if (shared_count) {
        hipLaunchKernelGGL(count_lane_kernel, dim3(blocks), dim3(BLOCK), 0, st, r.a);
        SGL_LAUNCH_CHECK();
        if (r.a.scanned) {
            hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, r.a, (int)blocks);
            SGL_LAUNCH_CHECK();
        }
    } else {
        hipLaunchKernelGGL(count_lane_dual_kernel, dim3(2 * blocks), dim3(BLOCK), 0, st, r.a, u.a);
        SGL_LAUNCH_CHECK();
        if (r.a.scanned) {
            hipLaunchKernelGGL(scan_dual_kernel, dim3(2), dim3(SCAN_BLOCK), 0, st, r.a, u.a, (int)blocks);
            SGL_LAUNCH_CHECK();
        }
    }
    const size_t lds = uniform_flat_lds(u.a.k);
    if (u.Gf == 16) hipLaunchKernelGGL((fill_dual_kernel<16, UFLAT_SLOTS, 2>), dim3(2 * blocks), dim3(BLOCK), lds, st, r.a, u.a);
    else hipLaunchKernelGGL((fill_dual_kernel<32, UFLAT_SLOTS, 4>), dim3(2 * blocks), dim3(BLOCK), lds, st, r.a, u.a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}


Fused2Args fused2_args(const sgl_tcsr* g, const RootSpec* spec, int64_t S0, const sgl_sample_params* p,
                       const sgl_hop_out* outs, unsigned long long* desc) {
    Fused2Args f{};
    HopArgs& a = f.h;
    a.n = g->n; a.m = g->m; a.row_ptr = g->row_ptr; a.col = g->col; a.ts = g->ts; a.eid = g->eid; a.hint = g->hop_hint; a.rec = g->rec;
    a.S_max = S0; a.derive = 1;
    a.root_hint = p->equal_root_time ? nullptr : p->root_hint;
    a.R = spec->R; a.S_pos = spec->S_pos; a.roots = spec->roots; a.ts_ptr = spec->ts_ptr;
    a.root_ts = spec->root_ts; a.neg_roots = spec->neg_roots; a.neg_ts = spec->neg_ts;
    a.slot_node_out = spec->slot_node_out; a.slot_ts_out = spec->slot_ts_out;
    a.type = p->type; a.k = p->fanout; a.allowed_offset = p->allowed_offset;
    a.equal_root_time = p->equal_root_time; a.keep_root_time = p->keep_root_time;
    a.replace = p->replace; a.hop = 0; a.seed = p->seed;
    a.mark = p->mark_state ? remap_flags(p->mark_state, p->mark_universe) : nullptr;
    a.mark_universe = p->mark_universe;
    a.mark_bytes = remap_byte_flags(p->mark_universe) ? 1 : 0;
    a.root_start_ptr = outs[0].root_start_ptr; a.root_end_ptr = outs[0].root_end_ptr;
    a.nbr = outs[0].neighbors; a.nbr_ts = outs[0].neighbors_ts; a.nbr_eid = outs[0].neighbors_eid;
    a.nbr_dt = outs[0].neighbors_dt; a.counts = outs[0].counts;
    f.rsp1 = outs[1].root_start_ptr; f.rep1 = outs[1].root_end_ptr;
    f.nbr1 = outs[1].neighbors; f.nbr_ts1 = outs[1].neighbors_ts; f.nbr_eid1 = outs[1].neighbors_eid;
    f.nbr_dt1 = outs[1].neighbors_dt; f.counts1 = outs[1].counts;
    f.desc = desc;
    f.spin_limit = wait_limit();
    return f;
}

size_t pick_lds_bytes(int32_t k) { return (size_t)k * BLOCK * sizeof(int64_t); }

bool fused2_fits(int32_t layers, const sgl_sample_params* p, int64_t S0) {
    return layers == 2 && p->fanout >= 1 && p->fanout <= FG && S0 >= 1 && S0 <= FUSED_MAX_SLOTS &&
           !(p->flags & SGL_SAMPLE_MULTI_LAUNCH);
}

int32_t run_fused2(const sgl_tcsr* g, const RootSpec* spec, int64_t S0, const sgl_sample_params* p,
                   const sgl_hop_out* outs, void* ws, size_t ws_bytes, hipStream_t st) {
    if (ws_bytes < hop_workspace_bytes(S0) || !ws)
        return fail(SGL_ENOMEM, "sample: workspace %zu < %zu bytes", ws_bytes, hop_workspace_bytes(S0));
    Arena ar(ws, ws_bytes);
    const int blocks = (int)ceil_div<int64_t>(S0, FSPB);
    unsigned long long* desc = reinterpret_cast<unsigned long long*>(ar.take<int64_t>(blocks));
    if (!ar.ok()) return fail(SGL_ENOMEM, "sample: workspace too small");
    const Fused2Args f = fused2_args(g, spec, S0, p, outs, desc);
    hipLaunchKernelGGL(fused_clear_kernel, dim3((unsigned)ceil_div<int>(blocks, BLOCK)), dim3(BLOCK), 0, st, f.desc, blocks,
                       f.h.counts, f.counts1, (int64_t*)nullptr, (int64_t*)nullptr);
    SGL_LAUNCH_CHECK();
    if (p->type == SGL_SAMPLE_UNIFORM)
        hipLaunchKernelGGL(fused2_kernel<true>, dim3((unsigned)blocks), dim3(BLOCK), pick_lds_bytes(p->fanout), st, f);
    else
        hipLaunchKernelGGL(fused2_kernel<false>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, f);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

// a most-recent and a uniform call over the same roots: one launch (fused2_pair_kernel)
int32_t run_fused2_pair(const sgl_tcsr* g, const RootSpec* spec, int64_t S0, const sgl_sample_params* p_rec,
                        const sgl_hop_out* outs_rec, const sgl_sample_params* p_uni, const sgl_hop_out* outs_uni,
                        void* ws, size_t ws_bytes, hipStream_t st) {
    if (ws_bytes < 2 * hop_workspace_bytes(S0) || !ws)
        return fail(SGL_ENOMEM, "sample: workspace %zu < %zu bytes", ws_bytes, 2 * hop_workspace_bytes(S0));
    Arena ar(ws, ws_bytes);
    const int blocks = (int)ceil_div<int64_t>(S0, FSPB);
    unsigned long long* desc = reinterpret_cast<unsigned long long*>(ar.take<int64_t>(2 * (size_t)blocks));
    if (!ar.ok()) return fail(SGL_ENOMEM, "sample: workspace too small");
    const Fused2Args fr = fused2_args(g, spec, S0, p_rec, outs_rec, desc);
    const Fused2Args fu = fused2_args(g, spec, S0, p_uni, outs_uni, desc + blocks);
    hipLaunchKernelGGL(fused_clear_kernel, dim3((unsigned)ceil_div<int>(2 * blocks, BLOCK)), dim3(BLOCK), 0, st, desc,
                       2 * blocks, fr.h.counts, fr.counts1, fu.h.counts, fu.counts1);
    SGL_LAUNCH_CHECK();
    const int same_window = p_rec->allowed_offset == p_uni->allowed_offset &&
                            (p_rec->equal_root_time != 0) == (p_uni->equal_root_time != 0) &&
                            fr.h.root_hint == fu.h.root_hint;
    hipLaunchKernelGGL(fused2_pair_kernel, dim3((unsigned)blocks), dim3(BLOCK), pick_lds_bytes(p_uni->fanout), st,
                       fr, fu, same_window);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
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
    return run_hop(g, slot_node, slot_ts, nullptr, S_max, S_dev, p, out, ws, ws_bytes, as_stream(stream));
}

// ---- sgl_sample_hop_static: the hop's scratch (window starts and lengths, block sums) lives in
// device memory that belongs to the library image instead of a caller's workspace, for callers that
// cannot allocate.  Each GPU holds its own copy of the array; host code never uses the array's name
// as an address, only what hipGetSymbolAddress returned for the device that is current.
constexpr size_t STATIC_SCRATCH_BYTES = hop_workspace_bytes(SGL_STATIC_HOP_MAX_SLOTS);
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[STATIC_MAX_DEVICES];   // per device, resolved at the first call on it

int32_t static_scratch(void** out) {
    int dev = -1;
    SGL_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return fail(SGL_ENOTSUP, "sample_hop_static: device %d not supported", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        SGL_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return fail(SGL_EHIP, "sample_hop_static: no address for the scratch array on device %d", dev);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SGL_OK;
}
}  // namespace

extern "C" int32_t sgl_sample_hop_static(const sgl_tcsr* g, const int64_t* slot_node, const int64_t* slot_ts,
                                         int64_t S_max, const int64_t* S_dev, const sgl_sample_params* p,
                                         const sgl_hop_out* out, void* stream) {
    int32_t rc;
    if ((rc = check_graph(g)) != SGL_OK) return rc;
    if ((rc = check_params(p)) != SGL_OK) return rc;
    if (S_max < 0) return fail(SGL_EINVAL, "sample_hop_static: S_max < 0");
    if (S_max > SGL_STATIC_HOP_MAX_SLOTS)
        return fail(SGL_ENOMEM, "sample_hop_static: %lld slots exceed the limit of %lld (use sgl_sample_hop with a workspace)",
                    (long long)S_max, (long long)SGL_STATIC_HOP_MAX_SLOTS);
    if ((rc = check_out(out, S_max, p->fanout)) != SGL_OK) return rc;
    void* ws = nullptr;
    if ((rc = static_scratch(&ws)) != SGL_OK) return rc;
    // every word of the scratch that a launch reads was written by an earlier launch of the same call
    // (count_kernel writes the window arrays and block sums that scan/fill read): nothing to clear
    return run_hop(g, slot_node, slot_ts, nullptr, S_max, S_dev, p, out, ws, STATIC_SCRATCH_BYTES, as_stream(stream));
}

static int64_t worst_slots(int64_t S0, int32_t layer, int32_t k) {
    int64_t s = S0;
    for (int32_t l = 0; l < layer; ++l) {
        if (k != 0 && s > INT64_MAX / (k > 0 ? k : 1)) return INT64_MAX;
        s *= k;
    }
    return s;
}

// the two arrays through which a hop hands the index entries of its edges to the next hop's slots
static size_t hint_carry_bytes(int64_t worst) { return 2 * align_up((size_t)(worst + 1) * 8); }

extern "C" size_t sgl_sample_khop_workspace_bytes(int64_t S0, int32_t layers, int32_t fanout) {
    if (S0 < 0 || layers <= 0 || fanout < 0) return hop_workspace_bytes(0);
    int64_t worst = S0;
    for (int32_t l = 0; l < layers; ++l) {
        const int64_t s = worst_slots(S0, l, fanout);
        if (s > worst) worst = s;
    }
    return hop_workspace_bytes(worst) + (layers > 1 ? hint_carry_bytes(worst) : 0);
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
    if (R < 0 || S_pos < 0 || N_neg < 0 || layers < 1) return fail(SGL_EINVAL, "sample_khop: negative size or layers < 1");
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
    RootSpec spec{R, S_pos, roots, ts_ptr, root_ts, neg_roots, neg_ts, slot_node0, slot_ts0};
    if (fused2_fits(layers, p, S0)) return run_fused2(g, &spec, S0, p, outs, ws, ws_bytes, st);
    const int64_t* sn = nullptr;
    const int64_t* stt = nullptr;
    const int64_t* S_dev = nullptr;
    // With the graph's next-hop index the slots of hops >= 1 need no search: hop l stores the index
    // entry of every edge it emits, hop l+1 reads it as the end of that slot's window.  (Only for
    // strictly-before windows whose slot time is the edge's own time.)
    int64_t worst = S0;
    for (int32_t l = 0; l < layers; ++l) worst = worst_slots(S0, l, p->fanout) > worst ? worst_slots(S0, l, p->fanout) : worst;
    const size_t hop_ws = hop_workspace_bytes(worst);
    const bool carry = layers > 1 && g->hop_hint != nullptr && !p->equal_root_time &&
                       !(p->type == SGL_SAMPLE_UNIFORM && p->keep_root_time) && ws != nullptr &&
                       ws_bytes >= hop_ws + hint_carry_bytes(worst);
    int64_t* carry_buf[2] = {nullptr, nullptr};
    if (carry) {
        carry_buf[0] = reinterpret_cast<int64_t*>(static_cast<char*>(ws) + hop_ws);
        carry_buf[1] = reinterpret_cast<int64_t*>(static_cast<char*>(ws) + hop_ws + align_up((size_t)(worst + 1) * 8));
    }
    for (int32_t l = 0; l < layers; ++l) {
        sgl_sample_params pl = *p;
        pl.hop = l;
        const int64_t s_max = worst_slots(S0, l, p->fanout);
        rc = run_hop(g, sn, stt, l == 0 ? &spec : nullptr, s_max, S_dev, &pl, &outs[l], ws, carry ? hop_ws : ws_bytes, st,
                     (carry && l > 0) ? carry_buf[(l - 1) & 1] : nullptr, (carry && l + 1 < layers) ? carry_buf[l & 1] : nullptr);
        if (rc != SGL_OK) return rc;
        sn = outs[l].neighbors;
        stt = outs[l].neighbors_ts;
        S_dev = outs[l].counts + 1;
    }
    return SGL_OK;
}

extern "C" size_t sgl_sample_khop_multi_workspace_bytes(int64_t S0, int32_t layers, int32_t fanout, int32_t Q) {
    return (size_t)(Q > 0 ? Q : 1) * sgl_sample_khop_workspace_bytes(S0, layers, fanout);
}

extern "C" int32_t sgl_sample_khop_multi(const sgl_tcsr* g, int64_t R, const int64_t* roots,
                                         const int64_t* ts_ptr, int64_t S_pos, const int64_t* root_ts,
                                         int64_t N_neg, const int64_t* neg_roots, const int64_t* neg_ts,
                                         int32_t layers, int32_t Q, const sgl_sample_params* p,
                                         int64_t* slot_node0, int64_t* slot_ts0, const sgl_hop_out* outs,
                                         void* ws, size_t ws_bytes, void* stream) {
    if (Q < 0 || (Q > 0 && (!p || !outs)) || layers < 1) return fail(SGL_EINVAL, "sample_khop_multi: bad Q, layers or NULL argument");
    int32_t fan = 0;
    for (int32_t q = 0; q < Q; ++q) fan = p[q].fanout > fan ? p[q].fanout : fan;
    const int64_t S0 = (S_pos > 0 ? S_pos : 0) + (N_neg > 0 ? N_neg : 0);
    const size_t per = sgl_sample_khop_workspace_bytes(S0, layers, fan);
    if (Q > 0 && (!ws || ws_bytes < (size_t)Q * per))
        return fail(SGL_ENOMEM, "sample_khop_multi: workspace %zu < %zu bytes", ws_bytes, (size_t)Q * per);
    // one most-recent and one uniform 2-hop call of the single-launch size share a launch
    if (Q == 2 && p[0].type != p[1].type && fused2_fits(layers, &p[0], S0) && fused2_fits(layers, &p[1], S0) &&
        R >= 0 && S_pos >= 0 && N_neg >= 0 && slot_node0 && slot_ts0 &&
        (S_pos == 0 || (R > 0 && roots && ts_ptr && root_ts)) && (N_neg == 0 || (neg_roots && neg_ts))) {
        int32_t rc;
        if ((rc = check_graph(g)) != SGL_OK) return rc;
        for (int32_t q = 0; q < 2; ++q) {
            if ((rc = check_params(&p[q])) != SGL_OK) return rc;
            for (int32_t l = 0; l < 2; ++l)
                if ((rc = check_out(&outs[q * 2 + l], worst_slots(S0, l, p[q].fanout), p[q].fanout)) != SGL_OK) return rc;
        }
        const int r = p[0].type == SGL_SAMPLE_RECENT ? 0 : 1, u = 1 - r;
        RootSpec spec{R, S_pos, roots, ts_ptr, root_ts, neg_roots, neg_ts, slot_node0, slot_ts0};
        return run_fused2_pair(g, &spec, S0, &p[r], &outs[r * 2], &p[u], &outs[u * 2], ws, ws_bytes, as_stream(stream));
    }
    for (int32_t q = 0; q < Q; ++q) {
        const int32_t rc = sgl_sample_khop(g, R, roots, ts_ptr, S_pos, root_ts, N_neg, neg_roots, neg_ts, layers, &p[q],
                                           slot_node0, slot_ts0, outs + (size_t)q * layers,
                                           static_cast<char*>(ws) + (size_t)q * per, per, stream);
        if (rc != SGL_OK) return rc;
    }
    return SGL_OK;
}

// ---- sgl_sample_khop_batched: the root slots of B mini-batches sampled as one k-hop call --------------
namespace {
constexpr int SEG_MAX_CHAINS = 16;      // queries x layers one launch of batch_seg_kernel follows
struct SegArgs {
    int32_t B, layers, Q;
    int64_t S_max;
    const int64_t* batch_ptr;
    const int64_t* rsp[SEG_MAX_CHAINS];      // [q * layers + l]: root_start_ptr of hop l of query q
    int64_t cap[SEG_MAX_CHAINS];             // its capacity_slots
    int64_t* seg;                            // [Q][layers + 1][B + 1]
};
// What scan_kernel publishes for a hop, for a second query that shares the hop's counting pass
__global__ void share_counts_kernel(const int64_t* src_counts, int64_t* counts, int64_t* rsp, int64_t* rep, int64_t cap) {
    const int64_t S = src_counts[0], E = src_counts[1];
    counts[0] = S;
    counts[1] = E;
    counts[2] = src_counts[2];
    if (S >= 0 && S <= cap) {
        rsp[S] = E;
        rep[S] = E;
    }
}
// seg[q][0][b] = first root slot of batch b; seg[q][l+1][b] = root_start_ptr_l[seg[q][l][b]]: where batch b's
// edges of hop l begin (hop l's terminating entry root_start_ptr[S_l] = E_l closes the last batch).
__global__ void batch_seg_kernel(SegArgs a) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b > a.B) return;
    const int64_t S = live_count(a.batch_ptr + a.B, a.S_max);
    int64_t x0 = a.batch_ptr[b];
    x0 = x0 < 0 ? 0 : (x0 > S ? S : x0);
    for (int q = 0; q < a.Q; ++q) {
        int64_t* out = a.seg + (size_t)q * (a.layers + 1) * (a.B + 1);
        int64_t x = x0;
        out[b] = x;
        for (int l = 0; l < a.layers; ++l) {
            const int64_t cap = a.cap[q * a.layers + l];        // (an index is kept inside the array whatever it holds)
            x = a.rsp[q * a.layers + l][x < 0 ? 0 : (x > cap ? cap : x)];
            out[(size_t)(l + 1) * (a.B + 1) + b] = x;
        }
    }
}
}  // namespace

extern "C" size_t sgl_sample_khop_batched_workspace_bytes(int64_t S_max, int32_t layers, int32_t fanout, int32_t Q) {
    return (size_t)(Q > 0 ? Q : 1) * sgl_sample_khop_workspace_bytes(S_max, layers, fanout);
}

extern "C" int32_t sgl_sample_khop_batched(const sgl_tcsr* g, int32_t B, const int64_t* batch_ptr, int64_t S_max,
                                           const int64_t* slot_node, const int64_t* slot_ts, const int64_t* slot_hint,
                                           int32_t layers, int32_t Q, const sgl_sample_params* p,
                                           const sgl_hop_out* outs, int64_t* seg, void* ws, size_t ws_bytes,
                                           void* stream) {
    int32_t rc;
    if ((rc = check_graph(g)) != SGL_OK) return rc;
    if (B < 1 || !batch_ptr || S_max < 0 || layers < 1 || Q < 1 || !p || !outs || !seg)
        return fail(SGL_EINVAL, "sample_khop_batched: bad B, S_max, layers, Q or NULL argument");
    if (S_max > 0 && (!slot_node || !slot_ts)) return fail(SGL_EINVAL, "sample_khop_batched: slot array is NULL");
    if ((int64_t)Q * layers > SEG_MAX_CHAINS)
        return fail(SGL_ENOTSUP, "sample_khop_batched: Q * layers > %d", SEG_MAX_CHAINS);
    int32_t fan = 0;
    for (int32_t q = 0; q < Q; ++q) {
        if ((rc = check_params(&p[q])) != SGL_OK) return rc;
        if (p[q].mark_state) return fail(SGL_EINVAL, "sample_khop_batched: mark_state is not supported (the batches have id spaces of their own)");
        fan = p[q].fanout > fan ? p[q].fanout : fan;
        for (int32_t l = 0; l < layers; ++l) {
            const int64_t s = worst_slots(S_max, l, p[q].fanout);
            if (s == INT64_MAX) return fail(SGL_ENOTSUP, "sample_khop_batched: worst-case slot count overflows");
            if ((rc = check_out(&outs[(size_t)q * layers + l], s, p[q].fanout)) != SGL_OK) return rc;
        }
    }
    const size_t per = sgl_sample_khop_workspace_bytes(S_max, layers, fan);
    if (!ws || ws_bytes < (size_t)Q * per)
        return fail(SGL_ENOMEM, "sample_khop_batched: workspace %zu < %zu bytes", ws_bytes, (size_t)Q * per);
    hipStream_t st = as_stream(stream);
    // Hop-major order: a query that asks for the same windows and fanout as query 0 runs only the fill of hop 0,
    // on query 0's window arrays and block sums (its root slots are the same; they are searched once).
    const int64_t* sn[SEG_MAX_CHAINS];
    const int64_t* stt[SEG_MAX_CHAINS];
    const int64_t* S_dev[SEG_MAX_CHAINS];
    for (int32_t q = 0; q < Q; ++q) {
        sn[q] = slot_node;
        stt[q] = slot_ts;
        S_dev[q] = batch_ptr + B;
    }
    const int Gf0 = pick_group(&p[0], S_max);
    const HopGrid grid0 = hop_grid(S_max, pick_search_group(Gf0, S_max), Gf0);
    PreparedHop ph[SEG_MAX_CHAINS];
    bool shares[SEG_MAX_CHAINS];
    for (int32_t l = 0; l < layers; ++l) {
        for (int32_t q = 0; q < Q; ++q) {
            const sgl_sample_params* pq = &p[q];
            const sgl_hop_out* oq = outs + (size_t)q * layers;
            char* wq = static_cast<char*>(ws) + (size_t)q * per;
            int64_t worst = S_max;
            for (int32_t j = 0; j < layers; ++j) worst = worst_slots(S_max, j, pq->fanout) > worst ? worst_slots(S_max, j, pq->fanout) : worst;
            const size_t hop_ws = hop_workspace_bytes(worst);
            // as sgl_sample_khop: with the graph's next-hop index the slots of hops >= 1 are not searched
            const bool carry = layers > 1 && g->hop_hint != nullptr && !pq->equal_root_time &&
                               !(pq->type == SGL_SAMPLE_UNIFORM && pq->keep_root_time) && per >= hop_ws + hint_carry_bytes(worst);
            int64_t* carry_buf[2] = {nullptr, nullptr};
            if (carry) {
                carry_buf[0] = reinterpret_cast<int64_t*>(wq + hop_ws);
                carry_buf[1] = reinterpret_cast<int64_t*>(wq + hop_ws + align_up((size_t)(worst + 1) * 8));
            }
            sgl_sample_params pl = *pq;
            pl.hop = l;
            const int64_t s_max = worst_slots(S_max, l, pq->fanout);
            const int64_t* hint_in = l == 0 ? (pq->equal_root_time ? nullptr : slot_hint) : (carry ? carry_buf[(l - 1) & 1] : nullptr);
            bool share = false;
            if (l == 0 && q > 0) {
                const int Gfq = pick_group(pq, S_max);
                const HopGrid gq = hop_grid(S_max, pick_search_group(Gfq, S_max), Gfq);
                share = pq->fanout == p[0].fanout && pq->allowed_offset == p[0].allowed_offset &&
                        (pq->equal_root_time != 0) == (p[0].equal_root_time != 0) && gq.align == grid0.align &&
                        gq.blocks == grid0.blocks;      // (a hop's scratch is carved by its own slot count: same places)
            }
            shares[q] = share;
            rc = prepare_hop(g, sn[q], stt[q], nullptr, s_max, S_dev[q], &pl, &oq[l], share ? static_cast<char*>(ws) : wq,
                             carry ? hop_ws : per, hint_in, (carry && l + 1 < layers) ? carry_buf[l & 1] : nullptr, l == 0, &ph[q]);
            if (rc != SGL_OK) return rc;
        }
        // a most-recent query followed by a uniform one over grids of the same size: their kernels of this hop side by side
        const bool dual = Q == 2 && dual_hop_fits(ph[0], ph[1]);
        if (dual) {
            if ((rc = launch_dual_hop(ph[0], ph[1], st, shares[1])) != SGL_OK) return rc;
        }
        for (int32_t q = 0; q < Q; ++q) {
            const sgl_hop_out* oq = outs + (size_t)q * layers;
            if (!dual && (rc = launch_hop(ph[q].a, st, ph[q].Gc, ph[q].Gf, !shares[q], true)) != SGL_OK) return rc;
            if (shares[q] && grid0.blocks > FUSED_PREFIX_MAX) {   // the scan launch of query 0 published that query's counts only
                hipLaunchKernelGGL(share_counts_kernel, dim3(1), dim3(1), 0, st, outs[0].counts, oq[0].counts,
                                   oq[0].root_start_ptr, oq[0].root_end_ptr, oq[0].capacity_slots);
                SGL_LAUNCH_CHECK();
            }
            sn[q] = oq[l].neighbors;
            stt[q] = oq[l].neighbors_ts;
            S_dev[q] = oq[l].counts + 1;
        }
    }
    SegArgs sa{};
    sa.B = B; sa.layers = layers; sa.Q = Q; sa.S_max = S_max; sa.batch_ptr = batch_ptr; sa.seg = seg;
    for (int32_t i = 0; i < Q * layers; ++i) {
        sa.rsp[i] = outs[i].root_start_ptr;
        sa.cap[i] = outs[i].capacity_slots;
    }
    hipLaunchKernelGGL(batch_seg_kernel, dim3((unsigned)ceil_div<int>(B + 1, 256)), dim3(256), 0, st, sa);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
