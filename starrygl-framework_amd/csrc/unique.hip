// Unique + compaction of sampled node ids to dense local ids for gfx950.
//
// Dense-universe path (ids in [0, universe), `state` given):
//   the persistent state holds a 64-bit table entry per id
//   (epoch << 32 | local id) and a "pending" flag per id: a byte for universes
//   of up to 16M ids, a bit beyond.  Per group
//     mark   : ids whose table entry is not of the current epoch set their flag
//              (plain byte store, or atomicOr on the bitmap), duplicates
//              collapse for free;
//     reduce : per-tile popcount sums over the flag words;
//     assign : every set flag gets local id = base + rank of the flag, which is
//              the ascending-id order the reference obtains by sort + unique;
//              the entry, the local->global list and the cleared word are
//              written in the same pass;
//     commit : the call's epoch and id count become the committed ones (the
//              last group's commit is done by one thread of the lookup launch);
//   then one lookup launch rewrites every input array through the table.
//   No sort, no hash probing; the result is deterministic.
//   Grouped mode (per array: the ids new to the epoch, ascending, appended) is
//   one numbering pass as well when the flags are bytes: array g sets flags in
//   plane g of the pending set, an id belongs to the first plane that has it,
//   and the offsets of all (group, tile) buckets are one exclusive scan over
//   the group-major counts.  With a bitmap the arrays are numbered one by one.
//   Up to SINGLE_PASS_MAX tiles, reduce and assign of the sorted mode are one launch: every tile
//   publishes its count in a descriptor kept in the state (tagged with the
//   state's pass counter, so descriptors never need clearing) and adds up the
//   descriptors of the tiles before it as they appear.
//
// Replaces Remapper::remapper / insert, mark_new_ids_kernel and
// update_new_ids_kernel (csrc/include/starrygl/sample.cu.hpp:1719-1854).
#include "common.hpp"

namespace sgl {

// hash-set path, defined in unique_hash.hip
size_t hash_unique_workspace_bytes(int32_t G, const int64_t* len_max);
int32_t hash_unique_compact(int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev, int64_t* const* local_out,
                            int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, hipStream_t st);

namespace {

constexpr int BLOCK = 256;
constexpr int MAXG = 8;
constexpr int TILE = BLOCK;            // flag words (8 ids each) per block in reduce/assign (one per thread)
constexpr int SCAN_BLOCK = 1024;
constexpr int MAX_GRID = 2048;         // grid cap of the per-id kernels (grid-stride loops)
constexpr int FUSED_SCAN_MAX = 4096;   // up to this many tiles assign sums the preceding tiles itself
constexpr int SINGLE_PASS_MAX = 2048;  // up to this many tiles the counts are exchanged inside the assign launch
constexpr size_t HEADER_BYTES = REMAP_HEADER_BYTES;

struct Header {
    uint64_t epoch;     // committed epoch (low 32 bits are stamped into the table)
    int64_t id_count;   // committed number of local ids handed out in this epoch
    uint64_t pass;      // numbering passes committed so far (tags the tile descriptors)
    int64_t poisoned;   // sticky: a tile once gave up waiting for an earlier tile's descriptor
};

struct State {
    Header* hdr;
    uint64_t* table;
    uint64_t* bitmap;   // the pending flags, one byte per id, addressed as 8-byte words by reduce/assign
    uint64_t* desc;     // one descriptor per tile of flag words: pass tag << 32 | flags set in the tile
    int64_t universe, words;
    int32_t bytes;      // 1: a flag byte per id (8 ids per word), 0: a bit per id (64 ids per word)
    int32_t planes;     // copies of the pending set (one per array of a grouped call)
};

State carve(void* state, int64_t universe) {
    State s;
    char* p = static_cast<char*>(state);
    s.universe = universe;
    s.bytes = remap_byte_flags(universe) ? 1 : 0;
    s.words = ceil_div<int64_t>(universe, s.bytes ? 8 : 64);
    s.hdr = reinterpret_cast<Header*>(p);
    s.table = reinterpret_cast<uint64_t*>(p + HEADER_BYTES);
    s.bitmap = s.table + universe;           // s.planes planes of s.words words each; plane 0 first
    s.planes = s.bytes ? MAXG : 1;           // (a bitmap state numbers the arrays of a grouped call one by one)
    s.desc = s.bitmap + (int64_t)s.planes * s.words;
    return s;
}

// Epoch stamp / first local id a call works with.  The header is only written
// by commit_kernel, so every kernel of a call derives the same values from it.
__device__ __forceinline__ uint64_t eff_epoch(const State& s, int reset) {
    uint64_t e = s.hdr->epoch;
    if (reset) {
        e += 1;
        if ((e & 0xFFFFFFFFull) == 0) e += 1;  // stamp 0 means "never mapped"
    }
    return e;
}
__device__ __forceinline__ uint32_t eff_stamp(const State& s, int reset) {
    return (uint32_t)(eff_epoch(s, reset) & 0xFFFFFFFFull);
}
__device__ __forceinline__ int64_t eff_base(const State& s, int reset) { return reset ? 0 : s.hdr->id_count; }
// Tag of the numbering pass in flight: never 0, the value of a descriptor nobody has written yet.
__device__ __forceinline__ uint64_t next_pass(uint64_t pass) {
    pass += 1;
    if ((pass & 0xFFFFFFFFull) == 0) pass += 1;
    return pass;
}
__device__ __forceinline__ uint32_t eff_tag(const State& s) { return (uint32_t)(next_pass(s.hdr->pass) & 0xFFFFFFFFull); }

struct Arrays {
    int32_t G;
    const int64_t* ids[MAXG];
    int64_t* out[MAXG];
    const int64_t* len_dev[MAXG];
    int64_t len_max[MAXG];
    int64_t start[MAXG + 1];  // flat index space over len_max
};

__global__ void init_state_kernel(State s) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = t; i < s.universe; i += stride) s.table[i] = 0;
    for (int64_t i = t; i < (int64_t)s.planes * s.words; i += stride) s.bitmap[i] = 0;
    for (int64_t i = t; i < ceil_div<int64_t>(s.words, TILE); i += stride) s.desc[i] = 0;
    if (t == 0) {
        s.hdr->epoch = 1;
        s.hdr->id_count = 0;
        s.hdr->pass = 0;
        s.hdr->poisoned = 0;
    }
}

// Sets the flag of every id that has no local id in this epoch yet: one id per
// thread and an unconditional fire-and-forget store / atomicOr.  (Measured on
// MI355X: on a small universe the atomics of a batch serialise on the few cache
// lines of the bitmap and cost twice what byte stores do; on a 100M-id universe
// sweeping a byte per id in reduce/assign costs more than the atomics.  Testing
// the flag first, or folding the block's ids through an LDS hash set first,
// lengthens the dependent chain and runs 2-3x slower in both layouts.)
__global__ __launch_bounds__(BLOCK) void mark_kernel(State s, Arrays a, int reset, int grouped) {
    const uint32_t stamp = eff_stamp(s, reset);
    // Index i is processed for every array at once (loads of the different arrays are
    // independent and issue together: one dependent chain id -> table -> atomic per
    // thread instead of one per array), with a grid stride bounded by the longest LIVE
    // length: capacities are worst cases (slots x fanout), most of them is dead.
    int64_t len[MAXG];
    int64_t max_len = 0;
#pragma unroll
    for (int g = 0; g < MAXG; ++g) {
        len[g] = g < a.G ? live_count(a.len_dev[g], a.len_max[g]) : 0;
        max_len = len[g] > max_len ? len[g] : max_len;
    }
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < max_len; i += (int64_t)gridDim.x * BLOCK) {
        int64_t id[MAXG];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) id[g] = (g < a.G && i < len[g]) ? a.ids[g][i] : -1;
        uint64_t e[MAXG];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) {
            const bool ok = id[g] >= 0 && id[g] < s.universe;
            e[g] = ok ? s.table[id[g]] : ((uint64_t)stamp << 32);   // out of range: treated as already numbered
        }
#pragma unroll
        for (int g = 0; g < MAXG; ++g)
            if ((uint32_t)(e[g] >> 32) != stamp)      // grouped: array g has plane g of the pending set
                remap_set_pending(s.bitmap + (grouped ? (int64_t)g * s.words : 0), s.bytes, id[g]);
    }
}

__global__ __launch_bounds__(BLOCK) void reduce_kernel(State s, int64_t* tile_sum) {
    __shared__ int32_t s_w[BLOCK / WAVE];
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    int32_t c = (w < s.words) ? __popcll(s.bitmap[w]) : 0;
    for (int d = WAVE / 2; d > 0; d >>= 1) c += __shfl_down(c, d);
    if (threadIdx.x % WAVE == 0) s_w[threadIdx.x / WAVE] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t sum = 0;
        for (int q = 0; q < BLOCK / WAVE; ++q) sum += s_w[q];
        tile_sum[blockIdx.x] = sum;
    }
}

// exclusive scan of `nt` tile sums in place (+ the grand total at [nt]), by one block, in pieces of SCAN_PIECE
// sums: coalesced loads into LDS (a block that reads 8 consecutive sums per thread straight from memory issues
// strided 64-byte reads, which one CU serves slowly), thread t then owns the 8 consecutive sums of its stretch, one
// round of shuffles per wavefront scans the stretch totals, and the offsets leave through LDS, coalesced again.
constexpr int SCAN_PER = 8;
constexpr int SCAN_PIECE = SCAN_BLOCK * SCAN_PER;
__global__ __launch_bounds__(SCAN_BLOCK) void scan_tiles_kernel(int64_t* tile_sum, int64_t nt) {
    constexpr int NW = SCAN_BLOCK / WAVE;
    __shared__ int64_t s_v[SCAN_PIECE + SCAN_PIECE / 32];      // (a pad word per 32: the stretches start in different banks)
    __shared__ int64_t s_w[NW];
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    auto at = [](int i) { return i + (i >> 5); };
    int64_t base = 0;
    for (int64_t p0 = 0; p0 < nt; p0 += SCAN_PIECE) {          // block-uniform
        __syncthreads();
#pragma unroll
        for (int q = 0; q < SCAN_PER; ++q) {
            const int i = q * SCAN_BLOCK + threadIdx.x;
            s_v[at(i)] = p0 + i < nt ? tile_sum[p0 + i] : 0;
        }
        __syncthreads();
        int64_t v[SCAN_PER], sum = 0;
#pragma unroll
        for (int q = 0; q < SCAN_PER; ++q) {
            v[q] = s_v[at(threadIdx.x * SCAN_PER + q)];
            sum += v[q];
        }
        int64_t inc = sum;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int64_t y = shfl_i64(inc, lane >= d ? lane - d : lane);
            if (lane >= d) inc += y;
        }
        if (lane == WAVE - 1) s_w[wid] = inc;
        __syncthreads();
        int64_t run = base + inc - sum, total = 0;
#pragma unroll
        for (int q = 0; q < NW; ++q) {
            if (q < wid) run += s_w[q];
            total += s_w[q];
        }
#pragma unroll
        for (int q = 0; q < SCAN_PER; ++q) {
            s_v[at(threadIdx.x * SCAN_PER + q)] = run;
            run += v[q];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < SCAN_PER; ++q) {
            const int i = q * SCAN_BLOCK + threadIdx.x;
            if (p0 + i < nt) tile_sum[p0 + i] = s_v[at(i)];
        }
        base += total;
    }
    if (threadIdx.x == 0) tile_sum[nt] = base;
}

// Numbers the set bits in ascending id order.
// MODE 0: tile_sum holds raw sums and the block adds up the tiles before it, MODE 1: tile_sum
// holds exclusive offsets (+ total at [nt]), MODE 2: no tile_sum - the tiles
// exchange their counts through the state's descriptors inside this launch (a tile waits, bounded,
// only for tiles with a smaller index, which the dispatcher started no later than itself).
template <int MODE>
__global__ __launch_bounds__(BLOCK) void assign_kernel(State s, const int64_t* tile_sum, int64_t nt,
                                                       int reset, int64_t* unique_out,
                                                       int64_t unique_capacity, int64_t* U_dev, uint32_t* stamp_ws,
                                                       int32_t spin_limit) {
    __shared__ int64_t s_red[BLOCK / WAVE];
    __shared__ int32_t s_wave[BLOCK / WAVE];
    __shared__ int s_gave[BLOCK / WAVE];
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int64_t base = eff_base(s, reset);
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    uint64_t word = (w < s.words) ? s.bitmap[w] : 0ull;
    const int32_t c = __popcll(word);
    int32_t inc = c;
    for (int d = 1; d < WAVE; d <<= 1) {
        const int32_t x = __shfl_up(inc, d);
        if (lane >= d) inc += x;
    }
    if (lane == WAVE - 1) s_wave[wid] = inc;
    __syncthreads();
    int32_t wave_off = 0, block_total = 0;
    for (int q = 0; q < BLOCK / WAVE; ++q) {
        if (q < wid) wave_off += s_wave[q];
        block_total += s_wave[q];
    }
    int64_t tile_off = 0;
    int gave_up = 0;
    if constexpr (MODE == 1) {
        tile_off = tile_sum[blockIdx.x];
    } else {
        int64_t part = 0;
        if constexpr (MODE == 0) {
            for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += BLOCK) part += tile_sum[b];
        } else {
            const uint64_t tag = (uint64_t)eff_tag(s) << 32;
            if (threadIdx.x == 0)
                __hip_atomic_store(&s.desc[blockIdx.x], tag | (uint64_t)(uint32_t)block_total, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += BLOCK) {
                uint64_t d;
                int spins = 0;
                while (((d = __hip_atomic_load(&s.desc[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) &
                        0xFFFFFFFF00000000ull) != tag) {
                    if (++spins > spin_limit) {
                        gave_up = 1;
                        d = 0;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                part += (int64_t)(d & 0xFFFFFFFFull);
            }
        }
        for (int d = WAVE / 2; d > 0; d >>= 1) {   // butterfly: all lanes hold the wave sum
            part += shfl_i64(part, lane ^ d);
            gave_up |= __shfl(gave_up, lane ^ d);
        }
        if (lane == 0) {
            s_red[wid] = part;
            s_gave[wid] = gave_up;
        }
        __syncthreads();
        gave_up = 0;
        for (int q = 0; q < BLOCK / WAVE; ++q) {
            tile_off += s_red[q];
            gave_up |= s_gave[q];
        }
    }
    if (blockIdx.x == nt - 1 && threadIdx.x == 0) {  // publish the counts and the stamp of this call
        U_dev[0] = base + tile_off + block_total;
        stamp_ws[0] = eff_stamp(s, reset);
    }
    // a tile that gave up waiting poisons the state: every later commit reports INT64_MAX ids
    if (gave_up && threadIdx.x == 0) s.hdr->poisoned = 1;
    if (c == 0) return;
    int64_t local = base + tile_off + wave_off + (inc - c);
    const uint64_t stamp = (uint64_t)eff_stamp(s, reset) << 32;
    const int64_t id0 = w * (s.bytes ? 8 : 64);
    const int shift = s.bytes ? 3 : 0;
    while (word) {
        const int bit = __ffsll((unsigned long long)word) - 1;
        word &= word - 1;
        const int64_t id = id0 + (bit >> shift);
        s.table[id] = stamp | (uint64_t)(uint32_t)local;
        if (local < unique_capacity) unique_out[local] = id;
        ++local;
    }
    s.bitmap[w] = 0;
}

// Grouped mode, counting: tile_cnt[g * nt + tile] = ids of the tile whose first plane is g.
__global__ __launch_bounds__(BLOCK) void reduce_groups_kernel(State s, int G, int64_t nt, int64_t* tile_cnt) {
    __shared__ int32_t s_w[MAXG][BLOCK / WAVE];
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    uint64_t seen = 0;
#pragma unroll
    for (int g = 0; g < MAXG; ++g) {
        int32_t c = 0;
        if (g < G) {
            const uint64_t m = (w < s.words) ? s.bitmap[(int64_t)g * s.words + w] : 0ull;
            c = __popcll(m & ~seen);
            seen |= m;
        }
        for (int d = WAVE / 2; d > 0; d >>= 1) c += __shfl_down(c, d);
        if (lane == 0) s_w[g][wid] = c;
    }
    __syncthreads();
    if ((int)threadIdx.x < G) {
        int64_t sum = 0;
        for (int q = 0; q < BLOCK / WAVE; ++q) sum += s_w[threadIdx.x][q];
        tile_cnt[(int64_t)threadIdx.x * nt + blockIdx.x] = sum;
    }
}

// Grouped mode, numbering.  The local id of an id of group g in tile t is
//   base + (ids of groups < g, all tiles) + (ids of group g, tiles < t) + rank inside the tile,
// and the two middle terms are the exclusive prefix of tile_cnt at g * nt + t (group-major order).
// `scanned`: tile_cnt already holds that prefix (+ the grand total at [G * nt]); otherwise raw counts.
__global__ __launch_bounds__(BLOCK) void assign_groups_kernel(State s, int G, const int64_t* tile_cnt, int64_t nt,
                                                              int scanned, int reset, int64_t* unique_out,
                                                              int64_t unique_capacity, int64_t* U_dev, uint32_t* stamp_ws) {
    __shared__ int64_t s_red[MAXG + 1][BLOCK / WAVE];
    __shared__ int32_t s_wave[BLOCK / WAVE];
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int64_t flat = (int64_t)G * nt;
    int64_t off[MAXG], total = 0;
    if (scanned) {
#pragma unroll
        for (int g = 0; g < MAXG; ++g) off[g] = g < G ? tile_cnt[(int64_t)g * nt + blockIdx.x] : 0;
        total = tile_cnt[flat];
    } else {
        int64_t part[MAXG + 1];
#pragma unroll
        for (int g = 0; g <= MAXG; ++g) part[g] = 0;
        for (int64_t i = threadIdx.x; i < flat; i += BLOCK) {
            const int64_t v = tile_cnt[i];
            part[MAXG] += v;
#pragma unroll
            for (int g = 0; g < MAXG; ++g)
                if (g < G && i < (int64_t)g * nt + blockIdx.x) part[g] += v;
        }
#pragma unroll
        for (int g = 0; g <= MAXG; ++g) {
            int64_t x = part[g];
            for (int d = WAVE / 2; d > 0; d >>= 1) x += shfl_i64(x, lane ^ d);
            if (lane == 0) s_red[g][wid] = x;
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < MAXG; ++g) {
            off[g] = 0;
            for (int q = 0; q < BLOCK / WAVE; ++q) off[g] += s_red[g][q];
        }
        for (int q = 0; q < BLOCK / WAVE; ++q) total += s_red[MAXG][q];
    }
    const int64_t base = eff_base(s, reset);
    if (blockIdx.x == nt - 1 && threadIdx.x == 0) {  // publish the counts and the stamp of this call
        U_dev[0] = base + total;
        stamp_ws[0] = eff_stamp(s, reset);
    }
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    const uint64_t stamp = (uint64_t)eff_stamp(s, reset) << 32;
    const int64_t id0 = w * (s.bytes ? 8 : 64);
    const int shift = s.bytes ? 3 : 0;
    uint64_t seen = 0;
    for (int g = 0; g < G; ++g) {
        const uint64_t m = (w < s.words) ? s.bitmap[(int64_t)g * s.words + w] : 0ull;
        uint64_t word = m & ~seen;
        seen |= m;
        const int32_t c = __popcll(word);
        int32_t inc = c;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int32_t x = __shfl_up(inc, d);
            if (lane >= d) inc += x;
        }
        __syncthreads();
        if (lane == WAVE - 1) s_wave[wid] = inc;
        __syncthreads();
        int32_t wave_off = 0;
        for (int q = 0; q < wid; ++q) wave_off += s_wave[q];
        int64_t local = base + off[g] + wave_off + (inc - c);
        while (word) {
            const int bit = __ffsll((unsigned long long)word) - 1;
            word &= word - 1;
            const int64_t id = id0 + (bit >> shift);
            s.table[id] = stamp | (uint64_t)(uint32_t)local;
            if (local < unique_capacity) unique_out[local] = id;
            ++local;
        }
        if (m != 0) s.bitmap[(int64_t)g * s.words + w] = 0;
    }
}

// Makes the call's epoch and id count the committed ones.  `first`: U_dev[1]
// (ids numbered before this call) is recorded.  `has_new` == 0: no assign ran.
__device__ __forceinline__ void commit(const State& s, int reset, int first, int has_new, int64_t* U_dev) {
    const int64_t base = eff_base(s, reset);
    const uint64_t epoch = eff_epoch(s, reset);
    if (first) U_dev[1] = base;
    if (!has_new) U_dev[0] = base;
    s.hdr->epoch = epoch;
    s.hdr->pass = next_pass(s.hdr->pass);
    if (s.hdr->poisoned) {        // numbers handed out by a pass that gave up are meaningless
        s.hdr->id_count = 0;
        U_dev[0] = INT64_MAX;
    } else {
        s.hdr->id_count = U_dev[0];
    }
}

__global__ void commit_kernel(State s, int reset, int first, int has_new, int64_t* U_dev) {
    commit(s, reset, first, has_new, U_dev);
}

// Rewrites every input array through the table.  `fold` != 0: the call's last commit
// has not run yet; the kernel takes the stamp from `stamp_ws` (written by the single
// thread of stamp_kernel / assign's publisher before this launch, never from the header)
// and thread 0 of block 0 commits, so no thread of this launch reads what it writes.
__global__ __launch_bounds__(BLOCK) void lookup_kernel(State s, Arrays a, int fold, int reset, int first, int has_new,
                                                       const uint32_t* stamp_ws, int64_t* U_dev) {
    const uint32_t stamp = fold ? stamp_ws[0] : (uint32_t)(s.hdr->epoch & 0xFFFFFFFFull);
    if (fold && blockIdx.x == 0 && threadIdx.x == 0) commit(s, reset, first, has_new, U_dev);
    int64_t len[MAXG];
    int64_t max_len = 0;
#pragma unroll
    for (int g = 0; g < MAXG; ++g) {
        len[g] = g < a.G ? live_count(a.len_dev[g], a.len_max[g]) : 0;
        max_len = len[g] > max_len ? len[g] : max_len;
    }
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < max_len; i += (int64_t)gridDim.x * BLOCK) {
        int64_t id[MAXG];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) id[g] = (g < a.G && i < len[g]) ? a.ids[g][i] : -1;   // ids may alias out
        uint64_t e[MAXG];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) e[g] = (id[g] >= 0 && id[g] < s.universe) ? s.table[id[g]] : 0ull;
#pragma unroll
        for (int g = 0; g < MAXG; ++g)
            if (g < a.G && i < len[g])
                a.out[g][i] = ((uint32_t)(e[g] >> 32) == stamp) ? (int64_t)(e[g] & 0xFFFFFFFFull) : -1;
    }
}

// ---------------------------------------------------------------------------------------
// Batched call: B mini-batches, each with a local-id space of its own, numbered by ONE launch sequence.
// Batch b's ids live at [b * stride, b * stride + universe) of a state over B * stride ids (stride: the
// universe rounded up to whole tiles of flag words, so that a tile belongs to one batch); array g's
// elements [seg[g][b], seg[g][b+1]) belong to batch b.  Ascending numbering over the big universe is
// batch-major and ascending inside a batch: batch b's local id = global rank - rank of the batch's first
// tile.  There is no id -> local id table: numbering leaves, per group of 64 ids, the 64 pending bits and the
// batch-local rank of the group's first pending id (16 bytes per 64 ids: 256 KB for a million ids, which an L2
// holds, where a 4-byte entry per id made every lookup a sector of its own out of a table that no L2 held), and
// a lookup is that one 16-byte load and a popcount of the bits below the id's own.  Every call numbers afresh
// and looks up only ids it has numbered itself, so nothing needs epoch stamps or clearing.
constexpr int BATCH_MAX = SGL_BATCH_MAX;
constexpr int64_t BATCH_STRIDE_ALIGN = (int64_t)TILE * 64;   // ids per tile: a thread of reduce / assign owns a group of 64

struct Batched {
    int32_t B;
    int64_t stride, universe;
    const int64_t* seg[MAXG];
};

struct alignas(16) RankWord {
    uint64_t mask;      // pending bits of ids [64 w, 64 w + 64)
    int64_t rank;       // batch-local rank of the first of them
};

struct BState {
    RankWord* rank;     // [B * stride / 64]
    uint64_t* flags;    // pending flags: a byte per id (8 per word) or a bit per id
    int64_t universe, words, groups;
    int32_t bytes;
};

// A flag byte per id up to 64M ids in all (B x the universe): a batch's marks are plain stores, and the sweeps
// over the flags cost less than atomics on a bitmap do (20 x 1M ids: 7.6 against 11.9 us per batch for the whole call).
constexpr int64_t BATCHED_BYTE_FLAGS_MAX = 1ll << 26;
inline bool batched_byte_flags(int64_t big) { return big <= BATCHED_BYTE_FLAGS_MAX; }
inline int64_t batch_stride(int64_t universe) { return ceil_div<int64_t>(universe, BATCH_STRIDE_ALIGN) * BATCH_STRIDE_ALIGN; }

BState carve_batched(void* state, int64_t universe, int32_t B) {
    BState s;
    char* p = static_cast<char*>(state);
    s.universe = (int64_t)B * batch_stride(universe);
    s.bytes = batched_byte_flags(s.universe) ? 1 : 0;
    s.words = s.universe / (s.bytes ? 8 : 64);
    s.groups = s.universe / 64;
    s.rank = reinterpret_cast<RankWord*>(p + HEADER_BYTES);                 // HEADER_BYTES is a multiple of 16
    s.flags = reinterpret_cast<uint64_t*>(s.rank + s.groups);
    return s;
}

__global__ void init_batched_kernel(BState s) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < s.words; i += stride) s.flags[i] = 0;
}

__device__ __forceinline__ void stage_segs(const Batched& bt, int G, int64_t (*s_seg)[BATCH_MAX + 1]) {
    for (int x = threadIdx.x; x < G * (bt.B + 1); x += blockDim.x) {
        const int g = x / (bt.B + 1), b = x - g * (bt.B + 1);
        s_seg[g][b] = bt.seg[g][b];
    }
    __syncthreads();
}

// LOOKUP == false: sets the flag of every id (a new numbering per call: no table read);
// LOOKUP == true : rewrites every array through the table.
//
// Which block walks which batch follows the chip: workgroups go to the 8 XCDs in turn (block i runs on XCD i % 8) and
// every XCD has an L2 of its own, so all blocks of one XCD work on the same batch at the same time (batch b belongs to
// the blocks of class b % V; V = 8 from eight batches on, the largest power of two <= B below).  A batch's flags (1 MB
// for a million ids) and its slice of the table (4 MB) then stay in one L2 while the batch is walked: with every block
// striding over all batches the lookup walk of 16 batches fetched a 64-byte sector per element (240 MB for 19 MB of
// ids) and the marking walk wrote one per flag byte.  Only the speed depends on that placement, the result does not.
constexpr int XCDS = 8;
constexpr int WALK_ILP = 4;
constexpr int WALK_SEGS = (BATCH_MAX / XCDS) * MAXG;        // (batch, array) pieces one class of blocks can own
static_assert(BATCH_MAX % XCDS == 0 && WALK_SEGS <= WAVE && MAXG <= XCDS, "the pieces of a class are listed by one wavefront");

template <bool LOOKUP>
__global__ __launch_bounds__(BLOCK) void walk_batched_kernel(BState s, Arrays a, Batched bt) {
    __shared__ int64_t s_seg[MAXG][BATCH_MAX + 1];
    __shared__ int64_t s_pref[WALK_SEGS + 1], s_lo[WALK_SEGS], s_base[WALK_SEGS];
    __shared__ const int64_t* s_ids[WALK_SEGS];
    __shared__ int64_t* s_out[WALK_SEGS];
    stage_segs(bt, a.G, s_seg);
    int V = XCDS;
    while (V > bt.B) V >>= 1;                                   // classes of blocks (a power of two, >= 1)
    const int x = blockIdx.x % XCDS;
    const int cls = x % V;
    // this block's place among the blocks of its class, and how many those are (the grid is a multiple of XCDS)
    const int64_t worker = (int64_t)(blockIdx.x / XCDS) * (XCDS / V) + x / V;
    const int64_t step = (int64_t)(gridDim.x / XCDS) * (XCDS / V) * BLOCK;
    // The class's pieces - array g's elements of batch b, for every batch of the class - laid end to end as one
    // index range, so that every lane has an element whatever the pieces' sizes are (a batch's root list is a
    // twentieth of its hop-2 list).  Piece e = (e / MAXG)-th batch of the class, array e % MAXG.
    if (threadIdx.x < WAVE) {
        const int e = threadIdx.x;
        const int g = e % MAXG, b = cls + (e / MAXG) * V;
        int64_t lo = 0, n = 0;
        if (e < WALK_SEGS && g < a.G && b < bt.B) {
            int64_t top = s_seg[g][bt.B];
            top = top < 0 ? 0 : (top > a.len_max[g] ? a.len_max[g] : top);
            lo = s_seg[g][b];
            int64_t hi = s_seg[g][b + 1];
            lo = lo < 0 ? 0 : lo;
            hi = hi > top ? top : hi;
            n = hi > lo ? hi - lo : 0;
        }
        int64_t inc = n;
        for (int d = 1; d < WAVE; d <<= 1) {
            const int64_t y = __shfl_up(inc, d);
            if (e >= d) inc += y;
        }
        if (e < WALK_SEGS) {
            s_pref[e] = inc - n;
            s_lo[e] = lo;
            s_base[e] = (int64_t)b * bt.stride;
            s_ids[e] = g < a.G ? a.ids[g] : nullptr;
            s_out[e] = g < a.G ? a.out[g] : nullptr;
        }
        if (e == WALK_SEGS - 1) s_pref[WALK_SEGS] = inc;
    }
    __syncthreads();
    const int64_t total = s_pref[WALK_SEGS];
    for (int64_t j0 = worker * BLOCK + threadIdx.x; j0 < total; j0 += step * WALK_ILP) {
        int64_t id[WALK_ILP], at[WALK_ILP];
        int64_t* dst[WALK_ILP];
#pragma unroll
        for (int u = 0; u < WALK_ILP; ++u) {
            const int64_t j = j0 + u * step;
            id[u] = -1;
            at[u] = 0;
            dst[u] = nullptr;
            if (j < total) {
                int e = 0;                                  // the last piece that starts at or before j
#pragma unroll
                for (int h = WALK_SEGS / 2; h > 0; h >>= 1)
                    if (s_pref[e + h] <= j) e += h;
                const int64_t i = s_lo[e] + (j - s_pref[e]);
                id[u] = s_ids[e][i];                        // ids may alias out: every element is read before it is written
                at[u] = s_base[e] + id[u];
                dst[u] = s_out[e] + i;
            }
        }
        if constexpr (LOOKUP) {
            RankWord v[WALK_ILP];
#pragma unroll
            for (int u = 0; u < WALK_ILP; ++u) v[u] = (id[u] >= 0 && id[u] < bt.universe) ? s.rank[at[u] >> 6] : RankWord{0ull, -1};
#pragma unroll
            for (int u = 0; u < WALK_ILP; ++u)
                if (dst[u])
                    *dst[u] = (id[u] >= 0 && id[u] < bt.universe)
                                  ? v[u].rank + __popcll(v[u].mask & ((1ull << (at[u] & 63)) - 1ull)) : -1;
        } else {
#pragma unroll
            for (int u = 0; u < WALK_ILP; ++u)
                if (id[u] >= 0 && id[u] < bt.universe) remap_set_pending(s.flags, s.bytes, at[u]);
        }
    }
}

// the eight flag bytes (0 or 1 each) of a word as eight bits, byte i -> bit i
__device__ __forceinline__ uint64_t pack_flag_bytes(uint64_t w) {
    return (((w << 7) & 0x8080808080808080ull) * 0x0002040810204081ull) >> 56;
}

// Thread w owns ids [64 w, 64 w + 64): it turns their flags into the group's 64 pending bits (left in rank[w].mask),
// clears the flags for the next call and counts; a block's count is its tile's sum.
// A batch none of whose arrays holds an element in this call (a group of batches with fewer live ones than the state
// has room for): its flags are all clear and nobody will look its ids up, so reduce and assign leave its tiles alone
// (both ask the same question, so a tile's pending bits are read by assign only when reduce wrote them in this call).
__device__ __forceinline__ bool batch_live(const Batched& bt, int G, int64_t b) {
    bool live = false;
#pragma unroll
    for (int g = 0; g < MAXG; ++g)
        if (g < G && bt.seg[g][b + 1] > bt.seg[g][b]) live = true;
    return live;
}

__global__ __launch_bounds__(BLOCK) void reduce_batched_kernel(BState s, int64_t* tile_sum, Batched bt, int G) {
    __shared__ int32_t s_w[BLOCK / WAVE];
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    if (!batch_live(bt, G, (int64_t)blockIdx.x / (bt.stride / BATCH_STRIDE_ALIGN))) {      // block-uniform
        if (threadIdx.x == 0) tile_sum[blockIdx.x] = 0;
        return;
    }
    uint64_t mask = 0;
    if (w < s.groups) {
        if (s.bytes) {
            const ulonglong2* f = reinterpret_cast<const ulonglong2*>(s.flags + w * 8);
            ulonglong2 q[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) q[j] = f[j];
#pragma unroll
            for (int j = 0; j < 4; ++j) mask |= (pack_flag_bytes(q[j].x) | (pack_flag_bytes(q[j].y) << 8)) << (16 * j);
            if (mask) {
                ulonglong2* fw = reinterpret_cast<ulonglong2*>(s.flags + w * 8);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (q[j].x | q[j].y) fw[j] = ulonglong2{0ull, 0ull};
            }
        } else {
            mask = s.flags[w];
            if (mask) s.flags[w] = 0;
        }
        s.rank[w].mask = mask;
    }
    int32_t c = __popcll(mask);
    for (int d = WAVE / 2; d > 0; d >>= 1) c += __shfl_down(c, d);
    if (threadIdx.x % WAVE == 0) s_w[threadIdx.x / WAVE] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t sum = 0;
        for (int q = 0; q < BLOCK / WAVE; ++q) sum += s_w[q];
        tile_sum[blockIdx.x] = sum;
    }
}

// Numbers the pending ids (tile_sum holds the exclusive tile offsets, the total at [nt]): an id's local id is its
// rank inside its batch, i.e. the global rank minus the offset of the batch's first tile; the first tile of
// every batch records where the batch's list begins.
__global__ __launch_bounds__(BLOCK) void assign_batched_kernel(BState s, const int64_t* tile_sum, int64_t nt, Batched bt, int G,
                                                               int64_t* unique_out, int64_t unique_capacity, int64_t* U_off) {
    __shared__ int32_t s_wave[BLOCK / WAVE];
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int64_t w = (int64_t)blockIdx.x * TILE + threadIdx.x;
    const bool live = batch_live(bt, G, (int64_t)blockIdx.x / (bt.stride / BATCH_STRIDE_ALIGN));       // block-uniform
    uint64_t word = (live && w < s.groups) ? s.rank[w].mask : 0ull;
    const int32_t c = __popcll(word);
    int32_t inc = c;
    for (int d = 1; d < WAVE; d <<= 1) {
        const int32_t x = __shfl_up(inc, d);
        if (lane >= d) inc += x;
    }
    if (lane == WAVE - 1) s_wave[wid] = inc;
    __syncthreads();
    int32_t wave_off = 0;
    for (int q = 0; q < wid; ++q) wave_off += s_wave[q];
    const int64_t tile_off = tile_sum[blockIdx.x];
    const int64_t tiles_per_batch = bt.stride / BATCH_STRIDE_ALIGN;
    const int64_t b = (int64_t)blockIdx.x / tiles_per_batch;        // the tile's batch (a stride is a whole number of tiles)
    const int64_t batch_off = tile_sum[b * tiles_per_batch];
    if (threadIdx.x == 0) {
        if ((int64_t)blockIdx.x == b * tiles_per_batch) U_off[b] = tile_off;
        if (blockIdx.x == nt - 1) U_off[bt.B] = tile_sum[nt];
    }
    if (!live || w >= s.groups) return;
    int64_t rank = tile_off + wave_off + (inc - c);
    s.rank[w].rank = rank - batch_off;
    const int64_t id0 = w * 64 - b * bt.stride;
    while (word) {
        const int bit = __ffsll((unsigned long long)word) - 1;
        word &= word - 1;
        if (rank < unique_capacity) unique_out[rank] = id0 + bit;
        ++rank;
    }
}

size_t batched_workspace_bytes(int64_t universe, int32_t B) {
    const int64_t big = (int64_t)B * batch_stride(universe);
    return align_up((size_t)(big / BATCH_STRIDE_ALIGN + 2) * 8) + 512;
}

size_t dense_workspace_bytes(int64_t universe) {
    const int64_t words = ceil_div<int64_t>(universe, remap_byte_flags(universe) ? 8 : 64);
    return align_up((size_t)(MAXG * ceil_div<int64_t>(words, TILE) + 2) * 8) + 512;
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_remap_state_bytes(int64_t universe) {
    if (universe < 0) return 0;
    const int64_t words = ceil_div<int64_t>(universe, remap_byte_flags(universe) ? 8 : 64);
    const size_t planes = remap_byte_flags(universe) ? MAXG : 1;
    return HEADER_BYTES + (size_t)universe * 8 + planes * (size_t)words * 8 + (size_t)ceil_div<int64_t>(words, TILE) * 8 + 8;
}

extern "C" int32_t sgl_remap_init(void* state, size_t state_bytes, int64_t universe, void* stream) {
    if (!state || universe < 0) return fail(SGL_EINVAL, "remap_init: state is NULL or universe < 0");
    if (universe > 0xFFFFFFFFll) return fail(SGL_ENOTSUP, "remap_init: universe > 2^32");
    if (state_bytes < sgl_remap_state_bytes(universe))
        return fail(SGL_ENOMEM, "remap_init: state %zu < %zu bytes", state_bytes, sgl_remap_state_bytes(universe));
    if (reinterpret_cast<uintptr_t>(state) % 8) return fail(SGL_EINVAL, "remap_init: state must be 8-byte aligned");
    State s = carve(state, universe);
    int64_t blocks = ceil_div<int64_t>(universe > 0 ? universe : 1, 256);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(init_state_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), s);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" size_t sgl_unique_workspace_bytes(int64_t universe, int32_t G, const int64_t* len_max) {
    if (universe > 0) return dense_workspace_bytes(universe);
    return hash_unique_workspace_bytes(G, len_max);
}

extern "C" int32_t sgl_unique_compact(void* state, int64_t universe, int32_t reset, int32_t mode,
                                      int32_t G, const int64_t* const* ids, const int64_t* len_max,
                                      const int64_t* const* len_dev, int64_t* const* local_out,
                                      int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev,
                                      void* ws, size_t ws_bytes, void* stream) {
    if (G < 0 || (G > 0 && (!ids || !len_max || !local_out)) || !U_dev)
        return fail(SGL_EINVAL, "unique_compact: NULL argument");
    const bool premarked = (mode & SGL_UNIQUE_PREMARKED) != 0;
    const bool multi_launch = (mode & SGL_UNIQUE_MULTI_LAUNCH) != 0;
    mode &= ~(SGL_UNIQUE_PREMARKED | SGL_UNIQUE_MULTI_LAUNCH);
    if (mode != SGL_UNIQUE_SORTED && mode != SGL_UNIQUE_GROUPED) return fail(SGL_EINVAL, "unique_compact: bad mode");
    if (premarked && (mode != SGL_UNIQUE_SORTED || !reset || !state))
        return fail(SGL_EINVAL, "unique_compact: PREMARKED needs the dense state, SORTED mode and reset = 1");
    if (G > MAXG) return fail(SGL_ENOTSUP, "unique_compact: more than %d arrays", MAXG);
    if (unique_capacity < 0 || (unique_capacity > 0 && !unique_out))
        return fail(SGL_EINVAL, "unique_compact: unique_out is NULL");
    for (int32_t g = 0; g < G; ++g) {
        if (len_max[g] < 0) return fail(SGL_EINVAL, "unique_compact: negative length");
        if (len_max[g] > 0 && (!ids[g] || !local_out[g])) return fail(SGL_EINVAL, "unique_compact: array %d is NULL", g);
    }
    hipStream_t st = as_stream(stream);
    if (!state) {
        if (!reset) return fail(SGL_ENOTSUP, "unique_compact: hash path needs reset=1");
        return hash_unique_compact(mode, G, ids, len_max, len_dev, local_out, unique_out, unique_capacity,
                                   U_dev, ws, ws_bytes, st);
    }
    if (universe < 0 || universe > 0xFFFFFFFFll) return fail(SGL_EINVAL, "unique_compact: bad universe");
    if (!ws || ws_bytes < dense_workspace_bytes(universe))
        return fail(SGL_ENOMEM, "unique_compact: workspace %zu < %zu bytes", ws_bytes, dense_workspace_bytes(universe));
    State s = carve(state, universe);
    Arena ar(ws, ws_bytes);
    const int64_t nt = ceil_div<int64_t>(s.words > 0 ? s.words : 1, TILE);

    Arrays all;
    all.G = G;
    all.start[0] = 0;
    for (int g = 0; g < MAXG; ++g) {
        const bool live = g < G;
        all.ids[g] = live ? ids[g] : nullptr;
        all.out[g] = live ? local_out[g] : nullptr;
        all.len_dev[g] = (live && len_dev) ? len_dev[g] : nullptr;
        all.len_max[g] = live ? len_max[g] : 0;
        all.start[g + 1] = all.start[g] + all.len_max[g];
    }
    const int64_t total = all.start[MAXG];
    if (ceil_div<int64_t>(total, BLOCK) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "unique_compact: too many ids");

    // Grouped mode over a byte-flag state: one numbering pass for all arrays (array g marks plane g).
    // Over a bitmap state the arrays are numbered one after the other: there the marks are atomics,
    // and an id that an earlier array has already numbered is skipped by the later array's marking
    // pass - popular ids come back thousands of times in the deeper hops, and that many atomics on
    // one word cost more (906 us against 262 us for 14.7M ids) than the extra passes.
    const bool planes = mode == SGL_UNIQUE_GROUPED && s.bytes;
    int64_t* tile_sum = ar.take<int64_t>((planes ? (int64_t)G : 1) * nt + 2);
    uint32_t* stamp_ws = ar.take<uint32_t>(4);
    if (!ar.ok()) return fail(SGL_ENOMEM, "unique_compact: workspace too small");
    const int n_groups = (mode == SGL_UNIQUE_SORTED || planes) ? (G > 0 ? 1 : 0) : G;
    // groups that have anything to number; the commit of the last one is folded into the
    // lookup launch (one launch less per call), the others commit with a kernel of their own
    int runnable[MAXG], n_run = 0;
    for (int grp = 0; grp < n_groups; ++grp) {
        const int64_t sub_total = (mode == SGL_UNIQUE_GROUPED && !planes) ? all.len_max[grp] : total;
        if (sub_total > 0 && universe > 0) runnable[n_run++] = grp;
    }
    const bool fold = n_run > 0 && total > 0;
    int first = 1, rst = reset ? 1 : 0;
    for (int r = 0; r < n_run; ++r) {
        const int grp = runnable[r];
        Arrays sub = all;
        if (mode == SGL_UNIQUE_GROUPED && !planes) {  // only array `grp`
            sub.G = 1;
            sub.ids[0] = all.ids[grp]; sub.out[0] = all.out[grp];
            sub.len_dev[0] = all.len_dev[grp]; sub.len_max[0] = all.len_max[grp];
            sub.start[0] = 0;
            for (int g = 1; g <= MAXG; ++g) sub.start[g] = sub.len_max[0];
        }
        int64_t longest = 0;
        for (int g = 0; g < sub.G; ++g) longest = sub.len_max[g] > longest ? sub.len_max[g] : longest;
        int64_t mb = ceil_div<int64_t>(longest, BLOCK);
        if (mb > MAX_GRID) mb = MAX_GRID;
        if (!premarked) {
            hipLaunchKernelGGL(mark_kernel, dim3((unsigned)mb), dim3(BLOCK), 0, st, s, sub, rst, planes ? 1 : 0);
            SGL_LAUNCH_CHECK();
        }
        if (planes) {
            hipLaunchKernelGGL(reduce_groups_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, (int)G, nt, tile_sum);
            SGL_LAUNCH_CHECK();
            const int scanned = (int64_t)G * nt > FUSED_SCAN_MAX ? 1 : 0;
            if (scanned) {
                hipLaunchKernelGGL(scan_tiles_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, tile_sum, (int64_t)G * nt);
                SGL_LAUNCH_CHECK();
            }
            hipLaunchKernelGGL(assign_groups_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, (int)G, tile_sum, nt, scanned,
                               rst, unique_out, unique_capacity, U_dev, stamp_ws);
            SGL_LAUNCH_CHECK();
        } else if (nt <= SINGLE_PASS_MAX && !multi_launch) {
            hipLaunchKernelGGL(assign_kernel<2>, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum, nt, rst,
                               unique_out, unique_capacity, U_dev, stamp_ws, wait_limit());
            SGL_LAUNCH_CHECK();
        } else {
            hipLaunchKernelGGL(reduce_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum);
            SGL_LAUNCH_CHECK();
            if (nt > FUSED_SCAN_MAX) {
                hipLaunchKernelGGL(scan_tiles_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, tile_sum, nt);
                SGL_LAUNCH_CHECK();
                hipLaunchKernelGGL(assign_kernel<1>, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum, nt, rst,
                                   unique_out, unique_capacity, U_dev, stamp_ws, wait_limit());
            } else {
                hipLaunchKernelGGL(assign_kernel<0>, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum, nt, rst,
                                   unique_out, unique_capacity, U_dev, stamp_ws, wait_limit());
            }
            SGL_LAUNCH_CHECK();
        }
        if (fold && r == n_run - 1) break;   // committed by the lookup launch below
        hipLaunchKernelGGL(commit_kernel, dim3(1), dim3(1), 0, st, s, rst, first, 1, U_dev);
        SGL_LAUNCH_CHECK();
        first = 0;
        rst = 0;  // the epoch has been opened; later groups continue it
    }
    if (n_run == 0) {  // nothing was numbered: still open the epoch / report the counts
        hipLaunchKernelGGL(commit_kernel, dim3(1), dim3(1), 0, st, s, rst, 1, 0, U_dev);
        SGL_LAUNCH_CHECK();
    }
    if (total > 0) {
        int64_t longest = 0;
        for (int g = 0; g < all.G; ++g) longest = all.len_max[g] > longest ? all.len_max[g] : longest;
        int64_t lb = ceil_div<int64_t>(longest, BLOCK);
        if (lb > MAX_GRID) lb = MAX_GRID;
        hipLaunchKernelGGL(lookup_kernel, dim3((unsigned)lb), dim3(BLOCK), 0, st, s, all, fold ? 1 : 0, rst, first, 1,
                           stamp_ws, U_dev);
        SGL_LAUNCH_CHECK();
    }
    return SGL_OK;
}

// ---- batched: B mini-batches with local-id spaces of their own in one launch sequence ------------------
extern "C" size_t sgl_remap_batched_state_bytes(int64_t universe, int32_t B) {
    if (universe <= 0 || B < 1 || B > BATCH_MAX) return 0;
    const int64_t big = (int64_t)B * batch_stride(universe);
    return HEADER_BYTES + (size_t)(big / 64) * sizeof(RankWord) + (size_t)(big / (batched_byte_flags(big) ? 1 : 8)) + 16;
}

extern "C" int32_t sgl_remap_batched_init(void* state, size_t state_bytes, int64_t universe, int32_t B, void* stream) {
    if (!state || universe <= 0) return fail(SGL_EINVAL, "remap_batched_init: state is NULL or universe <= 0");
    if (B < 1 || B > BATCH_MAX) return fail(SGL_ENOTSUP, "remap_batched_init: B must be 1..%d", BATCH_MAX);
    if ((int64_t)B * batch_stride(universe) > 0xFFFFFFFFll) return fail(SGL_ENOTSUP, "remap_batched_init: B * universe > 2^32");
    if (state_bytes < sgl_remap_batched_state_bytes(universe, B))
        return fail(SGL_ENOMEM, "remap_batched_init: state %zu < %zu bytes", state_bytes, sgl_remap_batched_state_bytes(universe, B));
    if (reinterpret_cast<uintptr_t>(state) % 16) return fail(SGL_EINVAL, "remap_batched_init: state must be 16-byte aligned");
    BState s = carve_batched(state, universe, B);
    int64_t blocks = ceil_div<int64_t>(s.words, 256);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(init_batched_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), s);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" size_t sgl_unique_batched_workspace_bytes(int64_t universe, int32_t B) {
    if (universe <= 0 || B < 1 || B > BATCH_MAX) return 512;
    return batched_workspace_bytes(universe, B);
}

extern "C" int32_t sgl_unique_compact_batched(void* state, int64_t universe, int32_t B, int32_t G,
                                              const int64_t* const* ids, const int64_t* len_max,
                                              const int64_t* const* seg, int64_t* const* local_out,
                                              int64_t* unique_out, int64_t unique_capacity, int64_t* U_off,
                                              void* ws, size_t ws_bytes, void* stream) {
    if (!state || G < 1 || !ids || !len_max || !seg || !local_out || !U_off)
        return fail(SGL_EINVAL, "unique_compact_batched: NULL argument or G < 1");
    if (universe <= 0 || B < 1 || B > BATCH_MAX || (int64_t)B * batch_stride(universe) > 0xFFFFFFFFll)
        return fail(SGL_EINVAL, "unique_compact_batched: bad universe or B (1..%d)", BATCH_MAX);
    if (G > MAXG) return fail(SGL_ENOTSUP, "unique_compact_batched: more than %d arrays", MAXG);
    if (unique_capacity < 0 || (unique_capacity > 0 && !unique_out))
        return fail(SGL_EINVAL, "unique_compact_batched: unique_out is NULL");
    if (reinterpret_cast<uintptr_t>(state) % 16) return fail(SGL_EINVAL, "unique_compact_batched: state must be 16-byte aligned");
    if (!ws || ws_bytes < batched_workspace_bytes(universe, B))
        return fail(SGL_ENOMEM, "unique_compact_batched: workspace %zu < %zu bytes", ws_bytes, batched_workspace_bytes(universe, B));
    Arrays all;
    all.G = G;
    all.start[0] = 0;
    Batched bt;
    bt.B = B; bt.universe = universe; bt.stride = batch_stride(universe);
    int64_t longest = 0;
    for (int g = 0; g < MAXG; ++g) {
        const bool live = g < G;
        if (live && (len_max[g] < 0 || !seg[g] || (len_max[g] > 0 && (!ids[g] || !local_out[g]))))
            return fail(SGL_EINVAL, "unique_compact_batched: array %d: negative length or NULL pointer", g);
        all.ids[g] = live ? ids[g] : nullptr;
        all.out[g] = live ? local_out[g] : nullptr;
        all.len_dev[g] = nullptr;
        all.len_max[g] = live ? len_max[g] : 0;
        all.start[g + 1] = all.start[g] + all.len_max[g];
        bt.seg[g] = live ? seg[g] : nullptr;
        longest = all.len_max[g] > longest ? all.len_max[g] : longest;
    }
    if (ceil_div<int64_t>(all.start[MAXG], BLOCK) > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "unique_compact_batched: too many ids");
    hipStream_t st = as_stream(stream);
    BState s = carve_batched(state, universe, B);
    Arena ar(ws, ws_bytes);
    const int64_t nt = s.groups / TILE;
    int64_t* tile_sum = ar.take<int64_t>(nt + 2);
    if (!ar.ok()) return fail(SGL_ENOMEM, "unique_compact_batched: workspace too small");
    // a whole number of blocks per XCD; the walk deals the batches to classes of blocks, so the grid follows the
    // ids in all, not the longest array
    int64_t mb = ceil_div<int64_t>(ceil_div<int64_t>(all.start[MAXG] > 0 ? all.start[MAXG] : 1, BLOCK * WALK_ILP), XCDS) * XCDS;
    if (mb > MAX_GRID) mb = MAX_GRID;
    if (longest > 0) {
        hipLaunchKernelGGL(walk_batched_kernel<false>, dim3((unsigned)mb), dim3(BLOCK), 0, st, s, all, bt);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(reduce_batched_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum, bt, G);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_tiles_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, tile_sum, nt);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(assign_batched_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, s, tile_sum, nt, bt, G, unique_out,
                       unique_capacity, U_off);
    SGL_LAUNCH_CHECK();
    if (longest > 0) {
        hipLaunchKernelGGL(walk_batched_kernel<true>, dim3((unsigned)mb), dim3(BLOCK), 0, st, s, all, bt);
        SGL_LAUNCH_CHECK();
    }
    return SGL_OK;
}
