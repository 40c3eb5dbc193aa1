// Hash-set unique + compaction for ids without a dense universe (gfx950).
//
// For ids that are arbitrary non-negative 63-bit values (partition-encoded ids,
// say), where no table indexed by id can be kept.  The set is an open-addressing
// table of 8-byte keys with a parallel array of 4-byte local ids; it lives
// either in a persistent "hashed state" of a stated capacity (an epoch of local
// ids can then continue over several calls, as with the dense state) or, for
// one-shot calls, in the call's workspace.  A call is a fixed sequence of
// launches on the caller's stream, sized on the host from the worst case and
// driven by device-side counts - no host synchronisation, HIP-graph capturable:
//
//   prep    : empties the table (everything for a workspace table; for a
//             persistent one only on reset, and then only the slots the last
//             epoch used when those are few) and zeroes the bucket counters;
//             for calls of up to 2^20 ids it also leaves OR and AND over the
//             call's ids, one pair per block, for the insert to fold;
//   insert  : a block folds its tile of ids through an LDS set, so an id that
//             repeats inside the tile reaches the global table once; the
//             element that put an id into the LDS set probes the table for it
//             (a plain load first: most ids of a sampled batch are repeats and
//             end there; atomicCAS only on an empty slot).  Every input element
//             remembers the table slot of its id (4 bytes), so nothing is ever
//             probed twice.  The ids a block added are appended - id and slot -
//             to the call's list with ONE returning atomic per block; OR and
//             AND over them are kept.  Calls of up to 2^20 ids are bound by the
//             chain of round trips, not by the number of atomics: their probes
//             are an atomicCAS straight away (one round trip per probe instead
//             of two), the table is sparser (load <= 1/3), and the insert
//             itself counts the bucket sizes (the squeezed key below is then
//             made from the bits in which the call's ids differ, known from
//             prep, a superset of the bits in which the new ones do).
//             In grouped mode (an id belongs to the first
//             array that holds it) the arrays are inserted by one launch each, in
//             array order, so the ids an array adds are exactly those new to it;
//   order   : the new ids have to be numbered in ascending order.  The bits in
//             which they differ at all (OR ^ AND) are squeezed together into a
//             short key that keeps the order (in grouped mode the array that
//             owns the id is the top digit), and the top bits of that key cut
//             the ids into buckets of a few ids each:
//             - calls of up to 2^20 ids: the insert counts the bucket sizes with one
//               returning atomic per new id (what comes back is the id's place inside
//               its bucket); scatter moves the ids to their bucket's segment, every
//               block making the prefix of the at most 8192 sizes for itself in LDS
//               (its first block leaves the first places and the list of oversized
//               buckets in memory for the numbering launch);
//             - larger calls, where an atomic per id costs more than a pass
//               over the data: three 8-bit passes of the library's radix sort
//               on the top 24 bits of the key;
//   number  : an id's rank = first place of its bucket + ids of the bucket
//             that are smaller (a handful, compared from a tile of ids parked in
//             LDS); rank + ids numbered before = local id, written to the table and
//             the local->global list.  Oversized buckets (skewed id distributions)
//             are sorted by a block each with a bitonic network in place;
//   lookup  : out[i] = local id at the slot element i remembered.
//
// Numbering is by ascending id inside each group, so the result equals the dense
// path and the reference's sort + unique (csrc/include/starrygl/sample.cu.hpp:
// 1786-1852) bit for bit.
#include <algorithm>
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int MAXG = 8;
constexpr unsigned long long EMPTY = ~0ull;
constexpr uint32_t NONE = 0xFFFFFFFFu;   // slot of an element whose id is negative
constexpr uint32_t UNNUMBERED = 0x7FFFFFFFu;  // value of a slot whose id has no local id yet
constexpr int64_t MAX_CAPACITY = 0x7FFFFF00ll;
constexpr int NB_MIN_LOG = 8, NB_MAX_LOG = 13;   // buckets of the atomic route: at least one per thread of a block, at most what a block scans in LDS
constexpr int64_t ATOMIC_ROUTE_MAX = 1ll << 20;  // most ids a call may add for the atomic route to be taken
constexpr int SORT_KEY_LOG = 24;         // bucket bits of the radix route (three 8-bit passes)
constexpr int SORT_KEY_SHIFT = 64 - SORT_KEY_LOG;
constexpr int SMALL_BUCKET = 512;        // buckets up to this size are ranked by counting
constexpr int IDS_PER_BUCKET = 32;      // of the atomic route, when every id of the call is new
constexpr int64_t SPARSE_CAPACITY = 1ll << 20;   // tables up to this capacity are three times the capacity
constexpr int NMASK = BLOCK;             // most blocks of prep that leave an OR / AND pair
constexpr int MAX_GRID = 4096;

// Every field that blocks of one launch hammer with atomics has a 128-byte line of its own: a line that
// holds a contended counter serves nothing else at a useful rate.
struct Header {
    unsigned long long total;     // ids numbered in the current epoch (committed by the last launch of a call)
    unsigned long long nbig;      // oversized buckets of the running call (0 between calls)
    unsigned long long pad0[14];
    struct { unsigned long long n, pad[15]; } added[MAXG];   // ids the running call has added, per array group (0 between calls)
    unsigned long long or_mask;   // OR / AND over the ids the running call has added (0 / ~0 between calls)
    unsigned long long and_mask;
    unsigned long long pad2[14];
    unsigned long long overflow;  // sticky: more ids than the capacity, or no free slot
    unsigned long long pad3[15];
};
constexpr size_t HEADER_BYTES = 384 + 128 * MAXG;
static_assert(sizeof(Header) == HEADER_BYTES, "hashed state header layout");

struct Table {
    Header* hdr;
    unsigned long long* keys;   // [slots]
    uint32_t* vals;             // [slots] local id, or UNNUMBERED
    uint32_t* used;             // [capacity] slot of the k-th id of the epoch
    int64_t capacity, slots;
};

// (small tables are cheap to empty, and a short probe sequence is what a small call's time is made of)
int64_t slots_of(int64_t capacity) { return (capacity <= SPARSE_CAPACITY ? 3 * capacity : capacity + capacity / 2) + 64; }

size_t state_bytes(int64_t capacity) {
    const int64_t s = slots_of(capacity);
    return HEADER_BYTES + align_up((size_t)s * 8) + align_up((size_t)s * 4) + align_up((size_t)(capacity + 1) * 4);
}

Table carve(void* state, int64_t capacity) {
    Table t;
    char* p = static_cast<char*>(state);
    t.capacity = capacity;
    t.slots = slots_of(capacity);
    t.hdr = reinterpret_cast<Header*>(p);
    p += HEADER_BYTES;
    t.keys = reinterpret_cast<unsigned long long*>(p);
    p += align_up((size_t)t.slots * 8);
    t.vals = reinterpret_cast<uint32_t*>(p);
    p += align_up((size_t)t.slots * 4);
    t.used = reinterpret_cast<uint32_t*>(p);
    return t;
}

// Per-call scratch.  Atomic route: list_b, list_r, part_*, cnt, off, mask_part.  Radix route: key_a/b (bucket << 40 | table
// slot) with the ids as the sort's values (id_a/b), and the sort's own workspace.
struct Scratch {
    uint32_t* slot_of;          // [total] table slot of every input element (NONE: negative id)
    unsigned long long* list_id;  // [ncap] ids added by this call, in the order of their appends
    uint32_t* list_b;           // [ncap] their buckets
    uint32_t* list_r;           // [ncap] how many ids the bucket held when they were counted into it
    unsigned long long* part_id;  // [ncap] the same ids grouped by bucket
    uint32_t* part_slot;        // [ncap]
    uint32_t* part_b;           // [ncap]
    uint32_t* cnt;              // [nb + 1] bucket sizes
    uint32_t* off;              // [nb + 1] first places of the buckets, left by the first block of the scatter launch
    unsigned long long* mask_part;  // [2 * NMASK] OR / AND over the call's ids, one pair per block of prep
    uint32_t* big;              // [ncap / SMALL_BUCKET + 2] oversized buckets (atomic route) / their first places (radix route)
    uint64_t* key_a;            // [ncap] radix route
    uint64_t* key_b;
    int64_t* id_b;              // (id_a is list_id)
    void* sort_ws;
    size_t sort_ws_bytes;
    int64_t ncap;               // most ids one call can add
    int32_t nb_log;             // log2 of the number of buckets
    int32_t radix;              // 1: radix route
    int32_t nmask;              // pairs in mask_part
};

bool radix_route(int64_t ncap) { return ncap > ATOMIC_ROUTE_MAX; }

// entries of Scratch::big: a call that adds at most ncap ids has fewer than ncap / SMALL_BUCKET oversized buckets
__host__ __device__ constexpr int64_t big_capacity(int64_t ncap) { return ncap / SMALL_BUCKET + 2; }

int nb_log_of(int64_t ncap) {
    if (radix_route(ncap)) return SORT_KEY_LOG;
    int l = NB_MIN_LOG;
    while (l < NB_MAX_LOG && ((int64_t)IDS_PER_BUCKET << l) < ncap) ++l;
    return l;
}

size_t scratch_bytes(int64_t total, int64_t ncap) {
    const int64_t nb = 1ll << nb_log_of(ncap);
    size_t b = align_up((size_t)(total + 1) * 4) + align_up((size_t)(ncap + 1) * 8) +
               align_up((size_t)big_capacity(ncap) * 4) + 1024;
    if (radix_route(ncap))
        b += 3 * align_up((size_t)(ncap + 1) * 8) + radix_sort_workspace_bytes(ncap) + 256;
    else
        b += align_up((size_t)(ncap + 1) * 8) + 4 * align_up((size_t)(ncap + 1) * 4) + 2 * align_up((size_t)(nb + 1) * 4) +
             align_up((size_t)2 * NMASK * 8);
    return b;
}

Scratch carve_scratch(Arena& ar, int64_t total, int64_t ncap) {
    Scratch s{};
    s.ncap = ncap;
    s.nb_log = nb_log_of(ncap);
    s.radix = radix_route(ncap) ? 1 : 0;
    const int64_t nb = 1ll << s.nb_log;
    s.slot_of = ar.take<uint32_t>(total + 1);
    s.list_id = ar.take<unsigned long long>(ncap + 1);
    s.big = ar.take<uint32_t>(big_capacity(ncap));
    if (s.radix) {
        s.key_a = ar.take<uint64_t>(ncap + 1);
        s.key_b = ar.take<uint64_t>(ncap + 1);
        s.id_b = ar.take<int64_t>(ncap + 1);
        s.sort_ws_bytes = radix_sort_workspace_bytes(ncap);
        s.sort_ws = ar.take<char>(s.sort_ws_bytes);
    } else {
        s.part_id = ar.take<unsigned long long>(ncap + 1);
        s.list_b = ar.take<uint32_t>(ncap + 1);
        s.list_r = ar.take<uint32_t>(ncap + 1);
        s.part_slot = ar.take<uint32_t>(ncap + 1);
        s.part_b = ar.take<uint32_t>(ncap + 1);
        s.cnt = ar.take<uint32_t>(nb + 1);
        s.off = ar.take<uint32_t>(nb + 1);
        s.mask_part = ar.take<unsigned long long>(2 * NMASK);
    }
    return s;
}

__device__ __forceinline__ uint64_t mix(uint64_t x) {  // splitmix64 finaliser
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27; x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}

struct Arrays {
    int32_t G;
    const int64_t* ids[MAXG];
    int64_t* out[MAXG];
    const int64_t* len_dev[MAXG];
    int64_t len_max[MAXG];
    int64_t start[MAXG + 1];
};

__device__ __forceinline__ bool locate(const Arrays& a, int64_t t, int* g_out, int64_t* i_out) {
    if (t >= a.start[a.G]) return false;
    int g = 0;
#pragma unroll
    for (int q = 1; q < MAXG; ++q)
        if (q < a.G && t >= a.start[q]) g = q;
    const int64_t i = t - a.start[g];
    if (i >= live_count(a.len_dev[g], a.len_max[g])) return false;
    *g_out = g;
    *i_out = i;
    return true;
}

// What a call works with: ids numbered before it and (from the order launches on) ids it added.
__device__ __forceinline__ int64_t ids_before(const Table& t, int reset) { return reset ? 0 : (int64_t)t.hdr->total; }
__device__ __forceinline__ int64_t ids_added(const Table& t, const Scratch& s, int64_t before) {
    int64_t n = 0;
#pragma unroll
    for (int g = 0; g < MAXG; ++g) n += (int64_t)t.hdr->added[g].n;
    const int64_t room = t.capacity - before;
    if (n > room) n = room;
    if (n > s.ncap) n = s.ncap;
    return n < 0 ? 0 : n;
}
// array group of the k-th id the call added (groups are appended one after the other)
__device__ __forceinline__ uint32_t group_of(const Table& t, int64_t k) {
    uint32_t g = 0;
    int64_t end = 0;
#pragma unroll
    for (int q = 0; q < MAXG - 1; ++q) {
        end += (int64_t)t.hdr->added[q].n;
        g += k >= end ? 1u : 0u;
    }
    return g;
}
__device__ __forceinline__ void clear_call_fields(Header* h) {
#pragma unroll
    for (int g = 0; g < MAXG; ++g) h->added[g].n = 0;
    h->or_mask = 0;
    h->and_mask = ~0ull;
    h->nbig = 0;
}

// The bits in which the new ids differ, squeezed into a key that keeps their order: up to three runs
// of such bits from the top, then one span down to the lowest of them (it may hold bits that do not
// differ; only the top bits of the key select the bucket).
struct Codec {
    int32_t sh[4], dst[4];
    uint64_t mask[4];
    int32_t nb;   // bits of the key
};

__device__ inline Codec make_codec(uint64_t or_mask, uint64_t and_mask) {
    Codec c;
    uint64_t diff = (or_mask ^ and_mask) & 0x7FFFFFFFFFFFFFFFull;
    int32_t width[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        c.sh[n] = 0;
        c.mask[n] = 0;
        width[n] = 0;
        if (diff != 0) {
            const int top = 63 - __clzll((long long)diff);
            int lo;
            if (n < 3) {
                // the run of ones that ends at `top`
                const uint64_t below = ~diff & ((2ull << top) - 1ull);          // zeros at or below top
                lo = below == 0 ? 0 : 64 - __clzll((long long)below);        // first zero below the run, + 1
            } else {
                lo = __ffsll((unsigned long long)diff) - 1;
            }
            const int w = top - lo + 1;
            c.sh[n] = lo;
            c.mask[n] = (1ull << w) - 1ull;      // w <= 63
            width[n] = w;
            diff &= (lo == 0) ? 0ull : ((1ull << lo) - 1ull);
        }
    }
    c.nb = width[0] + width[1] + width[2] + width[3];
    int acc = c.nb;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        acc -= width[r];
        c.dst[r] = acc;
    }
    return c;
}

__device__ __forceinline__ uint64_t squeeze(const Codec& c, uint64_t id) {
    uint64_t k = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) k |= ((id >> c.sh[r]) & c.mask[r]) << c.dst[r];
    return k;
}

// bucket of an id of array group g: g is the top digit (glog bits), the key's top bits the rest
__device__ __forceinline__ uint32_t bucket_of(const Codec& c, uint64_t id, uint32_t g, int nb_log, int glog) {
    const int kb = nb_log - glog;
    const uint64_t key = squeeze(c, id);
    const uint64_t top = c.nb > kb ? key >> (c.nb - kb) : key;
    return (g << kb) | (uint32_t)top;
}

__global__ __launch_bounds__(BLOCK) void init_kernel(Table t) {
    const int64_t tid = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    for (int64_t i = tid; i < t.slots; i += (int64_t)gridDim.x * BLOCK) {
        t.keys[i] = EMPTY;
        t.vals[i] = UNNUMBERED;
    }
    if (tid == 0) {
        t.hdr->total = 0;
        t.hdr->overflow = 0;
        clear_call_fields(t.hdr);
    }
}

// OR / AND over the values of a block's threads, left in s_or / s_and (both set up before the call)
__device__ __forceinline__ void block_or_and(unsigned long long o, unsigned long long n, unsigned long long* s_or,
                                             unsigned long long* s_and) {
#pragma unroll
    for (int d = WAVE / 2; d > 0; d >>= 1) {
        o |= __shfl_xor(o, d);
        n &= __shfl_xor(n, d);
    }
    if (threadIdx.x % WAVE == 0) {
        atomicOr(s_or, o);
        atomicAnd(s_and, n);
    }
}

__global__ __launch_bounds__(BLOCK) void prep_kernel(Arrays a, Table t, Scratch s, int fresh, int reset) {
    __shared__ unsigned long long s_or, s_and;
    const int64_t tid = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * BLOCK;
    // every block reads the header before anyone writes it: only a fresh (workspace) table's header is
    // written here, and nobody reads that one.  Only the keys are emptied: whoever claims a slot sets its value.
    const int64_t prev = fresh ? 0 : (int64_t)t.hdr->total;
    if (fresh || (reset && prev * 4 >= t.slots)) {
        for (int64_t i = tid; i < t.slots; i += stride) t.keys[i] = EMPTY;
    } else if (reset) {
        for (int64_t k = tid; k < prev; k += stride) t.keys[t.used[k]] = EMPTY;
    }
    if (!s.radix) {
        const int64_t nb = 1ll << s.nb_log;
        for (int64_t i = tid; i <= nb; i += stride) s.cnt[i] = 0;
        if ((int)blockIdx.x < s.nmask) {     // block-uniform
            if (threadIdx.x == 0) {
                s_or = 0;
                s_and = ~0ull;
            }
            __syncthreads();
            unsigned long long o = 0, n = ~0ull;
            for (int64_t x = tid; x < a.start[a.G]; x += (int64_t)s.nmask * BLOCK) {
                int g;
                int64_t i;
                if (!locate(a, x, &g, &i)) continue;
                const int64_t id = a.ids[g][i];
                if (id >= 0) {
                    o |= (unsigned long long)id;
                    n &= (unsigned long long)id;
                }
            }
            block_or_and(o, n, &s_or, &s_and);
            __syncthreads();
            if (threadIdx.x == 0) {
                s.mask_part[2 * blockIdx.x] = s_or;
                s.mask_part[2 * blockIdx.x + 1] = s_and;
            }
        }
    }
    if (fresh && tid == 0) {
        t.hdr->total = 0;
        t.hdr->overflow = 0;
        clear_call_fields(t.hdr);
    }
}

// IPT ids per thread: a tile of 256 * IPT ids per block (small calls take small tiles so that the chip has
// blocks to run; large ones take large tiles, which fold more repeats before the table is touched).
// grp: the array group whose ids this launch adds (grouped mode: one launch per array, in array order, so that
// an id belongs to the first array that holds it; otherwise one launch, group 0, over all arrays).  flat_base:
// index of the launch's first element among the elements of all arrays (slot_of is indexed over all of them).
// SMALL (calls of the atomic route): probes are an atomicCAS straight away, and the ids the block adds are
// counted into their buckets here, with the key made from the masks prep left; otherwise a probe is a plain load
// first and OR / AND over the added ids go to the header for the launches that follow.
template <int IPT, bool SMALL>
__global__ __launch_bounds__(BLOCK) void insert_kernel(Arrays a, Table t, Scratch s, int reset, int grp, int glog,
                                                       int64_t flat_base) {
    constexpr int TILE = BLOCK * IPT;
    constexpr int LDS_SLOTS = 2 * TILE;      // load <= 0.5
    __shared__ unsigned long long s_key[LDS_SLOTS];
    __shared__ uint32_t s_aux[LDS_SLOTS];       // table slot of the id
    __shared__ int32_t s_won;
    __shared__ long long s_base;
    __shared__ unsigned long long s_or, s_and;  // SMALL: over the call's ids; otherwise over the ids the block added
#pragma unroll
    for (int q = 0; q < LDS_SLOTS / BLOCK; ++q) {
        s_key[q * BLOCK + threadIdx.x] = EMPTY;
    }
    if (threadIdx.x == 0) {
        s_won = 0;
        s_or = 0;
        s_and = ~0ull;
    }
    const int64_t t0 = (int64_t)blockIdx.x * TILE + threadIdx.x;
    // the tile's ids (every load issued before the first LDS probe)
    int64_t id[IPT];
    bool live[IPT];
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        // the id is loaded beside the array's live length, not after it (the arrays hold len_max entries)
        const int64_t x = t0 + (int64_t)q * BLOCK;
        id[q] = -1;
        live[q] = false;
        if (x < a.start[a.G]) {
            int g = 0;
#pragma unroll
            for (int w = 1; w < MAXG; ++w)
                if (w < a.G && x >= a.start[w]) g = w;
            const int64_t i = x - a.start[g];
            const int64_t v = a.ids[g][i];
            live[q] = i < live_count(a.len_dev[g], a.len_max[g]);
            if (live[q]) id[q] = v;
        }
    }
    unsigned long long part_or = 0, part_and = ~0ull;
    if constexpr (SMALL) {
        if ((int)threadIdx.x < s.nmask) {
            part_or = s.mask_part[2 * threadIdx.x];
            part_and = s.mask_part[2 * threadIdx.x + 1];
        }
    }
    __syncthreads();
    if constexpr (SMALL) block_or_and(part_or, part_and, &s_or, &s_and);
    int32_t ls[IPT];                      // LDS slot of the id; -1: negative id or no element
    bool owner[IPT];                      // this element put the id into the LDS set
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        ls[q] = -1;
        owner[q] = false;
        if (id[q] < 0) continue;
        uint32_t h = (uint32_t)mix((uint64_t)id[q]) & (LDS_SLOTS - 1);
        while (true) {
            const unsigned long long prev = atomicCAS(&s_key[h], EMPTY, (unsigned long long)id[q]);
            if (prev == EMPTY) owner[q] = true;
            if (prev == EMPTY || prev == (unsigned long long)id[q]) break;
            h = (h + 1) & (LDS_SLOTS - 1);
        }
        ls[q] = (int32_t)h;
    }
    // every owner finds or claims the table slot of its id: first probes of all its ids in flight together
    const int64_t before = ids_before(t, reset);
    uint64_t h[IPT];
    unsigned long long k0[IPT];
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        h[q] = 0;
        k0[q] = 0;
        if (owner[q]) {
            h[q] = __umul64hi(mix((uint64_t)id[q]), (uint64_t)t.slots);
            if constexpr (SMALL) k0[q] = atomicCAS(&t.keys[h[q]], EMPTY, (unsigned long long)id[q]);
            else k0[q] = t.keys[h[q]];  // a slot never changes once it holds an id: a cached value is good
        }
    }
    Codec codec{};
    if constexpr (SMALL) {
        __syncthreads();                 // the masks are folded
        codec = make_codec(s_or, s_and);
    }
    bool won[IPT];
    int32_t pos[IPT];
    uint32_t bkt[IPT], rnk[IPT];          // SMALL: bucket of a new id and how many ids the bucket held before it
    unsigned long long my_or = 0, my_and = ~0ull;
    bool lost = false;
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        won[q] = false;
        pos[q] = 0;
        bkt[q] = rnk[q] = 0;
        if (!owner[q]) continue;
        const unsigned long long me = (unsigned long long)id[q];
        unsigned long long k = k0[q];
        bool placed = false;
        for (int64_t probes = 0; probes < t.slots; ++probes) {
            if constexpr (SMALL) {
                if (probes > 0) k = atomicCAS(&t.keys[h[q]], EMPTY, me);
                if (k == EMPTY) {
                    won[q] = true;
                    k = me;
                }
            } else {
                if (probes > 0) k = t.keys[h[q]];
                if (k == EMPTY) {
                    k = atomicCAS(&t.keys[h[q]], EMPTY, me);
                    if (k == EMPTY) {
                        won[q] = true;
                        k = me;
                    }
                }
            }
            if (k == me) {
                placed = true;
                break;
            }
            h[q] = h[q] + 1 == (uint64_t)t.slots ? 0 : h[q] + 1;
        }
        if (!placed) {          // the table is full
            lost = true;
            won[q] = false;
            s_aux[ls[q]] = NONE;
            continue;
        }
        s_aux[ls[q]] = (uint32_t)h[q];
        if (won[q]) {
            pos[q] = atomicAdd(&s_won, 1);
            t.vals[h[q]] = UNNUMBERED;
            if constexpr (SMALL) {       // counted here, so that this round trip runs beside the block's append
                bkt[q] = bucket_of(codec, me, (uint32_t)grp, s.nb_log, glog);
                rnk[q] = atomicAdd(&s.cnt[bkt[q]], 1u);
            }
            my_or |= me;
            my_and &= me;
        }
    }
    if constexpr (!SMALL) {
        if (my_or != 0 || my_and != ~0ull) {
            atomicOr(&s_or, my_or);
            atomicAnd(&s_and, my_and);
        }
    }
    if (lost) atomicOr(&t.hdr->overflow, 1ull);
    __syncthreads();
    if (threadIdx.x == 0 && s_won > 0) {
        long long prev = 0;                 // ids added by the launches of the groups before this one
        for (int g = 0; g < grp; ++g) prev += (long long)t.hdr->added[g].n;
        s_base = prev + (long long)atomicAdd(&t.hdr->added[grp].n, (unsigned long long)s_won);
        if (before + s_base + s_won > t.capacity || s_base + s_won > s.ncap) atomicOr(&t.hdr->overflow, 1ull);
    }
    if constexpr (!SMALL) {
        // lanes of two other waves, so that the three round trips to the header run side by side.  The two masks
        // settle after the first few blocks: an atomic only when this block still changes them (they move one
        // way only, so a stale reading costs a redundant atomic, never a missing one)
        if (threadIdx.x == WAVE && s_won > 0 &&
            (s_or & ~__hip_atomic_load(&t.hdr->or_mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)))
            atomicOr(&t.hdr->or_mask, s_or);
        if (threadIdx.x == 2 * WAVE && s_won > 0 &&
            (~s_and & __hip_atomic_load(&t.hdr->and_mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)))
            atomicAnd(&t.hdr->and_mask, s_and);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        if (won[q]) {
            const int64_t k = s_base + pos[q];
            if (k < s.ncap && before + k < t.capacity) {
                s.list_id[k] = (unsigned long long)id[q];
                t.used[before + k] = (uint32_t)h[q];
                if constexpr (SMALL) {
                    s.list_b[k] = bkt[q];
                    s.list_r[k] = rnk[q];
                }
            }
        }
        if (live[q]) s.slot_of[flat_base + t0 + (int64_t)q * BLOCK] = ls[q] < 0 ? NONE : s_aux[ls[q]];
    }
}

// ---- atomic route -------------------------------------------------------------------------------
// Exclusive prefix of the nb <= 2^NB_MAX_LOG bucket sizes (and their total at [nb]) into LDS, by every block for
// itself: thread t loads its nb / BLOCK consecutive sizes (16 bytes at a time) and adds them up, the block scans
// the sums.  Entry i sits at i + i / 32, so that the threads' runs do not all start in the same bank.
constexpr int NB_MAX = 1 << NB_MAX_LOG;
constexpr int PRE_WORDS = NB_MAX + NB_MAX / 32 + 2;
__device__ __forceinline__ int pre_at(int i) { return i + (i >> 5); }

__device__ void block_prefix(const uint32_t* __restrict__ cnt, int nb, uint32_t* s_pre, uint32_t* s_wave) {
    constexpr int NW = BLOCK / WAVE;
    constexpr int PER_MAX = NB_MAX / BLOCK;
    const int per = nb / BLOCK;                // nb is a power of two >= BLOCK
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    uint32_t v[PER_MAX];
#pragma unroll
    for (int j = 0; j < PER_MAX; ++j) v[j] = 0;
    if (per >= 4) {
        const uint4* src = reinterpret_cast<const uint4*>(cnt + (size_t)threadIdx.x * per);   // (the counters are 256-byte aligned)
#pragma unroll
        for (int j = 0; j < PER_MAX / 4; ++j) {
            if (4 * j < per) {
                const uint4 x = src[j];
                v[4 * j] = x.x; v[4 * j + 1] = x.y; v[4 * j + 2] = x.z; v[4 * j + 3] = x.w;
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            if (j < per) v[j] = cnt[threadIdx.x * per + j];
    }
    uint32_t sum = 0;
#pragma unroll
    for (int j = 0; j < PER_MAX; ++j) sum += v[j];
    uint32_t inc = sum;
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const uint32_t y = __shfl_up(inc, d);
        if (lane >= d) inc += y;
    }
    if (lane == WAVE - 1) s_wave[wid] = inc;
    __syncthreads();
    uint32_t o = inc - sum, total = 0;
#pragma unroll
    for (int q = 0; q < NW; ++q) {
        const uint32_t x = s_wave[q];
        if (q < wid) o += x;
        total += x;
    }
#pragma unroll
    for (int j = 0; j < PER_MAX; ++j) {
        if (j < per) {
            s_pre[pre_at(threadIdx.x * per + j)] = o;
            o += v[j];
        }
    }
    if (threadIdx.x == 0) s_pre[pre_at(nb)] = total;
    __syncthreads();
}

// An id's place: first place of its bucket + the count the insert got back when it counted the id into the bucket.
// The list entries are loaded before the number of live ones is known (the arrays hold ncap entries).
__global__ __launch_bounds__(BLOCK) void scatter_kernel(Table t, Scratch s, int reset) {
    __shared__ uint32_t s_pre[PRE_WORDS];
    __shared__ uint32_t s_wave[BLOCK / WAVE];
    constexpr int PER = 2;
    const int64_t k0 = (int64_t)blockIdx.x * (PER * BLOCK) + threadIdx.x;
    uint32_t b[PER], r[PER];
    unsigned long long id[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t k = k0 + j * BLOCK;
        b[j] = r[j] = 0;
        id[j] = 0;
        if (k < s.ncap) {
            b[j] = s.list_b[k];
            r[j] = s.list_r[k];
            id[j] = s.list_id[k];
        }
    }
    const int nb = 1 << s.nb_log;
    // After an overflow (more ids than the capacity, or a full table) the counts the insert got back no longer
    // number the listed ids 0..n-1 bucket by bucket (ids without a place in the list were counted too), so places
    // would stay unwritten: the result is void anyway, and neither this launch nor the numbering one touches it.
    if (t.hdr->overflow != 0) return;                  // the same for every thread of the launch
    const int64_t before = ids_before(t, reset);       // (read before the barriers of the prefix, not after)
    const int64_t n = ids_added(t, s, before);
    block_prefix(s.cnt, nb, s_pre, s_wave);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t k = k0 + j * BLOCK;
        if (k >= n) continue;
        const int64_t p = (int64_t)s_pre[pre_at((int)(b[j] & (uint32_t)(nb - 1)))] + r[j];
        if (p >= n) continue;            // (cannot happen without an overflow)
        s.part_id[p] = id[j];
        s.part_slot[p] = t.used[before + k];
        s.part_b[p] = b[j];
    }
    if (blockIdx.x == 0) {               // for the numbering launch: the first places, and which buckets are oversized
        __shared__ uint32_t s_nbig;
        if (threadIdx.x == 0) s_nbig = 0;
        __syncthreads();
        for (int i = threadIdx.x; i <= nb; i += BLOCK) {
            const uint32_t f = s_pre[pre_at(i)];
            s.off[i] = f;
            if (i < nb && s_pre[pre_at(i + 1)] - f > (uint32_t)SMALL_BUCKET) {
                const uint32_t q = atomicAdd(&s_nbig, 1u);
                if ((int64_t)q < big_capacity(s.ncap)) s.big[q] = (uint32_t)i;    // (more only after an overflow)
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) t.hdr->nbig = (int64_t)s_nbig < big_capacity(s.ncap) ? s_nbig : (uint32_t)big_capacity(s.ncap);
    }
}

// In-place ascending sort of ids[0..n) (all distinct) with a companion array, by one block: a bitonic
// network in which every comparator puts the smaller id at the lower index, so that the positions from n
// up to the next power of two act as +infinity and their comparators are simply skipped.
template <typename IdT, typename PayloadT>
__device__ void block_sort(IdT* ids, PayloadT* payload, int64_t n) {
    int64_t p2 = 1;
    while (p2 < n) p2 <<= 1;
    for (int64_t k = 2; k <= p2; k <<= 1) {
        for (int64_t j = k >> 1; j > 0; j >>= 1) {
            for (int64_t c = threadIdx.x; c < p2 / 2; c += BLOCK) {
                int64_t i, l;
                if (j == (k >> 1)) {       // first step of a merge: mirror inside the block of k
                    const int64_t blk = c / j, r = c % j;
                    i = blk * k + r;
                    l = blk * k + k - 1 - r;
                } else {
                    i = 2 * j * (c / j) + (c % j);
                    l = i + j;
                }
                if (l < n) {
                    const IdT x = ids[i], y = ids[l];
                    if (x > y) {
                        ids[i] = y;
                        ids[l] = x;
                        const PayloadT sx = payload[i], sy = payload[l];
                        payload[i] = sy;
                        payload[l] = sx;
                    }
                }
            }
            __syncthreads();
        }
    }
}

// A block takes NUMBER_TILE consecutive places and parks their ids in LDS: an id is ranked against the ids of
// its bucket from there (a chain of LDS reads instead of one of trips to the L2); only the part of a bucket that
// lies outside the tile is read from memory.  Oversized buckets (skewed id distributions), listed by the scatter
// launch, are taken in turn by the blocks and sorted in place.
constexpr int NUMBER_TILE = 2 * BLOCK;
__global__ __launch_bounds__(BLOCK) void number_kernel(Table t, Scratch s, int reset, int64_t* __restrict__ unique_out,
                                                       int64_t unique_capacity) {
    __shared__ unsigned long long s_id[NUMBER_TILE];
    constexpr int PER = NUMBER_TILE / BLOCK;
    const int64_t p0 = (int64_t)blockIdx.x * NUMBER_TILE;
    const int nb = 1 << s.nb_log;
    if (t.hdr->overflow != 0) return;                  // the scatter launch left nothing to number (see there)
    uint32_t slot[PER];
    int64_t lo[PER], hi[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {       // loaded before the number of live places is known (the arrays hold ncap entries)
        const int64_t p = p0 + j * BLOCK + threadIdx.x;
        slot[j] = 0;
        lo[j] = hi[j] = 0;
        if (p < s.ncap) {
            s_id[j * BLOCK + threadIdx.x] = s.part_id[p];
            slot[j] = s.part_slot[p];
            const uint32_t bucket = s.part_b[p] & (uint32_t)(nb - 1);
            lo[j] = s.off[bucket];
            hi[j] = s.off[bucket + 1];
        }
    }
    const int64_t before = ids_before(t, reset);
    const int64_t n = ids_added(t, s, before);
    const int64_t nbig = (int64_t)t.hdr->nbig;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t p = p0 + j * BLOCK + threadIdx.x;
        if (p >= n) continue;
        if (lo[j] > n) lo[j] = n;         // (beyond n only after an overflow)
        if (hi[j] > n) hi[j] = n;
        if (hi[j] - lo[j] > SMALL_BUCKET) continue;       // sorted below
        const unsigned long long id = s_id[j * BLOCK + threadIdx.x];
        int64_t r = lo[j];
        if (lo[j] >= p0 && hi[j] <= p0 + NUMBER_TILE) {    // the whole bucket is in the tile (all but the buckets at its ends)
            const int a = (int)(lo[j] - p0), e = (int)(hi[j] - p0);
            int q = a;
            for (; q + 4 <= e; q += 4) {
                const unsigned long long o0 = s_id[q], o1 = s_id[q + 1], o2 = s_id[q + 2], o3 = s_id[q + 3];
                r += (o0 < id ? 1 : 0) + (o1 < id ? 1 : 0) + (o2 < id ? 1 : 0) + (o3 < id ? 1 : 0);
            }
            for (; q < e; ++q) r += s_id[q] < id ? 1 : 0;
        } else {
            for (int64_t q = lo[j]; q < hi[j]; ++q) {
                const int64_t rel = q - p0;
                const unsigned long long other = (rel >= 0 && rel < NUMBER_TILE) ? s_id[rel] : s.part_id[q];
                r += other < id ? 1 : 0;
            }
        }
        const int64_t local = before + r;
        if (local < unique_capacity) unique_out[local] = (int64_t)id;
        if ((int64_t)slot[j] < t.slots) t.vals[slot[j]] = (uint32_t)local;
    }
    for (int64_t q = blockIdx.x; q < nbig; q += gridDim.x) {
        const uint32_t bucket = s.big[q];
        int64_t blo = s.off[bucket], bhi = s.off[bucket + 1];
        if (blo > n) blo = n;
        if (bhi > n) bhi = n;
        const int64_t len = bhi - blo;
        __syncthreads();
        block_sort(s.part_id + blo, s.part_slot + blo, len);
        for (int64_t j = threadIdx.x; j < len; j += BLOCK) {
            const int64_t local = before + blo + j;
            if (local < unique_capacity) unique_out[local] = (int64_t)s.part_id[blo + j];
            t.vals[s.part_slot[blo + j]] = (uint32_t)local;
        }
    }
}

// ---- radix route --------------------------------------------------------------------------------
// sort key of the k-th new id: bucket << 40 | table slot (the sort only looks at the bucket); value: the id
__global__ __launch_bounds__(BLOCK) void sortkey_kernel(Table t, Scratch s, int reset, int grouped, int glog, int64_t* n_out) {
    __shared__ Codec s_codec;
    if (threadIdx.x == 0) s_codec = make_codec(t.hdr->or_mask, t.hdr->and_mask);
    __syncthreads();
    const Codec c = s_codec;
    const int64_t before = ids_before(t, reset);
    const int64_t n = ids_added(t, s, before);
    if (blockIdx.x == 0 && threadIdx.x == 0) *n_out = n;      // the sort's live length
    for (int64_t k = (int64_t)blockIdx.x * BLOCK + threadIdx.x; k < n; k += (int64_t)gridDim.x * BLOCK) {
        const uint32_t slot = t.used[before + k];
        const uint32_t b = bucket_of(c, s.list_id[k], grouped ? group_of(t, k) : 0, SORT_KEY_LOG, glog);
        s.key_a[k] = ((uint64_t)b << SORT_KEY_SHIFT) | slot;
    }
}

// keys/ids: the new ids ordered by bucket.  A bucket is a run of equal keys >> 40; a thread finds the ends of
// its run by walking (runs hold tens of ids), counting the smaller ids on the way.  A run longer than
// SMALL_BUCKET is left to sorted_runs_kernel: its first place is listed by the thread that stands there.
__global__ __launch_bounds__(BLOCK) void rank_kernel(Table t, Scratch s, const uint64_t* __restrict__ keys,
                                                     const int64_t* __restrict__ ids, int reset,
                                                     int64_t* __restrict__ unique_out, int64_t unique_capacity) {
    const int64_t before = ids_before(t, reset);
    const int64_t n = ids_added(t, s, before);
    for (int64_t p = (int64_t)blockIdx.x * BLOCK + threadIdx.x; p < n; p += (int64_t)gridDim.x * BLOCK) {
        const uint64_t key = keys[p];
        const uint64_t top = key >> SORT_KEY_SHIFT;
        const int64_t id = ids[p];
        int64_t smaller = 0, left = 0, right = 0;
        bool open = false;
        for (int64_t q = p - 1;; --q) {               // to the left
            if (q < 0 || (keys[q] >> SORT_KEY_SHIFT) != top) break;
            if (++left > SMALL_BUCKET) { open = true; break; }
            smaller += ids[q] < id ? 1 : 0;
        }
        for (int64_t q = p + 1; !open; ++q) {         // to the right
            if (q >= n || (keys[q] >> SORT_KEY_SHIFT) != top) break;
            if (++right > SMALL_BUCKET) { open = true; break; }
            smaller += ids[q] < id ? 1 : 0;
        }
        if (open || left + right + 1 > SMALL_BUCKET) {
            if (left == 0) s.big[atomicAdd(&t.hdr->nbig, 1ull)] = (uint32_t)p;
            continue;
        }
        const int64_t local = before + (p - left) + smaller;
        if (local < unique_capacity) unique_out[local] = id;
        t.vals[(uint32_t)key] = (uint32_t)local;
    }
}

__global__ __launch_bounds__(BLOCK) void sorted_runs_kernel(Table t, Scratch s, uint64_t* keys, int64_t* ids, int reset,
                                                            int64_t* __restrict__ unique_out, int64_t unique_capacity) {
    __shared__ int64_t s_end;
    const int64_t before = ids_before(t, reset);
    const int64_t n = ids_added(t, s, before);
    const int64_t nbig = (int64_t)t.hdr->nbig;
    for (int64_t q = blockIdx.x; q < nbig; q += gridDim.x) {
        const int64_t lo = s.big[q];
        const uint64_t top = keys[lo] >> SORT_KEY_SHIFT;
        // the run's end: the first place from lo on whose bucket differs
        if (threadIdx.x == 0) s_end = n;
        __syncthreads();
        for (int64_t base = lo; base < n; base += BLOCK) {
            const int64_t x = base + threadIdx.x;
            if (x < n && (keys[x] >> SORT_KEY_SHIFT) != top) atomicMin(reinterpret_cast<unsigned long long*>(&s_end), (unsigned long long)x);
            __syncthreads();
            const int64_t e = s_end;
            __syncthreads();              // (nobody writes s_end again before everybody has read it)
            if (e < n) break;
        }
        const int64_t len = s_end - lo;
        __syncthreads();
        block_sort(ids + lo, keys + lo, len);
        for (int64_t j = threadIdx.x; j < len; j += BLOCK) {
            const int64_t local = before + lo + j;
            if (local < unique_capacity) unique_out[local] = ids[lo + j];
            t.vals[(uint32_t)keys[lo + j]] = (uint32_t)local;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(BLOCK) void lookup_kernel(Arrays a, Table t, Scratch s, int reset, int64_t* U_dev) {
    const int64_t i0 = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    // the call's totals, committed by one thread: no other thread of this launch reads the header
    if (i0 == 0) {
        const int64_t before = ids_before(t, reset);
        const int64_t n = ids_added(t, s, before);
        const bool void_result = t.hdr->overflow != 0;
        U_dev[0] = void_result ? INT64_MAX : before + n;
        U_dev[1] = before;
        t.hdr->total = (unsigned long long)(before + n);
        clear_call_fields(t.hdr);
    }
    for (int64_t x = i0; x < a.start[a.G]; x += (int64_t)gridDim.x * BLOCK) {
        int g;
        int64_t i;
        if (!locate(a, x, &g, &i)) continue;
        const uint32_t h = s.slot_of[x];
        int64_t local = -1;
        if (h != NONE) {
            const uint32_t v = t.vals[h];
            if (v != UNNUMBERED) local = (int64_t)v;
        }
        a.out[g][i] = local;
    }
}

int32_t check_capacity(int64_t capacity) {
    if (capacity < 0 || capacity > MAX_CAPACITY)
        return fail(SGL_EINVAL, "hashed remap state: capacity %lld outside [0, %lld]", (long long)capacity, (long long)MAX_CAPACITY);
    return SGL_OK;
}

using InsertKernel = void (*)(Arrays, Table, Scratch, int, int, int, int64_t);

int32_t run(Table t, bool fresh, int32_t reset, int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
            const int64_t* const* len_dev, int64_t* const* local_out, int64_t* unique_out, int64_t unique_capacity,
            int64_t* U_dev, Arena& ar, hipStream_t st) {
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
    if (total > MAX_CAPACITY) return fail(SGL_ENOTSUP, "unique_compact: too many ids");
    const int64_t ncap = total < t.capacity ? total : t.capacity;
    Scratch s = carve_scratch(ar, total, ncap);
    int64_t* n_sort = ar.take<int64_t>(1);
    if (!ar.ok()) return fail(SGL_ENOMEM, "unique_compact: workspace too small");
    const int grouped = (mode == SGL_UNIQUE_GROUPED && G > 1) ? 1 : 0;
    int glog = 0;
    while (grouped && (1 << glog) < G) ++glog;

    auto grid = [](int64_t work, int per_block) {
        int64_t b = ceil_div<int64_t>(work > 0 ? work : 1, per_block);
        return dim3((unsigned)(b > MAX_GRID ? MAX_GRID : b));
    };
    int64_t prep_work = (fresh || reset) ? t.slots : 1;
    if (!s.radix) prep_work = std::max<int64_t>(prep_work, std::max<int64_t>(1ll << s.nb_log, total));
    const dim3 prep_grid = grid(prep_work, 4 * BLOCK);
    s.nmask = s.radix ? 0 : (int32_t)std::min<unsigned>(prep_grid.x, (unsigned)NMASK);
    hipLaunchKernelGGL(prep_kernel, prep_grid, dim3(BLOCK), 0, st, all, t, s, fresh ? 1 : 0, reset);
    SGL_LAUNCH_CHECK();
    if (total > 0) {
        // tile of the insert: 1024 ids per block (larger tiles fold more repeats before the table is touched but
        // leave fewer waves per compute unit to hide the table's latency: 2048 ids per block is 10 % slower
        // on 15.6M ids); small launches take smaller tiles so that the chip still has a few hundred blocks
        auto launch_insert = [&](const Arrays& arr, int64_t n, int grp, int64_t flat_base) -> int32_t {
            int ipt = 4;
            while (ipt > 1 && n / (BLOCK * ipt) < 256) ipt >>= 1;
            const InsertKernel ins = s.radix ? (ipt == 4 ? insert_kernel<4, false> : ipt == 2 ? insert_kernel<2, false> : insert_kernel<1, false>)
                                             : (ipt == 4 ? insert_kernel<4, true> : ipt == 2 ? insert_kernel<2, true> : insert_kernel<1, true>);
            hipLaunchKernelGGL(ins, dim3((unsigned)ceil_div<int64_t>(n, BLOCK * ipt)), dim3(BLOCK), 0, st, arr, t, s, reset, grp, glog, flat_base);
            SGL_LAUNCH_CHECK();
            return SGL_OK;
        };
        int32_t rc_ins = SGL_OK;
        if (!grouped) {
            rc_ins = launch_insert(all, total, 0, 0);
        } else {
            for (int g = 0; g < G && rc_ins == SGL_OK; ++g) {   // array by array: an id belongs to the first array that holds it
                if (all.len_max[g] == 0) continue;
                Arrays sub = all;
                sub.G = 1;
                sub.ids[0] = all.ids[g]; sub.out[0] = all.out[g];
                sub.len_dev[0] = all.len_dev[g]; sub.len_max[0] = all.len_max[g];
                sub.start[0] = 0;
                for (int q = 1; q <= MAXG; ++q) sub.start[q] = sub.len_max[0];
                rc_ins = launch_insert(sub, sub.len_max[0], g, all.start[g]);
            }
        }
        if (rc_ins != SGL_OK) return rc_ins;
        if (!s.radix) {
            hipLaunchKernelGGL(scatter_kernel, dim3((unsigned)ceil_div<int64_t>(std::max<int64_t>(ncap, 1), 2 * BLOCK)), dim3(BLOCK), 0, st, t, s, reset);
            SGL_LAUNCH_CHECK();
            hipLaunchKernelGGL(number_kernel, dim3((unsigned)ceil_div<int64_t>(std::max<int64_t>(ncap, 1), NUMBER_TILE)), dim3(BLOCK), 0, st, t, s, reset,
                               unique_out, unique_capacity);
            SGL_LAUNCH_CHECK();
        } else {
            hipLaunchKernelGGL(sortkey_kernel, grid(ncap, BLOCK), dim3(BLOCK), 0, st, t, s, reset, grouped, glog, n_sort);
            SGL_LAUNCH_CHECK();
            int in_b = 0;
            int64_t* id_a = reinterpret_cast<int64_t*>(s.list_id);
            const int32_t rc = radix_sort_pairs(s.key_a, id_a, s.key_b, s.id_b, ncap, n_sort, SORT_KEY_SHIFT, 64, &in_b, s.sort_ws,
                                                s.sort_ws_bytes, st);
            if (rc != SGL_OK) return rc;
            uint64_t* keys = in_b ? s.key_b : s.key_a;
            int64_t* sorted_ids = in_b ? s.id_b : id_a;
            hipLaunchKernelGGL(rank_kernel, grid(ncap, BLOCK), dim3(BLOCK), 0, st, t, s, keys, sorted_ids, reset, unique_out, unique_capacity);
            SGL_LAUNCH_CHECK();
            hipLaunchKernelGGL(sorted_runs_kernel, dim3(256), dim3(BLOCK), 0, st, t, s, keys, sorted_ids, reset, unique_out, unique_capacity);
            SGL_LAUNCH_CHECK();
        }
    }
    hipLaunchKernelGGL(lookup_kernel, grid(total, BLOCK), dim3(BLOCK), 0, st, all, t, s, reset, U_dev);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

int64_t total_of(int32_t G, const int64_t* len_max) {
    int64_t total = 0;
    for (int32_t g = 0; g < G && len_max; ++g) total += len_max[g] > 0 ? len_max[g] : 0;
    return total;
}

}  // namespace

// ---- one-shot calls (sgl_unique_compact without a state): the table lives in the workspace ----
size_t hash_unique_workspace_bytes(int32_t G, const int64_t* len_max) {
    const int64_t total = total_of(G, len_max);
    return state_bytes(total) + scratch_bytes(total, total) + 1024;
}

int32_t hash_unique_compact(int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev, int64_t* const* local_out,
                            int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, hipStream_t st) {
    if (!ws || ws_bytes < hash_unique_workspace_bytes(G, len_max))
        return fail(SGL_ENOMEM, "unique_compact: workspace %zu < %zu bytes", ws_bytes, hash_unique_workspace_bytes(G, len_max));
    const int64_t total = total_of(G, len_max);
    if (total > MAX_CAPACITY) return fail(SGL_ENOTSUP, "unique_compact: too many ids");
    Arena ar(ws, ws_bytes);
    void* state = ar.take<char>(state_bytes(total));
    return run(carve(state, total), true, 1, mode, G, ids, len_max, len_dev, local_out, unique_out, unique_capacity, U_dev, ar, st);
}

}  // namespace sgl

using namespace sgl;

extern "C" size_t sgl_remap_hashed_state_bytes(int64_t capacity) {
    return state_bytes(capacity < 0 ? 0 : (capacity > MAX_CAPACITY ? MAX_CAPACITY : capacity));
}

extern "C" int32_t sgl_remap_hashed_init(void* state, size_t bytes, int64_t capacity, void* stream) {
    int32_t rc;
    if ((rc = check_capacity(capacity)) != SGL_OK) return rc;
    if (capacity < 1) return fail(SGL_EINVAL, "remap_hashed_init: capacity < 1");
    if (!state || bytes < state_bytes(capacity))
        return fail(SGL_EINVAL, "remap_hashed_init: state is NULL or smaller than %zu bytes", state_bytes(capacity));
    Table t = carve(state, capacity);
    int64_t b = ceil_div<int64_t>(t.slots, 4 * BLOCK);
    if (b > MAX_GRID) b = MAX_GRID;
    hipLaunchKernelGGL(init_kernel, dim3((unsigned)b), dim3(BLOCK), 0, as_stream(stream), t);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" size_t sgl_unique_hashed_workspace_bytes(int64_t capacity, int32_t G, const int64_t* len_max) {
    const int64_t total = total_of(G, len_max);
    const int64_t cap = capacity < 0 ? 0 : capacity;
    return scratch_bytes(total, total < cap ? total : cap) + 1024;
}

extern "C" int32_t sgl_unique_compact_hashed(void* state, int64_t capacity, int32_t reset, int32_t mode, int32_t G,
                                             const int64_t* const* ids, const int64_t* len_max,
                                             const int64_t* const* len_dev, int64_t* const* local_out,
                                             int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                                             size_t ws_bytes, void* stream) {
    int32_t rc;
    if (!state) return fail(SGL_EINVAL, "unique_compact_hashed: state is NULL");
    if ((rc = check_capacity(capacity)) != SGL_OK) return rc;
    if (capacity < 1) return fail(SGL_EINVAL, "unique_compact_hashed: capacity < 1");
    if (G < 0 || (G > 0 && (!ids || !len_max || !local_out)) || !U_dev)
        return fail(SGL_EINVAL, "unique_compact_hashed: NULL argument");
    if (mode != SGL_UNIQUE_SORTED && mode != SGL_UNIQUE_GROUPED) return fail(SGL_EINVAL, "unique_compact_hashed: bad mode");
    if (G > MAXG) return fail(SGL_ENOTSUP, "unique_compact_hashed: more than %d arrays", MAXG);
    if (unique_capacity < 0 || (unique_capacity > 0 && !unique_out))
        return fail(SGL_EINVAL, "unique_compact_hashed: unique_out is NULL");
    for (int32_t g = 0; g < G; ++g) {
        if (len_max[g] < 0) return fail(SGL_EINVAL, "unique_compact_hashed: negative length");
        if (len_max[g] > 0 && (!ids[g] || !local_out[g])) return fail(SGL_EINVAL, "unique_compact_hashed: array %d is NULL", g);
    }
    if (!ws || ws_bytes < sgl_unique_hashed_workspace_bytes(capacity, G, len_max))
        return fail(SGL_ENOMEM, "unique_compact_hashed: workspace %zu < %zu bytes", ws_bytes,
                    sgl_unique_hashed_workspace_bytes(capacity, G, len_max));
    Arena ar(ws, ws_bytes);
    return run(carve(state, capacity), false, reset ? 1 : 0, mode, G, ids, len_max, len_dev, local_out, unique_out,
               unique_capacity, U_dev, ar, as_stream(stream));
}
