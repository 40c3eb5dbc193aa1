// Hash-set unique + compaction for ids without a dense universe (gfx950).
//
// Used when the caller has no remap state (ids are arbitrary non-negative
// 63-bit values, e.g. partition-encoded ids).  Per group of input arrays:
//   insert  : a block folds its 1024 ids through an LDS open-addressing set, so
//             an id that repeats inside the tile reaches the global table
//             once; block-unique ids are claimed in the global table with
//             atomicCAS; the ids a block wins are appended to the group's list
//             with ONE global atomicAdd per block (same-address atomics cost
//             ~11 ns each on MI355X, per-id appends would dominate);
//   (one host read of the per-group counts and the largest id)
//   sort    : the group's new ids are radix-sorted on the bits actually used;
//   number  : rank r of the sorted list gets local id base + r, written into the
//             table's value array and the local->global list;
// then one lookup launch rewrites every input array.  Numbering is by ascending
// id inside each group, so the result equals the dense path and the reference's
// sort + unique (csrc/include/starrygl/sample.cu.hpp:1786-1811) bit for bit.
// The call synchronises with the host once.
#include "common.hpp"
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int MAXG = 8;
constexpr int IPT = 4;
constexpr int TILE = BLOCK * IPT;        // ids per block
constexpr int LDS_SLOTS = 2 * TILE;      // load <= 0.5
constexpr unsigned long long EMPTY = ~0ull;

struct Counters {
    long long count[MAXG];  // new ids of each group
    long long max_id;
};

__device__ __forceinline__ uint64_t mix(uint64_t x) {  // splitmix64 finaliser
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27; x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}

__global__ void fill_empty_kernel(unsigned long long* keys, int64_t cap, Counters* c) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = t; i < cap; i += stride) keys[i] = EMPTY;
    if (t == 0) {
        for (int g = 0; g < MAXG; ++g) c->count[g] = 0;
        c->max_id = 0;
    }
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

__global__ __launch_bounds__(BLOCK) void insert_kernel(Arrays a, unsigned long long* __restrict__ keys,
                                                       int64_t cap_mask, int grp, Counters* c,
                                                       int64_t* __restrict__ list) {
    __shared__ unsigned long long s_set[LDS_SLOTS];
    __shared__ int32_t s_won;
    __shared__ long long s_base, s_max;
    for (int q = threadIdx.x; q < LDS_SLOTS; q += BLOCK) s_set[q] = EMPTY;
    if (threadIdx.x == 0) { s_won = 0; s_max = 0; }
    __syncthreads();
    const int64_t t0 = (int64_t)blockIdx.x * TILE + threadIdx.x;
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
        int g;
        int64_t i;
        if (!locate(a, t0 + (int64_t)q * BLOCK, &g, &i)) continue;
        const int64_t id = a.ids[g][i];
        if (id < 0) continue;
        uint32_t h = (uint32_t)mix((uint64_t)id) & (LDS_SLOTS - 1);
        while (true) {
            const unsigned long long prev = atomicCAS(&s_set[h], EMPTY, (unsigned long long)id);
            if (prev == EMPTY || prev == (unsigned long long)id) break;
            h = (h + 1) & (LDS_SLOTS - 1);
        }
    }
    __syncthreads();
    // every occupied LDS slot is one block-unique id: claim it in the global table
    unsigned long long won[LDS_SLOTS / BLOCK];
    int32_t pos[LDS_SLOTS / BLOCK];
    long long mx = 0;
#pragma unroll
    for (int q = 0; q < LDS_SLOTS / BLOCK; ++q) {
        const unsigned long long id = s_set[q * BLOCK + threadIdx.x];
        won[q] = EMPTY;
        pos[q] = 0;
        if (id == EMPTY) continue;
        uint64_t h = mix(id) & (uint64_t)cap_mask;
        while (true) {
            const unsigned long long prev = atomicCAS(&keys[h], EMPTY, id);
            if (prev == EMPTY) { won[q] = id; break; }
            if (prev == id) break;
            h = (h + 1) & (uint64_t)cap_mask;
        }
        if (won[q] != EMPTY) {
            pos[q] = atomicAdd(&s_won, 1);
            mx = (long long)id > mx ? (long long)id : mx;
        }
    }
    if (mx > 0) atomicMax(&s_max, mx);
    __syncthreads();
    if (threadIdx.x == 0 && s_won > 0) {
        s_base = (long long)atomicAdd(reinterpret_cast<unsigned long long*>(&c->count[grp]), (unsigned long long)s_won);
        atomicMax(&c->max_id, s_max);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < LDS_SLOTS / BLOCK; ++q)
        if (won[q] != EMPTY) list[s_base + pos[q]] = (int64_t)won[q];
}

__device__ __forceinline__ int64_t find_slot(const unsigned long long* __restrict__ keys, int64_t cap_mask,
                                             unsigned long long id) {
    uint64_t h = mix(id) & (uint64_t)cap_mask;
    while (true) {
        const unsigned long long k = keys[h];
        if (k == id) return (int64_t)h;
        if (k == EMPTY) return -1;
        h = (h + 1) & (uint64_t)cap_mask;
    }
}

__global__ __launch_bounds__(BLOCK) void number_kernel(const uint64_t* __restrict__ sorted, int64_t count,
                                                       int64_t base, const unsigned long long* __restrict__ keys,
                                                       int64_t* __restrict__ vals, int64_t cap_mask,
                                                       int64_t* __restrict__ unique_out, int64_t unique_capacity) {
    const int64_t r = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (r >= count) return;
    const unsigned long long id = sorted[r];
    const int64_t slot = find_slot(keys, cap_mask, id);
    if (slot >= 0) vals[slot] = base + r;
    if (base + r < unique_capacity) unique_out[base + r] = (int64_t)id;
}

__global__ __launch_bounds__(BLOCK) void lookup_kernel(Arrays a, const unsigned long long* __restrict__ keys,
                                                       const int64_t* __restrict__ vals, int64_t cap_mask) {
    const int64_t t = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    int g;
    int64_t i;
    if (!locate(a, t, &g, &i)) return;
    const int64_t id = a.ids[g][i];
    int64_t local = -1;
    if (id >= 0) {
        const int64_t slot = find_slot(keys, cap_mask, (unsigned long long)id);
        if (slot >= 0) local = vals[slot];
    }
    a.out[g][i] = local;
}

__global__ void publish_kernel(int64_t* U_dev, int64_t total) {
    U_dev[0] = total;
    U_dev[1] = 0;
}

int64_t table_capacity(int64_t total) {
    int64_t c = 1024;
    while (c < 2 * total) c <<= 1;
    return c;
}

int bits_of(uint64_t x) {
    int b = 0;
    while (x) { ++b; x >>= 1; }
    return b;
}

}  // namespace

size_t hash_unique_workspace_bytes(int32_t G, const int64_t* len_max) {
    int64_t total = 0, longest = 0;
    for (int32_t g = 0; g < G && len_max; ++g) {
        const int64_t l = len_max[g] > 0 ? len_max[g] : 0;
        total += l;
    }
    longest = total;  // sorted mode sorts all ids as one group
    const int64_t cap = table_capacity(total);
    return 2 * align_up((size_t)cap * 8) + 3 * align_up((size_t)(total + 1) * 8) + align_up((size_t)(longest + 1) * 8) +
           radix_sort_workspace_bytes(longest) + 8192;
}

int32_t hash_unique_compact(int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev, int64_t* const* local_out,
                            int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, hipStream_t st) {
    if (!ws || ws_bytes < hash_unique_workspace_bytes(G, len_max))
        return fail(SGL_ENOMEM, "unique_compact: workspace %zu < %zu bytes", ws_bytes, hash_unique_workspace_bytes(G, len_max));
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
    const int64_t cap = table_capacity(total);
    Arena ar(ws, ws_bytes);
    Counters* d_cnt = ar.take<Counters>(1);
    unsigned long long* keys = ar.take<unsigned long long>(cap);
    int64_t* vals = ar.take<int64_t>(cap);
    int64_t* list = ar.take<int64_t>(total + 1);    // group g's new ids start at all.start[g] (sorted mode: 0)
    uint64_t* sort_b = ar.take<uint64_t>(total + 1);
    int64_t* dummy_a = ar.take<int64_t>(total + 1);  // the sort carries a value array; it is not used
    int64_t* dummy_b = ar.take<int64_t>(total + 1);
    const size_t rws_bytes = radix_sort_workspace_bytes(total);
    void* rws = ar.take<char>(rws_bytes);
    if (!ar.ok()) return fail(SGL_ENOMEM, "unique_compact: workspace too small");

    int64_t fb = ceil_div<int64_t>(cap, 1024);
    if (fb > 65536) fb = 65536;
    hipLaunchKernelGGL(fill_empty_kernel, dim3((unsigned)fb), dim3(256), 0, st, keys, cap, d_cnt);
    SGL_LAUNCH_CHECK();
    const int n_groups = (mode == SGL_UNIQUE_SORTED) ? (G > 0 ? 1 : 0) : G;
    for (int grp = 0; grp < n_groups; ++grp) {
        Arrays sub = all;
        int64_t list_off = 0;
        if (mode == SGL_UNIQUE_GROUPED) {
            sub.G = 1;
            sub.ids[0] = all.ids[grp]; sub.out[0] = all.out[grp];
            sub.len_dev[0] = all.len_dev[grp]; sub.len_max[0] = all.len_max[grp];
            sub.start[0] = 0;
            for (int g = 1; g <= MAXG; ++g) sub.start[g] = sub.len_max[0];
            list_off = all.start[grp];
        }
        const int64_t sub_total = sub.start[sub.G];
        if (sub_total == 0) continue;
        hipLaunchKernelGGL(insert_kernel, dim3((unsigned)ceil_div<int64_t>(sub_total, TILE)), dim3(BLOCK), 0, st, sub,
                           keys, cap - 1, grp, d_cnt, list + list_off);
        SGL_LAUNCH_CHECK();
    }
    Counters h;
    SGL_HIP_TRY(hipMemcpyAsync(&h, d_cnt, sizeof h, hipMemcpyDeviceToHost, st));
    SGL_HIP_TRY(hipStreamSynchronize(st));
    const int bits = bits_of((uint64_t)h.max_id);
    int64_t base = 0;
    for (int grp = 0; grp < n_groups; ++grp) {
        const int64_t cnt = h.count[grp];
        if (cnt == 0) continue;
        const int64_t list_off = (mode == SGL_UNIQUE_GROUPED) ? all.start[grp] : 0;
        uint64_t* seg = reinterpret_cast<uint64_t*>(list + list_off);
        int in_b = 0;
        int32_t rc = radix_sort_pairs(seg, dummy_a, sort_b, dummy_b, cnt, nullptr, 0, bits, &in_b, rws, rws_bytes, st);
        if (rc != SGL_OK) return rc;
        hipLaunchKernelGGL(number_kernel, dim3((unsigned)ceil_div<int64_t>(cnt, BLOCK)), dim3(BLOCK), 0, st,
                           in_b ? sort_b : seg, cnt, base, keys, vals, cap - 1, unique_out, unique_capacity);
        SGL_LAUNCH_CHECK();
        base += cnt;
    }
    if (total > 0) {
        hipLaunchKernelGGL(lookup_kernel, dim3((unsigned)ceil_div<int64_t>(total, BLOCK)), dim3(BLOCK), 0, st, all, keys,
                           vals, cap - 1);
        SGL_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(publish_kernel, dim3(1), dim3(1), 0, st, U_dev, base);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

}  // namespace sgl
