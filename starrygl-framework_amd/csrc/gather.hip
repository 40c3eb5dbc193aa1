// Two-tier row gather / scatter through the cache index for gfx950.
//
// A block owns RPB consecutive output rows.  Phase 1: one thread per row walks
// the lookup chain id -> key -> local row -> hot slot once and parks the row's
// source address in LDS.  Phase 2: all 256 threads stream the block's
// RPB * row_bytes output bytes as flat, fully coalesced 16-byte chunks (8- or
// 4-byte chunks when the row size or a base address is not 16-byte aligned),
// several independent loads in flight per lane.  Hot rows come from HBM, cold
// rows are read in place from device-visible pinned host memory.
//
// Replaces IDMapper.to_local + DistNodeState.__getitem__/update
// (starrygl/utils/partition_book.py:106-133, starrygl/cache/NodeState.py:36-61)
// and tensor_gather (csrc/include/starrygl/feature.cu.hpp:42-88).
#include "common.hpp"

namespace sgl {

// the hash-set unique of unique_hash.hip (numbers the distinct cold rows a call asks for)
size_t hash_unique_workspace_bytes(int32_t G, const int64_t* len_max);
int32_t hash_unique_compact(int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev, int64_t* const* local_out,
                            int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, hipStream_t st);

namespace {

constexpr int BLOCK = 256;
constexpr int UNROLL = 4;
// Grids are capped and blocks walk tiles with a grid stride: the live row count is a
// device value, and launching the worst-case number of blocks costs ~0.2 ns per dead
// block (10 us for 50 000 of them), more than the whole copy of a small batch.
constexpr int MAX_GRID = 4096;
constexpr int MULTI_MAX_GRID = 1024;    // grid cap of the multi-segment gather
// gather_multi writes its rows past the caches from this many output bytes (worst case) on
constexpr int64_t NT_STORE_MIN_BYTES = 64ll << 20;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct GatherArgs {
    sgl_cache c;
    const int64_t* ids;
    int64_t N_max;
    const int64_t* N_dev;
    char* out;
    int64_t* out_ts;
    int64_t* stats;
    int32_t rpb;  // rows per block
    int32_t cpr;  // chunks per row
};

__host__ __device__ __forceinline__ int64_t cold_stride(const sgl_cache& c) { return c.cold_stride ? c.cold_stride : c.row_bytes; }
__host__ __device__ __forceinline__ int64_t ts_cold_stride(const sgl_cache& c) { return c.ts_cold_stride ? c.ts_cold_stride : 8; }
__host__ __device__ __forceinline__ int64_t hot_stride(const sgl_cache& c) { return c.hot_stride ? c.hot_stride : c.row_bytes; }

// lc / cpr for a chunk index inside a block's tile (lc < 2^22: a tile holds at most 1024 rows of at most 1024
// chunks, or one row of at most 65536): one multiply and a fix-up in place of an integer division per chunk.
__device__ __forceinline__ int32_t row_of_chunk(int32_t lc, int32_t cpr, float inv_cpr) {
    int32_t r = (int32_t)(((float)lc + 0.5f) * inv_cpr);
    r -= (r * cpr > lc) ? 1 : 0;
    r += ((r + 1) * cpr <= lc) ? 1 : 0;
    return r;
}

// id -> (source row address, last-update time); nullptr when not resident.
// tier: 0 hot, 1 cold, 2 absent.
__device__ __forceinline__ const char* resolve(const sgl_cache& c, int64_t id, int64_t* ts_out,
                                               int* tier) {
    *ts_out = 0;
    *tier = 2;
    if (id < 0) return nullptr;
    int64_t key = id & c.id_mask;
    if (c.g2l != nullptr) {
        if (key < 0 || key >= c.g2l_len) return nullptr;
        key = c.g2l[key];
    }
    if (key < 0 || key >= c.rows) return nullptr;
    const int64_t slot = c.hot_slot != nullptr ? (int64_t)c.hot_slot[key] : key;
    if (slot >= 0) {
        *tier = 0;
        if (c.ts_hot != nullptr) *ts_out = c.ts_hot[slot];
        return static_cast<const char*>(c.hot) + slot * hot_stride(c);
    }
    *tier = 1;
    if (c.ts_cold != nullptr)
        *ts_out = *reinterpret_cast<const int64_t*>(reinterpret_cast<const char*>(c.ts_cold) + key * ts_cold_stride(c));
    return static_cast<const char*>(c.cold) + key * cold_stride(c);
}

// NT: non-temporal loads and stores, for outputs much larger than the last-level
// cache (measured: +5..13 % beyond ~0.5 GB, -15 % at 70 MB, so small calls keep
// the cached path where repeated rows hit in L2).  NT_STORE alone: cached loads,
// streaming stores - for calls whose live size is a device-side count (140 MB moved
// under a capacity of 1.6 GB: 36 us against 42 us all-streaming).
template <typename V, bool NT, bool NT_STORE = NT>
__global__ __launch_bounds__(BLOCK) void gather_kernel(GatherArgs a) {
    extern __shared__ const char* s_src[];  // [rpb]
    __shared__ int32_t s_tier[3];
    const int64_t N = live_count(a.N_dev, a.N_max);
    if (threadIdx.x < 3) s_tier[threadIdx.x] = 0;
    const int32_t cpr = a.cpr;
    const float inv_cpr = 1.0f / (float)cpr;
    const int64_t first_row = (int64_t)blockIdx.x * a.rpb;
    if (a.stats != nullptr) __syncthreads();  // s_tier is zero before the first atomicAdd
    for (int64_t row0 = first_row; row0 < N; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
        if (row0 != first_row) __syncthreads();  // s_src of the previous tile has been consumed
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            int64_t ts;
            int tier;
            s_src[r] = resolve(a.c, a.ids[row0 + r], &ts, &tier);
            if (a.out_ts != nullptr) a.out_ts[row0 + r] = ts;
            if (a.stats != nullptr) atomicAdd(&s_tier[tier], 1);
        }
        __syncthreads();
        const int32_t total = rows * cpr;
        V* __restrict__ dst = reinterpret_cast<V*>(a.out + row0 * a.c.row_bytes);
        for (int32_t base = 0; base < total; base += BLOCK * UNROLL) {
            V val[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int32_t lc = base + u * BLOCK + threadIdx.x;
                V v = {};
                if (lc < total) {
                    const int32_t r = row_of_chunk(lc, cpr, inv_cpr);
                    const int32_t part = lc - r * cpr;
                    const V* src = reinterpret_cast<const V*>(s_src[r]);
                    if (src != nullptr) v = NT ? __builtin_nontemporal_load(src + part) : src[part];
                }
                val[u] = v;
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int32_t lc = base + u * BLOCK + threadIdx.x;
                if (lc < total) {
                    if (NT_STORE) __builtin_nontemporal_store(val[u], dst + lc);
                    else dst[lc] = val[u];
                }
            }
        }
    }
    if (a.stats != nullptr) __syncthreads();
    if (a.stats != nullptr && threadIdx.x < 3 && s_tier[threadIdx.x] != 0)
        atomicAdd(reinterpret_cast<unsigned long long*>(a.stats + threadIdx.x),
                  (unsigned long long)s_tier[threadIdx.x]);
}


struct MultiSeg {
    sgl_cache c;
    const int64_t* ids;
    int64_t N_max;
    const int64_t* N_dev;
    char* out;
    int64_t* out_ts;
    int32_t rpb, cpr;
};
struct MultiArgs {
    int32_t T;
    MultiSeg seg[SGL_GATHER_MAX_SEGMENTS];
};

// Several gathers in one launch: every block walks its grid-stride share of the
// tiles of segment 0, then of segment 1, ...  16-byte chunks only.
// NT_STORE: the output rows are written with non-temporal stores.  The kernel itself runs as
// fast either way (5.5 TB/s on 257 MB); what changes is that ~130 MB of rows nobody reads
// again soon do not displace the graph arrays from the last-level cache: the sampler and
// unique kernels of the neighbouring batches finish sooner (whole step -4 % with one batch
// in flight, -8 % with three).
template <bool NT_STORE>
__global__ __launch_bounds__(BLOCK) void gather_multi_kernel(MultiArgs m) {
    extern __shared__ const char* s_src[];
#pragma unroll 1
    for (int t = 0; t < m.T; ++t) {
        const MultiSeg& a = m.seg[t];
        const int64_t N = live_count(a.N_dev, a.N_max);
        const int32_t cpr = a.cpr;
        const float inv_cpr = 1.0f / (float)cpr;
        for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < N; row0 += (int64_t)gridDim.x * a.rpb) {
            const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
            __syncthreads();  // s_src of the previous tile has been consumed
            for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
                int64_t ts;
                int tier;
                s_src[r] = resolve(a.c, a.ids[row0 + r], &ts, &tier);
                if (a.out_ts != nullptr) a.out_ts[row0 + r] = ts;
            }
            __syncthreads();
            const int32_t total = rows * cpr;
            u32x4* __restrict__ dst = reinterpret_cast<u32x4*>(a.out + row0 * a.c.row_bytes);
            for (int32_t base = 0; base < total; base += BLOCK * UNROLL) {
                u32x4 val[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const int32_t lc = base + u * BLOCK + threadIdx.x;
                    u32x4 v = {};
                    if (lc < total) {
                        const int32_t r = row_of_chunk(lc, cpr, inv_cpr);
                        const int32_t part = lc - r * cpr;
                        const u32x4* src = reinterpret_cast<const u32x4*>(s_src[r]);
                        if (src != nullptr) v = src[part];
                    }
                    val[u] = v;
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const int32_t lc = base + u * BLOCK + threadIdx.x;
                    if (lc < total) {
                        if (NT_STORE) __builtin_nontemporal_store(val[u], dst + lc);
                        else dst[lc] = val[u];
                    }
                }
            }
        }
    }
}

// ---- gather with the cold tier fetched once per distinct row -------------------------------------------
// Requests of a batch repeat rows; a cold row crosses PCIe once per REQUEST in the kernels above.  Here:
//   classify : key[i] = local row of request i when that row is cold, -1 otherwise;
//   (the hash-set unique numbers the distinct keys: slot[i] = place of request i's row in the staging buffer)
//   phase A  : one launch, two segments walked by all blocks in turn - the distinct cold rows from pinned host
//              memory into the HBM staging buffer (PCIe bound, few tiles), then every request whose row is hot
//              (HBM bound; blocks that have finished their staging tiles start on these while the others still
//              wait for the link) and zero rows for absent ids;
//   phase B  : the requests of cold rows, served from the staging buffer (HBM to HBM).
struct DedupArgs {
    sgl_cache c;
    const int64_t* ids;
    int64_t N_max;
    const int64_t* N_dev;
    char* out;
    int64_t* out_ts;
    int64_t* stats;         // [4] or nullptr: hot requests, cold requests, absent, distinct cold rows
    int64_t* key;           // [N_max]
    const int64_t* slot;    // [N_max] written by the unique
    const int64_t* uniq;    // [<= N_max] distinct cold rows
    const int64_t* U_dev;   // their number
    char* staging;          // [staging_rows, row_bytes] HBM
    int64_t* staging_ts;    // [staging_rows] or nullptr
    int64_t staging_rows;
    int32_t rpb, cpr;
};

// where the local row `loc` of the cold tier lives, and its time
__device__ __forceinline__ const char* cold_row(const sgl_cache& c, int64_t loc, int64_t* ts_out) {
    *ts_out = c.ts_cold != nullptr ? *reinterpret_cast<const int64_t*>(reinterpret_cast<const char*>(c.ts_cold) + loc * ts_cold_stride(c)) : 0;
    return static_cast<const char*>(c.cold) + loc * cold_stride(c);
}

__global__ __launch_bounds__(BLOCK) void dedup_classify_kernel(DedupArgs a) {
    __shared__ int32_t s_tier[3];
    if (threadIdx.x < 3) s_tier[threadIdx.x] = 0;
    __syncthreads();
    const int64_t N = live_count(a.N_dev, a.N_max);
    for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < N; i += (int64_t)gridDim.x * BLOCK) {
        const int64_t id = a.ids[i];
        int64_t key = -1;
        int tier = 2;
        if (id >= 0) {
            int64_t loc = id & a.c.id_mask;
            bool ok = true;
            if (a.c.g2l != nullptr) {
                ok = loc >= 0 && loc < a.c.g2l_len;
                if (ok) loc = a.c.g2l[loc];
            }
            if (ok && loc >= 0 && loc < a.c.rows) {
                const bool cold = a.c.hot_slot != nullptr && a.c.hot_slot[loc] < 0;
                tier = cold ? 1 : 0;
                if (cold) key = loc;
            }
        }
        a.key[i] = key;
        if (a.stats != nullptr) atomicAdd(&s_tier[tier], 1);
    }
    if (a.stats == nullptr) return;
    __syncthreads();
    if (threadIdx.x < 3 && s_tier[threadIdx.x] != 0)
        atomicAdd(reinterpret_cast<unsigned long long*>(a.stats + threadIdx.x), (unsigned long long)s_tier[threadIdx.x]);
}

// the flat, coalesced copy of one tile whose source rows are parked in s_src (nullptr: zeros, SKIP: leave the row alone)
__device__ __forceinline__ void copy_tile(const char* const* s_src, char* out_tile, int32_t rows, int32_t cpr, float inv_cpr, bool stream_out) {
    const char* const SKIP = reinterpret_cast<const char*>(uintptr_t(1));
    const int32_t total = rows * cpr;
    u32x4* __restrict__ dst = reinterpret_cast<u32x4*>(out_tile);
    for (int32_t base = 0; base < total; base += BLOCK * UNROLL) {
        u32x4 val[UNROLL];
        bool on[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int32_t lc = base + u * BLOCK + threadIdx.x;
            u32x4 v = {};
            on[u] = false;
            if (lc < total) {
                const int32_t r = row_of_chunk(lc, cpr, inv_cpr);
                const char* src = s_src[r];
                on[u] = src != SKIP;
                if (src != nullptr && src != SKIP) v = reinterpret_cast<const u32x4*>(src)[lc - r * cpr];
            }
            val[u] = v;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int32_t lc = base + u * BLOCK + threadIdx.x;
            if (on[u]) {
                if (stream_out) __builtin_nontemporal_store(val[u], dst + lc);
                else dst[lc] = val[u];
            }
        }
    }
}

__global__ __launch_bounds__(BLOCK) void dedup_phase_a_kernel(DedupArgs a) {
    extern __shared__ const char* s_src[];
    const char* const SKIP = reinterpret_cast<const char*>(uintptr_t(1));
    const int32_t cpr = a.cpr;
    const float inv_cpr = 1.0f / (float)cpr;
    // segment 1: distinct cold rows -> staging (those that fit; the others are read in place by phase B)
    int64_t U = a.U_dev[0];
    if (a.stats != nullptr && blockIdx.x == 0 && threadIdx.x == 0) a.stats[3] += U;
    U = U < a.staging_rows ? U : a.staging_rows;
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < U; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((U - row0) < a.rpb ? (U - row0) : a.rpb);
        __syncthreads();
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            int64_t ts;
            s_src[r] = cold_row(a.c, a.uniq[row0 + r], &ts);
            if (a.staging_ts != nullptr) a.staging_ts[row0 + r] = ts;
        }
        __syncthreads();
        copy_tile(s_src, a.staging + row0 * a.c.row_bytes, rows, cpr, inv_cpr, false);
    }
    // segment 2: the requests of hot rows (and zero rows for absent ids)
    const int64_t N = live_count(a.N_dev, a.N_max);
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < N; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
        __syncthreads();
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            if (a.key[row0 + r] >= 0) {
                s_src[r] = SKIP;
            } else {
                int64_t ts;
                int tier;
                s_src[r] = resolve(a.c, a.ids[row0 + r], &ts, &tier);
                if (a.out_ts != nullptr) a.out_ts[row0 + r] = ts;
            }
        }
        __syncthreads();
        copy_tile(s_src, a.out + row0 * a.c.row_bytes, rows, cpr, inv_cpr, true);
    }
}

__global__ __launch_bounds__(BLOCK) void dedup_phase_b_kernel(DedupArgs a) {
    extern __shared__ const char* s_src[];
    const char* const SKIP = reinterpret_cast<const char*>(uintptr_t(1));
    const int32_t cpr = a.cpr;
    const float inv_cpr = 1.0f / (float)cpr;
    const int64_t N = live_count(a.N_dev, a.N_max);
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < N; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
        __syncthreads();
        int any = 0;
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            const int64_t key = a.key[row0 + r];
            const char* src = SKIP;
            if (key >= 0) {
                const int64_t sl = a.slot[row0 + r];
                int64_t ts;
                if (sl >= 0 && sl < a.staging_rows) {
                    src = a.staging + sl * a.c.row_bytes;
                    ts = a.staging_ts != nullptr ? a.staging_ts[sl] : 0;
                } else {
                    src = cold_row(a.c, key, &ts);       // (a staging buffer smaller than the call's distinct cold rows)
                }
                if (a.out_ts != nullptr) a.out_ts[row0 + r] = ts;
                any = 1;
            }
            s_src[r] = src;
        }
        if (__syncthreads_or(any)) copy_tile(s_src, a.out + row0 * a.c.row_bytes, rows, cpr, inv_cpr, true);
    }
}

struct ScatterArgs {
    sgl_cache c;
    char* hot_rw;
    char* cold_rw;
    int64_t* ts_hot_rw;
    int64_t* ts_cold_rw;
    const int64_t* ids;
    int64_t N;
    const char* values;
    const int64_t* ts;
    int32_t rpb, cpr;
};

template <typename V>
__global__ __launch_bounds__(BLOCK) void scatter_kernel(ScatterArgs a) {
    extern __shared__ char* s_dst[];
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < a.N; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((a.N - row0) < a.rpb ? (a.N - row0) : a.rpb);
        __syncthreads();
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            int64_t ts_unused;
            int tier;
            const char* p = resolve(a.c, a.ids[row0 + r], &ts_unused, &tier);
            char* d = nullptr;
            if (tier == 0) {
                const int64_t slot = (p - static_cast<const char*>(a.c.hot)) / hot_stride(a.c);
                d = a.hot_rw + slot * hot_stride(a.c);
                if (a.ts != nullptr && a.ts_hot_rw != nullptr) a.ts_hot_rw[slot] = a.ts[row0 + r];
            } else if (tier == 1) {
                const int64_t loc = (p - static_cast<const char*>(a.c.cold)) / cold_stride(a.c);
                d = a.cold_rw + loc * cold_stride(a.c);
                if (a.ts != nullptr && a.ts_cold_rw != nullptr)
                    *reinterpret_cast<int64_t*>(reinterpret_cast<char*>(a.ts_cold_rw) + loc * ts_cold_stride(a.c)) = a.ts[row0 + r];
            }
            s_dst[r] = d;
        }
        __syncthreads();
        const int32_t cpr = a.cpr;
        const float inv_cpr = 1.0f / (float)cpr;
        const int32_t total = rows * cpr;
        const V* __restrict__ src = reinterpret_cast<const V*>(a.values + row0 * a.c.row_bytes);
        for (int32_t lc = threadIdx.x; lc < total; lc += BLOCK) {
            const int32_t r = row_of_chunk(lc, cpr, inv_cpr);
            const int32_t part = lc - r * cpr;
            V* d = reinterpret_cast<V*>(s_dst[r]);
            if (d != nullptr) d[part] = src[lc];
        }
    }
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

int32_t check_cache(const sgl_cache* c) {
    if (!c) return fail(SGL_EINVAL, "cache is NULL");
    if (c->rows < 0 || c->hot_rows < 0 || c->g2l_len < 0) return fail(SGL_EINVAL, "cache: negative size");
    if (c->row_bytes <= 0 || c->row_bytes % 4 != 0)
        return fail(SGL_EINVAL, "cache: row_bytes %lld must be a positive multiple of 4", (long long)c->row_bytes);
    if (c->row_bytes > (1 << 20)) return fail(SGL_ENOTSUP, "cache: row_bytes > 1 MiB");
    if (c->hot_slot == nullptr && c->hot == nullptr && c->rows > 0)
        return fail(SGL_EINVAL, "cache: hot table is NULL while hot_slot is NULL");
    if (c->hot_slot == nullptr && c->rows > c->hot_rows)
        return fail(SGL_EINVAL, "cache: without hot_slot every logical row must be a hot row");
    if (c->hot_slot != nullptr && c->cold == nullptr && c->rows > 0)
        return fail(SGL_EINVAL, "cache: hot_slot given but cold table is NULL");
    if (c->cold_stride != 0 && (c->cold_stride < c->row_bytes || c->cold_stride % 4 != 0))
        return fail(SGL_EINVAL, "cache: cold_stride %lld must be 0 or a multiple of 4 >= row_bytes", (long long)c->cold_stride);
    if (c->hot_stride != 0 && (c->hot_stride < c->row_bytes || c->hot_stride % 4 != 0))
        return fail(SGL_EINVAL, "cache: hot_stride %lld must be 0 or a multiple of 4 >= row_bytes", (long long)c->hot_stride);
    if (c->ts_cold_stride != 0 && (c->ts_cold_stride < 8 || c->ts_cold_stride % 8 != 0))
        return fail(SGL_EINVAL, "cache: ts_cold_stride %lld must be 0 or a multiple of 8", (long long)c->ts_cold_stride);
    return SGL_OK;
}

// widest chunk every involved address / the row size allows
int pick_vec(int64_t row_bytes, int64_t stride_bytes, std::initializer_list<const void*> ptrs) {
    int v = 16;      // (stride_bytes: the cold and the hot row stride OR-ed together - a common divisor test)
    if (row_bytes % 16 || stride_bytes % 16) v = (row_bytes % 8 || stride_bytes % 8) ? 4 : 8;
    for (const void* p : ptrs) {
        if (!p) continue;
        while (v > 4 && !aligned(p, v)) v >>= 1;
    }
    return v;
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" int32_t sgl_gather(const sgl_cache* c, const int64_t* ids, int64_t N_max,
                              const int64_t* N_dev, void* out, int64_t* out_ts, int64_t* stats,
                              void* stream) {
    int32_t rc;
    if ((rc = check_cache(c)) != SGL_OK) return rc;
    if (N_max < 0) return fail(SGL_EINVAL, "gather: N_max < 0");
    if (N_max == 0) return SGL_OK;
    if (!ids || !out) return fail(SGL_EINVAL, "gather: ids/out is NULL");
    const int vec = pick_vec(c->row_bytes, cold_stride(*c) | hot_stride(*c), {c->hot, c->cold, out});
    GatherArgs a;
    a.c = *c; a.ids = ids; a.N_max = N_max; a.N_dev = N_dev;
    a.out = static_cast<char*>(out); a.out_ts = out_ts; a.stats = stats;
    a.cpr = (int32_t)(c->row_bytes / vec);
    // about BLOCK*UNROLL chunks per block, at least one row, at most 1024 rows
    int64_t rpb = (int64_t)BLOCK * UNROLL / a.cpr;
    rpb = rpb < 1 ? 1 : (rpb > 1024 ? 1024 : rpb);
    a.rpb = (int32_t)rpb;
    // a device-side live count usually is far below the capacity: cap the grid; a host-known
    // count gets one block per tile (measured 15 % faster on 2M-row gathers than striding)
    int64_t blocks = ceil_div<int64_t>(N_max, rpb);
    if (N_dev != nullptr && blocks > MAX_GRID) blocks = MAX_GRID;
    if (blocks > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "gather: too many rows for one launch");
    const size_t shmem = (size_t)rpb * sizeof(char*);
    hipStream_t st = as_stream(stream);
    // host-known row count: loads and stores past the caches from 256 MB of output on; device-side count
    // (the capacity says little about the live size): cached loads, streaming stores from 64 MB of capacity on
    const double cap_bytes = (double)N_max * (double)c->row_bytes;
    const bool nt = N_dev == nullptr && cap_bytes >= 256.0 * 1024 * 1024;
    const bool nt_store = N_dev != nullptr && cap_bytes >= (double)NT_STORE_MIN_BYTES;
    const dim3 grid((unsigned)blocks), blk(BLOCK);
    if (vec == 16 && nt) hipLaunchKernelGGL((gather_kernel<u32x4, true>), grid, blk, shmem, st, a);
    else if (vec == 16 && nt_store) hipLaunchKernelGGL((gather_kernel<u32x4, false, true>), grid, blk, shmem, st, a);
    else if (vec == 16) hipLaunchKernelGGL((gather_kernel<u32x4, false>), grid, blk, shmem, st, a);
    else if (vec == 8) hipLaunchKernelGGL((gather_kernel<u32x2, false>), grid, blk, shmem, st, a);
    else hipLaunchKernelGGL((gather_kernel<uint32_t, false>), grid, blk, shmem, st, a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}


extern "C" int32_t sgl_gather_multi(int32_t T, const sgl_gather_seg* segs, void* stream) {
    if (T < 0 || (T > 0 && !segs)) return fail(SGL_EINVAL, "gather_multi: bad segment list");
    if (T > SGL_GATHER_MAX_SEGMENTS) return fail(SGL_ENOTSUP, "gather_multi: more than %d segments", SGL_GATHER_MAX_SEGMENTS);
    MultiArgs m;
    m.T = 0;
    int64_t max_rpb = 1, want_blocks = 1, out_bytes = 0;
    for (int32_t t = 0; t < T; ++t) {
        const sgl_gather_seg& g = segs[t];
        int32_t rc;
        if ((rc = check_cache(g.cache)) != SGL_OK) return rc;
        if (g.N_max < 0) return fail(SGL_EINVAL, "gather_multi: N_max < 0");
        if (g.N_max == 0) continue;
        if (!g.ids || !g.out) return fail(SGL_EINVAL, "gather_multi: ids/out is NULL");
        if (pick_vec(g.cache->row_bytes, cold_stride(*g.cache) | hot_stride(*g.cache), {g.cache->hot, g.cache->cold, g.out}) != 16)
            return fail(SGL_ENOTSUP, "gather_multi: segment %d is not 16-byte aligned / sized", t);
        MultiSeg& a = m.seg[m.T++];
        a.c = *g.cache; a.ids = g.ids; a.N_max = g.N_max; a.N_dev = g.N_dev;
        a.out = static_cast<char*>(g.out); a.out_ts = g.out_ts;
        a.cpr = (int32_t)(g.cache->row_bytes / 16);
        int64_t rpb = (int64_t)BLOCK * UNROLL / a.cpr;
        rpb = rpb < 1 ? 1 : (rpb > 1024 ? 1024 : rpb);
        a.rpb = (int32_t)rpb;
        max_rpb = rpb > max_rpb ? rpb : max_rpb;
        const int64_t b = ceil_div<int64_t>(g.N_max, rpb);
        want_blocks = b > want_blocks ? b : want_blocks;
        out_bytes += g.N_max * g.cache->row_bytes;
    }
    if (m.T == 0) return SGL_OK;
    // Four blocks per CU (256 CUs), each walking many tiles: a launch over the rows of 16 mini-batches (4.6 GB) moves
    // 6.4-6.7 TB/s from 1024 blocks against 6.0-6.3 TB/s from 4096, and kernels of other streams find wave slots
    // beside it (step of the batched bench 0.055-0.058 against 0.059-0.063 ms).
    if (want_blocks > MULTI_MAX_GRID) want_blocks = MULTI_MAX_GRID;
    auto kern = out_bytes >= NT_STORE_MIN_BYTES ? gather_multi_kernel<true> : gather_multi_kernel<false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)want_blocks), dim3(BLOCK), (size_t)max_rpb * sizeof(char*),
                       as_stream(stream), m);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" int32_t sgl_scatter_update(const sgl_cache* c, void* hot_rw, void* cold_rw,
                                      int64_t* ts_hot_rw, int64_t* ts_cold_rw, const int64_t* ids,
                                      int64_t N, const void* values, const int64_t* ts, void* stream) {
    int32_t rc;
    if ((rc = check_cache(c)) != SGL_OK) return rc;
    if (N < 0) return fail(SGL_EINVAL, "scatter_update: N < 0");
    if (N == 0) return SGL_OK;
    if (!ids || !values) return fail(SGL_EINVAL, "scatter_update: ids/values is NULL");
    if (c->hot != nullptr && hot_rw == nullptr) return fail(SGL_EINVAL, "scatter_update: hot_rw is NULL");
    if (c->hot_slot != nullptr && cold_rw == nullptr) return fail(SGL_EINVAL, "scatter_update: cold_rw is NULL");
    const int vec = pick_vec(c->row_bytes, cold_stride(*c) | hot_stride(*c), {hot_rw, cold_rw, values});
    ScatterArgs a;
    a.c = *c; a.hot_rw = static_cast<char*>(hot_rw); a.cold_rw = static_cast<char*>(cold_rw);
    a.ts_hot_rw = ts_hot_rw; a.ts_cold_rw = ts_cold_rw; a.ids = ids; a.N = N;
    a.values = static_cast<const char*>(values); a.ts = ts;
    a.cpr = (int32_t)(c->row_bytes / vec);
    int64_t rpb = (int64_t)BLOCK * UNROLL / a.cpr;
    rpb = rpb < 1 ? 1 : (rpb > 1024 ? 1024 : rpb);
    a.rpb = (int32_t)rpb;
    int64_t blocks = ceil_div<int64_t>(N, rpb);
    if (blocks > 0x3FFFFFll) blocks = 0x3FFFFFll;
    const size_t shmem = (size_t)rpb * sizeof(char*);
    hipStream_t st = as_stream(stream);
    switch (vec) {
        case 16: hipLaunchKernelGGL(scatter_kernel<u32x4>, dim3((unsigned)blocks), dim3(BLOCK), shmem, st, a); break;
        case 8: hipLaunchKernelGGL(scatter_kernel<u32x2>, dim3((unsigned)blocks), dim3(BLOCK), shmem, st, a); break;
        default: hipLaunchKernelGGL(scatter_kernel<uint32_t>, dim3((unsigned)blocks), dim3(BLOCK), shmem, st, a); break;
    }
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

extern "C" size_t sgl_gather_dedup_workspace_bytes(int64_t N_max) {
    if (N_max < 0) N_max = 0;
    const int64_t lens[1] = {N_max};
    return 3 * align_up((size_t)(N_max + 1) * 8) + align_up(16) + hash_unique_workspace_bytes(1, lens) + 1024;
}

extern "C" int32_t sgl_gather_dedup(const sgl_cache* c, const int64_t* ids, int64_t N_max, const int64_t* N_dev,
                                    void* out, int64_t* out_ts, int64_t* stats, void* staging, int64_t* staging_ts,
                                    int64_t staging_rows, void* ws, size_t ws_bytes, void* stream) {
    int32_t rc;
    if ((rc = check_cache(c)) != SGL_OK) return rc;
    if (N_max < 0 || staging_rows < 0) return fail(SGL_EINVAL, "gather_dedup: negative size");
    if (N_max == 0) return SGL_OK;
    if (!ids || !out) return fail(SGL_EINVAL, "gather_dedup: ids/out is NULL");
    if (staging_rows > 0 && !staging) return fail(SGL_EINVAL, "gather_dedup: staging is NULL");
    if (pick_vec(c->row_bytes, cold_stride(*c) | hot_stride(*c), {c->hot, c->cold, out, staging}) != 16)
        return fail(SGL_ENOTSUP, "gather_dedup: rows and tables must be 16-byte aligned / sized (use sgl_gather)");
    if (!ws || ws_bytes < sgl_gather_dedup_workspace_bytes(N_max))
        return fail(SGL_ENOMEM, "gather_dedup: workspace %zu < %zu bytes", ws_bytes, sgl_gather_dedup_workspace_bytes(N_max));
    hipStream_t st = as_stream(stream);
    Arena ar(ws, ws_bytes);
    DedupArgs a;
    a.c = *c; a.ids = ids; a.N_max = N_max; a.N_dev = N_dev;
    a.out = static_cast<char*>(out); a.out_ts = out_ts; a.stats = stats;
    a.key = ar.take<int64_t>(N_max + 1);
    int64_t* slot = ar.take<int64_t>(N_max + 1);
    int64_t* uniq = ar.take<int64_t>(N_max + 1);
    int64_t* U_dev = ar.take<int64_t>(2);
    a.slot = slot; a.uniq = uniq; a.U_dev = U_dev;
    a.staging = static_cast<char*>(staging); a.staging_ts = (c->ts_cold != nullptr) ? staging_ts : nullptr;
    a.staging_rows = (c->ts_cold != nullptr && out_ts != nullptr && !staging_ts) ? 0 : staging_rows;
    a.cpr = (int32_t)(c->row_bytes / 16);
    int64_t rpb = (int64_t)BLOCK * UNROLL / a.cpr;
    rpb = rpb < 1 ? 1 : (rpb > 1024 ? 1024 : rpb);
    a.rpb = (int32_t)rpb;
    const size_t used = align_up(ar.used);
    if (!ar.ok() || used > ws_bytes) return fail(SGL_ENOMEM, "gather_dedup: workspace too small");
    int64_t cb = ceil_div<int64_t>(N_max, BLOCK);
    if (cb > 2048) cb = 2048;
    hipLaunchKernelGGL(dedup_classify_kernel, dim3((unsigned)cb), dim3(BLOCK), 0, st, a);
    SGL_LAUNCH_CHECK();
    const int64_t* kp[1] = {a.key};
    int64_t* sp[1] = {slot};
    const int64_t lens[1] = {N_max};
    const int64_t* ld[1] = {N_dev};
    rc = hash_unique_compact(SGL_UNIQUE_SORTED, 1, kp, lens, ld, sp, uniq, N_max, U_dev, static_cast<char*>(ws) + used,
                             ws_bytes - used, st);
    if (rc != SGL_OK) return rc;
    int64_t blocks = ceil_div<int64_t>(N_max, rpb);
    if (blocks > MAX_GRID) blocks = MAX_GRID;
    const size_t shmem = (size_t)rpb * sizeof(char*);
    hipLaunchKernelGGL(dedup_phase_a_kernel, dim3((unsigned)blocks), dim3(BLOCK), shmem, st, a);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(dedup_phase_b_kernel, dim3((unsigned)blocks), dim3(BLOCK), shmem, st, a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
