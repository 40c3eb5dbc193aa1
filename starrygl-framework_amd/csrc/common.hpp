// Shared host/device helpers of libsgl_hot.so (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/sgl_hot.h"

namespace sgl {

constexpr int WAVE = 64;

// ---- status plumbing (thread-local error string, no exceptions) -------------
char* err_buf();
constexpr size_t ERR_BUF = 512;

int32_t fail(int32_t code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define SGL_HIP_TRY(expr)                                                              \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess)                                                          \
            return ::sgl::fail(SGL_EHIP, "%s: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                               __FILE__, __LINE__);                                    \
    } while (0)

// Launch check: a bad launch configuration is reported by hipGetLastError.
#define SGL_LAUNCH_CHECK() SGL_HIP_TRY(hipGetLastError())

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

template <typename T>
__host__ __device__ constexpr T ceil_div(T a, T b) { return (a + b - 1) / b; }

constexpr size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }

// Bump allocator over a caller-provided workspace.
struct Arena {
    char*  base;
    size_t size, used;
    Arena(void* p, size_t n) : base(static_cast<char*>(p)), size(n), used(0) {}
    template <typename T>
    T* take(size_t count) {
        size_t off = align_up(used);
        used = off + count * sizeof(T);
        return reinterpret_cast<T*>(base + off);
    }
    bool ok() const { return base != nullptr && used <= size; }
};

// ---- device helpers ---------------------------------------------------------
#if defined(__HIPCC__)

// Layout of a remap state (sgl_remap_init): header, table[universe] of 8-byte entries, then the
// "pending" set: one flag byte per id for universes up to REMAP_BYTE_FLAGS_MAX ids (set by plain
// stores), one bit per id beyond (set by atomicOr; sweeping a byte per id would cost more there
// than the atomics do).  unique.hip owns the state; the sampler only sets flags.
// polls of one descriptor before a waiting lane gives up (sgl_set_wait_limit)
constexpr int32_t WAIT_LIMIT_DEFAULT = 1 << 20;
int32_t wait_limit();

// The fourth field of an interleaved edge record (sgl_tcsr_records_build) is the edge's next-hop index entry - the
// position where the window of the slot (col[e], ts[e]) ends - with the LENGTH of that window in its upper bits:
// bits 0..39 the position (graphs of up to 2^40 edges), bits 40..62 a field f: 0 = not recorded, 1..HINT_LEN_SAT-1 =
// length + 1, HINT_LEN_SAT = longer than the field holds.  A slot of a deeper hop whose index entry came out of a
// record then knows its whole window [position - length, position) without reading the row pointers of its node.
// A plain index entry (from the hop_hint array, a caller's root hint) has f = 0; -1 stays -1.
constexpr int HINT_POS_BITS = 40;
constexpr int64_t HINT_POS_MASK = (1ll << HINT_POS_BITS) - 1;
constexpr int64_t HINT_LEN_SAT = (1ll << 23) - 1;
__host__ __device__ __forceinline__ int64_t hint_pos(int64_t h) { return h < 0 ? h : (h & HINT_POS_MASK); }
// window length recorded in an entry, or -1
__host__ __device__ __forceinline__ int64_t hint_len(int64_t h) {
    if (h < 0) return -1;
    const int64_t f = h >> HINT_POS_BITS;
    return (f == 0 || f >= HINT_LEN_SAT) ? -1 : f - 1;
}
__host__ __device__ __forceinline__ int64_t hint_pack(int64_t pos, int64_t len) {
    const int64_t f = len + 1 < HINT_LEN_SAT ? len + 1 : HINT_LEN_SAT;
    return pos | (f << HINT_POS_BITS);
}

constexpr size_t REMAP_HEADER_BYTES = 256;
constexpr int64_t REMAP_BYTE_FLAGS_MAX = 1ll << 24;
inline bool remap_byte_flags(int64_t universe) { return universe <= REMAP_BYTE_FLAGS_MAX; }
inline void* remap_flags(void* state, int64_t universe) {
    return static_cast<char*>(state) + REMAP_HEADER_BYTES + (size_t)universe * 8;
}
// Marks the remap state whose pending flags are `flags` as void (the sticky field of its header, see
// unique.hip): what a sampler launch that gave up does to the state it was recording ids in.
__device__ __forceinline__ void remap_poison(void* flags, int64_t universe) {
    char* base = static_cast<char*>(flags) - REMAP_HEADER_BYTES - (size_t)universe * 8;
    reinterpret_cast<int64_t*>(base)[3] = 1;
}
__device__ __forceinline__ void remap_set_pending(void* flags, int bytes, int64_t id) {
    if (bytes) {
        static_cast<uint8_t*>(flags)[id] = 1;
    } else {
        atomicOr(static_cast<unsigned long long*>(flags) + (id >> 6), 1ull << (id & 63));
    }
}

// Ballot restricted to the G-lane group that starts at bit `gshift` of the wave.
template <int G>
__device__ __forceinline__ uint64_t group_ballot(bool pred, int gshift) {
    uint64_t b = __ballot(pred);
    if constexpr (G == 64) {
        (void)gshift;
        return b;
    } else {
        return (b >> gshift) & ((1ull << G) - 1ull);
    }
}

__device__ __forceinline__ int64_t shfl_i64(int64_t v, int src_lane) {
    int lo = __shfl(static_cast<int>(v & 0xFFFFFFFFll), src_lane);
    int hi = __shfl(static_cast<int>(v >> 32), src_lane);
    return (static_cast<int64_t>(hi) << 32) | static_cast<uint32_t>(lo);
}

// Live element count of a launch: *n_dev clamped to [0, n_max] when given.
__device__ __forceinline__ int64_t live_count(const int64_t* n_dev, int64_t n_max) {
    if (n_dev == nullptr) return n_max;
    int64_t n = *n_dev;
    return n < 0 ? 0 : (n > n_max ? n_max : n);
}

#endif  // __HIPCC__

}  // namespace sgl
