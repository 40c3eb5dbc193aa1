// Stable LSD radix sort of (int64 key, int64 value) pairs and a device-wide
// exclusive scan, for gfx950.  Both are building blocks of the T-CSR build
// (the reference's thrust::sort with EdgeComparator, sample.cu.hpp:51-63,1078)
// and of the hash-set unique (thrust::sort + unique, sample.cu.hpp:1794-1795).
//
// One 8-bit pass = three launches:
//   hist    : per 4096-key tile, digit histogram in LDS -> hist[digit][tile];
//   scan    : exclusive scan over the digit-major histogram (all digit-0 tiles,
//             then all digit-1 tiles, ...) = the global base of every
//             (digit, tile) bucket;
//   scatter : 512 threads take 8 keys each; inside a wave the rank of a key
//             among equal digits comes from 8 ballots (one per digit bit),
//             across waves and rounds from a small LDS table, so equal keys
//             keep their input order (stable).  The tile is then put in sorted
//             order in LDS and leaves it with consecutive threads writing
//             consecutive places of a digit's run (coalesced stores instead of
//             one scattered 8-byte store per key and array).
#include "radix.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;            // scan kernels
constexpr int WAVES = BLOCK / WAVE;
constexpr int RADIX = 256;
constexpr int SORT_BLOCK = 512;       // threads of a sort block
constexpr int ITEMS = 8;              // keys per thread
constexpr int TILE = SORT_BLOCK * ITEMS;
constexpr int SORT_WAVES = SORT_BLOCK / WAVE;
constexpr int SCAN_BLOCK = 1024;
constexpr int SCAN_TILE = 2048;
constexpr int64_t SCAN_SINGLE_MAX = 16384;   // up to here one block scans the whole input
// dynamic LDS of scatter_kernel: the (round, wave, digit) counters, later reused to stage the tile
constexpr size_t CNT_BYTES = (size_t)ITEMS * SORT_WAVES * RADIX * sizeof(uint16_t);
constexpr size_t STAGE_BYTES = (size_t)TILE * 16;
constexpr size_t SCATTER_LDS = CNT_BYTES > STAGE_BYTES ? CNT_BYTES : STAGE_BYTES;

__global__ __launch_bounds__(SORT_BLOCK) void hist_kernel(const uint64_t* __restrict__ keys, int64_t n_max,
                                                          const int64_t* n_dev, int shift, int64_t nb,
                                                          int64_t* __restrict__ hist) {
    __shared__ uint32_t s_h[RADIX];
    const int64_t n = live_count(n_dev, n_max);
    if (threadIdx.x < RADIX) s_h[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * TILE;
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
        const int64_t i = base + r * SORT_BLOCK + threadIdx.x;
        if (i < n) atomicAdd(&s_h[(keys[i] >> shift) & 0xFF], 1u);
    }
    __syncthreads();
    if (threadIdx.x < RADIX) hist[(int64_t)threadIdx.x * nb + blockIdx.x] = s_h[threadIdx.x];
}

__global__ __launch_bounds__(SORT_BLOCK) void scatter_kernel(const uint64_t* __restrict__ keys,
                                                             const int64_t* __restrict__ vals, int64_t n_max,
                                                             const int64_t* n_dev, int shift, int64_t nb,
                                                             const int64_t* __restrict__ hist_scanned,
                                                             uint64_t* __restrict__ keys_out,
                                                             int64_t* __restrict__ vals_out) {
    extern __shared__ __align__(16) unsigned char s_dyn[];
    // s_cnt[round][wave][digit]: keys of that digit in that (round, wave); later their exclusive prefix
    uint16_t (*s_cnt)[SORT_WAVES][RADIX] = reinterpret_cast<uint16_t (*)[SORT_WAVES][RADIX]>(s_dyn);
    __shared__ uint32_t s_dbase[RADIX];   // first place of digit d inside the sorted tile
    __shared__ int64_t s_goff[RADIX];     // global place of the tile's first key of digit d, minus s_dbase[d]
    __shared__ uint32_t s_wtot[RADIX / WAVE];
    const int64_t n = live_count(n_dev, n_max);
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    const int64_t base = (int64_t)blockIdx.x * TILE;
    if (base >= n) return;
    for (int q = threadIdx.x; q < ITEMS * SORT_WAVES * RADIX; q += SORT_BLOCK) (&s_cnt[0][0][0])[q] = 0;
    __syncthreads();
    uint64_t key[ITEMS];
    int64_t val[ITEMS];
    uint16_t rank[ITEMS];
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
        const int64_t i = base + r * SORT_BLOCK + threadIdx.x;
        const bool live = i < n;
        key[r] = live ? keys[i] : ~0ull;
        val[r] = live ? vals[i] : 0;
        const uint32_t d = (uint32_t)(key[r] >> shift) & 0xFF;
        // lanes of this wave holding the same digit (dead lanes only match dead lanes)
        uint64_t peers = __ballot(live) ;
        peers = live ? peers : ~peers;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const uint64_t m = __ballot((d >> b) & 1);
            peers &= ((d >> b) & 1) ? m : ~m;
        }
        const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
        rank[r] = (uint16_t)__popcll(peers & lt);
        if (live && rank[r] == 0) s_cnt[r][wid][d] = (uint16_t)__popcll(peers);
    }
    __syncthreads();
    uint32_t run = 0;
    if (threadIdx.x < RADIX) {   // thread d: exclusive prefix over the (round, wave) sequence of digit d
        const int d = threadIdx.x;
#pragma unroll
        for (int r = 0; r < ITEMS; ++r)
#pragma unroll
            for (int w = 0; w < SORT_WAVES; ++w) {
                const uint32_t c = s_cnt[r][w][d];
                s_cnt[r][w][d] = (uint16_t)run;
                run += c;
            }
    }
    // exclusive prefix of the digit totals over the 256 digits (threads 0..255 = waves 0..3)
    uint32_t inc = run;
    for (int dd = 1; dd < WAVE; dd <<= 1) {
        const uint32_t x = __shfl_up(inc, dd);
        if (lane >= dd) inc += x;
    }
    if (threadIdx.x < RADIX && lane == WAVE - 1) s_wtot[wid] = inc;
    __syncthreads();
    if (threadIdx.x < RADIX) {
        uint32_t off = inc - run;
        for (int w = 0; w < wid; ++w) off += s_wtot[w];
        s_dbase[threadIdx.x] = off;
        s_goff[threadIdx.x] = hist_scanned[(int64_t)threadIdx.x * nb + blockIdx.x] - (int64_t)off;
    }
    __syncthreads();
    // place of every key inside the sorted tile (registers), then the counters make room for the tile itself
    uint16_t lpos[ITEMS];
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
        const uint32_t d = (uint32_t)(key[r] >> shift) & 0xFF;
        lpos[r] = (uint16_t)(s_dbase[d] + s_cnt[r][wid][d] + rank[r]);
    }
    __syncthreads();
    uint64_t* s_key = reinterpret_cast<uint64_t*>(s_dyn);
    int64_t* s_val = reinterpret_cast<int64_t*>(s_dyn + (size_t)TILE * 8);
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
        if (base + r * SORT_BLOCK + threadIdx.x < n) {
            s_key[lpos[r]] = key[r];
            s_val[lpos[r]] = val[r];
        }
    }
    __syncthreads();
    // the tile leaves LDS in sorted order: consecutive threads write consecutive places of a digit's run
    const int64_t live_n = n - base < TILE ? n - base : TILE;
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
        const int i = r * SORT_BLOCK + threadIdx.x;
        if (i < live_n) {
            const uint64_t k = s_key[i];
            const int64_t pos = s_goff[(uint32_t)(k >> shift) & 0xFF] + i;
            keys_out[pos] = k;
            vals_out[pos] = s_val[i];
        }
    }
}

// ---- device-wide exclusive scan (int64), three launches ---------------------
__global__ __launch_bounds__(BLOCK) void scan_reduce_kernel(const int64_t* __restrict__ in, int64_t n,
                                                            int64_t* __restrict__ tile_sum) {
    __shared__ int64_t s_w[WAVES];
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE;
    int64_t sum = 0;
#pragma unroll
    for (int r = 0; r < SCAN_TILE / BLOCK; ++r) {
        const int64_t i = base + r * BLOCK + threadIdx.x;
        if (i < n) sum += in[i];
    }
    const int lane = threadIdx.x % WAVE;
    for (int d = WAVE / 2; d > 0; d >>= 1) sum += shfl_i64(sum, lane ^ d);
    if (lane == 0) s_w[threadIdx.x / WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t t = 0;
        for (int w = 0; w < WAVES; ++w) t += s_w[w];
        tile_sum[blockIdx.x] = t;
    }
}

// One block scans n values: thread t owns a contiguous run.  `in` may equal `out`.
__global__ __launch_bounds__(SCAN_BLOCK) void scan_single_kernel(const int64_t* in, int64_t* out, int64_t n,
                                                                 int64_t* total_out) {
    __shared__ int64_t s_part[SCAN_BLOCK];
    const int64_t per = ceil_div<int64_t>(n, SCAN_BLOCK);
    const int64_t b0 = (int64_t)threadIdx.x * per;
    const int64_t b1 = b0 + per < n ? b0 + per : n;
    int64_t sum = 0;
    for (int64_t b = b0; b < b1; ++b) sum += in[b];
    s_part[threadIdx.x] = sum;
    __syncthreads();
    for (int d = 1; d < SCAN_BLOCK; d <<= 1) {
        int64_t x = 0;
        if ((int)threadIdx.x >= d) x = s_part[threadIdx.x - d];
        __syncthreads();
        s_part[threadIdx.x] += x;
        __syncthreads();
    }
    int64_t run = s_part[threadIdx.x] - sum;
    for (int64_t b = b0; b < b1; ++b) {
        const int64_t x = in[b];
        out[b] = run;
        run += x;
    }
    if (threadIdx.x == SCAN_BLOCK - 1 && total_out != nullptr) *total_out = s_part[SCAN_BLOCK - 1];
}

__global__ __launch_bounds__(BLOCK) void scan_apply_kernel(const int64_t* __restrict__ in, int64_t n,
                                                           const int64_t* __restrict__ tile_off,
                                                           int64_t* __restrict__ out) {
    // the tile is cut into BLOCK runs of 8 consecutive elements, one run per thread
    __shared__ int64_t s_w[WAVES];
    constexpr int PER = SCAN_TILE / BLOCK;
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * PER;
    int64_t v[PER];
    int64_t sum = 0;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        v[r] = (base + r < n) ? in[base + r] : 0;
        sum += v[r];
    }
    const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
    int64_t inc = sum;
    for (int d = 1; d < WAVE; d <<= 1) {
        const int64_t x = shfl_i64(inc, lane >= d ? lane - d : lane);
        if (lane >= d) inc += x;
    }
    if (lane == WAVE - 1) s_w[wid] = inc;
    __syncthreads();
    int64_t run = tile_off[blockIdx.x] + (inc - sum);
    for (int w = 0; w < wid; ++w) run += s_w[w];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        if (base + r < n) out[base + r] = run;
        run += v[r];
    }
}

}  // namespace

size_t exclusive_scan_workspace_bytes(int64_t n) {
    return align_up((size_t)(ceil_div<int64_t>(n > 0 ? n : 1, SCAN_TILE) + 1) * 8) + 256;
}

int32_t exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out, void* ws,
                           size_t ws_bytes, hipStream_t st) {
    if (n < 0) return fail(SGL_EINVAL, "scan: n < 0");
    if (ws_bytes < exclusive_scan_workspace_bytes(n) || !ws) return fail(SGL_ENOMEM, "scan: workspace too small");
    int64_t* tile_sum = static_cast<int64_t*>(ws);
    const int64_t nt = ceil_div<int64_t>(n > 0 ? n : 1, SCAN_TILE);
    if (nt > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "scan: too many elements");
    if (n <= SCAN_SINGLE_MAX) {   // short inputs: one launch instead of three
        hipLaunchKernelGGL(scan_single_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, in, out, n, total_out);
        SGL_LAUNCH_CHECK();
        return SGL_OK;
    }
    hipLaunchKernelGGL(scan_reduce_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, in, n, tile_sum);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_single_kernel, dim3(1), dim3(SCAN_BLOCK), 0, st, tile_sum, tile_sum, nt, total_out);
    SGL_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)nt), dim3(BLOCK), 0, st, in, n, tile_sum, out);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}

size_t radix_sort_workspace_bytes(int64_t n_max) {
    const int64_t nb = ceil_div<int64_t>(n_max > 0 ? n_max : 1, TILE);
    return align_up((size_t)nb * RADIX * 8) + exclusive_scan_workspace_bytes(nb * RADIX) + 256;
}

int32_t radix_sort_pairs(uint64_t* keys_a, int64_t* vals_a, uint64_t* keys_b, int64_t* vals_b, int64_t n_max,
                         const int64_t* n_dev, int begin_bit, int end_bit, int* result_in_b, void* ws,
                         size_t ws_bytes, hipStream_t st) {
    if (n_max < 0 || begin_bit < 0 || end_bit > 64 || begin_bit > end_bit) return fail(SGL_EINVAL, "radix: bad range");
    if (ws_bytes < radix_sort_workspace_bytes(n_max) || !ws) return fail(SGL_ENOMEM, "radix: workspace too small");
    *result_in_b = 0;
    if (n_max == 0) return SGL_OK;
    // (the staged tile needs more than the 64 KB of LDS a kernel gets by default)
    const hipError_t lds_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(scatter_kernel),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)SCATTER_LDS);
    if (lds_ok != hipSuccess) return fail(SGL_EHIP, "radix: %s", hipGetErrorString(lds_ok));
    const int64_t nb = ceil_div<int64_t>(n_max, TILE);
    if (nb > 0x7FFFFFFFll / 2) return fail(SGL_ENOTSUP, "radix: too many keys");
    Arena ar(ws, ws_bytes);
    int64_t* hist = ar.take<int64_t>(nb * RADIX);
    const size_t scan_ws_bytes = exclusive_scan_workspace_bytes(nb * RADIX);
    void* scan_ws = ar.take<char>(scan_ws_bytes);
    if (!ar.ok()) return fail(SGL_ENOMEM, "radix: workspace too small");
    uint64_t* kin = keys_a; int64_t* vin = vals_a; uint64_t* kout = keys_b; int64_t* vout = vals_b;
    for (int shift = begin_bit; shift < end_bit; shift += 8) {
        hipLaunchKernelGGL(hist_kernel, dim3((unsigned)nb), dim3(SORT_BLOCK), 0, st, kin, n_max, n_dev, shift, nb, hist);
        SGL_LAUNCH_CHECK();
        int32_t rc = exclusive_scan_i64(hist, hist, nb * RADIX, nullptr, scan_ws, scan_ws_bytes, st);
        if (rc != SGL_OK) return rc;
        hipLaunchKernelGGL(scatter_kernel, dim3((unsigned)nb), dim3(SORT_BLOCK), SCATTER_LDS, st, kin, vin, n_max, n_dev,
                           shift, nb, hist, kout, vout);
        SGL_LAUNCH_CHECK();
        uint64_t* tk = kin; kin = kout; kout = tk;
        int64_t* tv = vin; vin = vout; vout = tv;
        *result_in_b ^= 1;
    }
    return SGL_OK;
}

}  // namespace sgl
