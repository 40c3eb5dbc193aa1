// cos(w * dt + b) time encoding for gfx950.
//
// out[i, j] = cos(fl32(fl32(w[j] * float(dt[i])) + b[j])): the product and the
// sum are rounded separately (no FMA contraction), which is what a K=1
// `nn.Linear` followed by `torch.cos` computes.  One pass over the output: the
// [N, dim] tensor is written once, in 16-byte stores (4-byte stores when dim is
// not a multiple of 4), instead of written, re-read and re-written by a GEMM +
// cos pair; the cosine is computed by cos_core / cos_f32 below.  The kernel is
// bound by the cosine's fp64 arithmetic, with the stores hidden behind it as long
// as a wave does not load from global memory between two stores
// (time_encode_cols_kernel); time_encode_kernel is the general form (any dim).
//
// Replaces TimeEncoder.forward (starrygl/nn/model/time_encoder.py:29-31).
#include "common.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;
constexpr int MAX_RPB = 256;

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct TEArgs {
    const void* dt;
    int32_t dt_dtype;
    int64_t N_max;
    const int64_t* N_dev;
    const float* w;
    const float* b;
    int32_t dim;
    float* out;
    int32_t rpb;
};

// cos of an fp32 argument with an absolute error of at most 1.2e-7 (one ulp at 1.0; near the zeros of the
// cosine, where the result is small, that is many ulps of the result) for every
// magnitude the path produces (|a| up to 2^40 and beyond): the argument is reduced
// in double precision by multiples of pi (two-constant Cody-Waite, exact through
// FMA) to r in [-pi/2, pi/2]; then cos(r) = 1 - 2 sin^2(r/2) with one odd
// polynomial for sqrt(2) sin on [-pi/4, pi/4] - no quadrant-dependent coefficients, so no
// selects - and the sign (-1)^n is applied to the sign bit of the result.  14 fp64
// operations and two conversions, all straight-line.  The library cosf takes ~2.5x as long (its
// large-argument path is a Payne-Hanek reduction).  Arguments beyond 2^45 (not
// reachable from int64 timestamps times w <= 1 in practice) take the library routine.
constexpr float COS_CORE_LIMIT = 3.5e13f;
// |af| < COS_CORE_LIMIT
__device__ __forceinline__ float cos_core(float af) {
    const double x = (double)af;
    // n = nearest integer to x/pi without a rounding instruction: adding 1.5 * 2^52 leaves n in the low
    // mantissa bits of the sum (|x/pi| < 2^44 here), whose lowest bit is the parity of n
    constexpr double SHIFT = 6755399441055744.0;
    const double t = __builtin_fma(x, 0.31830988618379067154, SHIFT);   // 1/pi
    const uint32_t odd = (uint32_t)__double_as_longlong(t) & 1u;
    const double n = t - SHIFT;
    double r = __builtin_fma(-n, 3.14159265358979311600e+00, x);        // pi, high part
    r = __builtin_fma(-n, 1.22464679914735317723e-16, r);               // pi, low part
    // cos r = 1 - 2 sin^2(r/2) = 1 - q^2 with q = sqrt(2) sin(r/2), odd in u = r/sqrt(2) on [-1.12, 1.12]:
    // q = u + u*u2*Q(u2), Q the cubic through (q/u - 1)/u2 at the four Chebyshev points of [0, 1.235]
    // (|cos r - result| < 4e-11 before the rounding to fp32, as with the series up to u^11)
    const double u = 0.70710678118654752440 * r, u2 = u * u;
    double p = 1.7031108097175238e-07;
    p = __builtin_fma(p, u2, -2.4800106945370714e-05);
    p = __builtin_fma(p, u2, 2.083332968131731e-03);
    p = __builtin_fma(p, u2, -8.33333333192484e-02);
    const double q = __builtin_fma(p, u * u2, u);
    const float c = (float)__builtin_fma(-q, q, 1.0);                   // cos(r)
    // (-1)^n: flip the sign bit of the rounded result
    return __uint_as_float(__float_as_uint(c) ^ (odd << 31));
}

__device__ __forceinline__ float cos_f32(float af) {
    if (!(__builtin_fabsf(af) < COS_CORE_LIMIT)) return cosf(af);   // also NaN / inf
    return cos_core(af);
}

__device__ __forceinline__ float enc(float w, float x, float b) {
    return cos_f32(__fadd_rn(__fmul_rn(w, x), b));
}

// four columns of one row; the test for the library fallback is made once for the four
__device__ __forceinline__ f32x4 enc4(const f32x4 w, float x, const f32x4 b) {
    const float a0 = __fadd_rn(__fmul_rn(w.x, x), b.x), a1 = __fadd_rn(__fmul_rn(w.y, x), b.y);
    const float a2 = __fadd_rn(__fmul_rn(w.z, x), b.z), a3 = __fadd_rn(__fmul_rn(w.w, x), b.w);
    const float m = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(a0), __builtin_fabsf(a1)),
                                    __builtin_fmaxf(__builtin_fabsf(a2), __builtin_fabsf(a3)));
    // (the maximum drops a NaN operand; cos_core turns a NaN into a NaN, so one may take either route)
    f32x4 y;
    if (m < COS_CORE_LIMIT) {
        y.x = cos_core(a0); y.y = cos_core(a1); y.z = cos_core(a2); y.w = cos_core(a3);
    } else {
        y.x = cos_f32(a0); y.y = cos_f32(a1); y.z = cos_f32(a2); y.w = cos_f32(a3);
    }
    return y;
}

// dim % 4 == 0 and dim / 4 <= BLOCK: a thread owns one 4-column chunk for its whole life and keeps the
// chunk's w and b in registers; the block's threads form RPI = BLOCK / (dim / 4) rows of such chunks and
// walk a tile of `un` * RPI rows, RPI rows (one contiguous piece of the output) per trip.  The tile's dt
// values are converted once and parked in LDS together with w and b (dynamic LDS: un * RPI + 2 * dim
// floats), so after the one barrier of a tile a wave issues no global load: loads and stores return
// through one in-order counter, and a wave that loads w, b or dt between two stores waits for the first
// store's completion as well, with the arithmetic units idling behind the latency of the stores.  What a
// block pays before its first result (launch, the loads, the barrier) is paid once per tile: tiles of
// 8 * RPI rows and more take 0.8 of the time of tiles of 4 * RPI rows (1.32M x 100); the host shrinks the
// tile when the call is too small to give every CU several blocks.
constexpr int COLS_UN_MAX = 16;
constexpr int COLS_MIN_BLOCKS = 512;
__global__ __launch_bounds__(BLOCK) void time_encode_cols_kernel(TEArgs a, int32_t un) {
    extern __shared__ __align__(16) float s_dyn[];
    const int32_t cpr = a.dim / 4;
    const int32_t rpi = BLOCK / cpr;
    const int32_t tile = rpi * un;
    float* __restrict__ s_w = s_dyn;
    float* __restrict__ s_b = s_dyn + a.dim;
    float* __restrict__ s_x = s_dyn + 2 * a.dim;
    const int32_t rl = threadIdx.x / cpr;
    const int32_t j = (threadIdx.x - rl * cpr) * 4;
    const bool active = rl < rpi;
    for (int32_t i = threadIdx.x; i < a.dim; i += BLOCK) {
        s_w[i] = a.w[i];
        s_b[i] = a.b[i];
    }
    f32x4 w = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
    const int64_t N = live_count(a.N_dev, a.N_max);
    bool first = true;
    for (int64_t row0 = (int64_t)blockIdx.x * tile; row0 < N; row0 += (int64_t)gridDim.x * tile) {
        const int32_t rows = (int32_t)((N - row0) < tile ? (N - row0) : tile);
        __syncthreads();
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            s_x[r] = a.dt_dtype == SGL_DT_I64 ? (float)static_cast<const int64_t*>(a.dt)[row0 + r]
                                               : static_cast<const float*>(a.dt)[row0 + r];
        }
        __syncthreads();
        if (first && active) {
            w = *reinterpret_cast<const f32x4*>(s_w + j);
            b = *reinterpret_cast<const f32x4*>(s_b + j);
        }
        first = false;
        float* __restrict__ dst = a.out + (row0 + rl) * a.dim + j;
        const int64_t step = (int64_t)rpi * a.dim;
        for (int32_t r = rl; r < rows; r += rpi, dst += step) {
            if (active) *reinterpret_cast<f32x4*>(dst) = enc4(w, s_x[r], b);
        }
    }
}

template <int VEC>
__global__ __launch_bounds__(BLOCK) void time_encode_kernel(TEArgs a) {
    __shared__ float s_x[MAX_RPB];
    const int64_t N = live_count(a.N_dev, a.N_max);
    const int32_t cpr = a.dim / VEC;
    // capped grid, tiles walked with a grid stride (dead blocks of a worst-case grid are not free)
    for (int64_t row0 = (int64_t)blockIdx.x * a.rpb; row0 < N; row0 += (int64_t)gridDim.x * a.rpb) {
        const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
        __syncthreads();
        for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
            s_x[r] = a.dt_dtype == SGL_DT_I64 ? (float)static_cast<const int64_t*>(a.dt)[row0 + r]
                                               : static_cast<const float*>(a.dt)[row0 + r];
        }
        __syncthreads();
        const int32_t total = rows * cpr;
        float* __restrict__ dst = a.out + row0 * a.dim;
        const float inv_cpr = 1.0f / (float)cpr;
        for (int32_t lc = threadIdx.x; lc < total; lc += BLOCK) {
            // lc / cpr for lc < 2^16 (a tile has at most MAX_RPB * BLOCK chunks): one multiply and a fix-up
            int32_t r = (int32_t)(((float)lc + 0.5f) * inv_cpr);
            r -= (r * cpr > lc) ? 1 : 0;
            r += ((r + 1) * cpr <= lc) ? 1 : 0;
            const int32_t j = (lc - r * cpr) * VEC;
            const float x = s_x[r];
            if constexpr (VEC == 4) {
                const f32x4 w = *reinterpret_cast<const f32x4*>(a.w + j);
                const f32x4 b = *reinterpret_cast<const f32x4*>(a.b + j);
                f32x4 y;
                y.x = enc(w.x, x, b.x);
                y.y = enc(w.y, x, b.y);
                y.z = enc(w.z, x, b.z);
                y.w = enc(w.w, x, b.w);
                reinterpret_cast<f32x4*>(dst)[lc] = y;
            } else {
                dst[lc] = enc(a.w[j], x, a.b[j]);
            }
        }
    }
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" int32_t sgl_time_encode(const void* dt, int32_t dt_dtype, int64_t N_max,
                                   const int64_t* N_dev, const float* w, const float* b,
                                   int32_t dim, float* out, void* stream) {
    if (N_max < 0 || dim <= 0) return fail(SGL_EINVAL, "time_encode: N_max < 0 or dim <= 0");
    if (!w || !b) return fail(SGL_EINVAL, "time_encode: w/b is NULL");
    if (dt_dtype != SGL_DT_I64 && dt_dtype != SGL_DT_F32) return fail(SGL_EINVAL, "time_encode: bad dt dtype");
    if (N_max == 0) return SGL_OK;
    if (!dt || !out) return fail(SGL_EINVAL, "time_encode: dt/out is NULL");
    const bool vec4 = dim % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0;
    TEArgs a{dt, dt_dtype, N_max, N_dev, w, b, dim, out, 0};
    const int cpr = vec4 ? dim / 4 : dim;
    int64_t rpb = (int64_t)BLOCK * 4 / cpr;
    rpb = rpb < 1 ? 1 : (rpb > MAX_RPB ? MAX_RPB : rpb);
    a.rpb = (int32_t)rpb;
    int64_t blocks = ceil_div<int64_t>(N_max, rpb);
    if (N_dev != nullptr && blocks > 8192) blocks = 8192;   // live count usually far below capacity
    if (blocks > 0x3FFFFFll) blocks = 0x3FFFFFll;
    hipStream_t st = as_stream(stream);
    if (vec4 && cpr <= BLOCK) {
        const int64_t rpi = BLOCK / cpr;
        int64_t un = N_max / (rpi * COLS_MIN_BLOCKS);
        un = un < 1 ? 1 : (un > COLS_UN_MAX ? COLS_UN_MAX : un);
        blocks = ceil_div<int64_t>(N_max, rpi * un);
        if (N_dev != nullptr && blocks > 8192) blocks = 8192;
        if (blocks > 0x3FFFFFll) blocks = 0x3FFFFFll;
        const size_t lds = (size_t)(rpi * un + 2 * dim) * sizeof(float);     // <= 16 KB + 8 KB
        hipLaunchKernelGGL(time_encode_cols_kernel, dim3((unsigned)blocks), dim3(BLOCK), lds, st, a, (int32_t)un);
    } else if (vec4)
        hipLaunchKernelGGL(time_encode_kernel<4>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
    else
        hipLaunchKernelGGL(time_encode_kernel<1>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
