// cos(w * dt + b) time encoding for gfx950.
//
// out[i, j] = cos(fl32(fl32(w[j] * float(dt[i])) + b[j])): the product and the
// sum are rounded separately (no FMA contraction), which is what a K=1
// `nn.Linear` followed by `torch.cos` computes.  A block owns RPB rows: their
// converted dt values are parked in LDS, then all threads emit the block's
// RPB x dim outputs as flat, coalesced 16-byte stores (4-byte stores when dim
// is not a multiple of 4).  One pass over the output: the [N, dim] tensor is
// written once instead of written, re-read and re-written by a GEMM + cos pair.
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

__device__ __forceinline__ float enc(float w, float x, float b) {
    return cosf(__fadd_rn(__fmul_rn(w, x), b));
}

template <int VEC>
__global__ __launch_bounds__(BLOCK) void time_encode_kernel(TEArgs a) {
    __shared__ float s_x[MAX_RPB];
    const int64_t N = live_count(a.N_dev, a.N_max);
    const int64_t row0 = (int64_t)blockIdx.x * a.rpb;
    if (row0 >= N) return;
    const int32_t rows = (int32_t)((N - row0) < a.rpb ? (N - row0) : a.rpb);
    for (int32_t r = threadIdx.x; r < rows; r += BLOCK) {
        s_x[r] = a.dt_dtype == SGL_DT_I64 ? (float)static_cast<const int64_t*>(a.dt)[row0 + r]
                                           : static_cast<const float*>(a.dt)[row0 + r];
    }
    __syncthreads();
    const int32_t cpr = a.dim / VEC;
    const int32_t total = rows * cpr;
    float* __restrict__ dst = a.out + row0 * a.dim;
    for (int32_t lc = threadIdx.x; lc < total; lc += BLOCK) {
        const int32_t r = lc / cpr;
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
    const int64_t blocks = ceil_div<int64_t>(N_max, rpb);
    if (blocks > 0x7FFFFFFFll) return fail(SGL_ENOTSUP, "time_encode: too many rows for one launch");
    hipStream_t st = as_stream(stream);
    if (vec4)
        hipLaunchKernelGGL(time_encode_kernel<4>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
    else
        hipLaunchKernelGGL(time_encode_kernel<1>, dim3((unsigned)blocks), dim3(BLOCK), 0, st, a);
    SGL_LAUNCH_CHECK();
    return SGL_OK;
}
