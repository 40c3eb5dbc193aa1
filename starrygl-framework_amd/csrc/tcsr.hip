// T-CSR validation and construction for gfx950.
#include "common.hpp"

namespace sgl {
namespace {

constexpr int BLOCK = 256;

// flag bits: 1 row_ptr ends, 2 row_ptr not monotone, 4 col out of range, 8 ts not ascending
__global__ void validate_rows_kernel(sgl_tcsr g, int32_t* flag) {
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v == 0 && (g.row_ptr[0] != 0 || g.row_ptr[g.n] != g.m)) atomicOr(flag, 1);
    if (v < g.n && g.row_ptr[v + 1] < g.row_ptr[v]) atomicOr(flag, 2);
}

__global__ void validate_edges_kernel(sgl_tcsr g, int32_t* flag) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= g.m) return;
    const int64_t c = g.col[e];
    if (c < 0 || c >= g.n) atomicOr(flag, 4);
    if (e + 1 < g.m && g.ts[e + 1] < g.ts[e]) {
        // a descent is legal only across a row boundary: find the row of e
        int64_t lo = 0, hi = g.n;  // last v with row_ptr[v] <= e
        while (hi - lo > 1) {
            const int64_t mid = lo + ((hi - lo) >> 1);
            if (g.row_ptr[mid] <= e) lo = mid; else hi = mid;
        }
        if (g.row_ptr[lo + 1] > e + 1) atomicOr(flag, 8);
    }
}

}  // namespace
}  // namespace sgl

using namespace sgl;

extern "C" int32_t sgl_tcsr_validate(const sgl_tcsr* g, void* ws, size_t ws_bytes, void* stream) {
    if (!g || g->n < 0 || g->m < 0 || !g->row_ptr) return fail(SGL_EINVAL, "tcsr_validate: NULL graph");
    if (g->m > 0 && (!g->col || !g->ts || !g->eid)) return fail(SGL_EINVAL, "tcsr_validate: NULL array");
    if (!ws || ws_bytes < 8) return fail(SGL_ENOMEM, "tcsr_validate: workspace < 8 bytes");
    hipStream_t st = as_stream(stream);
    int32_t* flag = static_cast<int32_t*>(ws);
    SGL_HIP_TRY(hipMemsetAsync(flag, 0, 8, st));
    hipLaunchKernelGGL(validate_rows_kernel, dim3((unsigned)ceil_div<int64_t>(g->n + 1, BLOCK)), dim3(BLOCK), 0, st, *g, flag);
    SGL_LAUNCH_CHECK();
    if (g->m > 0) {
        hipLaunchKernelGGL(validate_edges_kernel, dim3((unsigned)ceil_div<int64_t>(g->m, BLOCK)), dim3(BLOCK), 0, st, *g, flag);
        SGL_LAUNCH_CHECK();
    }
    int32_t h = 0;
    SGL_HIP_TRY(hipMemcpyAsync(&h, flag, 4, hipMemcpyDeviceToHost, st));
    SGL_HIP_TRY(hipStreamSynchronize(st));
    if (h & 1) return fail(SGL_ERANGE, "tcsr_validate: row_ptr[0] != 0 or row_ptr[n] != m");
    if (h & 2) return fail(SGL_ERANGE, "tcsr_validate: row_ptr not monotone");
    if (h & 4) return fail(SGL_ERANGE, "tcsr_validate: col outside [0,n)");
    if (h & 8) return fail(SGL_ERANGE, "tcsr_validate: ts not ascending in row");
    return SGL_OK;
}

extern "C" size_t sgl_tcsr_build_workspace_bytes(int64_t n, int64_t m) {
    (void)n; (void)m;
    return 256;
}

extern "C" int32_t sgl_tcsr_build(int64_t n, int64_t m, const int64_t* src, const int64_t* dst,
                                  const int64_t* ts, const int64_t* eid, int64_t* row_ptr, int64_t* col,
                                  int64_t* col_ts, int64_t* col_eid, void* ws, size_t ws_bytes,
                                  void* stream) {
    (void)n; (void)m; (void)src; (void)dst; (void)ts; (void)eid; (void)row_ptr; (void)col; (void)col_ts;
    (void)col_eid; (void)ws; (void)ws_bytes; (void)stream;
    return fail(SGL_ENOTSUP, "tcsr_build: device build is not built yet");
}
