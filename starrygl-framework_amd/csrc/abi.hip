// Status plumbing of libsgl_hot.so.
#include <stdarg.h>

#include <atomic>

#include "common.hpp"

namespace sgl {

char* err_buf() {
    static thread_local char buf[ERR_BUF];
    return buf;
}

int32_t fail(int32_t code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), ERR_BUF, fmt, ap);
    va_end(ap);
    return code;
}

namespace {
std::atomic<int32_t> g_wait_limit{WAIT_LIMIT_DEFAULT};
}

int32_t wait_limit() { return g_wait_limit.load(std::memory_order_relaxed); }

}  // namespace sgl

extern "C" int32_t sgl_set_wait_limit(int32_t polls) {
    return sgl::g_wait_limit.exchange(polls > 0 ? polls : sgl::WAIT_LIMIT_DEFAULT, std::memory_order_relaxed);
}

extern "C" const char* sgl_last_error_string(void) { return sgl::err_buf(); }
extern "C" int32_t sgl_abi_version(void) { return SGL_ABI_VERSION; }
extern "C" size_t sgl_struct_bytes(int32_t which) {
    switch (which) {
        case 0: return sizeof(sgl_tcsr);
        case 1: return sizeof(sgl_sample_params);
        case 2: return sizeof(sgl_hop_out);
        case 3: return sizeof(sgl_cache);
        case 4: return sizeof(sgl_gather_seg);
        case 5: return sizeof(sgl_seed_query);
        case 6: return sizeof(sgl_window_params);
        default: return 0;
    }
}
