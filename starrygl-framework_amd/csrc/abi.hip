// Status plumbing of libsgl_hot.so.
#include <stdarg.h>

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

}  // namespace sgl

extern "C" const char* sgl_last_error_string(void) { return sgl::err_buf(); }
extern "C" int32_t sgl_abi_version(void) { return SGL_ABI_VERSION; }
