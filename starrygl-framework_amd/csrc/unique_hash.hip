// Hash-set unique for ids without a dense universe (gfx950).
#include "common.hpp"

namespace sgl {

size_t hash_unique_workspace_bytes(int32_t G, const int64_t* len_max) {
    (void)G; (void)len_max;
    return 256;
}

int32_t hash_unique_compact(int32_t mode, int32_t G, const int64_t* const* ids, const int64_t* len_max,
                            const int64_t* const* len_dev, int64_t* const* local_out,
                            int64_t* unique_out, int64_t unique_capacity, int64_t* U_dev, void* ws,
                            size_t ws_bytes, hipStream_t st) {
    (void)mode; (void)G; (void)ids; (void)len_max; (void)len_dev; (void)local_out; (void)unique_out;
    (void)unique_capacity; (void)U_dev; (void)ws; (void)ws_bytes; (void)st;
    return fail(SGL_ENOTSUP, "unique_compact: hash-set path is not built yet");
}

}  // namespace sgl
