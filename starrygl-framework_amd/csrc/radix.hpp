// Internal sort / scan primitives of libsgl_hot.so (see radix.hip).
#pragma once
#include "common.hpp"

namespace sgl {

// Exclusive prefix sum of n int64 values (in == out allowed).  *total_out, when
// given, receives the grand total (device pointer).
size_t  exclusive_scan_workspace_bytes(int64_t n);
int32_t exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out, void* ws,
                           size_t ws_bytes, hipStream_t st);

// Stable LSD radix sort of pairs on key bits [begin_bit, end_bit), 8 bits per
// pass, ping-ponging between the (a) and (b) buffers; *result_in_b tells where
// the sorted pairs ended up.  The live length is *n_dev when given (<= n_max).
size_t  radix_sort_workspace_bytes(int64_t n_max);
int32_t radix_sort_pairs(uint64_t* keys_a, int64_t* vals_a, uint64_t* keys_b, int64_t* vals_b, int64_t n_max,
                         const int64_t* n_dev, int begin_bit, int end_bit, int* result_in_b, void* ws,
                         size_t ws_bytes, hipStream_t st);

}  // namespace sgl
