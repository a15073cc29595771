// Stable radix sort of (tile key, entry index) pairs for the analysis of the
// tiled two-phase SpMV.  This is the one place where a library routine
// (rocPRIM's device radix sort, header-only) is used: it runs once per matrix,
// outside the multiply path.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "tile_sort.hpp"

namespace asamd {

template <typename V>
static hipError_t sort_pairs(hipStream_t stream, unsigned* keys_in, unsigned* keys_out, V* vals_in, V* vals_out,
                             size_t n, unsigned end_bit) {
  size_t temp_bytes = 0;
  hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, keys_in, keys_out, vals_in, vals_out, n,
                                           0u, end_bit, stream);
  if (e != hipSuccess) return e;
  void* temp = nullptr;
  e = hipMalloc(&temp, temp_bytes ? temp_bytes : 1);
  if (e != hipSuccess) return e;
  e = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in, vals_out, n, 0u, end_bit,
                                stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(temp);
  return e;
}

hipError_t sort_pairs_u32(hipStream_t stream, unsigned* keys_in, unsigned* keys_out, unsigned* vals_in,
                          unsigned* vals_out, size_t n, unsigned end_bit) {
  return sort_pairs<unsigned>(stream, keys_in, keys_out, vals_in, vals_out, n, end_bit);
}

hipError_t sort_pairs_u32_u64(hipStream_t stream, unsigned* keys_in, unsigned* keys_out, unsigned long long* vals_in,
                              unsigned long long* vals_out, size_t n, unsigned end_bit) {
  return sort_pairs<unsigned long long>(stream, keys_in, keys_out, vals_in, vals_out, n, end_bit);
}

}  // namespace asamd
