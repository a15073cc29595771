// Stable radix sort of (tile key, entry index) pairs for the analysis of the
// tiled two-phase SpMV, and the running sum of the pieces' lengths for the
// slice-by-slice copy.  This is the one place where library routines (rocPRIM's
// device radix sort and scan, header-only) are used: they run once per matrix,
// outside the multiply path.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

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

// off[i] = sum over k < i of (seg[k + m] - seg[k]), i = 0 .. pieces (pieces + 1 results)
struct PieceLength {
  const int* seg;
  int m;
  long long pieces;
  __host__ __device__ int operator()(long long i) const { return i < pieces ? seg[i + m] - seg[i] : 0; }
};
hipError_t scan_piece_lengths(hipStream_t stream, const int* seg, int m, long long pieces, int* off) {
  auto lengths = rocprim::make_transform_iterator(rocprim::make_counting_iterator<long long>(0),
                                                  PieceLength{seg, m, pieces});
  size_t temp_bytes = 0;
  hipError_t e = rocprim::exclusive_scan(nullptr, temp_bytes, lengths, off, 0, (size_t)pieces + 1, rocprim::plus<int>(),
                                         stream);
  if (e != hipSuccess) return e;
  void* temp = nullptr;
  e = hipMalloc(&temp, temp_bytes ? temp_bytes : 1);
  if (e != hipSuccess) return e;
  e = rocprim::exclusive_scan(temp, temp_bytes, lengths, off, 0, (size_t)pieces + 1, rocprim::plus<int>(), stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(temp);
  return e;
}

}  // namespace asamd
