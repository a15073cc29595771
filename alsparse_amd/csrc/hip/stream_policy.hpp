// Which of a multiply's two matrix streams is loaded non-temporally (host side of kStreamNtValues /
// kStreamNtIndices in device_utils.hpp).
//
// Whatever is loaded plainly stays in the 256 MB memory-side cache until something pushes it out, and an
// iterative solver multiplies by the same matrix again and again: a matrix that fits, or nearly, is then read from
// that cache; one that does not should at least leave the part that fits alone; with streams of a gigabyte
// nothing is kept whatever is done.  Measured, in us, with neither / the values / the indices / both streams
// non-temporal:
//   524 288 x 524 288, 16 per row, fp32 (67 MB)           41.3   43.5   43.6   44.6
//   2 M x 65 536, 16 per row, fp32 (285 MB with x, y)    140.7  146.4  147.4  155.8
//   5-point Laplacian 2048^2, fp64 (168 + 84 MB)          67.6   59.9   50.7   65.5
//   4 M x 65 536, 8 per row, fp64 (268 + 134 MB)         191.5  177.5  183.0  191.2
//   8 M x 4 096, 5 per row, fp32 (168 + 168 MB)          105.7   88.3   88.2   98.0
//   27-point stencil 160^3, fp32 (437 + 437 MB)          208.5  206.3  205.8  198.7
//   27-point stencil 128^3, fp64 (446 + 223 MB)          148.6  149.8  147.4  162.7
//   power-law, 8 M rows, fp32 (379 + 379 MB)             595.8  583.0  582.6  567.3
// Both streams non-temporal pays with 4-byte values, and with wider ones in merge-path (power-law rows,
// complex64: 954 / 912 / 938 / 892 us) and the ELL kernel (that stencil, fp64: 280 / 279 / 277 / 252 us), not in the
// staged and the constant-row-length kernels (the stencil line above).  What is not a matrix stream (row offsets, x, y) is always kept.  ALSPARSE_AMD_STREAM_POLICY = 0..3 forces a combination (bit 0: values, bit 1: indices).
#pragma once

#include <cstddef>
#include <cstdlib>

#include "device_utils.hpp"

namespace asamd {

// entries: stored entries (padding included); rest_bytes: everything else the multiply touches; wide_both: whether
// the kernel gains from both streams non-temporal with values of 8 bytes and more; index_bytes: per entry (8 for
// the coordinate format's row and column)
inline int stream_policy(double entries, size_t val_size, double rest_bytes, bool wide_both = false,
                         double index_bytes = 4.0) {
  static const int forced = getenv("ALSPARSE_AMD_STREAM_POLICY") ? atoi(getenv("ALSPARSE_AMD_STREAM_POLICY")) : -1;
  if (forced >= 0) return forced & (kStreamNtValues | kStreamNtIndices);
  const double cache = 256.0e6;
  const double values = entries * (double)val_size, indices = entries * index_bytes;
  if (rest_bytes + values + indices <= 300.0e6) return 0;  // a little more than the cache holds still gains from it
  if (values >= indices) {
    if (rest_bytes + values <= cache) return kStreamNtIndices;
    if (rest_bytes + indices <= cache) return kStreamNtValues;
  } else {
    if (rest_bytes + indices <= cache) return kStreamNtValues;
    if (rest_bytes + values <= cache) return kStreamNtIndices;
  }
  return val_size == 4 || wide_both ? (kStreamNtValues | kStreamNtIndices) : kStreamNtIndices;
}

}  // namespace asamd
