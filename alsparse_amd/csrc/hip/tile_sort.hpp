// Internal: stable device sort of (key, value) pairs with 32-bit unsigned keys
// on the low `end_bit` bits of the key; synchronises the stream.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stddef.h>

namespace asamd {
hipError_t sort_pairs_u32(hipStream_t stream, unsigned* keys_in, unsigned* keys_out, unsigned* vals_in,
                          unsigned* vals_out, size_t n, unsigned end_bit);
// the same with 64-bit values (an entry's value and local indices travel with its key)
hipError_t sort_pairs_u32_u64(hipStream_t stream, unsigned* keys_in, unsigned* keys_out, unsigned long long* vals_in,
                              unsigned long long* vals_out, size_t n, unsigned end_bit);
// off[i] = seg[0 + m] - seg[0] + ... + seg[i - 1 + m] - seg[i - 1] for i = 0 .. pieces; waits for the stream
hipError_t scan_piece_lengths(hipStream_t stream, const int* seg, int m, long long pieces, int* off);
}
