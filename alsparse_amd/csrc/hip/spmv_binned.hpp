// CSR SpMV by row-length bins for gfx950 (wave64): one kernel launch per bin.
//
// For matrices whose rows differ so much in length that no single lane mapping fits them (a few very
// long rows among millions of short ones).  The analysis sorts the row numbers by length class (a stable
// sort: rows stay ascending inside a class, so neighbouring lanes still read neighbouring entries) and
// every class gets the mapping that suits it:
//
//   class 0  rows of at most kBinShort entries     4 lanes per row     spmv_bin_rows_kernel<T, 4>
//   class 1  ... of at most kBinMid entries        16 lanes per row    spmv_bin_rows_kernel<T, 16>
//   class 2  ... of at most kBinWave entries       a wave per row      spmv_bin_rows_kernel<T, 64>
//   class 3  longer rows                           cut into chunks of kBinChunk entries, a workgroup per
//                                                  chunk (spmv_bin_chunk_kernel), then one lane per row adds
//                                                  the row's chunk sums in chunk order (spmv_bin_finish_kernel)
//
// Every row is summed by one lane group in a fixed order and every y is written once: no atomics, results
// identical from run to run.  Values, columns and row offsets are read from the caller's arrays; what the
// analysis keeps is the list of row numbers and the chunk table.
//
// The reference builds such length classes on the host (ComputeRowBlocks,
// src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267, long rows at :100-115) but has no kernel that
// reads them; the arithmetic per row is that of src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-54.
#pragma once

#include "device_utils.hpp"
#include "spmv_rows.hpp"

namespace asamd {

constexpr int kBinShort = 8;
constexpr int kBinMid = 64;
constexpr int kBinWave = 2048;
constexpr int kBinChunk = 4096;  // entries per workgroup of the long-row kernel
constexpr int kBinClasses = 4;

struct BinChunk {
  int row;       // the long row this chunk belongs to
  int begin;     // entry range, zero-based offsets into the CSR streams
  int end;
};

__device__ __forceinline__ int bin_class(int len) {
  return len <= kBinShort ? 0 : (len <= kBinMid ? 1 : (len <= kBinWave ? 2 : 3));
}

// key[r] = length class of row r, idx[r] = r
static __global__ __launch_bounds__(256) void bin_keys_kernel(int m, const int* __restrict__ row_ptr, unsigned* __restrict__ key,
                                                       unsigned* __restrict__ idx, int* __restrict__ count) {
  __shared__ int s_count[kBinClasses];
  if (threadIdx.x < kBinClasses) s_count[threadIdx.x] = 0;
  __syncthreads();
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r < m) {
    const int c = bin_class(row_ptr[r + 1] - row_ptr[r]);
    key[r] = (unsigned)c;
    idx[r] = (unsigned)r;
    atomicAdd(&s_count[c], 1);
  }
  __syncthreads();
  if (threadIdx.x < kBinClasses && s_count[threadIdx.x]) atomicAdd(&count[threadIdx.x], s_count[threadIdx.x]);
}

// (row_ptr[r], row_ptr[r + 1]) of the listed rows, for the host that cuts the long rows into chunks
static __global__ __launch_bounds__(256) void bin_row_bounds_kernel(int count, const int* __restrict__ rows,
                                                             const int* __restrict__ row_ptr, int* __restrict__ bounds) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  const int r = rows[i];
  bounds[2 * i] = row_ptr[r];
  bounds[2 * i + 1] = row_ptr[r + 1];
}

// W consecutive lanes share one of the `count` listed rows.
template <typename T, int W>
__global__ __launch_bounds__(kRowsBlock) void spmv_bin_rows_kernel(
    int count, const int* __restrict__ rows, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  constexpr int kRowsPerBlock = kRowsBlock / W;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int lane = threadIdx.x % W;
  const int64_t i = (int64_t)bid * kRowsPerBlock + threadIdx.x / W;
  if (i >= count) return;  // whole lane groups leave together
  const int64_t row = rows[i];
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* __restrict__ xb = x - base;
  T sum = T(0);
  int64_t j = start + lane;
  if constexpr (W >= 64) {
    // four entries per lane and trip: a wave that owns a row of a thousand entries lives on its loads in flight
    for (; j + 3 * W < end; j += 4 * W) {
      T v[4];
      int c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        v[u] = val[j + u * W];
        c[u] = col_ind[j + u * W];
      }
      T xv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) xv[u] = xb[c[u]];
#pragma unroll
      for (int u = 0; u < 4; ++u) sum = fma_t(v[u], xv[u], sum);
    }
  }
  for (; j + W < end; j += 2 * W) {
    const T v0 = val[j];
    const T v1 = val[j + W];
    const int c0 = col_ind[j];
    const int c1 = col_ind[j + W];
    const T x0 = xb[c0];
    const T x1 = xb[c1];
    sum = fma_t(v0, x0, sum);
    sum = fma_t(v1, x1, sum);
  }
  if (j < end) sum = fma_t(val[j], xb[col_ind[j]], sum);
  sum = group_sum<W>(sum);
  if (lane == 0) store_axpby(y, row, alpha, sum, beta);
}

// One workgroup per chunk of a long row: every lane adds up its entries (stride 256), the lanes of a wave
// meet in a butterfly, the four waves in wave order.
template <typename T>
__global__ __launch_bounds__(kRowsBlock) void spmv_bin_chunk_kernel(
    int chunks, const BinChunk* __restrict__ chunk, const T* __restrict__ val, const int* __restrict__ col_ind,
    const T* __restrict__ x, int base, T* __restrict__ partial) {
  __shared__ T s_wave[kRowsBlock / kWave];
  const int cidx = blockIdx.x;
  if (cidx >= chunks) return;
  const BinChunk ch = chunk[cidx];
  const T* __restrict__ xb = x - base;
  T sum = T(0);
  int64_t j = (int64_t)ch.begin + threadIdx.x;
  const int64_t end = ch.end;
  for (; j + 3 * kRowsBlock < end; j += 4 * kRowsBlock) {
    T v[4];
    int c[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      v[u] = val[j + u * kRowsBlock];
      c[u] = col_ind[j + u * kRowsBlock];
    }
    T xv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) xv[u] = xb[c[u]];
#pragma unroll
    for (int u = 0; u < 4; ++u) sum = fma_t(v[u], xv[u], sum);
  }
  for (; j < end; j += kRowsBlock) sum = fma_t(val[j], xb[col_ind[j]], sum);
  sum = group_sum<kWave>(sum);
  if (threadIdx.x % kWave == 0) s_wave[threadIdx.x / kWave] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    T total = s_wave[0];
#pragma unroll
    for (int w = 1; w < kRowsBlock / kWave; ++w) total += s_wave[w];
    partial[cidx] = total;
  }
}

// Lane i adds the chunk sums of long row i in chunk order and writes its y.
template <typename T>
__global__ __launch_bounds__(256) void spmv_bin_finish_kernel(int nlong, const int* __restrict__ long_rows,
                                                              const int* __restrict__ first_chunk,
                                                              const T* __restrict__ partial, T alpha, T beta,
                                                              T* __restrict__ y) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= nlong) return;
  T sum = T(0);
  for (int c = first_chunk[i]; c < first_chunk[i + 1]; ++c) sum += partial[c];
  store_axpby(y, (int64_t)long_rows[i], alpha, sum, beta);
}

}  // namespace asamd
