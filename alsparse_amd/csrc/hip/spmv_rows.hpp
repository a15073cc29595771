// Row-parallel CSR SpMV kernels for gfx950 (wave64): one lane group per row.
//
//   spmv_vector_kernel<T, W>    W consecutive lanes share a row, W picked from
//                               the mean row length; coalesced col/val streaming,
//                               DPP group reduction.
//   spmv_rowconst_kernel<T, G>  every row has exactly 4*G entries starting at
//                               row*4*G: no row_ptr traffic, one 128-bit load of
//                               values and one of indices per lane.
//   spmv_scalar_kernel<T>       one lane per row (diagnostic baseline).
//   spmv_stream_kernel<T>       rows of at most 16 entries: a workgroup stages the
//                               products of 256 consecutive rows in LDS, one lane
//                               per row sums them.
//
// They stand in for the reference's only CSR SpMV kernel, csr_gemv_vector
// (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57): same arithmetic
// (fma accumulation per lane, then y = beta*y + alpha*sum), different mapping.
// beta == 0 never reads y.  All element offsets are formed in 64 bits.
#pragma once

#include "device_utils.hpp"

namespace asamd {

constexpr int kRowsBlock = 256;  // threads per workgroup of the row kernels

template <typename T, int W>
__global__ __launch_bounds__(kRowsBlock) void spmv_vector_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  constexpr int kRowsPerBlock = kRowsBlock / W;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int lane = threadIdx.x % W;
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / W;
  if (row >= m) return;  // whole lane groups leave together
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* __restrict__ xb = x - base;
  T sum = T(0);
  int64_t j = start + lane;
  // two entries per lane and trip keep two gathers in flight
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

template <typename T>
__global__ __launch_bounds__(kRowsBlock) void spmv_scalar_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  const int64_t row = (int64_t)blockIdx.x * kRowsBlock + threadIdx.x;
  if (row >= m) return;
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* __restrict__ xb = x - base;
  T sum = T(0);
  for (int64_t j = start; j < end; ++j) sum = fma_t(val[j], xb[col_ind[j]], sum);
  store_axpby(y, row, alpha, sum, beta);
}

// ---- short rows: LDS-staged row blocks ---------------------------------------
// A workgroup owns kStreamRows consecutive rows, none longer than
// kStreamMaxLen.  Their entries are one contiguous range of the CSR streams: it
// is read fully coalesced (lane k takes entries k, k + 256, ...), multiplied
// with the gathered x and staged in LDS; after one barrier every lane sums the
// few products of its own row from LDS (a lane's run is contiguous and runs of
// neighbouring lanes are adjacent, so the reads spread over the banks) and
// writes y unit stride.  No searches, no scans: this is what rows of 3-5
// entries (stencils) want.
constexpr int kStreamRows = 256;
constexpr int kStreamMaxLen = 16;

// CAP: compile-time bound on the row length (4, 8 or 16): sizes the LDS staging
// area, so shorter rows leave room for more resident workgroups.
template <typename T, int CAP>
__global__ __launch_bounds__(kStreamRows) void spmv_stream_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  __shared__ T s_prod[kStreamRows * CAP];
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row0 = (int64_t)bid * kStreamRows;
  const int64_t row = row0 + threadIdx.x;
  int64_t row_last = row0 + kStreamRows;
  if (row_last > m) row_last = m;
  const int64_t e0 = (int64_t)row_ptr[row0] - base;
  const int n = (int)((int64_t)row_ptr[row_last] - base - e0);  // <= kStreamRows * CAP by contract
  int my_begin = 0, my_end = 0;
  if (row < m) {
    my_begin = (int)((int64_t)row_ptr[row] - base - e0);
    my_end = (int)((int64_t)row_ptr[row + 1] - base - e0);
  }
  const T* __restrict__ xb = x - base;
  T v[CAP];
  int c[CAP];
#pragma unroll
  for (int s = 0; s < CAP; ++s) {
    const int k = threadIdx.x + s * kStreamRows;
    if (k < n) {
      v[s] = val[e0 + k];
      c[s] = col_ind[e0 + k];
    }
  }
#pragma unroll
  for (int s = 0; s < CAP; ++s) {
    const int k = threadIdx.x + s * kStreamRows;
    if (k < n) s_prod[k] = v[s] * xb[c[s]];
  }
  __syncthreads();
  if (row >= m) return;
  T sum = T(0);
  for (int k = my_begin; k < my_end; ++k) sum += s_prod[k];
  store_axpby(y, row, alpha, sum, beta);
}

// ---- constant row length ----------------------------------------------------
template <typename T>
struct Quad;  // four consecutive values loaded as 128-bit pieces
template <>
struct Quad<float> {
  Float4 q;
  __device__ __forceinline__ void load(const float* p) { q = *reinterpret_cast<const Float4*>(p); }
  __device__ __forceinline__ float get(int i) const { return i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : q.w; }
};
template <>
struct Quad<double> {
  Double2 a, b;
  __device__ __forceinline__ void load(const double* p) {
    a = *reinterpret_cast<const Double2*>(p);
    b = *reinterpret_cast<const Double2*>(p + 2);
  }
  __device__ __forceinline__ double get(int i) const { return i == 0 ? a.x : i == 1 ? a.y : i == 2 ? b.x : b.y; }
};

// G lanes per row, each owning 4 consecutive entries: L = 4*G.  R rows per
// lane group and launch keep 4*R gathers per lane in flight.
template <typename T, int G, int R>
__global__ __launch_bounds__(kRowsBlock) void spmv_rowconst_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ col_ind,
    const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  constexpr int kGroups = kRowsBlock / G;  // lane groups per workgroup
  constexpr int L = 4 * G;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int lane = threadIdx.x % G;
  const int group = threadIdx.x / G;
  const int64_t row0 = (int64_t)bid * (kGroups * R) + group;
  const T* __restrict__ xb = x - base;

  Quad<T> v[R];
  Int4 c[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + (int64_t)r * kGroups;
    if (row < m) {
      const int64_t off = row * L + lane * 4;
      v[r].load(val + off);
      c[r] = *reinterpret_cast<const Int4*>(col_ind + off);
    }
  }
  T xs[R][4];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + (int64_t)r * kGroups;
    if (row < m) {
      xs[r][0] = xb[c[r].x];
      xs[r][1] = xb[c[r].y];
      xs[r][2] = xb[c[r].z];
      xs[r][3] = xb[c[r].w];
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + (int64_t)r * kGroups;
    if (row < m) {
      T sum = v[r].get(0) * xs[r][0];
      sum = fma_t(v[r].get(1), xs[r][1], sum);
      sum = fma_t(v[r].get(2), xs[r][2], sum);
      sum = fma_t(v[r].get(3), xs[r][3], sum);
      sum = group_sum<G>(sum);
      if (lane == 0) store_axpby(y, row, alpha, sum, beta);
    }
  }
}

}  // namespace asamd
