// Transposed CSR SpMV, y = alpha*A^T*x + beta*y (A is m x n: x has m entries, y has n).
//
// Two routes:
//   * a CSR copy of A^T built once by the analysis (stable radix sort of the
//     entries by column, so rows stay ascending inside every column and the
//     layout is deterministic); multiplies then run the ordinary row kernels on
//     that copy: same bytes, same rooflines, bit-reproducible.
//   * without such a copy, the scatter below: y is scaled by beta, then every
//     entry adds alpha*val*x[row] to y[col] with a hardware float atomic.  This
//     is what the reference always does, one lane per row
//     (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_x_csr_trans.cpp:11-45; its beta
//     pass covers m elements of y where n are meant, :61-64); here W lanes share
//     a row so that the entry loads coalesce.  CONJ conjugates the values on
//     the way: y = alpha*A^H*x + beta*y, the reference's
//     csr_gemv_conj_scalar_atomicadd (dcu_gemv_c_csr_conj.cpp:22-48).
#pragma once

#include "device_utils.hpp"

namespace asamd {

// key[k] = zero-based column of entry k, idx[k] = k
static __global__ __launch_bounds__(256) void transpose_keys_kernel(int nnz, const int* __restrict__ col_ind, int base,
                                                             unsigned* __restrict__ key,
                                                             unsigned* __restrict__ idx) {
  for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz;
       k += (int64_t)gridDim.x * blockDim.x) {
    key[k] = (unsigned)(col_ind[k] - base);
    idx[k] = (unsigned)k;
  }
}

// entries of A^T in column-sorted order: zero-based row of A as the new column index
// (CONJ: values conjugated, which makes the copy A^H)
template <typename T, bool CONJ>
__global__ __launch_bounds__(256) void transpose_gather_kernel(int nnz, const unsigned* __restrict__ perm,
                                                               const int* __restrict__ coo_row,
                                                               const T* __restrict__ val, int base,
                                                               int* __restrict__ t_col, T* __restrict__ t_val) {
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < nnz;
       q += (int64_t)gridDim.x * blockDim.x) {
    const unsigned k = perm[q];
    t_col[q] = coo_row[k] - base;
    t_val[q] = CONJ ? conj_t(val[k]) : val[k];
  }
}

// y <- beta*y over n elements (beta == 0 stores zeros without reading)
template <typename T>
__global__ __launch_bounds__(256) void scale_vec_kernel(int n, T beta, T* __restrict__ y) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  y[i] = beta == T(0) ? T(0) : y[i] * beta;
}

constexpr int kTransThreads = 256;

template <typename T, int W, bool CONJ>
__global__ __launch_bounds__(kTransThreads) void csrmv_trans_scatter_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T* __restrict__ y, int base) {
  const int64_t row = ((int64_t)blockIdx.x * kTransThreads + threadIdx.x) / W;
  const int sub = threadIdx.x % W;
  if (row >= m) return;
  const T t = alpha * x[row];
  const int64_t b = (int64_t)row_ptr[row] - base, e = (int64_t)row_ptr[row + 1] - base;
  for (int64_t k = b + sub; k < e; k += W) {
    const int c = col_ind[k] - base;
    if ((unsigned)c < (unsigned)n) atomic_add(&y[c], (CONJ ? conj_t(val[k]) : val[k]) * t);
  }
}

}  // namespace asamd
