// ELL SpMV, y = alpha*A*x + beta*y with A in column-major ELL (slot s of row r
// at [s*m + r]): one lane per row, so the lanes of a wave read consecutive
// addresses in every slot and nothing but the x gathers is irregular.  Slots
// whose index (minus base) falls outside [0, n) do not count.  Same traversal
// as src/kernel/dcu/level2/mv/dcu_gemv_x_ell.cpp:10-43; the slot loop is
// unrolled so that four independent gathers are in flight per lane.
// Used by the ELL entry points and by the CSR plan's ELL copy (matrices whose
// rows are short and nearly equal, where it beats every CSR traversal: no
// row_ptr, no LDS staging, full-width coalescing).
#pragma once

#include "device_utils.hpp"

namespace asamd {

constexpr int kEllThreads = 256;
constexpr int kEllUnroll = 4;

template <typename T>
__global__ __launch_bounds__(kEllThreads) void ellmv_kernel(int m, int n, T alpha,
                                                            const T* __restrict__ ell_val,
                                                            const int* __restrict__ ell_col, int width,
                                                            int base, const T* __restrict__ x, T beta,
                                                            T* __restrict__ y) {
  const int64_t row = (int64_t)blockIdx.x * kEllThreads + threadIdx.x;
  if (row >= m) return;
  T sum = T(0);
  int s = 0;
  for (; s + kEllUnroll <= width; s += kEllUnroll) {
    int c[kEllUnroll];
    T v[kEllUnroll], xv[kEllUnroll];
#pragma unroll
    for (int u = 0; u < kEllUnroll; ++u) {
      const int64_t idx = (int64_t)(s + u) * m + row;
      c[u] = __builtin_nontemporal_load(&ell_col[idx]) - base;
      v[u] = nt_load(&ell_val[idx]);
    }
#pragma unroll
    for (int u = 0; u < kEllUnroll; ++u) xv[u] = (unsigned)c[u] < (unsigned)n ? x[c[u]] : T(0);
#pragma unroll
    for (int u = 0; u < kEllUnroll; ++u)
      if ((unsigned)c[u] < (unsigned)n) sum = fma_t(v[u], xv[u], sum);
  }
  for (; s < width; ++s) {
    const int64_t idx = (int64_t)s * m + row;
    const int c = ell_col[idx] - base;
    if ((unsigned)c < (unsigned)n) sum = fma_t(ell_val[idx], x[c], sum);
  }
  store_axpby(y, row, alpha, sum, beta);
}

}  // namespace asamd
