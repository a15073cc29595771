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

// R consecutive rows per lane: when the number of rows is a multiple of R every slot starts at a multiple of
// R, so the lane's R values and R indices of a slot are aligned vector loads (for 8-byte values and R = 2:
// 16 / 8 bytes per lane instead of 8 / 4): 1 / R as many memory instructions for the same bytes.  Measured on
// the 5-point Laplacian of 4 M rows, fp64 (one row per lane, both streams non-temporal: 56.0 us): R = 2 with
// the indices non-temporal and the values not 50.0 us, both non-temporal 53.4, values only 51.6, neither
// 59.3; R = 1 with that mix 54.4; R = 4 65.5 (too few lanes in flight).  NTV / NTC: which stream bypasses the
// caches; the launch picks them from the sizes of the streams (stream_policy.hpp).
template <typename T, int R, bool NTV = false, bool NTC = true>
__global__ __launch_bounds__(kEllThreads) void ellmv_multi_kernel(int m, int n, T alpha,
                                                                  const T* __restrict__ ell_val,
                                                                  const int* __restrict__ ell_col, int width,
                                                                  int base, const T* __restrict__ x, T beta,
                                                                  T* __restrict__ y) {
  struct alignas(R * sizeof(T) > 16 ? 16 : R * sizeof(T)) ValR {
    T e[R];
  };
  struct alignas(4 * R) ColR {
    int e[R];
  };
  const int64_t row = ((int64_t)blockIdx.x * kEllThreads + threadIdx.x) * R;
  if (row >= m) return;
  T sum[R];
#pragma unroll
  for (int i = 0; i < R; ++i) sum[i] = T(0);
  constexpr int kU = R >= 4 ? 2 : 4;
  int s = 0;
  for (; s + kU <= width; s += kU) {
    ColR c[kU];
    ValR v[kU];
    T xv[kU][R];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int64_t idx = (int64_t)(s + u) * m + row;
      c[u] = NTC ? nt_load_object(reinterpret_cast<const ColR*>(ell_col + idx)) : *reinterpret_cast<const ColR*>(ell_col + idx);
      v[u] = NTV ? nt_load_object(reinterpret_cast<const ValR*>(ell_val + idx)) : *reinterpret_cast<const ValR*>(ell_val + idx);
    }
#pragma unroll
    for (int u = 0; u < kU; ++u)
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int col = c[u].e[i] - base;
        xv[u][i] = (unsigned)col < (unsigned)n ? x[col] : T(0);
      }
#pragma unroll
    for (int u = 0; u < kU; ++u)
#pragma unroll
      for (int i = 0; i < R; ++i)
        if ((unsigned)(c[u].e[i] - base) < (unsigned)n) sum[i] = fma_t(v[u].e[i], xv[u][i], sum[i]);
  }
  for (; s < width; ++s) {
    const int64_t idx = (int64_t)s * m + row;
    const ColR c = *reinterpret_cast<const ColR*>(ell_col + idx);
    const ValR v = *reinterpret_cast<const ValR*>(ell_val + idx);
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int col = c.e[i] - base;
      if ((unsigned)col < (unsigned)n) sum[i] = fma_t(v.e[i], x[col], sum[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) store_axpby(y, row + i, alpha, sum[i], beta);
}

}  // namespace asamd
