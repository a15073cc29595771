// CSR SpMM  C = alpha*A*B + beta*C  for gfx950 (wave64).
//
//   spmm_rowmajor_kernel<T, V>  unit stride along the dense columns (row-major
//       B and C, or column-major with op(B) = B^T read as row-major): one wave
//       per row of A and per chunk of 64*V dense columns; the row's
//       (col, alpha*val) pairs are read coalesced 64 at a time and broadcast
//       with v_readlane, so every B row is fetched with one wave-wide load of
//       64*V contiguous elements; C is read-modified-written once.
//       This is the layout the reference cannot run on the GPU at all
//       (dcu_gemm_?_csr_row returns NOT_SUPPORTED,
//       src/kernel/dcu/level3/mm/csrmm/dcu_gemm_x_csr_row.cpp:15-36).
//   spmm_rowmajor_group_kernel<T, G, V> / spmm_rowmajor_short_kernel<T, NV, W>
//       the same layout with at most 32 / at most 16 dense columns: several
//       rows of A per wave (described at the kernels).
//   dense_transpose_kernel<T> + spmm_colmajor_kernel<T>   column-major B and C
//       (the layout the reference's GPU path does run): B is first transposed
//       into a row-major workspace, 64 x 64 tiles through LDS, both sides
//       coalesced; then a workgroup takes 64 consecutive rows of A and 64 dense
//       columns, its waves form the rows' sums exactly as above (one wave-wide
//       load per B row), park them in an LDS tile and the workgroup writes the
//       tile to column-major C transposed: 64 consecutive rows of one column
//       per wave instruction.  Gathering column-major B directly costs one
//       128-byte line per ELEMENT instead of per row (44 ms against 1.3 ms on
//       a 2^20 x 2^20 matrix with 32 entries per row and 64 columns).
//   spmm_strided_kernel<T>      any strides: one lane per (row, dense column),
//       lanes of a wave on consecutive rows, so column-major C is written
//       coalesced and B(:, c) is gathered like an SpMV x.  Stands in for
//       csr_gemm_plain_device (dcu_gemm_csr_col_plain.h:9-39).
//
// Arithmetic follows the row-major plain kernel
// (src/plain/kernel/level3/mm/gemm/gemm_x_csr_row_plain.c:11-19): alpha is
// folded into each value, products are accumulated with fma in entry order,
// then C = beta*C + acc.  beta == 0 never reads C.

#include <hip/hip_runtime.h>

#include <cstdlib>
#include <mutex>

#include "alsparse_amd_kernels.h"
#include "device_utils.hpp"

using namespace asamd;

constexpr int kSpmmBlock = 256;
constexpr int kSpmmWaves = kSpmmBlock / kWave;

template <typename T, int V>
struct alignas(sizeof(T) * V) Vec {
  T e[V];
};

// N consecutive elements that are only known to be aligned like a single one: the compiler may
// still fetch them with one wide load (global memory takes unaligned wide accesses).
template <typename T, int N>
struct __attribute__((packed, aligned(alignof(T)))) Packed {
  T e[N];
};
template <typename T>
using Quad4 = Packed<T, 4>;

// The first `valid` (<= V) elements at p, zeros behind them: whole groups of four through one load each.
template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_short_row(const T* p, int valid) {
  Vec<T, V> r;
#pragma unroll
  for (int i = 0; i < V; i += 4) {
    if (V - i >= 4 && i + 4 <= valid) {
      const Quad4<T> q = *reinterpret_cast<const Quad4<T>*>(p + i);
#pragma unroll
      for (int u = 0; u < 4; ++u) r.e[i + u] = q.e[u];
    } else {
#pragma unroll
      for (int u = 0; u < 4 && i + u < V; ++u) r.e[i + u] = i + u < valid ? p[i + u] : T(0);
    }
  }
  return r;
}

template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_vec(const T* p, bool vector_ok, int valid) {
  Vec<T, V> r;
  if (vector_ok && valid == V) {
    r = *reinterpret_cast<const Vec<T, V>*>(p);
  } else if (valid == V) {
    const Packed<T, V> q = *reinterpret_cast<const Packed<T, V>*>(p);
#pragma unroll
    for (int i = 0; i < V; ++i) r.e[i] = q.e[i];
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) r.e[i] = i < valid ? p[i] : T(0);
  }
  return r;
}

__device__ __forceinline__ float readlane_t(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ double readlane_t(double v, int l) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, l);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), l);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

template <typename R>
__device__ __forceinline__ Cx<R> readlane_t(Cx<R> v, int l) {
  return Cx<R>(readlane_t(v.re, l), readlane_t(v.im, l));
}

// grid.x covers rows (one wave each), grid.y covers chunks of 64*V columns.
template <typename T, int V>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc, bool vector_ok) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row = (int64_t)bid * kSpmmWaves + wave;
  if (row >= m) return;  // wave-uniform
  const int c0 = (blockIdx.y * kWave + lane) * V;  // first dense column of this lane
  int valid = n - c0;
  valid = valid > V ? V : (valid < 0 ? 0 : valid);

  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = T(0);

  for (int64_t j0 = start; j0 < end; j0 += kWave) {
    const int64_t j = j0 + lane;
    int my_col = 0;
    T my_val = T(0);
    if (j < end) {
      // A and C are touched once: non-temporal, so that they do not push rows of B out of the caches
      my_col = nt_load(col_ind + j) - base;
      my_val = alpha * nt_load(val + j);
    }
    const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
    int t = 0;
    constexpr int kU = 4;  // B rows in flight per wave (8 and 16 measured no faster)
    for (; t + kU <= cnt; t += kU) {
      Vec<T, V> b[kU];
      T a[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int col = __builtin_amdgcn_readlane(my_col, t + u);
        a[u] = readlane_t(my_val, t + u);
        b[u] = load_vec<T, V>(B + (int64_t)col * ldb + c0, vector_ok, valid);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
      }
    }
    for (; t < cnt; ++t) {
      const int col = __builtin_amdgcn_readlane(my_col, t);
      const T a = readlane_t(my_val, t);
      const Vec<T, V> b = load_vec<T, V>(B + (int64_t)col * ldb + c0, vector_ok, valid);
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] = fma_t(a, b.e[i], acc[i]);
    }
  }

  T* crow = C + row * ldc + c0;
  if (vector_ok && valid == V) {
    Vec<T, V> out;
    if (beta == T(0)) {
#pragma unroll
      for (int i = 0; i < V; ++i) out.e[i] = acc[i];
    } else {
      const Vec<T, V> old = *reinterpret_cast<const Vec<T, V>*>(crow);
#pragma unroll
      for (int i = 0; i < V; ++i) out.e[i] = old.e[i] * beta + acc[i];
    }
    *reinterpret_cast<Vec<T, V>*>(crow) = out;
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      if (i < valid) {
        const T res = beta == T(0) ? acc[i] : nt_load(crow + i) * beta + acc[i];
        nt_store(res, crow + i);
      }
    }
  }
}

// Four entries of a row per wave instruction: the wave's lanes form four groups of 16, lane l of a group owns
// the E = 16 / sizeof(T) dense columns from (blockIdx.y * 16 + l) * E on and loads them with one 128-bit load,
// so one instruction fetches 16 * E contiguous elements of FOUR rows of B (group g takes the row's entries
// 4i + g), and all the loads of up to 32 entries are in flight at once: a 32-entry row waits for B once, not
// eight times in turn.  The four partial sums meet at the end (two exchanges across the groups).  Needs B and C
// rows that 128-bit loads can address: pointers and row strides multiples of 16 bytes, n a multiple of E.
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_quad_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc) {
  constexpr int E = 16 / (int)sizeof(T);
  constexpr int kU = 8;  // loads in flight per lane
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row = (int64_t)bid * kSpmmWaves + wave;
  if (row >= m) return;  // wave-uniform
  const int g = lane / 16;
  const int c0 = (blockIdx.y * 16 + lane % 16) * E;
  const bool owns = c0 < n;
  // lanes past the last dense column load what the group's first lane loads (the same cache line: no request
  // of their own) and add nothing
  const T* bcol = B + (owns ? c0 : blockIdx.y * 16 * E);

  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T acc[E];
#pragma unroll
  for (int i = 0; i < E; ++i) acc[i] = T(0);

  for (int64_t j0 = start; j0 < end; j0 += kWave) {
    const int64_t j = j0 + lane < end ? j0 + lane : j0;  // lanes past the end repeat the chunk's first entry
    // A and C are touched once: non-temporal, so that they do not push rows of B out of the caches
    const int my_col = nt_load(col_ind + j) - base;
    const T my_val = alpha * nt_load(val + j);
    const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
    for (int t0 = 0; t0 < cnt; t0 += 4 * kU) {
      Vec<T, E> b[kU];
      T a[kU];
      // every load is issued whatever the group needs (a group past the end loads the chunk's first row of
      // B again and adds nothing): loads under branches would wait for one another
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int t = t0 + 4 * u + g;
        const int src = t < cnt ? t : 0;
        const int col = lane_get(my_col, src);
        a[u] = lane_get(my_val, src);
        b[u] = *reinterpret_cast<const Vec<T, E>*>(bcol + (int64_t)col * ldb);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        if (t0 + 4 * u + g < cnt) {
#pragma unroll
          for (int i = 0; i < E; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < E; ++i) {
    acc[i] += lane_xor(acc[i], 16);
    acc[i] += lane_xor(acc[i], 32);
  }
  if (g == 0 && owns) {
    T* crow = C + row * ldc + c0;
    Vec<T, E> out;
    if (beta == T(0)) {
#pragma unroll
      for (int i = 0; i < E; ++i) out.e[i] = acc[i];
    } else {
      const Vec<T, E> old = *reinterpret_cast<const Vec<T, E>*>(crow);
#pragma unroll
      for (int i = 0; i < E; ++i) out.e[i] = old.e[i] * beta + acc[i];
    }
    *reinterpret_cast<Vec<T, E>*>(crow) = out;
  }
}

// Dense operands narrower than a wave, lane-group form: G lanes per row of A, 64 / G rows per wave,
// lane c of a group owns V consecutive dense columns.  The group walks its row four entries at a
// time; the entry loads are the same address for all lanes of a group (one request), each B row is
// one load of G*V contiguous elements, so one wave instruction fetches 64 / G rows of B.  A wave per
// row would leave 64 - n lanes idle and issue 64 / G times as many loads.
template <typename T, int G, int V>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_group_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc, bool vector_ok) {
  constexpr int kRowsPerBlock = kSpmmBlock / G;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / G;
  if (row >= m) return;
  const int c0 = (blockIdx.y * G + threadIdx.x % G) * V;  // first dense column of this lane
  int valid = n - c0;
  valid = valid > V ? V : (valid < 0 ? 0 : valid);
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* bcol = B + c0;
  T acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = T(0);
  if constexpr (V == 1) {
    // four entries at a time, every lane of the group loading the same entry (one request per group):
    // measured faster than handing entries round when a lane has a single column (13 columns: 0.75 ms
    // against 0.81 ms on a 2^20 x 2^20 matrix with 32 entries per row)
    int64_t j = start;
    constexpr int kU = 4;
    for (; j + kU <= end; j += kU) {
      int col[kU];
      T a[kU], b[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        col[u] = col_ind[j + u] - base;
        a[u] = alpha * val[j + u];
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) b[u] = valid ? bcol[(int64_t)col[u] * ldb] : T(0);
#pragma unroll
      for (int u = 0; u < kU; ++u) acc[0] = fma_t(a[u], b[u], acc[0]);
    }
    for (; j < end; ++j)
      acc[0] = fma_t(alpha * val[j], valid ? bcol[(int64_t)(col_ind[j] - base) * ldb] : T(0), acc[0]);
  } else {
    const int gl = threadIdx.x % G;                  // lane inside the group
    const int g0 = (threadIdx.x % kWave) - gl;       // the group's first lane in the wave
    for (int64_t j0 = start; j0 < end; j0 += G) {
      // the group reads G entries of its row with one coalesced load, then hands them round
      const int64_t j = j0 + gl;
      int my_col = 0;
      T my_val = T(0);
      if (j < end) {
        my_col = nt_load(col_ind + j) - base;
        my_val = alpha * nt_load(val + j);
      }
      const int cnt = (int)(end - j0 < G ? end - j0 : G);
      int t = 0;
      constexpr int kU = 4;
      for (; t + kU <= cnt; t += kU) {
        T a[kU];
        Vec<T, V> b[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int col = lane_get(my_col, g0 + t + u);
          a[u] = lane_get(my_val, g0 + t + u);
          b[u] = load_vec<T, V>(bcol + (int64_t)col * ldb, vector_ok, valid);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
#pragma unroll
          for (int i = 0; i < V; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
        }
      }
      for (; t < cnt; ++t) {
        const int col = lane_get(my_col, g0 + t);
        const T a = lane_get(my_val, g0 + t);
        const Vec<T, V> b = load_vec<T, V>(bcol + (int64_t)col * ldb, vector_ok, valid);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = fma_t(a, b.e[i], acc[i]);
      }
    }
  }
  T* out = C + row * ldc + c0;
#pragma unroll
  for (int i = 0; i < V; ++i)
    if (i < valid) out[i] = beta == T(0) ? acc[i] : out[i] * beta + acc[i];
}

template <typename T, int G, int V>
static void launch_group(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci, int base,
                         const T* B, int64_t ldb, T beta, T* C, int64_t ldc) {
  constexpr int rows_per_block = kSpmmBlock / G;
  const dim3 grid((unsigned)(((int64_t)m + rows_per_block - 1) / rows_per_block), (unsigned)((n + G * V - 1) / (G * V)));
  const bool vector_ok = V > 1 && (uintptr_t)B % (V * sizeof(T)) == 0 && ldb % V == 0;
  spmm_rowmajor_group_kernel<T, G, V><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc,
                                                                  vector_ok);
}

// Narrow dense operands (n <= NV <= 16): W lanes share a row of A and read its entries coalesced, as
// in the lane-group SpMV kernel; every lane multiplies its entries with the whole (short) row of B
// -- one vector load of NV elements when B allows it -- and keeps NV partial sums; the group's sums
// meet through DPP and lane 0 writes the row of C.  Measured on a 2^20 x 2^20 matrix with 32 entries
// per row against the lane-group kernel above with a lane per column (n: ms -> ms): 1: 0.50 -> 0.21, 2: 0.68 -> 0.37,
// 4: 0.78 -> 0.48, 6: 0.82 -> 0.64, 8: 0.77 -> 0.55, 12: 0.73 -> 0.72, 16: 0.61 -> 0.60; 13: 0.75 -> 0.89,
// which is why widths above 8 that are not multiples of four stay with the kernel above.
template <typename T, int NV>
__device__ __forceinline__ Vec<T, NV> short_row(const T* p, bool vector_ok, int n) {
  if (vector_ok) return *reinterpret_cast<const Vec<T, NV>*>(p);  // n == NV and the row is aligned to its size
  return load_short_row<T, NV>(p, n);
}

template <typename T, int NV, int W>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_short_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t c_row_stride, int64_t c_col_stride, bool vector_ok) {
  constexpr int kRowsPerBlock = kSpmmBlock / W;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int lane = threadIdx.x % W;
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / W;
  if (row >= m) return;  // whole lane groups leave together
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = T(0);
  int64_t j = start + lane;
  // two entries per lane and trip keep two B rows in flight
  for (; j + W < end; j += 2 * W) {
    const T a0 = alpha * val[j], a1 = alpha * val[j + W];
    const int c0 = col_ind[j] - base, c1 = col_ind[j + W] - base;
    const Vec<T, NV> b0 = short_row<T, NV>(B + (int64_t)c0 * ldb, vector_ok, n);
    const Vec<T, NV> b1 = short_row<T, NV>(B + (int64_t)c1 * ldb, vector_ok, n);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a0, b0.e[i], acc[i]);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a1, b1.e[i], acc[i]);
  }
  if (j < end) {
    const T a0 = alpha * val[j];
    const Vec<T, NV> b0 = short_row<T, NV>(B + (int64_t)(col_ind[j] - base) * ldb, vector_ok, n);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a0, b0.e[i], acc[i]);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = group_sum<W>(acc[i]);
  if (lane == 0) {
    // row-major C: n consecutive elements; column-major C: the lanes 0 of a wave's groups hold
    // consecutive rows, so every dense column is written as one contiguous run
    T* crow = C + row * c_row_stride;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (i < n) crow[i * c_col_stride] = beta == T(0) ? acc[i] : crow[i * c_col_stride] * beta + acc[i];
  }
}

template <typename T, int NV, int W>
static void launch_short(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci, int base,
                         const T* B, int64_t ldb, T beta, T* C, int64_t scr, int64_t scc) {
  constexpr int rows_per_block = kSpmmBlock / W;
  const unsigned grid = (unsigned)(((int64_t)m + rows_per_block - 1) / rows_per_block);
  const bool vector_ok = n == NV && ldb % NV == 0 && (uintptr_t)B % (NV * sizeof(T)) == 0;
  spmm_rowmajor_short_kernel<T, NV, W><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, beta, C,
                                                                     scr, scc, vector_ok);
}

// lanes per row from the mean row length
template <typename T, int NV>
static void launch_short_w(hipStream_t s, int m, int n, int64_t nnz, T alpha, const T* val, const int* rp,
                           const int* ci, int base, const T* B, int64_t ldb, T beta, T* C, int64_t scr,
                           int64_t scc) {
  const double mean = (double)nnz / (double)m;
  if (mean < 8) launch_short<T, NV, 4>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (mean < 48) launch_short<T, NV, 16>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else launch_short<T, NV, 64>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
}

// B rows of n <= 16 contiguous elements, C with any two strides
template <typename T>
static void launch_short_n(hipStream_t s, int m, int n, int64_t nnz, T alpha, const T* val, const int* rp,
                           const int* ci, int base, const T* B, int64_t ldb, T beta, T* C, int64_t scr,
                           int64_t scc) {
  if (n <= 2) launch_short_w<T, 2>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (n <= 4) launch_short_w<T, 4>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (n <= 8) launch_short_w<T, 8>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else launch_short_w<T, 16>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
}

// out[r * out_ld + c] = in[r + c * in_ld] for r < rows, c < cols: 64 x 64 tiles, reads
// coalesced along r, writes along c.  grid = (ceil(rows/64), ceil(cols/64)).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void dense_transpose_kernel(int rows, int cols, const T* __restrict__ in,
                                                                     int64_t in_ld, T* __restrict__ out,
                                                                     int64_t out_ld) {
  __shared__ T tile[kWave][kWave + 1];
  const int tx = threadIdx.x % kWave, ty = threadIdx.x / kWave;
  const int64_t r0 = (int64_t)blockIdx.x * kWave;
  const int c0 = blockIdx.y * kWave;
#pragma unroll 4
  for (int i = ty; i < kWave; i += kSpmmWaves) {
    const int64_t r = r0 + tx;
    const int c = c0 + i;
    tile[i][tx] = (r < rows && c < cols) ? nt_load(in + r + (int64_t)c * in_ld) : T(0);
  }
  __syncthreads();
#pragma unroll 4
  for (int i = ty; i < kWave; i += kSpmmWaves) {
    const int64_t r = r0 + i;
    const int c = c0 + tx;
    if (r < rows && c < cols) out[r * out_ld + c] = tile[tx][i];
  }
}

// C (column-major, element (r, c) at r + c*ldc) = alpha*A*Bt + beta*C with Bt row-major
// (element (r, c) at r*ldbt + c).  grid = (ceil(m/64), ceil(n/64)).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void spmm_colmajor_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ Bt, int64_t ldbt, T beta,
    T* __restrict__ C, int64_t ldc) {
  __shared__ T tile[kWave][kWave + 1];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row0 = (int64_t)bid * kWave;
  const int c0 = blockIdx.y * kWave;
  const bool col_ok = c0 + lane < n;
  const T* bcol = Bt + c0 + lane;
  for (int rr = wave; rr < kWave; rr += kSpmmWaves) {
    const int64_t row = row0 + rr;
    T acc = T(0);
    if (row < m) {  // wave-uniform
      const int64_t start = (int64_t)row_ptr[row] - base;
      const int64_t end = (int64_t)row_ptr[row + 1] - base;
      for (int64_t j0 = start; j0 < end; j0 += kWave) {
        const int64_t j = j0 + lane;
        int my_col = 0;
        T my_val = T(0);
        if (j < end) {
          my_col = nt_load(col_ind + j) - base;
          my_val = alpha * nt_load(val + j);
        }
        const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
        int t = 0;
        constexpr int kU = 4;
        for (; t + kU <= cnt; t += kU) {
          T b[kU], a[kU];
#pragma unroll
          for (int u = 0; u < kU; ++u) {
            const int col = __builtin_amdgcn_readlane(my_col, t + u);
            a[u] = readlane_t(my_val, t + u);
            b[u] = col_ok ? bcol[(int64_t)col * ldbt] : T(0);
          }
#pragma unroll
          for (int u = 0; u < kU; ++u) acc = fma_t(a[u], b[u], acc);
        }
        for (; t < cnt; ++t) {
          const int col = __builtin_amdgcn_readlane(my_col, t);
          const T a = readlane_t(my_val, t);
          acc = fma_t(a, col_ok ? bcol[(int64_t)col * ldbt] : T(0), acc);
        }
      }
    }
    tile[rr][lane] = acc;
  }
  __syncthreads();
  const int64_t row = row0 + lane;
  if (row >= m) return;
  for (int cc = wave; cc < kWave; cc += kSpmmWaves) {
    const int c = c0 + cc;
    if (c >= n) break;
    T* out = C + row + (int64_t)c * ldc;
    const T acc = tile[lane][cc];
    const T res = beta == T(0) ? acc : nt_load(out) * beta + acc;
    nt_store(res, out);
  }
}

// One lane per (row, dense column); blockDim = (64 rows, 4 columns).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void spmm_strided_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t sbr, int64_t sbc,
    T beta, T* __restrict__ C, int64_t scr, int64_t scc) {
  const int64_t row = (int64_t)blockIdx.x * kWave + threadIdx.x;
  if (row >= m) return;
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  for (int64_t c = (int64_t)blockIdx.y * blockDim.y + threadIdx.y; c < n;
       c += (int64_t)gridDim.y * blockDim.y) {
    T acc = T(0);
    for (int64_t j = start; j < end; ++j) {
      const int64_t col = (int64_t)col_ind[j] - base;
      acc = fma_t(alpha * val[j], B[col * sbr + c * sbc], acc);
    }
    T* out = C + row * scr + c * scc;
    *out = beta == T(0) ? acc : *out * beta + acc;
  }
}

// column-major B (k x n) next to column-major C (m x n), more than one column:
// B has to be transposed into a workspace first
static bool colmajor_nn(const asamd_dense_strides* st, int n) {
  return n > 1 && st->b_row_stride == 1 && st->b_col_stride != 1 && st->c_row_stride == 1;
}

// ---- do neighbouring rows of A share columns? --------------------------------------------------
// Stencils and finite-element matrices do (a row of B fetched for one row of A is wanted again by the next
// rows), matrices with random columns do not, and which of the two row-major kernels is faster depends on it
// (27-point stencil, n = 64: four rows of B per wave instruction 0.56 ms, one per instruction 0.88 ms; random
// columns over a B of 64-256 MiB: 1.23 against 1.22 ms).  csrmm has no analysis call, so the first multiply of a
// matrix looks: kProbeRows rows scattered over the matrix, the share of their entries (the first 64 of each) whose column is in
// the next row as well.  One small kernel and one synchronisation, remembered per (row_ptr, col_ind, m, nnz);
// not done while the stream is being captured.
constexpr int kProbeRows = 2048;
__global__ __launch_bounds__(256) void spmm_reuse_probe_kernel(int m, const int* __restrict__ row_ptr,
                                                               const int* __restrict__ col_ind, int base,
                                                               unsigned* __restrict__ out) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= kProbeRows || m < 2) return;
  // scattered rows: evenly spaced ones fall on the same position of every grid line of a stencil
  const int64_t r = (int64_t)((((uint64_t)t + 1) * 0x9E3779B97F4A7C15ull >> 20) % (uint64_t)(m - 1));
  const int64_t b0 = (int64_t)row_ptr[r] - base, e0 = (int64_t)row_ptr[r + 1] - base, e1 = (int64_t)row_ptr[r + 2] - base;
  unsigned shared = 0, total = 0;
  for (int64_t j = b0; j < e0 && j < b0 + 64; ++j) {
    const int c = col_ind[j];
    int64_t lo = e0, hi = e1;  // rows with unsorted columns simply count as sharing nothing
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (col_ind[mid] < c) lo = mid + 1;
      else hi = mid;
    }
    shared += (lo < e1 && col_ind[lo] == c) ? 1u : 0u;
    ++total;
  }
  if (total) {
    atomicAdd(&out[0], shared);
    atomicAdd(&out[1], total);
  }
}

static bool rows_share_columns(hipStream_t s, int m, int nnz, const int* rp, const int* ci, int base) {
  struct Seen {
    const int *rp, *ci;
    int m, nnz;
    bool shares;
  };
  constexpr int kSeen = 16, kMaxDevices = 64;
  static std::mutex lock;
  static Seen seen[kSeen];
  static int next = 0;
  static unsigned* d_out[kMaxDevices];
  std::lock_guard<std::mutex> guard(lock);
  for (const Seen& e : seen)
    if (e.rp == rp && e.ci == ci && e.m == m && e.nnz == nnz) return e.shares;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return false;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
  if (!d_out[dev] && hipMalloc(&d_out[dev], 2 * sizeof(unsigned)) != hipSuccess) {
    (void)hipGetLastError();
    d_out[dev] = nullptr;
    return false;
  }
  unsigned h_out[2] = {0, 0};
  bool ok = hipMemsetAsync(d_out[dev], 0, sizeof(h_out), s) == hipSuccess;
  if (ok) {
    spmm_reuse_probe_kernel<<<kProbeRows / 256, 256, 0, s>>>(m, rp, ci, base, d_out[dev]);
    ok = hipGetLastError() == hipSuccess &&
         hipMemcpyAsync(h_out, d_out[dev], sizeof(h_out), hipMemcpyDeviceToHost, s) == hipSuccess &&
         hipStreamSynchronize(s) == hipSuccess;
  }
  if (!ok) {
    (void)hipGetLastError();
    return false;
  }
  const bool shares = h_out[1] > 0 && 4ull * h_out[0] >= (unsigned long long)h_out[1];
  seen[next] = Seen{rp, ci, m, nnz, shares};
  next = (next + 1) % kSeen;
  return shares;
}

static size_t workspace_bytes(size_t val_size, int n, int k, const asamd_dense_strides* st) {
  if (!st || n <= 0 || k <= 0 || !colmajor_nn(st, n)) return 0;
  return (((size_t)k * (size_t)n * val_size) + 255) & ~(size_t)255;
}

template <typename T>
static int csrmm_impl(hipStream_t s, int m, int n, int k, int nnz, T alpha, const T* val,
                      const int* rp, const int* ci, int base, const T* B, T beta, T* C,
                      const asamd_dense_strides* st, void* ws, size_t ws_bytes) {
  if (!val || !rp || !ci || !B || !C || !st || m <= 0 || n <= 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)B | (uintptr_t)C) % alignof(T)) return hipErrorInvalidValue;
  if (n > 1 && st->c_row_stride == 1 && st->c_col_stride != 1) {
    // column-major C: rows of op(B) must be contiguous for the wave-wide loads
    const T* Bt = nullptr;
    int64_t ldbt = 0;
    if (st->b_col_stride == 1) {  // op(B) = B^T of a column-major n x k array: already row-major k x n
      Bt = B;
      ldbt = st->b_row_stride;
    } else if (colmajor_nn(st, n) && ws && k > 0 && ws_bytes >= workspace_bytes(sizeof(T), n, k, st)) {
      const dim3 tgrid((unsigned)(((int64_t)k + kWave - 1) / kWave), (unsigned)((n + kWave - 1) / kWave));
      dense_transpose_kernel<T><<<tgrid, kSpmmBlock, 0, s>>>(k, n, B, st->b_col_stride, (T*)ws, (int64_t)n);
      Bt = (const T*)ws;
      ldbt = n;
    }
    if (Bt && n <= 16 && (n <= 8 || n % 4 == 0)) {
      // few dense columns: the entry-parallel kernel on the row-major B, C written through its strides
      launch_short_n<T>(s, m, n, nnz, alpha, val, rp, ci, base, Bt, ldbt, beta, C, 1, st->c_col_stride);
      return hipGetLastError();
    }
    if (Bt) {
      const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), (unsigned)((n + kWave - 1) / kWave));
      spmm_colmajor_kernel<T><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, Bt, ldbt, beta, C,
                                                          st->c_col_stride);
      return hipGetLastError();
    }
  }
  // a single dense column has unit stride along its one column whatever the layout says
  const bool unit_cols = (st->b_col_stride == 1 && st->c_col_stride == 1) || n == 1;
  if (unit_cols) {
    const int64_t ldb = st->b_row_stride, ldc = st->c_row_stride;
    if (n <= 16) {  // a wave per row would leave 64 - n lanes idle (0.93 ms whatever n is on the matrix below)
      // 9..16 columns that are not whole groups of four: a lane per column loads less padding
      if (n > 8 && n % 4 != 0) launch_group<T, 16, 1>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc);
      else launch_short_n<T>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, ldc, 1);
      return hipGetLastError();
    }
    if (n <= 32 && (uintptr_t)B % (2 * sizeof(T)) == 0 && ldb % 2 == 0) {
      // 17..32 columns in rows of B that pairs of elements can be loaded from: 16 lanes x 2 columns per row,
      // four rows of B per wave-wide load (n = 32: 0.95 ms with a wave per row -> 0.68 ms, n = 24: 1.00 -> 0.90).
      // Odd row strides were slower this way (n = 31: 1.23 ms against 1.13 ms), and wider groups or vectors
      // were no faster than a wave per row above 32 columns.
      launch_group<T, 16, 2>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc);
      return hipGetLastError();
    }
    const unsigned gx = (unsigned)(((int64_t)m + kSpmmWaves - 1) / kSpmmWaves);
    {
      // rows of B and C that 128-bit loads can address: four rows of B per wave instruction
      constexpr int E = 16 / (int)sizeof(T);
      static const bool quad_off = getenv("ALSPARSE_AMD_SPMM_QUAD") && atoi(getenv("ALSPARSE_AMD_SPMM_QUAD")) == 0;
      // Measured on 2^20 rows x 32 entries with random columns, n = 64, against one wave-wide load per row of B: B of
      // 4 / 16 / 32 MiB 0.64 / 0.95 / 1.10 ms against 0.97 / 1.05 / 1.11; 64-256 MiB 1.18-1.23 against 1.17-1.22 (the
      // L2-miss path is the limit either way); 512 MiB 1.22 against 1.38; n = 256 (1 GiB) 4.95 against 5.46.  Where
      // neighbouring rows of A share their columns the four-row form wins at any footprint (see above).
      const size_t b_bytes = (size_t)(k > 0 ? k : 0) * (size_t)n * sizeof(T);
      const bool eligible = !quad_off && n % E == 0 && ldb % E == 0 && ldc % E == 0 && (uintptr_t)B % 16 == 0 &&
                            (uintptr_t)C % 16 == 0;
      const bool quad_pays = eligible && (k <= 0 || b_bytes <= ((size_t)48 << 20) || b_bytes > ((size_t)384 << 20) ||
                                          rows_share_columns(s, m, nnz, rp, ci, base));
      if (quad_pays) {
        const dim3 grid(gx, (unsigned)((n + 16 * E - 1) / (16 * E)));
        spmm_rowmajor_quad_kernel<T><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc);
        return hipGetLastError();
      }
    }
    // widest per-lane vector that still gives every lane of a wave work
    constexpr int kMaxV = 32 / (int)sizeof(T) >= 4 ? 4 : 32 / (int)sizeof(T);  // at most 32 bytes per lane and load
    int V = 1;
    if (n >= 4 * kWave && kMaxV >= 4) V = 4;
    else if (n >= 2 * kWave && kMaxV >= 2) V = 2;
    // A B too large for the 256 MiB memory-side cache is better taken 64 dense columns at a time
    // (grid.y runs slowest, so one slice of B is live at a time and stays cached): measured on a
    // 2^20 x 2^20 matrix with 32 entries per row, n = 128: 3.10 ms with V = 2, against 2 x 1.23 ms.
    if (k > 0 && (size_t)k * (size_t)n * sizeof(T) > ((size_t)192 << 20)) V = 1;
    const size_t vbytes = (size_t)V * sizeof(T);
    const bool vector_ok = V > 1 && ((uintptr_t)B % vbytes == 0) && ((uintptr_t)C % vbytes == 0) &&
                           (ldb % V == 0) && (ldc % V == 0);
    const unsigned gy = (unsigned)((n + kWave * V - 1) / (kWave * V));
    const dim3 grid(gx, gy);
    if constexpr (kMaxV >= 4) {
      if (V == 4) {
        spmm_rowmajor_kernel<T, 4><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                               beta, C, ldc, vector_ok);
        return hipGetLastError();
      }
    }
    if (V == 2)
      spmm_rowmajor_kernel<T, 2><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                             beta, C, ldc, vector_ok);
    else
      spmm_rowmajor_kernel<T, 1><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                             beta, C, ldc, false);
  } else {
    const dim3 block(kWave, kSpmmBlock / kWave);
    unsigned gy = (unsigned)((n + block.y - 1) / block.y);
    if (gy > 65535u) gy = 65535u;
    const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), gy);
    spmm_strided_kernel<T><<<grid, block, 0, s>>>(m, n, alpha, val, rp, ci, base, B,
                                                  st->b_row_stride, st->b_col_stride, beta, C,
                                                  st->c_row_stride, st->c_col_stride);
  }
  return hipGetLastError();
}

extern "C" int asamd_s_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                             float alpha, const float* val, const int32_t* row_ptr,
                             const int32_t* col_ind, int32_t base, const float* B, float beta,
                             float* C, const asamd_dense_strides* strides) {
  return csrmm_impl<float>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C,
                           strides, nullptr, 0);
}

extern "C" size_t asamd_csrmm_workspace_bytes(int32_t val_size, int32_t m, int32_t n, int32_t k,
                                              const asamd_dense_strides* strides) {
  (void)m;
  return (val_size == 4 || val_size == 8 || val_size == 16) ? workspace_bytes((size_t)val_size, n, k, strides) : 0;
}

extern "C" int asamd_s_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, float alpha,
                                const float* val, const int32_t* row_ptr, const int32_t* col_ind, int32_t base,
                                const float* B, float beta, float* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  return csrmm_impl<float>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C, strides,
                           workspace, workspace_bytes);
}

extern "C" int asamd_d_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, double alpha,
                                const double* val, const int32_t* row_ptr, const int32_t* col_ind, int32_t base,
                                const double* B, double beta, double* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  return csrmm_impl<double>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C, strides,
                            workspace, workspace_bytes);
}

extern "C" int asamd_d_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                             double alpha, const double* val, const int32_t* row_ptr,
                             const int32_t* col_ind, int32_t base, const double* B, double beta,
                             double* C, const asamd_dense_strides* strides) {
  return csrmm_impl<double>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C,
                            strides, nullptr, 0);
}

// ---- the unanalysed, one-lane-per-element path ("plain"): entries of a row in storage order ---
template <typename T>
static int csrmm_plain_impl(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci,
                            int base, const T* B, T beta, T* C, const asamd_dense_strides* st) {
  if (!val || !rp || !ci || !B || !C || !st || m <= 0 || n <= 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)B | (uintptr_t)C) % alignof(T)) return hipErrorInvalidValue;
  const dim3 block(kWave, kSpmmBlock / kWave);
  unsigned gy = (unsigned)((n + block.y - 1) / block.y);
  if (gy > 65535u) gy = 65535u;
  const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), gy);
  spmm_strided_kernel<T><<<grid, block, 0, s>>>(m, n, alpha, val, rp, ci, base, B, st->b_row_stride,
                                                st->b_col_stride, beta, C, st->c_row_stride, st->c_col_stride);
  return hipGetLastError();
}

extern "C" int asamd_s_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, float alpha, const float* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, int32_t base, const float* B,
                                   float beta, float* C, const asamd_dense_strides* strides) {
  return csrmm_plain_impl<float>(stream, m, n, alpha, val, row_ptr, col_ind, base, B, beta, C, strides);
}

extern "C" int asamd_d_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, double alpha, const double* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, int32_t base, const double* B,
                                   double beta, double* C, const asamd_dense_strides* strides) {
  return csrmm_plain_impl<double>(stream, m, n, alpha, val, row_ptr, col_ind, base, B, beta, C, strides);
}

extern "C" int asamd_c_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex8 alpha,
                                   const asamd_complex8* val, const int32_t* row_ptr, const int32_t* col_ind,
                                   int32_t base, const asamd_complex8* B, asamd_complex8 beta, asamd_complex8* C,
                                   const asamd_dense_strides* strides) {
  using T = Cx<float>;
  return csrmm_plain_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                             (const T*)B, T(beta.real, beta.imag), (T*)C, strides);
}

extern "C" int asamd_z_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex16 alpha,
                                   const asamd_complex16* val, const int32_t* row_ptr, const int32_t* col_ind,
                                   int32_t base, const asamd_complex16* B, asamd_complex16 beta, asamd_complex16* C,
                                   const asamd_dense_strides* strides) {
  using T = Cx<double>;
  return csrmm_plain_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                             (const T*)B, T(beta.real, beta.imag), (T*)C, strides);
}

// ---- complex element types: the same kernels over Cx<float> / Cx<double> -------------------
static_assert(sizeof(asamd_complex8) == sizeof(Cx<float>) && sizeof(asamd_complex16) == sizeof(Cx<double>),
              "complex layouts");

extern "C" int asamd_c_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                                asamd_complex8 alpha, const asamd_complex8* val, const int32_t* row_ptr,
                                const int32_t* col_ind, int32_t base, const asamd_complex8* B, asamd_complex8 beta,
                                asamd_complex8* C, const asamd_dense_strides* strides, void* workspace,
                                size_t workspace_bytes) {
  using T = Cx<float>;
  return csrmm_impl<T>(stream, m, n, k, nnz, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                       (const T*)B, T(beta.real, beta.imag), (T*)C, strides, workspace, workspace_bytes);
}

extern "C" int asamd_z_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                                asamd_complex16 alpha, const asamd_complex16* val, const int32_t* row_ptr,
                                const int32_t* col_ind, int32_t base, const asamd_complex16* B,
                                asamd_complex16 beta, asamd_complex16* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  using T = Cx<double>;
  return csrmm_impl<T>(stream, m, n, k, nnz, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                       (const T*)B, T(beta.real, beta.imag), (T*)C, strides, workspace, workspace_bytes);
}
