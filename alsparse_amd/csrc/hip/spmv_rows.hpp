// Row-parallel CSR SpMV kernels for gfx950 (wave64): one lane group per row.
//
//   spmv_vector_kernel<T, W>    W consecutive lanes share a row, W picked from
//                               the mean row length; coalesced col/val streaming,
//                               DPP group reduction.
//   spmv_rowconst_kernel<T, G>  every row has exactly 4*G entries starting at
//                               row*4*G: no row_ptr traffic, one 128-bit load of
//                               values and one of indices per lane.
//   spmv_scalar_kernel<T>       one lane per row (diagnostic baseline).
//   spmv_stream_wide_kernel<T, CAP, G>, spmv_stream_kernel<T, CAP, G>
//                               rows of similar lengths, at most CAP * G entries: a workgroup
//                               stages the products of 256 / G consecutive rows in LDS (their
//                               entries are one contiguous range, read with 128-bit or 4-byte
//                               loads), G lanes per row sum them.
//
// They stand in for the reference's only CSR SpMV kernel, csr_gemv_vector
// (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57): same arithmetic
// (fma accumulation per lane, then y = beta*y + alpha*sum), different mapping.
// beta == 0 never reads y.  All element offsets are formed in 64 bits.
#pragma once
#include "device_utils.hpp"

namespace asamd {

constexpr int kRowsBlock = 256;  // threads per workgroup of the row kernels

// the rows of workgroup `bid`: W lanes per row
template <typename T, int W>
__device__ __forceinline__ void spmv_vector_block(unsigned bid, int m, T alpha, const T* __restrict__ val,
                                                  const int* __restrict__ row_ptr, const int* __restrict__ col_ind,
                                                  const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  constexpr int kRowsPerBlock = kRowsBlock / W;
  const int lane = threadIdx.x % W;
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / W;
  if (row >= m) return;  // whole lane groups leave together
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* __restrict__ xb = x - base;
  T sum = T(0);
  int64_t j = start + lane;
  if constexpr (W >= 64) {
    // four entries per lane and trip: a wave that owns a row of hundreds of entries lives on its loads in flight
    // (8 % on rows of 300 to 1 000 entries; non-temporal loads here: no gain or a loss)
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

template <typename T, int W>
__global__ __launch_bounds__(kRowsBlock) void spmv_vector_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  spmv_vector_block<T, W>(xcd_contiguous_id(blockIdx.x, gridDim.x), m, alpha, val, row_ptr, col_ind, x, beta, y, base);
}

// The stand-in for a kernel that a device-side guard may turn away: launched every time, with a small grid
// whose workgroups walk the row blocks in turn, so that the usual case -- *run_if == 0, nothing to do -- costs
// a few hundred empty workgroups instead of one per row block.
template <typename T, int W>
__global__ __launch_bounds__(kRowsBlock) void spmv_vector_standin_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base,
    unsigned nblocks, const int* __restrict__ run_if) {
  if (*run_if == 0) return;
  for (unsigned b = blockIdx.x; b < nblocks; b += gridDim.x)
    spmv_vector_block<T, W>(b, m, alpha, val, row_ptr, col_ind, x, beta, y, base);
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

// ---- regular rows: LDS-staged row blocks ---------------------------------------
// A workgroup owns kStreamRows / G consecutive rows, none longer than CAP * G
// entries.  Their entries are one contiguous range of the CSR streams: it
// is read fully coalesced (lane k takes entries k, k + 256, ...: every load of
// the workgroup is issued before the first is used), multiplied
// with the gathered x and staged in LDS; after one barrier G lanes sum the
// products of a row from LDS (with G = 1 a lane's run is contiguous and runs of
// neighbouring lanes are adjacent, so the reads spread over the banks), a butterfly
// joins them and the rows' y are written unit stride.  No searches, no scans: this is
// what rows of 3-5 entries (stencils, G = 1) want, and with G = 2 .. 16 rows of some tens of
// entries whose lengths differ too little to need merge-path (a lane group per row straight from
// global memory has three dependent loads per row and few of them in flight).
// Which stream bypasses the caches is the host's choice (the wide form's `policy`, see stream_policy.hpp);
// the 4-byte form loads its indices non-temporally and its values plainly.
constexpr int kStreamRows = 256;
constexpr int kStreamMaxLen = 16;        // longest row of the one-lane-per-row form
constexpr int kStreamMaxGroup = 16;      // most lanes per row

// What a workgroup of the staged kernels does when its rows hold more entries than its staging area: G lanes
// per row, straight from global memory.
template <typename T, int G>
__device__ __forceinline__ void stream_rows_direct(int m, int64_t row, int lane, T alpha, const T* __restrict__ val,
                                                   const int* __restrict__ row_ptr, const int* __restrict__ col_ind,
                                                   const T* __restrict__ xb, T beta, T* __restrict__ y, int base) {
  if (row >= m) return;  // whole lane groups leave together
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T sum = T(0);
  for (int64_t k = (int64_t)row_ptr[row] - base + lane; k < end; k += G) sum = fma_t(val[k], xb[col_ind[k]], sum);
  if constexpr (G > 1) sum = group_sum<G>(sum);
  if (lane == 0) store_axpby(y, row, alpha, sum, beta);
}

// CAP: entries per thread that the LDS staging area is sized for (256 * CAP products), G: lanes per row
template <typename T, int CAP, int G = 1>
__global__ __launch_bounds__(kStreamRows) void spmv_stream_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base) {
  constexpr int kRows = kStreamRows / G;
  __shared__ T s_prod[kStreamRows * CAP];
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row0 = (int64_t)bid * kRows;
  const int lane = threadIdx.x % G;
  const int64_t row = row0 + threadIdx.x / G;
  int64_t row_last = row0 + kRows;
  if (row_last > m) row_last = m;
  const int64_t e0 = (int64_t)row_ptr[row0] - base;
  const int64_t n64 = (int64_t)row_ptr[row_last] - base - e0;  // at most kStreamRows * CAP for the analysed structure
  const int n = n64 > INT32_MAX || n64 < 0 ? -1 : (int)n64;
  int my_begin = 0, my_end = 0;
  if (row < m) {
    my_begin = (int)((int64_t)row_ptr[row] - base - e0);
    my_end = (int)((int64_t)row_ptr[row + 1] - base - e0);
  }
  const T* __restrict__ xb = x - base;
  if (n < 0 || n > kStreamRows * CAP) {
    // The rows do not fit the staging area: row_ptr no longer holds the structure that the launch was sized
    // for.  (Workgroup-uniform.)  The lane groups take their rows straight from the arrays.
    stream_rows_direct<T, G>(m, row, lane, alpha, val, row_ptr, col_ind, xb, beta, y, base);
    return;
  }
  T v[CAP];
  int c[CAP];
#pragma unroll
  for (int s = 0; s < CAP; ++s) {
    const int k = threadIdx.x + s * kStreamRows;
    if (k < n) {
      v[s] = val[e0 + k];
      c[s] = nt_load(col_ind + e0 + k);
    }
  }
#pragma unroll
  for (int s = 0; s < CAP; ++s) {
    const int k = threadIdx.x + s * kStreamRows;
    if (k < n) s_prod[k] = v[s] * xb[c[s]];
  }
  __syncthreads();
  if (row >= m) return;  // whole lane groups leave together
  T sum = T(0);
  for (int k = my_begin + lane; k < my_end; k += G) sum += s_prod[k];
  if constexpr (G > 1) sum = group_sum<G>(sum);
  if (lane == 0) store_axpby(y, row, alpha, sum, beta);
}

// The same with 128-bit loads: the window of the workgroup's entries starts at the multiple of four entries
// at or before its first entry, thread t takes pieces t, t + 256, ... of four consecutive entries (values and
// indices; one more piece than CAP / 4 because of the up to three entries in front), and the entries outside
// the block are dropped.  A quarter of the memory instructions for the same bytes.  val and col_ind must be
// 16-byte aligned; `limit` is the number of entries in the arrays (counted like row_ptr - base): pieces that
// would reach past it -- in the last workgroup only -- are read entry by entry.
//
// REL16: the column numbers come from rel16 instead -- 16-bit signed distances from the workgroup's first row
// (rel16[k] = col_ind[k] - base - row0, nnz + 4 elements, made once by narrow_rel_columns_kernel for a structure that
// stays and a matrix whose entries lie within 32 767 columns of their rows: discretisations, bands), 2 instead of 4
// index bytes per entry.  col_ind is read by the fall-back only.  27-point stencil on 160^3 points: 0.204 -> 0.177 ms
// (fp32), 0.300 -> 0.273 (fp64); a matrix that the memory-side cache nearly holds gains nothing (5-point Laplacian on
// 2048^2, fp64: 0.050 -> 0.051 at best), so the distances are made for matrices well beyond it only.
typedef short StreamShort4 __attribute__((ext_vector_type(4)));
template <typename T, int CAP, int G, bool REL16 = false>
__global__ __launch_bounds__(kStreamRows) void spmv_stream_wide_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base, int64_t limit,
    int policy, const short* __restrict__ rel16 = nullptr) {
  constexpr int kRows = kStreamRows / G;
  constexpr int kPieces = CAP / 4 + 1;
  __shared__ T s_prod[kStreamRows * CAP];
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row0 = (int64_t)bid * kRows;
  const int lane = threadIdx.x % G;
  const int64_t row = row0 + threadIdx.x / G;
  int64_t row_last = row0 + kRows;
  if (row_last > m) row_last = m;
  const int64_t e0 = (int64_t)row_ptr[row0] - base;
  const int64_t n64 = (int64_t)row_ptr[row_last] - base - e0;  // at most kStreamRows * CAP for the analysed structure
  const int n = n64 > INT32_MAX || n64 < 0 ? -1 : (int)n64;
  int my_begin = 0, my_end = 0;
  if (row < m) {
    my_begin = (int)((int64_t)row_ptr[row] - base - e0);
    my_end = (int)((int64_t)row_ptr[row + 1] - base - e0);
  }
  const T* __restrict__ xb = x - base;
  if (n < 0 || n > kStreamRows * CAP) {
    // The rows do not fit the staging area: row_ptr no longer holds the structure that the launch was sized
    // for.  (Workgroup-uniform.)  The lane groups take their rows straight from the arrays.
    stream_rows_direct<T, G>(m, row, lane, alpha, val, row_ptr, col_ind, xb, beta, y, base);
    return;
  }
  if constexpr (REL16) xb = x + row0;  // (indexed with the distances)
  const int64_t a0 = e0 & ~(int64_t)3;
  const int head = (int)(e0 - a0);
  const int span = n + head;  // entries of the window
  Quad<T> v[kPieces];
  Int4 c[kPieces];
  StreamShort4 c16[kPieces];  // (REL16: kept as loaded until the gathers, so that no piece's loads wait for another's)
#pragma unroll
  for (int s = 0; s < kPieces; ++s) {
    const int k = 4 * (threadIdx.x + s * kStreamRows);
    if (k < span) {
      if (a0 + k + 4 <= limit) {
        if (policy & kStreamNtValues) v[s].load_nt(val + a0 + k);
        else v[s].load(val + a0 + k);
        if constexpr (REL16) {
          StreamShort4& d = c16[s];
          const StreamShort4* from = reinterpret_cast<const StreamShort4*>(rel16 + a0 + k);
          if (policy & kStreamNtIndices) {
            // (An address the compiler cannot tell from the other branch's: it would merge the two loads into a plain
            // one, and with one merged load its schedule of the piece's loads is the slower one even where this
            // branch is not taken: 27-point stencil on 160^3 points, fp64, 0.295 against 0.273 ms.)
            asm volatile("" : "+v"(from));
            d = nt_load_object(from);
          } else {
            d = *from;
          }
        } else {
          if (policy & kStreamNtIndices) c[s] = nt_load_object(reinterpret_cast<const Int4*>(col_ind + a0 + k));
          else c[s] = *reinterpret_cast<const Int4*>(col_ind + a0 + k);
        }
      } else {
        // the arrays end inside this piece
        alignas(32) T tv[4] = {T(0), T(0), T(0), T(0)};
        int tc[4] = {REL16 ? 0 : base, REL16 ? 0 : base, REL16 ? 0 : base, REL16 ? 0 : base};
        for (int j = 0; j < 4 && a0 + k + j < limit; ++j) {
          tv[j] = val[a0 + k + j];
          tc[j] = REL16 ? (int)rel16[a0 + k + j] : col_ind[a0 + k + j];
        }
        v[s].load(tv);
        if constexpr (REL16) c16[s] = StreamShort4{(short)tc[0], (short)tc[1], (short)tc[2], (short)tc[3]};
        else c[s] = Int4{tc[0], tc[1], tc[2], tc[3]};
      }
    }
  }
#pragma unroll
  for (int s = 0; s < kPieces; ++s) {
    const int k = 4 * (threadIdx.x + s * kStreamRows) - head;  // position of the piece's first entry in the block
    if (k + head < span) {
      int cc[4];
      if constexpr (REL16) cc[0] = c16[s].x, cc[1] = c16[s].y, cc[2] = c16[s].z, cc[3] = c16[s].w;
      else cc[0] = c[s].x, cc[1] = c[s].y, cc[2] = c[s].z, cc[3] = c[s].w;
      T xv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[j] = (k + j >= 0 && k + j < n) ? xb[cc[j]] : T(0);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (k + j >= 0 && k + j < n) s_prod[k + j] = v[s].get(j) * xv[j];
    }
  }
  __syncthreads();
  if (row >= m) return;  // whole lane groups leave together
  T sum = T(0);
  for (int k = my_begin + lane; k < my_end; k += G) sum += s_prod[k];
  if constexpr (G > 1) sum = group_sum<G>(sum);
  if (lane == 0) store_axpby(y, row, alpha, sum, beta);
}

// rel16[k] = col_ind[k] - base - (first row of the workgroup that takes entry k's row), 0 for the four elements behind
// the last entry; *too_far |= 1 if some distance does not fit 16 bits.  A workgroup per block of rows_per_group rows:
// the block's entries are one contiguous range and share their first row, so the lanes walk the range with unit stride
// (a lane per row read 27 scattered entries each: 1.95 ms for the 110 M entries of the 27-point stencil on 160^3 points).
static __global__ __launch_bounds__(256) void narrow_rel_columns_kernel(int m, int64_t nnz, int base, int rows_per_group,
                                                                        const int* __restrict__ row_ptr,
                                                                        const int* __restrict__ col_ind,
                                                                        short* __restrict__ rel16,
                                                                        int* __restrict__ too_far) {
  if (blockIdx.x == 0 && threadIdx.x < 4) rel16[nnz + threadIdx.x] = 0;
  const int64_t row0 = (int64_t)blockIdx.x * rows_per_group;
  if (row0 >= m) return;
  int64_t row_last = row0 + rows_per_group;
  if (row_last > m) row_last = m;
  int64_t lo = (int64_t)row_ptr[row0] - base, hi = (int64_t)row_ptr[row_last] - base;
  if (lo < 0) lo = 0;      // (offsets that do not describe the arrays: nothing outside them is touched)
  if (hi > nnz) hi = nnz;
  bool far = false;
  for (int64_t k = lo + threadIdx.x; k < hi; k += 256) {
    const int64_t d = (int64_t)col_ind[k] - base - row0;
    far |= d < -32768 || d > 32767;
    rel16[k] = (short)d;
  }
  if (__syncthreads_or(far) && threadIdx.x == 0) atomicOr(too_far, 1);
}

// ---- constant row length ----------------------------------------------------
// G lanes per row, each owning 4 consecutive entries: L = 4*G.  R rows per
// lane group and launch keep 4*R gathers per lane in flight.
template <typename T, int G, int R>
__global__ __launch_bounds__(kRowsBlock) void spmv_rowconst_kernel(
    int m, T alpha, const T* __restrict__ val, const int* __restrict__ col_ind,
    const T* __restrict__ x, T beta, T* __restrict__ y, int base, int policy) {
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
      // policy (kernel-uniform): which stream bypasses the caches, see kStreamNt*
      if (policy & kStreamNtValues) v[r].load_nt(val + off);
      else v[r].load(val + off);
      if (policy & kStreamNtIndices) c[r] = nt_load_object(reinterpret_cast<const Int4*>(col_ind + off));
      else c[r] = *reinterpret_cast<const Int4*>(col_ind + off);
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
