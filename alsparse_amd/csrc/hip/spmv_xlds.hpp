// CSR SpMV for matrices with so few columns that x fits the LDS of a compute unit (gfx950: 160 KB; wave64).
//
// The row kernels gather x from the caches: x[col] for 64 scattered columns is up to 64 cache-line requests per
// instruction, and with an x of a hundred KB, far larger than the 32 KB L1, nearly every one goes on to the L2 --
// a tall matrix (millions of rows, tens of thousands of columns, sixteen entries per row) then runs at a quarter
// of the memory's speed while its streams would allow three times that.  Here every compute unit holds ONE
// workgroup of 1 024 threads that copies x into LDS once and then walks its share of the rows, W lanes per row,
// gathering from LDS; the CSR arrays are read in place, so nothing is kept between calls and a caller's new values
// are seen by the next multiply.  The reference's kernel (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57)
// has the same row-to-lanes mapping and gathers from global memory.
//
// A lane group takes kXldsRows rows per trip (rows r, r + groups, r + 2 groups, ...: the groups of a wave sit on
// adjacent rows, whose entries are adjacent in memory), all their first loads in flight together: with one
// workgroup per compute unit the loads in flight per lane are what hides the memory's latency.  Rows of more
// than kXldsWaveRow * W entries are left to the whole wave, one after the other, 64 lanes and four entries per
// lane and trip.  Every row's sum is formed in an order that depends on W and the row alone.
//
// Measured (4 194 304 rows x 16 entries, fp32): this kernel, one entry per lane and load, 0.19 ms whatever the
// number of columns; the form below with four entries per lane and load 0.127 ms; the row kernels 0.105 / 0.125 /
// 0.20 / 0.25 / 0.29 ms with 4 / 16 / 32 / 64 / 128 KB of x.  What this one waits for is the memory pipeline (three
// quarters of the L1s' busy cycles are stalls on pending lines) -- two workgroups per compute unit where x leaves
// room changed nothing, nor did twelve rows per group and trip; fewer, wider requests did.  Two forms that stream
// the matrix 16 bytes per lane through a staging area in LDS (a workgroup's, with two barriers per trip; a wave's
// own, without) measured 0.25 and 0.21 ms and were dropped.  This form stays for complex values and for rows of
// fewer than four entries on average.
#pragma once
#include "device_utils.hpp"

namespace asamd {

constexpr int kXldsThreads = 1024;
constexpr int kXldsRows = 8;      // rows per lane group and trip
constexpr int kXldsWaveRow = 8;   // rows of more than this many entries per lane go to the wave

// NT: the first entries of the rows are loaded non-temporally (rows of at most W entries on average: every line
// of the streams is then wanted once; with longer rows the lines that the tails share with the next rows' heads
// would be fetched twice -- 33 entries per row: 0.34 against 0.26 ms).
template <typename T, int W, bool NT>
__global__ __launch_bounds__(kXldsThreads) void spmv_xlds_kernel(int m, int n, T alpha, const T* __restrict__ val,
                                                                 const int* __restrict__ row_ptr,
                                                                 const int* __restrict__ col_ind,
                                                                 const T* __restrict__ x, T beta, T* __restrict__ y,
                                                                 int base) {
  extern __shared__ __align__(16) unsigned char xlds_bytes[];
  T* __restrict__ xs = reinterpret_cast<T*>(xlds_bytes);
  constexpr int kGroups = kXldsThreads / W;
  constexpr int K = kXldsRows;
  const int lane = threadIdx.x % W;
  const int group = threadIdx.x / W;
  const int wave_lane = threadIdx.x % kWave;
  const int64_t stride = (int64_t)gridDim.x * (kGroups * K);
  int64_t row0 = (int64_t)blockIdx.x * (kGroups * K);
  // the offsets of a trip's rows are requested one trip ahead (the first ones in front of the copy of x)
  int start[K], end[K];
  auto request_offsets = [&](int64_t first, int* lo, int* hi) __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      // (rows past the last: the offset behind the last row, twice -- an empty row.  No load under a condition:
      // with loads in branches the compiler does not know how many are pending, and waits for all of them
      // wherever it waits for one.)
      const int64_t r = first + (int64_t)k * kGroups + group;
      lo[k] = row_ptr[r < m ? r : m];
      hi[k] = row_ptr[r < m ? r + 1 : m];
    }
  };
  request_offsets(row0, start, end);
  // x into LDS: 16 bytes per lane and load where x allows, a trip's loads all requested before the first is stored
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    typedef Int4 Wide;  // (16 bytes of x, whatever they hold)
    constexpr int kPer = 16 / (int)sizeof(T);
    const int wide_n = n / kPer;
    constexpr int kAhead = 4;
    int i = threadIdx.x;
    for (; i + (kAhead - 1) * kXldsThreads < wide_n; i += kAhead * kXldsThreads) {
      Wide w[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) w[u] = reinterpret_cast<const Wide*>(x)[i + u * kXldsThreads];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) reinterpret_cast<Wide*>(xs)[i + u * kXldsThreads] = w[u];
    }
    for (; i < wide_n; i += kXldsThreads) reinterpret_cast<Wide*>(xs)[i] = reinterpret_cast<const Wide*>(x)[i];
    for (int t = wide_n * kPer + threadIdx.x; t < n; t += kXldsThreads) xs[t] = x[t];
  } else {
    for (int i = threadIdx.x; i < n; i += kXldsThreads) xs[i] = x[i];
  }
  __syncthreads();
  const T* __restrict__ xb = xs - base;  // (indexed with the caller's column numbers)
  for (; row0 < m; row0 += stride) {
    // (a wave's memory operations complete in the order of their issue as far as its wait counter goes: entries
    // requested a trip ahead would be waited for with the first wait of this trip.  The offsets are waited for
    // at the top of the next trip, where nothing else is pending.)
    int next_start[K], next_end[K];
    request_offsets(row0 + stride, next_start, next_end);
    T sum[K];
    // ---- first entry of every lane in all K rows, requested together ----
    int c[K];
    T v[K];
    bool mine[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      start[k] -= base;
      end[k] -= base;
      const bool wave_row = end[k] - start[k] > kXldsWaveRow * W;
      const int j = start[k] + lane;
      mine[k] = j < end[k] && !wave_row;
      // (entry 0 exists: the launcher turns empty matrices away)
      c[k] = NT ? nt_load(col_ind + (mine[k] ? j : 0)) : col_ind[mine[k] ? j : 0];
      v[k] = NT ? nt_load(val + (mine[k] ? j : 0)) : val[mine[k] ? j : 0];
    }
#pragma unroll
    for (int k = 0; k < K; ++k) sum[k] = mine[k] ? v[k] * xb[c[k]] : T(0);
    // ---- the rest of rows longer than W, up to kXldsWaveRow entries per lane ----
#pragma unroll
    for (int k = 0; k < K; ++k) {
      if (end[k] - start[k] > kXldsWaveRow * W) continue;
      for (int j = start[k] + lane + W; j < end[k]; j += W) sum[k] = fma_t(val[j], xb[col_ind[j]], sum[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      sum[k] = group_sum<W>(sum[k]);
      const int64_t r = row0 + (int64_t)k * kGroups + group;
      if (lane == 0 && r < m && end[k] - start[k] <= kXldsWaveRow * W) store_axpby(y, r, alpha, sum[k], beta);
    }
    // ---- long rows: the wave takes them one at a time ----
#pragma unroll
    for (int k = 0; k < K; ++k) {
      unsigned long long todo = __ballot(lane == 0 && end[k] - start[k] > kXldsWaveRow * W);
      while (todo) {
        const int owner = __builtin_ctzll(todo);  // a group's first lane
        todo &= todo - 1;
        const int s = __builtin_amdgcn_readlane(start[k], owner), e = __builtin_amdgcn_readlane(end[k], owner);
        T acc = T(0);
        int j = s + wave_lane;
        for (; j + 3 * kWave < e; j += 4 * kWave) {
          T vv[4];
          int cc[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            vv[u] = val[j + u * kWave];
            cc[u] = col_ind[j + u * kWave];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) acc = fma_t(vv[u], xb[cc[u]], acc);
        }
        for (; j < e; j += kWave) acc = fma_t(val[j], xb[col_ind[j]], acc);
        acc = group_sum<kWave>(acc);
        if (wave_lane == 0) {
          const int64_t r = row0 + (int64_t)k * kGroups + (threadIdx.x / kWave) * (kWave / W) + owner / W;
          store_axpby(y, r, alpha, acc, beta);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      start[k] = next_start[k];
      end[k] = next_end[k];
    }
  }
}

// ---- four consecutive entries per lane and load (real element types) ----------------------------------------
// The same walk with 16 bytes of indices and 16 (32) bytes of values per lane and load: W lanes cover the first 4 W
// entries of a row, and a wave instruction fetches what sixteen of the loads above fetch one by one.  (Global
// loads of 16 bytes need no more than 4-byte alignment on this hardware, so rows may start anywhere.)  A piece
// that would reach past the arrays' end -- the last rows' lanes only -- is read as the arrays' last four entries
// and shifted into place; no load sits under a condition.  limit: entries in the arrays, at least 4.
constexpr int kXlds4Rows = 4;  // rows per lane group and trip

template <typename T>
struct XldsPiece {
  int c[4];
  T v[4];
};
typedef int XldsInt4 __attribute__((ext_vector_type(4), aligned(4)));
template <typename T>
struct XldsVal4 {
  typedef T type __attribute__((ext_vector_type(4), aligned(4)));
};

typedef unsigned short XldsShort4 __attribute__((ext_vector_type(4), aligned(2)));
template <typename C>
struct XldsCol4 {
  typedef XldsInt4 type;
};
template <>
struct XldsCol4<unsigned short> {
  typedef XldsShort4 type;
};

// C: int (the caller's column numbers) or unsigned short (columns counted from their slice's first, in a copy)
template <typename T, bool NT, typename C = int>
__device__ __forceinline__ XldsPiece<T> xlds_load_piece(const T* __restrict__ val, const C* __restrict__ col_ind,
                                                        int64_t j, int64_t limit) {
  // j > limit - 4: the window [limit - 4, limit) instead, its entries moved down by j - (limit - 4)
  const int64_t at = j + 4 <= limit ? j : limit - 4;
  const int shift = (int)(j - at);
  typedef typename XldsVal4<T>::type V4;
  typedef typename XldsCol4<C>::type C4;
  const C4 c = NT ? __builtin_nontemporal_load(reinterpret_cast<const C4*>(col_ind + at))
                  : *reinterpret_cast<const C4*>(col_ind + at);
  const V4 v = NT ? __builtin_nontemporal_load(reinterpret_cast<const V4*>(val + at))
                  : *reinterpret_cast<const V4*>(val + at);
  XldsPiece<T> p;
  if (shift == 0) {  // (all lanes but the matrix' last few)
    p.c[0] = c.x, p.c[1] = c.y, p.c[2] = c.z, p.c[3] = c.w;
    p.v[0] = v.x, p.v[1] = v.y, p.v[2] = v.z, p.v[3] = v.w;
  } else {
    const int cc[4] = {(int)c.x, (int)c.y, (int)c.z, (int)c.w};
    const T vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p.c[i] = cc[0];
      p.v[i] = T(0);
#pragma unroll
      for (int q = 1; q < 4; ++q)
        if (shift + i == q) p.c[i] = cc[q], p.v[i] = vv[q];  // (entries past the arrays' end: never summed)
    }
  }
  return p;
}

//
// Column slices (gridDim.y > 1): for an x of several LDS fills the matrix is cut into slices of slice_cols columns,
// workgroup row blockIdx.y taking slice blockIdx.y.  With ascending columns inside the rows a row's entries of one
// slice are a contiguous piece of the CSR arrays, so all a slice needs is where its piece of every row begins and
// ends: row_lo / row_hi then point at a table of slices + 1 rows of m offsets (offsets_per_slice = m apart; in
// row_ptr's convention, base included), and the kernel writes the slice's sums (alpha = 1, beta = 0) to
// y + blockIdx.y * y_per_slice for a second kernel to add up.  One slice: row_lo = row_ptr, row_hi = row_ptr + 1.
//
// A copy of the entries slice by slice (C = unsigned short): every slice is a CSR matrix of its own in val / col_ind,
// columns counted from the slice's first one; row_lo points at slices * m + 1 offsets into the copy (base 0,
// offsets_per_slice = m, row_hi = row_lo + 1) and the pieces of consecutive rows are consecutive in memory.
template <typename T, int W, bool NT, typename C = int>
__global__ __launch_bounds__(kXldsThreads) void spmv_xlds4_kernel(int m, int n_total, int slice_cols, int64_t limit,
                                                                  T alpha, const T* __restrict__ val,
                                                                  const int* __restrict__ row_lo,
                                                                  const int* __restrict__ row_hi,
                                                                  int64_t offsets_per_slice,
                                                                  const C* __restrict__ col_ind,
                                                                  const T* __restrict__ x, T beta, T* __restrict__ y,
                                                                  int64_t y_per_slice, int base) {
  extern __shared__ __align__(16) unsigned char xlds_bytes[];
  T* __restrict__ xs = reinterpret_cast<T*>(xlds_bytes);
  const int col0 = (int)blockIdx.y * slice_cols;  // the slice's first column
  const int n = n_total - col0 < slice_cols ? n_total - col0 : slice_cols;
  row_lo += (int64_t)blockIdx.y * offsets_per_slice;
  row_hi += (int64_t)blockIdx.y * offsets_per_slice;
  x += col0;
  y += (int64_t)blockIdx.y * y_per_slice;
  constexpr int kGroups = kXldsThreads / W;
  constexpr int K = kXlds4Rows;
  constexpr int kWaveLen = kXldsWaveRow * 4 * W;  // longer rows go to the whole wave
  const int lane = threadIdx.x % W;
  const int group = threadIdx.x / W;
  const int wave_lane = threadIdx.x % kWave;
  const int64_t stride = (int64_t)gridDim.x * (kGroups * K);
  int64_t row0 = (int64_t)blockIdx.x * (kGroups * K);
  int start[K], end[K];
  auto request_offsets = [&](int64_t first, int* lo, int* hi) __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      // (rows past the last: the last row's end, twice -- an empty row)
      const int64_t r = first + (int64_t)k * kGroups + group;
      hi[k] = row_hi[r < m ? r : m - 1];
      lo[k] = row_lo[r < m ? r : m - 1];
      lo[k] = r < m ? lo[k] : hi[k];
    }
  };
  request_offsets(row0, start, end);
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    constexpr int kPer = 16 / (int)sizeof(T);
    const int wide_n = n / kPer;
    constexpr int kAhead = 4;
    int i = threadIdx.x;
    for (; i + (kAhead - 1) * kXldsThreads < wide_n; i += kAhead * kXldsThreads) {
      Int4 w[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) w[u] = reinterpret_cast<const Int4*>(x)[i + u * kXldsThreads];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) reinterpret_cast<Int4*>(xs)[i + u * kXldsThreads] = w[u];
    }
    for (; i < wide_n; i += kXldsThreads) reinterpret_cast<Int4*>(xs)[i] = reinterpret_cast<const Int4*>(x)[i];
    for (int t = wide_n * kPer + threadIdx.x; t < n; t += kXldsThreads) xs[t] = x[t];
  } else {
    for (int i = threadIdx.x; i < n; i += kXldsThreads) xs[i] = x[i];
  }
  __syncthreads();
  const int first_col = sizeof(C) == 2 ? 0 : base + col0;
  const T* __restrict__ xb = xs - first_col;  // (indexed with the column numbers as the arrays hold them)
  // the lane's (up to four) entries from position j of a row that ends at e, times x, added up
  auto piece_sum = [&](const XldsPiece<T>& p, int j, int e, T sum) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool mine = j + i < e;
      const T xv = xb[mine ? p.c[i] : first_col];
      sum = mine ? fma_t(p.v[i], xv, sum) : sum;
    }
    return sum;
  };
  for (; row0 < m; row0 += stride) {
    int next_start[K], next_end[K];
    request_offsets(row0 + stride, next_start, next_end);
    XldsPiece<T> p[K];
    T sum[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      start[k] -= base;
      end[k] -= base;
      const int j = start[k] + 4 * lane;
      // (a lane with nothing to do, or a row for the wave: the matrix' first piece, never summed)
      const bool mine = j < end[k] && end[k] - start[k] <= kWaveLen;
      p[k] = xlds_load_piece<T, NT, C>(val, col_ind, mine ? (int64_t)j : 0, limit);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const bool group_row = end[k] - start[k] <= kWaveLen;
      sum[k] = piece_sum(p[k], start[k] + 4 * lane, group_row ? end[k] : start[k], T(0));
    }
    // ---- the rest of rows longer than 4 W, up to kXldsWaveRow pieces per lane ----
#pragma unroll
    for (int k = 0; k < K; ++k) {
      if (end[k] - start[k] > kWaveLen) continue;
      for (int j = start[k] + 4 * lane + 4 * W; j < end[k]; j += 4 * W)
        sum[k] = piece_sum(xlds_load_piece<T, false, C>(val, col_ind, j, limit), j, end[k], sum[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      sum[k] = group_sum<W>(sum[k]);
      const int64_t r = row0 + (int64_t)k * kGroups + group;
      if (lane == 0 && r < m && end[k] - start[k] <= kWaveLen) store_axpby(y, r, alpha, sum[k], beta);
    }
    // ---- long rows: the wave takes them one at a time ----
#pragma unroll
    for (int k = 0; k < K; ++k) {
      unsigned long long todo = __ballot(lane == 0 && end[k] - start[k] > kWaveLen);
      while (todo) {
        const int owner = __builtin_ctzll(todo);  // a group's first lane
        todo &= todo - 1;
        const int s = __builtin_amdgcn_readlane(start[k], owner), e = __builtin_amdgcn_readlane(end[k], owner);
        T acc = T(0);
        for (int j = s + 4 * wave_lane; j < e; j += 4 * kWave)
          acc = piece_sum(xlds_load_piece<T, false, C>(val, col_ind, j, limit), j, e, acc);
        acc = group_sum<kWave>(acc);
        if (wave_lane == 0) {
          const int64_t r = row0 + (int64_t)k * kGroups + (threadIdx.x / kWave) * (kWave / W) + owner / W;
          store_axpby(y, r, alpha, acc, beta);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      start[k] = next_start[k];
      end[k] = next_end[k];
    }
  }
}

// ---- the transposed product with y in LDS ---------------------------------------------------------------------
// y = alpha * op(A)^T x + beta * y for a matrix of few columns, without a copy of the transpose: the rows are walked as
// above (W lanes per row, eight rows per lane group and trip in flight), every entry adds a * x[row] to its column's
// sum in the workgroup's LDS (LDS atomics: the order of the additions inside a workgroup is not fixed), and the
// workgroup writes its n sums to partials + blockIdx.x * n; trans_partials_sum_kernel adds the workgroups' sums in
// order.  The scatter with global atomics (spmv_trans.hpp) takes 3.1 ms on 4 194 304 x 32 768 x 16, fp32: every one
// of its 67 M atomics travels to memory.
template <typename T, int W, bool CONJ>
__global__ __launch_bounds__(kXldsThreads) void spmv_trans_ylds_kernel(int m, int n, T alpha, const T* __restrict__ val,
                                                                       const int* __restrict__ row_ptr,
                                                                       const int* __restrict__ col_ind,
                                                                       const T* __restrict__ x, T* __restrict__ partials,
                                                                       int base) {
  extern __shared__ __align__(16) unsigned char xlds_bytes[];
  T* __restrict__ ys = reinterpret_cast<T*>(xlds_bytes);
  constexpr int kGroups = kXldsThreads / W;
  constexpr int K = kXldsRows;
  const int lane = threadIdx.x % W;
  const int group = threadIdx.x / W;
  const int64_t stride = (int64_t)gridDim.x * (kGroups * K);
  int64_t row0 = (int64_t)blockIdx.x * (kGroups * K);
  int start[K], end[K];
  auto request_offsets = [&](int64_t first, int* lo, int* hi) __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int64_t r = first + (int64_t)k * kGroups + group;
      lo[k] = row_ptr[r < m ? r : m];
      hi[k] = row_ptr[r < m ? r + 1 : m];
    }
  };
  request_offsets(row0, start, end);
  for (int i = threadIdx.x; i < n; i += kXldsThreads) ys[i] = T(0);
  __syncthreads();
  for (; row0 < m; row0 += stride) {
    int next_start[K], next_end[K];
    request_offsets(row0 + stride, next_start, next_end);
    int c[K];
    T v[K], t[K];
    bool mine[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int64_t r = row0 + (int64_t)k * kGroups + group;
      start[k] -= base;
      end[k] -= base;
      const int j = start[k] + lane;
      mine[k] = j < end[k];
      c[k] = nt_load(col_ind + (mine[k] ? j : 0));  // (entry 0 exists: the launcher turns empty matrices away)
      v[k] = nt_load(val + (mine[k] ? j : 0));
      t[k] = x[r < m ? r : 0];
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      t[k] = alpha * t[k];
      const int col = c[k] - base;
      if (mine[k] && (unsigned)col < (unsigned)n) atomic_add(&ys[col], (CONJ ? conj_t(v[k]) : v[k]) * t[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      for (int j = start[k] + lane + W; j < end[k]; j += W) {
        const int col = col_ind[j] - base;
        if ((unsigned)col < (unsigned)n) atomic_add(&ys[col], (CONJ ? conj_t(val[j]) : val[j]) * t[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      start[k] = next_start[k];
      end[k] = next_end[k];
    }
  }
  __syncthreads();
  T* __restrict__ out = partials + (int64_t)blockIdx.x * n;
  for (int i = threadIdx.x; i < n; i += kXldsThreads) out[i] = ys[i];
}
// y = beta * y + (the workgroups' sums, added in the order of the workgroups)
template <typename T>
__global__ __launch_bounds__(256) void trans_partials_sum_kernel(int n, int groups, const T* __restrict__ partials, T beta,
                                                                 T* __restrict__ y) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  T sum = partials[i];
  for (int g = 1; g < groups; ++g) sum += partials[(int64_t)g * n + i];
  y[i] = beta == T(0) ? sum : y[i] * beta + sum;
}

// ---- column slices: the table of offsets, and the sum of the slices' results ------------------------------------
// seg[s * m + r], s = 0 .. slices: where row r's entries of slice s begin (in row_ptr's convention, base included);
// needs ascending columns inside every row
static __global__ __launch_bounds__(256) void xlds_slice_offsets_kernel(int m, int slices, int slice_cols,
                                                                        const int* __restrict__ row_ptr,
                                                                        const int* __restrict__ col_ind, int base,
                                                                        int* __restrict__ seg) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= ((int64_t)slices + 1) * m) return;
  const int s = (int)(i / m), r = (int)(i % m);
  int lo = row_ptr[r] - base, hi = row_ptr[r + 1] - base;
  if (s == slices) lo = hi;
  if (s > 0 && s < slices) {
    const int64_t target = (int64_t)base + (int64_t)s * slice_cols;  // the slice's first column
    while (lo < hi) {
      const int mid = lo + (hi - lo) / 2;
      if ((int64_t)col_ind[mid] < target) lo = mid + 1;
      else hi = mid;
    }
  }
  seg[i] = lo + base;
}
// The same table from one walk over every row (a wave per row): entry k begins the slices behind its predecessor's
// up to its own, the row's first entry those up to its own, the row's end those behind its last entry.  One pass over
// col_ind instead of a binary search per row and slice (32 slices x 1 M rows: 2.5 ms of searches).
static __global__ __launch_bounds__(256) void xlds_slice_offsets_walk_kernel(int m, int slices, int slice_cols,
                                                                             const int* __restrict__ row_ptr,
                                                                             const int* __restrict__ col_ind, int base,
                                                                             int* __restrict__ seg) {
  const int64_t r = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (r >= m) return;
  const int lane = threadIdx.x % kWave;
  const int lo = row_ptr[r] - base, hi = row_ptr[r + 1] - base;
  // (column numbers outside the matrix land in the first or the last slice: nothing is written outside the table)
  auto slice_of = [&](int k) {
    const int s = (col_ind[k] - base) / slice_cols;
    return s < 0 ? 0 : (s >= slices ? slices - 1 : s);
  };
  for (int k = lo + lane; k < hi; k += kWave) {
    const int s = slice_of(k), before = k == lo ? -1 : slice_of(k - 1);
    for (int t = before + 1; t <= s; ++t) seg[(int64_t)t * m + r] = k + base;
  }
  if (lane == 0) {
    const int last = hi > lo ? slice_of(hi - 1) : -1;
    for (int t = last + 1; t <= slices; ++t) seg[(int64_t)t * m + r] = hi + base;
  }
}
// *unsorted |= 1 if the columns of some row do not ascend; a wave per row
static __global__ __launch_bounds__(256) void xlds_rows_ascend_kernel(int m, const int* __restrict__ row_ptr,
                                                                      const int* __restrict__ col_ind, int base,
                                                                      int* __restrict__ unsorted) {
  const int64_t r = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (r >= m) return;
  const int end = row_ptr[r + 1] - base;
  bool bad = false;
  for (int j = row_ptr[r] - base + (int)(threadIdx.x % kWave); j + 1 < end; j += kWave) bad |= col_ind[j] > col_ind[j + 1];
  if (__ballot(bad) != 0 && threadIdx.x % kWave == 0) atomicOr(unsorted, 1);
}
// The entries slice by slice: piece i = s * m + r (slice s of row r) goes from [seg[i], seg[i + m]) of the caller's
// arrays to off[i] .. of the copy, eight lanes per piece; col_ind == nullptr: the values only.  gate: nullptr, or a
// word that is 0 when there is nothing to do.
template <typename T>
__global__ __launch_bounds__(256) void xlds_copy_pieces_kernel(int64_t pieces, int m, int slice_cols, int base,
                                                               const int* __restrict__ seg, const int* __restrict__ off,
                                                               const T* __restrict__ val, const int* __restrict__ col_ind,
                                                               T* __restrict__ cval, unsigned short* __restrict__ ccol,
                                                               const int* __restrict__ gate) {
  if (gate && *gate == 0) return;
  constexpr int kLanes = 8;
  const int lane = threadIdx.x % kLanes;
  for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) / kLanes; i < pieces; i += (int64_t)gridDim.x * (256 / kLanes)) {
    const int from = seg[i] - base, len = seg[i + m] - base - from, to = off[i];
    const int first_col = base + (int)(i / m) * slice_cols;
    for (int k = lane; k < len; k += kLanes) {
      cval[to + k] = val[from + k];
      if (col_ind) ccol[to + k] = (unsigned short)(col_ind[from + k] - first_col);
    }
  }
}
// col16[i] = col_ind[i] - base for i < nnz, 0 for the four elements behind them
static __global__ __launch_bounds__(256) void narrow_columns_kernel(int64_t nnz, int base, const int* __restrict__ col_ind,
                                                                    unsigned short* __restrict__ col16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nnz + 4; i += (int64_t)gridDim.x * 256)
    col16[i] = i < nnz ? (unsigned short)(col_ind[i] - base) : (unsigned short)0;
}
// y = alpha * (the slices' sums, added in the order of the slices) + beta * y
template <typename T>
__global__ __launch_bounds__(256) void xlds_slices_sum_kernel(int m, int slices, T alpha, const T* __restrict__ part,
                                                              T beta, T* __restrict__ y) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= m) return;
  T sum = part[r];
  for (int s = 1; s < slices; ++s) sum += part[(int64_t)s * m + r];
  store_axpby(y, r, alpha, sum, beta);
}

}  // namespace asamd
