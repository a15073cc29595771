// Merge-path CSR SpMV for gfx950 (wave64).
//
// The work list is the merge of the m row-end offsets with the nnz entry
// indices (m + nnz items).  Every workgroup owns 256*IPT consecutive items
// of that list, every thread IPT consecutive items of its workgroup's
// share, so the load is balanced whatever the row-length distribution is: a
// 200 000-entry row simply spans ~100 workgroups, a run of empty rows costs
// one item each.
//
//   1. merge_partition_kernel   one binary search per workgroup boundary over
//                               row_ptr: first row not finished before the
//                               boundary (cached by the analysis when the
//                               structure is promised fixed).
//   2. spmv_merge_kernel        coalesced col/val streaming, x gathers,
//                               products and row ends staged in LDS; each
//                               thread walks its items, sums of finished rows go
//                               to an LDS row buffer; the unfinished tail of
//                               each thread is combined by a segmented scan
//                               (wave shuffles, then across the four waves in
//                               order) and completes the first row the next
//                               thread finishes; rows finished inside the
//                               workgroup are written unit stride as y = beta*y
//                               + alpha*sum.  The workgroup's first row may have
//                               begun in earlier workgroups: its partial sum
//                               goes to a head slot, the unfinished tail of the
//                               workgroup to a carry slot.
//   3. merge_fixup_kernel       one thread per workgroup that finished a row:
//                               sums the carries of the workgroups its first row
//                               crossed, in workgroup order, adds the head slot
//                               and writes that row's y once.
//
// No floating-point atomics anywhere: results are identical from run to run.
// The reference has no counterpart (its CSR-adaptive row blocks,
// src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267, are never read by
// a kernel); the arithmetic per entry is that of
// src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-54.
#pragma once

#include "device_utils.hpp"

namespace asamd {

constexpr int kMergeThreads = 256;
constexpr int kMergeWaves = kMergeThreads / kWave;

// LDS index with one pad word per 32 so that lanes reading at a stride of
// IPT words fall into distinct banks.
__device__ __forceinline__ int lds_pad(int i) { return i + (i >> 5); }

// block_row[b] = number of rows whose end offset is consumed before merge
// diagonal b*items_per_block, for b in [0, nblocks].
static __global__ __launch_bounds__(256) void merge_partition_kernel(int m, int nnz,
                                                              const int* __restrict__ row_ptr,
                                                              int base, int nblocks,
                                                              int items_per_block,
                                                              int* __restrict__ block_row) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b > nblocks) return;
  const int64_t total = (int64_t)m + nnz;
  int64_t d = (int64_t)b * items_per_block;
  if (d > total) d = total;
  int64_t lo = d > nnz ? d - nnz : 0;
  int64_t hi = d < m ? d : m;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    // row `mid` is finished before the diagonal iff its end offset does not
    // exceed the number of entries consumed alongside mid+1 rows
    if ((int64_t)row_ptr[mid + 1] - base <= d - mid - 1) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  block_row[b] = (int)lo;
}

// IPT items per thread, kMergeThreads * IPT items per workgroup.  WIDE: val and col_ind are 16-byte aligned
// and the workgroup's entries are read as pieces of four from the multiple of four at or before its first
// entry (a quarter of the memory instructions); a workgroup whose last piece would reach past the end of
// the arrays reads entry by entry.
template <typename T, int IPT, bool WIDE = false>
__global__ __launch_bounds__(kMergeThreads) void spmv_merge_kernel(
    int m, int nnz, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, const T* __restrict__ x, T beta, T* __restrict__ y, int base,
    const int* __restrict__ block_row, int* __restrict__ carry_row, T* __restrict__ carry_val,
    T* __restrict__ head_val, int policy = kStreamNtValues | kStreamNtIndices) {
  constexpr int kItems = kMergeThreads * IPT;
  __shared__ int s_rend[kItems + 1];  // row ends, local to this workgroup's entry range
  __shared__ T s_prod[kItems + kItems / 32 + 1];
  __shared__ T s_rsum[kItems];           // totals of rows finished here, for unit-stride writes of y
  __shared__ int s_crow[kMergeThreads];  // per-thread unfinished row
  __shared__ T s_cval[kMergeThreads];    // ... and its scanned partial sum
  __shared__ int s_wrow[kMergeWaves];
  __shared__ T s_wval[kMergeWaves];

  const int tid = threadIdx.x;
  // neighbouring workgroups gather neighbouring x: keep them on one XCD's L2
  const unsigned b = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t total = (int64_t)m + nnz;
  const int64_t d0 = (int64_t)b * kItems;
  const int64_t d1 = d0 + kItems < total ? d0 + kItems : total;
  const int row_b = block_row[b];
  const int row_e = block_row[b + 1];
  const int64_t nnz_b = d0 - row_b;
  const int64_t nnz_e = d1 - row_e;
  int rows_cnt = row_e - row_b;
  int nnz_cnt = (int)(nnz_e - nnz_b);
  // coordinates that do not describe this row_ptr (a stale cache) must not
  // drive any access out of bounds: clamp to what the LDS arrays and the
  // global arrays hold, results are then wrong but the launch is safe
  if (rows_cnt < 0 || rows_cnt > kItems || row_b < 0 || row_e > m) rows_cnt = 0;
  if (nnz_cnt < 0 || nnz_cnt > kItems || nnz_b < 0 || nnz_e > nnz) nnz_cnt = 0;
  const int items = rows_cnt + nnz_cnt;

  // ---- stage row ends (one extra: the row still open at the end) ----------
  for (int i = tid; i <= rows_cnt; i += kMergeThreads) {
    const int64_t r = (int64_t)row_b + i;
    const int64_t e = r < m ? (int64_t)row_ptr[r + 1] - base - nnz_b : (int64_t)kItems + 1;
    s_rend[i] = e > kItems ? kItems + 1 : (e < 0 ? 0 : (int)e);
  }
  // ---- stream entries, gather x, stage products ----------------------------
  const int64_t win0 = nnz_b & ~(int64_t)3;  // the window of whole pieces around the workgroup's entries
  const int head = (int)(nnz_b - win0);
  const int span = (nnz_cnt + head + 3) & ~3;
  if (WIDE && IPT % 4 == 0 && nnz_cnt > 0 && win0 + span <= nnz) {  // workgroup-uniform
    // Every load is issued unconditionally (a thread past the end of the window re-reads its first piece), and
    // so is every gather: the entries in front of and behind the workgroup's own are entries of the matrix too.
    const T* __restrict__ xb = x - base;
    constexpr int kPieces = IPT / 4;
    Quad<T> v[kPieces];
    Int4 c[kPieces];
#pragma unroll
    for (int s = 0; s < kPieces; ++s) {
      const int k = 4 * (tid + s * kMergeThreads);
      const int64_t kk = win0 + (k < span ? k : 0);
      if (policy & kStreamNtValues) v[s].load_nt(val + kk);
      else v[s].load(val + kk);
      if (policy & kStreamNtIndices) c[s] = nt_load_object(reinterpret_cast<const Int4*>(col_ind + kk));
      else c[s] = *reinterpret_cast<const Int4*>(col_ind + kk);
    }
    T xv[kPieces][4];
#pragma unroll
    for (int s = 0; s < kPieces; ++s) {
      xv[s][0] = xb[c[s].x];
      xv[s][1] = xb[c[s].y];
      xv[s][2] = xb[c[s].z];
      xv[s][3] = xb[c[s].w];
    }
#pragma unroll
    for (int s = 0; s < kPieces; ++s) {
      const int k = 4 * (tid + s * kMergeThreads) - head;  // the piece's first entry, counted from the workgroup's
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (k + j >= 0 && k + j < nnz_cnt) s_prod[lds_pad(k + j)] = v[s].get(j) * xv[s][j];
    }
    // a workgroup of nothing but entries that starts off a multiple of four has one piece more: thread 0 takes it
    if (tid == 0 && span > kItems) {
      const int k = kItems - head;
      for (int j = 0; j < 4; ++j)
        if (k + j < nnz_cnt) s_prod[lds_pad(k + j)] = nt_load(val + nnz_b + k + j) * xb[nt_load(col_ind + nnz_b + k + j)];
    }
  } else {
    // Every load is issued unconditionally (a thread past the end of the range re-reads the range's
    // first entry): loads under a branch make the compiler wait for ALL outstanding loads before
    // each use, which turned the IPT gathers of a thread into a chain of IPT memory latencies.
    const T* __restrict__ xb = x - base;
    const int64_t safe = nnz_cnt > 0 ? nnz_b : 0;
    T v[IPT];
    int c[IPT];
#pragma unroll
    for (int s = 0; s < IPT; ++s) {
      const int k = tid + s * kMergeThreads;
      const int64_t kk = k < nnz_cnt ? nnz_b + k : safe;
      // the streams are touched once: non-temporal, so that they do not push x out of the caches
      v[s] = nt_load(val + kk);
      c[s] = nt_load(col_ind + kk);
    }
    T xv[IPT];
#pragma unroll
    for (int s = 0; s < IPT; ++s) xv[s] = xb[c[s]];
#pragma unroll
    for (int s = 0; s < IPT; ++s) {
      const int k = tid + s * kMergeThreads;
      if (k < nnz_cnt) s_prod[lds_pad(k)] = v[s] * xv[s];
    }
  }
  __syncthreads();

  // ---- this thread's start on the workgroup-local merge path ---------------
  int dt = tid * IPT;
  if (dt > items) dt = items;
  int dt_end = dt + IPT;
  if (dt_end > items) dt_end = items;
  int lo = dt > nnz_cnt ? dt - nnz_cnt : 0;
  int hi = dt < rows_cnt ? dt : rows_cnt;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_rend[mid] <= dt - mid - 1) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  int i = lo;       // local row
  int j = dt - lo;  // local entry
  const int first_row = i;
  bool finished_any = false;
  T first_sum = T(0);  // this thread's part of the first row it finishes
  T acc = T(0);
#pragma unroll
  for (int step = 0; step < IPT; ++step) {
    if (dt + step < dt_end) {
      const bool take_entry = j < nnz_cnt && (i >= rows_cnt || j < s_rend[i]);
      if (take_entry) {
        acc += s_prod[lds_pad(j)];
        ++j;
      } else if (i < rows_cnt) {
        // exactly one thread finishes a given row.  The first row it finishes
        // may have been begun by the threads below and waits for their tails;
        // any further row lies entirely inside this thread's items.
        if (!finished_any) {
          first_sum = acc;
          finished_any = true;
        } else {
          s_rsum[i] = acc;
        }
        acc = T(0);
        ++i;
      }
    }
  }

  // ---- segmented inclusive scan of the unfinished tails, key = row --------
  // keys are non-decreasing in thread order, so "same key d lanes below"
  // implies every lane in between has that key too
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int key = i;
  T tail = acc;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const T up = lane_up(tail, d);
    const int kup = __shfl_up(key, d, kWave);
    if (lane >= d && kup == key) tail += up;
  }
  if (lane == kWave - 1) {
    s_wrow[wave] = key;
    s_wval[wave] = tail;
  }
  __syncthreads();
  for (int w = wave - 1; w >= 0; --w) {
    if (s_wrow[w] != key) break;
    tail += s_wval[w];
  }
  s_crow[tid] = key;
  s_cval[tid] = tail;
  __syncthreads();

  if (finished_any) {
    // add what the threads below contributed to this thread's first finished row
    if (tid > 0 && s_crow[tid - 1] == first_row) first_sum += s_cval[tid - 1];
    s_rsum[first_row] = first_sum;
  }
  if (tid == kMergeThreads - 1) {
    carry_row[b] = row_b + key;  // == row_e: the row still open, or m
    carry_val[b] = tail;
  }
  __syncthreads();

  // ---- rows finished here: y = beta*y + alpha*sum, unit stride -----------------
  // Local row 0 of every workgroup but the first may have begun in earlier
  // workgroups: the fix-up kernel completes it from head_val and the carries.
  const int first_direct = b > 0 ? 1 : 0;
  if (tid == 0 && b > 0) head_val[b] = rows_cnt > 0 ? s_rsum[0] : T(0);
  for (int r = tid + first_direct; r < rows_cnt; r += kMergeThreads)
    store_axpby(y, (int64_t)row_b + r, alpha, s_rsum[r], beta);
}

// Thread bb completes the first row of workgroup bb (bb >= 1) if that
// workgroup finished it: the row is carry_row[bb-1]; every earlier workgroup
// whose carry names the same row contributed a partial sum.  They are added in
// workgroup order, then the finishing workgroup's own part, then y is written
// once with the same rounding points as everywhere else.
template <typename T>
__global__ __launch_bounds__(256) void merge_fixup_kernel(int nblocks, int m, T alpha, T beta,
                                                          const int* __restrict__ carry_row,
                                                          const T* __restrict__ carry_val,
                                                          const T* __restrict__ head_val,
                                                          T* __restrict__ y) {
  const int bb = blockIdx.x * blockDim.x + threadIdx.x;
  if (bb < 1 || bb >= nblocks) return;
  const int r = carry_row[bb - 1];
  if (r < 0 || r >= m) return;
  if (carry_row[bb] == r) return;  // workgroup bb finished no row
  // the carries name rows in ascending order: the run of blocks that the row crossed starts at the first
  // carry that names it
  int first = bb - 1;
  if (first > 0 && carry_row[first - 1] == r) {
    int lo = 0, hi = first - 1;  // carry_row[hi] == r
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (carry_row[mid] < r) {
        lo = mid + 1;
      } else {
        hi = mid;
      }
    }
    first = lo;
  }
  T s = T(0);
  int k = first;
  for (; k + 4 <= bb; k += 4) {
    const T c0 = carry_val[k], c1 = carry_val[k + 1], c2 = carry_val[k + 2], c3 = carry_val[k + 3];
    s += c0;
    s += c1;
    s += c2;
    s += c3;
  }
  for (; k < bb; ++k) s += carry_val[k];
  s += head_val[bb];
  store_axpby(y, (int64_t)r, alpha, s, beta);
}

}  // namespace asamd
