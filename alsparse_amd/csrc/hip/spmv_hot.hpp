// Merge-path CSR SpMV with the x of the most popular columns held in LDS (gfx950, wave64).
//
// For matrices whose entries crowd into few columns (power-law graphs).  A compute unit's vector memory
// path keeps a limited number of cache-line requests in flight, so the rate of x gathers that leave the
// L1 is that number divided by their latency, whatever the bandwidth behind it; LDS gathers do not use
// that path at all, and gathers that hit the L2 wait a third as long as those that miss it.  The analysis
// ranks the columns by their number of entries and rewrites the column stream as one word per entry:
//     p <  h1      : x is hot[p] in LDS, the x of the p-th most popular column
//     p <  hc      : x is x_front[p], a compact array of the hc most popular columns' x that stays in the L2
//     p >= hc      : x is x[p - hc] (zero-based column)
// Before every multiply hot_prepare_kernel gathers the front; one PERSISTENT workgroup per compute unit
// copies the front's first h1 values into LDS and then each of its waves walks merge blocks of 64 * IPT
// items on its own: a wave needs no workgroup barrier, so the waves of a compute unit drift apart and the
// loads of one overlap the merge walk of another.  The values are read from the caller's array: the copy
// that the analysis keeps is structure only.
//
// The merge block is that of spmv_merge.hpp at wave size: products and row ends staged in LDS, every
// lane walks IPT consecutive items, the unfinished tails are combined by a segmented scan across the
// lanes, rows that cross blocks are completed by merge_fixup_kernel in block order; a block that lies
// inside one long row skips all that and adds its products up.  No floating-point atomics: results are
// identical from run to run.  The reference has no counterpart; the arithmetic per entry is that of
// src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-54.
#pragma once

#include "spmv_merge.hpp"

namespace asamd {

template <typename T, int IPT>
struct HotWaveSmem {
  static constexpr int kItems = kWave * IPT;
  T prod[kItems + kItems / 32 + 1];
  T rsum[kItems];                      // totals of rows finished here, for unit-stride writes of y
  unsigned short rend[kItems + 2];     // row ends, local to the block's entry range (at most kItems + 1)
};

template <typename T, int IPT, int NW>
struct HotDims {
  static constexpr int items = kWave * IPT;
  static constexpr int threads = kWave * NW;
  static constexpr int stage_bytes = (int)sizeof(HotWaveSmem<T, IPT>) * NW;
  // what is left of a compute unit's 160 KiB of LDS, in whole KiB of table
  static constexpr int table_bytes = (160 * 1024 - stage_bytes) / 1024 * 1024;
  static constexpr int lds_cols = table_bytes / (int)sizeof(T);
};

// Orders this wave's LDS traffic: the LDS works through a wave's instructions in order, so all that is
// needed is that the compiler keeps them in program order.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

template <typename T>
__global__ __launch_bounds__(256) void hot_prepare_kernel(int hc, const int* __restrict__ hot_cols,
                                                          const T* __restrict__ x, T* __restrict__ x_front) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < hc) x_front[i] = x[hot_cols[i]];
}

// Where a wave-sized merge block lies: items [b * K, (b + 1) * K) of the merge list with K = 64 * IPT.
struct HotCoords {
  int row_b, rows_cnt, nnz_cnt;
  int64_t nnz_b;
};
template <int IPT>
__device__ __forceinline__ HotCoords hot_coords(int b, bool exists, int m, int nnz, const int* __restrict__ block_row) {
  constexpr int kItems = kWave * IPT;
  HotCoords c;
  const int64_t total = (int64_t)m + nnz;
  const int64_t d0 = (int64_t)b * kItems;
  const int64_t d1 = d0 + kItems < total ? d0 + kItems : total;
  c.row_b = exists ? block_row[b] : 0;
  const int row_e = exists ? block_row[b + 1] : 0;
  c.nnz_b = d0 - c.row_b;
  const int64_t nnz_e = d1 - row_e;
  c.rows_cnt = row_e - c.row_b;
  c.nnz_cnt = (int)(nnz_e - c.nnz_b);
  // coordinates that do not describe this row_ptr must not drive any access out of bounds
  if (!exists || c.rows_cnt < 0 || c.rows_cnt > kItems || c.row_b < 0 || row_e > m) c.rows_cnt = 0;
  if (!exists || c.nnz_cnt < 0 || c.nnz_cnt > kItems || c.nnz_b < 0 || nnz_e > nnz) c.nnz_cnt = 0;
  if (c.nnz_cnt == 0) c.nnz_b = 0;
  return c;
}
// Which of the block's entries a lane holds in slot s of its registers.  Four-byte values: four consecutive
// entries per 128-bit load (slots 4q .. 4q+3 = entries 256q + 4 lane ..); else one entry per load, a wave's
// lanes side by side.
template <typename T, int IPT>
struct HotSlots {
  static constexpr bool wide = sizeof(T) == 4 && IPT % 4 == 0;
  static __device__ __forceinline__ int entry(int lane, int s) {
    return wide ? (s / 4) * (4 * kWave) + lane * 4 + s % 4 : lane + s * kWave;
  }
};
// The block's share of the value and position streams: every load is issued unconditionally: the compiler
// can only count outstanding loads that are certain to be issued.  Wide: through buffer resources that end
// with the block's entries, so the words past the end read as zero and ask memory for nothing (position 0 is
// a hot column: harmless); narrow: a lane past the end re-reads the range's first entry, a block that does
// not exist entry 0.
template <typename T, int IPT>
__device__ __forceinline__ void hot_load_streams(const HotCoords& c, int lane, const T* __restrict__ val,
                                                 const unsigned* __restrict__ pcol, T (&v)[IPT], unsigned (&p)[IPT]) {
  if constexpr (HotSlots<T, IPT>::wide) {
    const BufferRsrc rv = make_rsrc(val + c.nnz_b, c.nnz_cnt * (int)sizeof(T));
    const BufferRsrc rp = make_rsrc(pcol + c.nnz_b, c.nnz_cnt * (int)sizeof(unsigned));
#pragma unroll
    for (int q = 0; q < IPT / 4; ++q) {
      const int off = (q * 4 * kWave + lane * 4) * 4;
      const Float4 v4 = buffer_load<Float4, 2>(rv, off);
      const Int4 p4 = buffer_load<Int4, 2>(rp, off);
      v[4 * q + 0] = __builtin_bit_cast(T, v4.x);
      v[4 * q + 1] = __builtin_bit_cast(T, v4.y);
      v[4 * q + 2] = __builtin_bit_cast(T, v4.z);
      v[4 * q + 3] = __builtin_bit_cast(T, v4.w);
      p[4 * q + 0] = (unsigned)p4.x;
      p[4 * q + 1] = (unsigned)p4.y;
      p[4 * q + 2] = (unsigned)p4.z;
      p[4 * q + 3] = (unsigned)p4.w;
    }
  } else {
#pragma unroll
    for (int s = 0; s < IPT; ++s) {
      const int k = lane + s * kWave;
      const int64_t kk = c.nnz_b + (k < c.nnz_cnt ? k : 0);
      v[s] = nt_load(val + kk);
      p[s] = nt_load(pcol + kk);
    }
  }
}

// One merge block worked by one wave.  v and p hold the block's values and positions (loaded a block
// ahead); while this block's gathers are in flight the streams of the wave's next block are requested into
// vn and pn, so that they travel during the merge walk.
template <typename T, int IPT>
__device__ __forceinline__ void hot_wave_block(HotWaveSmem<T, IPT>& sm, const int lane, const int b, const HotCoords& c,
                                               const T (&v)[IPT], const unsigned (&p)[IPT], const HotCoords& cn,
                                               T (&vn)[IPT], unsigned (&pn)[IPT], const T* hot, const unsigned h1,
                                               const unsigned hc, const T* __restrict__ x_front,
                                               const T* __restrict__ x, int m, T alpha,
                                               const T* __restrict__ val, const int* __restrict__ row_ptr,
                                               const unsigned* __restrict__ pcol, T beta, T* __restrict__ y, int base,
                                               int* __restrict__ carry_row,
                                               T* __restrict__ carry_val, T* __restrict__ head_val) {
  constexpr int kItems = kWave * IPT;
  const int row_b = c.row_b, rows_cnt = c.rows_cnt, nnz_cnt = c.nnz_cnt;
  const int64_t nnz_b = c.nnz_b;
  const int items = rows_cnt + nnz_cnt;

  // ---- gathers, row ends, then the next block's streams ---------------------------
  T g[IPT];
#pragma unroll
  for (int s = 0; s < IPT; ++s) {
    // lanes served from LDS load the front's first word along with the others (one more lane of a line
    // costs nothing): every load is issued whatever the lanes need
    g[s] = p[s] < hc ? x_front[p[s] < h1 ? 0u : p[s]] : x[p[s] - hc];
  }
  // one row end per lane covers most blocks; the row still open at the end counts as one more
  int64_t rp0;
  {
    const int64_t r = (int64_t)row_b + (lane <= rows_cnt ? lane : 0);
    rp0 = r < m ? (int64_t)row_ptr[r + 1] : (int64_t)INT32_MAX;
  }
  hot_load_streams<T, IPT>(cn, lane, val, pcol, vn, pn);
  T l[IPT];
#pragma unroll
  for (int s = 0; s < IPT; ++s) l[s] = hot[p[s] < h1 ? p[s] : 0];
  if (rows_cnt == 0) {
    // no row ends inside this block (it lies inside one long row): no staging, no walk, one sum
    T acc = T(0);
#pragma unroll
    for (int s = 0; s < IPT; ++s) {
      const T pr = v[s] * (p[s] < h1 ? l[s] : g[s]);
      if (HotSlots<T, IPT>::entry(lane, s) < nnz_cnt) acc += pr;
    }
    acc = group_sum<kWave>(acc);
    if (lane == kWave - 1) {
      carry_row[b] = row_b;
      carry_val[b] = acc;
    }
    return;
  }
  if (lane <= rows_cnt) {
    const int64_t e = rp0 - base - nnz_b;
    sm.rend[lane] = (unsigned short)(e > kItems ? kItems + 1 : (e < 0 ? 0 : (int)e));
  }
  for (int i = lane + kWave; i <= rows_cnt; i += kWave) {
    const int64_t r = (int64_t)row_b + i;
    const int64_t e = r < m ? (int64_t)row_ptr[r + 1] - base - nnz_b : (int64_t)kItems + 1;
    sm.rend[i] = (unsigned short)(e > kItems ? kItems + 1 : (e < 0 ? 0 : (int)e));
  }
#pragma unroll
  for (int s = 0; s < IPT; ++s) {
    const int k = HotSlots<T, IPT>::entry(lane, s);
    if (k < nnz_cnt) sm.prod[lds_pad(k)] = v[s] * (p[s] < h1 ? l[s] : g[s]);
  }
  wave_lds_fence();

  // ---- this lane's start on the block-local merge path -----------------------
  int dt = lane * IPT;
  if (dt > items) dt = items;
  int dt_end = dt + IPT;
  if (dt_end > items) dt_end = items;
  int lo = dt > nnz_cnt ? dt - nnz_cnt : 0;
  int hi = dt < rows_cnt ? dt : rows_cnt;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if ((int)sm.rend[mid] <= dt - mid - 1) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  int i = lo;       // local row
  int j = dt - lo;  // local entry
  T acc = T(0);
  T first_sum = T(0);
  int first_row = -1;
  bool finished_any = false;
#pragma unroll
  for (int step = 0; step < IPT; ++step) {
    if (dt + step < dt_end) {
      const bool take_entry = j < nnz_cnt && (i >= rows_cnt || j < (int)sm.rend[i]);
      if (take_entry) {
        acc += sm.prod[lds_pad(j)];
        ++j;
      } else if (i < rows_cnt) {
        // exactly one lane finishes a given row; the first row it finishes may have begun in lanes below
        if (!finished_any) {
          first_row = i;
          first_sum = acc;
          finished_any = true;
        } else {
          sm.rsum[i] = acc;
        }
        acc = T(0);
        ++i;
      }
    }
  }

  // ---- segmented inclusive scan of the unfinished tails, key = row --------
  const int key = i;
  T tail = acc;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const T up = lane_up(tail, d);
    const int kup = __shfl_up(key, d, kWave);
    if (lane >= d && kup == key) tail += up;
  }
  {
    const T below = lane_up(tail, 1);
    const int kbelow = __shfl_up(key, 1, kWave);
    if (finished_any) {
      if (lane > 0 && kbelow == first_row) first_sum += below;
      sm.rsum[first_row] = first_sum;
    }
  }
  if (lane == kWave - 1) {
    carry_row[b] = row_b + key;  // == row_e: the row still open, or m
    carry_val[b] = tail;
  }
  wave_lds_fence();

  // ---- rows finished here: y = beta*y + alpha*sum, unit stride -----------------
  // Local row 0 of every block but the first may have begun in earlier blocks: the fix-up kernel
  // completes it from head_val and the carries.
  const int first_direct = b > 0 ? 1 : 0;
  if (lane == 0 && b > 0) head_val[b] = rows_cnt > 0 ? sm.rsum[0] : T(0);
  for (int r = lane + first_direct; r < rows_cnt; r += kWave)
    store_axpby(y, (int64_t)row_b + r, alpha, sm.rsum[r], beta);
  wave_lds_fence();  // the staging area is written again by the wave's next block
}

template <typename T, int IPT, int NW>
__global__ __launch_bounds__(kWave* NW) void spmv_merge_hot_kernel(
    int m, int nnz, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const unsigned* __restrict__ pcol, const T* __restrict__ x, const T* __restrict__ x_front, int h1, int hc,
    T beta, T* __restrict__ y, int base, const int* __restrict__ block_row, int* __restrict__ carry_row,
    T* __restrict__ carry_val, T* __restrict__ head_val, int nblocks) {
  using Dims = HotDims<T, IPT, NW>;
  extern __shared__ __align__(16) unsigned char smem[];
  T* hot = reinterpret_cast<T*>(smem);
  HotWaveSmem<T, IPT>* stage = reinterpret_cast<HotWaveSmem<T, IPT>*>(smem + Dims::table_bytes);
  for (int i = threadIdx.x; i < h1; i += Dims::threads) hot[i] = x_front[i];
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
  const int lane = (int)threadIdx.x % kWave;
  // every workgroup walks one contiguous share of the merge blocks, its waves taking turns; the shares
  // of the workgroups of one XCD are neighbours
  const unsigned w = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int per = (nblocks + (int)gridDim.x - 1) / (int)gridDim.x;
  const int b0 = (int)w * per;
  const int b1 = b0 + per < nblocks ? b0 + per : nblocks;
  T v[2][IPT];
  unsigned p[2][IPT];
  int b = b0 + wave;
  HotCoords c = hot_coords<IPT>(b, b < b1, m, nnz, block_row);
  hot_load_streams<T, IPT>(c, lane, val, pcol, v[0], p[0]);
  // two blocks per trip, so that the register sets swap roles without copies
  while (b < b1) {
    HotCoords cn = hot_coords<IPT>(b + NW, b + NW < b1, m, nnz, block_row);
    hot_wave_block<T, IPT>(stage[wave], lane, b, c, v[0], p[0], cn, v[1], p[1], hot, (unsigned)h1, (unsigned)hc, x_front, x,
                           m, alpha, val, row_ptr, pcol, beta, y, base, carry_row, carry_val, head_val);
    b += NW;
    if (b >= b1) break;
    c = hot_coords<IPT>(b + NW, b + NW < b1, m, nnz, block_row);
    hot_wave_block<T, IPT>(stage[wave], lane, b, cn, v[1], p[1], c, v[0], p[0], hot, (unsigned)h1, (unsigned)hc, x_front, x,
                           m, alpha, val, row_ptr, pcol, beta, y, base, carry_row, carry_val, head_val);
    b += NW;
  }
}

// ---- analysis of the hot columns ------------------------------------------------------------------
// Counts the entries of every column -- of one chunk of 256 entries in every 2^sample_shift: the atomics go
// to memory (about 10 G a second), and a quarter of a large matrix ranks its popular columns as well as all of
// it.  The same chunks every time: the same counts for the same matrix.
static __global__ __launch_bounds__(256) void col_count_kernel(int nnz, const int* __restrict__ col_ind, int base,
                                                        int sample_shift, unsigned* __restrict__ count) {
  const int64_t chunks = ((int64_t)nnz + 255) >> 8;
  const int64_t sampled = (chunks + ((int64_t)1 << sample_shift) - 1) >> sample_shift;
  for (int64_t c = blockIdx.x; c < sampled; c += gridDim.x) {
    const int64_t k = ((c << sample_shift) << 8) + threadIdx.x;
    if (k < nnz) atomicAdd(&count[nt_load(col_ind + k) - base], 1u);
  }
}
// key[c] = ~count[c] (an ascending sort then puts the most popular column first), idx[c] = c
static __global__ __launch_bounds__(256) void col_rank_keys_kernel(int n, const unsigned* __restrict__ count,
                                                            unsigned* __restrict__ key, unsigned* __restrict__ idx) {
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  key[c] = ~count[c];
  idx[c] = (unsigned)c;
}
// *total = the counts behind the first `first` sorted keys (one workgroup; the host wants this one number, and
// a copy of the keys themselves goes to the copy engine, whose first copy after a pause takes milliseconds)
static __global__ __launch_bounds__(256) void col_rank_head_sum_kernel(int first, const unsigned* __restrict__ key,
                                                                unsigned long long* __restrict__ total) {
  __shared__ unsigned long long part[256];
  unsigned long long sum = 0;
  for (int i = threadIdx.x; i < first; i += 256) sum += (unsigned long long)(~key[i]);
  part[threadIdx.x] = sum;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) *total = part[0];
}
// rank[sorted_col[i]] = i for i < hc (rank was filled with 0xFFFFFFFF)
static __global__ __launch_bounds__(256) void col_rank_scatter_kernel(int hc, const unsigned* __restrict__ sorted_col,
                                                               unsigned* __restrict__ rank, int* __restrict__ hot_cols) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= hc) return;
  rank[sorted_col[i]] = (unsigned)i;
  hot_cols[i] = (int)sorted_col[i];
}
// pcol[k] = rank of entry k's column if it is one of the hc most popular, else hc + column
static __global__ __launch_bounds__(256) void hot_pcol_kernel(int nnz, const int* __restrict__ col_ind, int base, int hc,
                                                       const unsigned* __restrict__ rank, unsigned* __restrict__ pcol) {
  for (int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x; k < nnz; k += (int64_t)gridDim.x * 256) {
    const unsigned c = (unsigned)(nt_load(col_ind + k) - base);
    const unsigned r = rank[c];
    pcol[k] = r != 0xFFFFFFFFu ? r : (unsigned)hc + c;
  }
}

}  // namespace asamd
