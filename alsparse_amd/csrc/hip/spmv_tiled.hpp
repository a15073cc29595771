// Tiled two-phase CSR SpMV for gfx950 (wave64): every x gather and every y
// update happens in LDS, HBM only sees unit-stride streams.
//
// Why: on matrices whose columns are spread over an x far larger than the 4 MiB
// L2 of an XCD, each x gather of the row-parallel kernels misses L2 and moves a
// whole 128-byte line for 4 useful bytes; measured on the 16 M-row uniform
// matrix that is 34.6 GB of fabric traffic for 2.4 GB of algorithmic bytes.
// Here the matrix is re-laid-out once (analysis) into tiles of
// TileDims::cols columns x kTileRows rows, tiles ordered by (column block, row
// block), entries inside a tile in CSR order (stable sort):
//
//   phase 1  tiled_products_kernel   one workgroup per chunk of a column block:
//            the block's x slice (128 KiB) is copied to LDS, then the chunk's
//            entries (value, 16-bit local column) are streamed and the products
//            val * x written back in the same order, unit stride.
//   phase 2  tiled_reduce_kernel     one WAVE per row block of TileDims::rows
//            rows: its accumulators live in a private slice of LDS; the wave
//            walks the tiles of its row block (one short contiguous run per
//            column block), streams products and 16-bit local rows and adds them
//            with plain LDS read-modify-writes.  No other wave ever touches those
//            accumulators, and entries of one row that share a wave instruction
//            (they are adjacent, the tile being in CSR order) are first combined
//            inside the wave, so no atomics are needed: LDS float atomics were
//            measured at ~0.45 lanes per clock, four times slower than the whole
//            phase takes without them.  The kRedWaves waves of a workgroup own
//            consecutive row blocks, whose tiles are adjacent in memory, and a
//            barrier per batch of column blocks keeps them in step, so DRAM sees
//            one multi-KiB burst per column block instead of scattered 256-byte
//            reads.  Tiles longer than kLongTile entries (long rows) are summed
//            by the whole workgroup beforehand, one LDS atomic per wave and row.
//            Finally y = beta*y + alpha*acc, unit stride.
//
// HBM traffic is 2*sizeof(T) + 4 bytes per entry more than plain CSR (the
// product round trip and the second index), all of it streamed.  The order of
// every addition is fixed by the layout, so results are bit-reproducible.
// The reference has no counterpart; per-entry arithmetic is that of
// src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-54.
#pragma once

#include "device_utils.hpp"

namespace asamd {

constexpr int kTileBytes = 128 * 1024;  // LDS bytes of an x slice (phase 1) / of a workgroup's accumulators (phase 2)
constexpr int kProdThreads = 1024;      // phase-1 workgroup
constexpr int kProdUnroll = 8;
constexpr int kRedWaves = 8;            // phase-2 workgroup: 8 waves = 8 consecutive row blocks,
constexpr int kRedThreads = kRedWaves * kWave;  // whose tiles are adjacent in memory for every column block
constexpr int kRedUnroll = 8;
constexpr int kRedBytes = kTileBytes / 2;  // LDS bytes of a phase-2 workgroup's accumulators
constexpr int kLongTile = 1024;         // tiles with more entries are summed by the whole workgroup
constexpr int kTiledMaxColBlocks = 2048;       // keeps the tile table small
constexpr int64_t kTiledMaxTiles = (int64_t)1 << 24;

template <typename T>
struct TileDims {
  static constexpr int cols = kTileBytes / (int)sizeof(T);            // 32768 fp32, 16384 fp64
  static constexpr int rows = kRedBytes / kRedWaves / (int)sizeof(T);  // rows per wave: 2048 fp32, 1024 fp64
  static constexpr int rows_log2 = sizeof(T) == 4 ? 11 : 10;
};

struct TiledChunk {
  int col_block;
  int begin;  // entry range [begin, end) in tile order
  int end;
};

struct TileRange {
  int begin, end;
};

struct LongTile {
  int begin, end;
  int row_block;
};

// ---- analysis ----------------------------------------------------------------
// key[k] = col_block * row_blocks + row_block of entry k; idx[k] = k.
// coo_row holds the row of every entry in the matrix's index base.
__global__ __launch_bounds__(256) void tile_keys_kernel(int nnz, const int* __restrict__ coo_row,
                                                        const int* __restrict__ col_ind, int base,
                                                        int tile_cols_log2, int tile_rows_log2,
                                                        int row_blocks, unsigned* __restrict__ key,
                                                        unsigned* __restrict__ idx) {
  for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz;
       k += (int64_t)gridDim.x * blockDim.x) {
    const unsigned cb = (unsigned)(col_ind[k] - base) >> tile_cols_log2;
    const unsigned rb = (unsigned)(coo_row[k] - base) >> tile_rows_log2;
    key[k] = cb * (unsigned)row_blocks + rb;
    idx[k] = (unsigned)k;
  }
}

// Entries in sorted order: values, local columns, local rows.
template <typename T>
__global__ __launch_bounds__(256) void tile_gather_kernel(
    int nnz, const unsigned* __restrict__ perm, const int* __restrict__ coo_row,
    const int* __restrict__ col_ind, const T* __restrict__ val, int base, int tile_cols_log2,
    int tile_rows_log2, T* __restrict__ t_val, unsigned short* __restrict__ t_col, unsigned short* __restrict__ t_row) {
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < nnz;
       q += (int64_t)gridDim.x * blockDim.x) {
    const unsigned k = perm[q];
    t_val[q] = val[k];
    t_col[q] = (unsigned short)((col_ind[k] - base) & ((1 << tile_cols_log2) - 1));
    t_row[q] = (unsigned short)((coo_row[k] - base) & ((1 << tile_rows_log2) - 1));
  }
}

// tile_ptr[t] = first position whose key is >= t, for t in [0, tiles].
__global__ __launch_bounds__(256) void tile_bounds_kernel(int nnz, const unsigned* __restrict__ sorted_key,
                                                          int64_t tiles, int* __restrict__ tile_ptr) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t > tiles) return;
  int lo = 0, hi = nnz;
  while (lo < hi) {
    const int mid = (int)(((int64_t)lo + hi) >> 1);
    if ((int64_t)sorted_key[mid] < t) lo = mid + 1;
    else hi = mid;
  }
  tile_ptr[t] = lo;
}

// Phase 2 reads the tile table row block by row block:
// ranges[rb * col_blocks + cb] = {tile_ptr[cb*row_blocks + rb], tile_ptr[cb*row_blocks + rb + 1]}.
// Tiles longer than kLongTile go to long_list instead (their range is left empty).
__global__ __launch_bounds__(256) void tile_ranges_kernel(int row_blocks, int col_blocks,
                                                          const int* __restrict__ tile_ptr,
                                                          TileRange* __restrict__ ranges,
                                                          LongTile* __restrict__ long_list,
                                                          int* __restrict__ long_count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)row_blocks * col_blocks) return;
  const int rb = (int)(i / col_blocks), cb = (int)(i % col_blocks);
  const int64_t t = (int64_t)cb * row_blocks + rb;
  int b = tile_ptr[t];
  const int e = tile_ptr[t + 1];
  if (e - b > kLongTile) {
    const int slot = atomicAdd(long_count, 1);
    long_list[slot].begin = b;
    long_list[slot].end = e;
    long_list[slot].row_block = rb;
    b = e;
  }
  ranges[i].begin = b;
  ranges[i].end = e;
}

// ---- phase 1 -------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kProdThreads) void tiled_products_kernel(
    int n, const TiledChunk* __restrict__ chunks, const T* __restrict__ t_val,
    const unsigned short* __restrict__ t_col, const T* __restrict__ x, T* __restrict__ prod) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* xs = reinterpret_cast<T*>(smem);
  const TiledChunk ch = chunks[blockIdx.x];
  const int64_t col0 = (int64_t)ch.col_block * TileDims<T>::cols;
  int64_t ncols = (int64_t)n - col0;
  if (ncols > TileDims<T>::cols) ncols = TileDims<T>::cols;
  for (int i = threadIdx.x; i < ncols; i += kProdThreads) xs[i] = x[col0 + i];
  __syncthreads();
  constexpr int kStep = kProdThreads * kProdUnroll;
  int k = ch.begin + threadIdx.x;
  for (; k + kStep - kProdThreads < ch.end; k += kStep) {
    T v[kProdUnroll];
    int c[kProdUnroll];  // widened at once: packing two 16-bit loads into one register would serialise them
#pragma unroll
    for (int u = 0; u < kProdUnroll; ++u) {
      v[u] = t_val[k + u * kProdThreads];
      c[u] = t_col[k + u * kProdThreads];
    }
#pragma unroll
    for (int u = 0; u < kProdUnroll; ++u) prod[k + u * kProdThreads] = v[u] * xs[c[u]];
  }
  for (; k < ch.end; k += kProdThreads) prod[k] = t_val[k] * xs[t_col[k]];
}

// ---- phase 2 -------------------------------------------------------------------
// acc[r] += v for the valid lanes of one wave instruction.  acc is private to
// the wave.  Entries of one row are adjacent (a tile is stored in CSR order), so
// lanes that share a row with their neighbour are combined inside the wave
// first and the read-modify-writes of one instruction never collide.  Isolated
// pairs (the usual case on short rows) cost three DPP wave shifts; longer runs
// take a segmented suffix sum.
template <bool Atomic, typename T>
__device__ __forceinline__ void rmw(T* p, T v) {
  if constexpr (Atomic) atomicAdd(p, v);
  else *p += v;
}

template <bool Atomic = false, typename T>
__device__ __forceinline__ void add_rows(T* acc, int r, T v, bool valid) {
  const int lane = threadIdx.x % kWave;
  const int r_up = __builtin_amdgcn_update_dpp(-1, r, 0x138, 0xF, 0xF, false);  // wave_shr:1, lane 0 keeps -1
  const bool same_as_prev = valid && lane > 0 && r_up == r;
  const uint64_t dup = __builtin_amdgcn_ballot_w64(same_as_prev);
  if (dup == 0) {
    if (valid) rmw<Atomic>(&acc[r], v);
  } else if ((dup & (dup << 1)) == 0) {
    // runs of exactly two: the first lane takes its neighbour's value
    const T v_next = dpp_mov<0x130>(v);  // wave_shl:1: value of lane + 1 (0 past the end)
    if ((dup >> 1 >> lane) & 1) v += v_next;
    if (valid && !same_as_prev) rmw<Atomic>(&acc[r], v);
  } else {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const T vd = __shfl_down(v, d, kWave);
      const int rd = __shfl_down(r, d, kWave);
      if (lane + d < kWave && rd == r) v += vd;
    }
    if (valid && !same_as_prev) rmw<Atomic>(&acc[r], v);
  }
}

template <typename T>
__global__ __launch_bounds__(kRedThreads) void tiled_reduce_kernel(
    int m, int row_blocks, int col_blocks, const TileRange* __restrict__ ranges,
    const int* __restrict__ long_ptr, const LongTile* __restrict__ long_tiles,
    const unsigned short* __restrict__ t_row, const T* __restrict__ prod, T alpha, T beta,
    T* __restrict__ y) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_acc = reinterpret_cast<T*>(smem);
  constexpr int kTileRows = TileDims<T>::rows;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int rb = blockIdx.x * kRedWaves + wave;
  const bool active = rb < row_blocks;  // wave-uniform; idle waves still meet the barriers
  T* acc = s_acc + wave * kTileRows;
  for (int i = lane; i < kTileRows; i += kWave) acc[i] = T(0);
  __syncthreads();

  // ---- long tiles of this workgroup: all waves, one LDS atomic per wave and row
  const int lt0 = long_ptr[blockIdx.x], lt1 = long_ptr[blockIdx.x + 1];
  for (int lt = lt0; lt < lt1; ++lt) {
    const LongTile t = long_tiles[lt];
    T* tacc = s_acc + (t.row_block - blockIdx.x * kRedWaves) * kTileRows;
    for (int k0 = t.begin; k0 < t.end; k0 += kRedThreads) {  // workgroup-uniform trip count
      const int k = k0 + threadIdx.x;
      const bool ok = k < t.end;
      const T v = ok ? prod[k] : T(0);
      const int r = ok ? (int)t_row[k] : -1 - lane;
      add_rows<true>(tacc, r, v, ok);
    }
  }
  if (lt1 > lt0) __syncthreads();

  // ---- short tiles: wave-private accumulators, batches of kRedUnroll column blocks
  const TileRange* my = ranges + (int64_t)(active ? rb : 0) * col_blocks;
  for (int cb0 = 0; cb0 < col_blocks; cb0 += kWave) {
    TileRange tr = {0, 0};
    if (active && cb0 + lane < col_blocks) tr = my[cb0 + lane];  // 64 tile ranges, one coalesced load
    const int ncb = col_blocks - cb0 < kWave ? col_blocks - cb0 : kWave;
    for (int j = 0; j < ncb; j += kRedUnroll) {
      // every lane takes up to two entries of each of kRedUnroll tiles, all loads in flight together
      T v[kRedUnroll][2];
      int r[kRedUnroll][2];
      int b[kRedUnroll], e[kRedUnroll];
#pragma unroll
      for (int u = 0; u < kRedUnroll; ++u) {
        const int src = j + u < ncb ? j + u : j;
        b[u] = __builtin_amdgcn_readlane(tr.begin, src);
        e[u] = j + u < ncb ? __builtin_amdgcn_readlane(tr.end, src) : b[u];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int k = b[u] + h * kWave + lane;
          const bool ok = k < e[u];
          v[u][h] = ok ? prod[k] : T(0);
          r[u][h] = ok ? (int)t_row[k] : -1 - lane;
        }
      }
#pragma unroll
      for (int u = 0; u < kRedUnroll; ++u) {
        add_rows(acc, r[u][0], v[u][0], r[u][0] >= 0);
        if (e[u] - b[u] > kWave) add_rows(acc, r[u][1], v[u][1], r[u][1] >= 0);  // wave-uniform
        for (int k = b[u] + 2 * kWave + lane; k - lane < e[u]; k += kWave) {  // tiles of 129 .. kLongTile entries
          const bool ok = k < e[u];
          const T v2 = ok ? prod[k] : T(0);
          const int r2 = ok ? (int)t_row[k] : -1 - lane;
          add_rows(acc, r2, v2, ok);
        }
      }
      __syncthreads();  // keeps the waves on neighbouring tiles: their reads form one burst
    }
  }
  if (!active) return;
  const int64_t row0 = (int64_t)rb * kTileRows;
  int64_t nrows = (int64_t)m - row0;
  if (nrows > kTileRows) nrows = kTileRows;
  for (int i = lane; i < nrows; i += kWave) store_axpby(y, row0 + i, alpha, acc[i], beta);
}

}  // namespace asamd
