// Tiled two-phase CSR SpMV for gfx950 (wave64): every x gather and every y
// update happens in LDS, HBM only sees unit-stride streams.
//
// Why: on matrices whose columns are spread over an x far larger than the 4 MiB
// L2 of an XCD, each x gather of the row-parallel kernels misses L2 and moves a
// whole 128-byte line for 4 useful bytes; measured on the 16 M-row uniform
// matrix that is 34.6 GB of fabric traffic for 2.4 GB of algorithmic bytes.
// Here the matrix is re-laid-out once (analysis) into tiles: column blocks of at
// most TileDims::cols columns and row blocks of at most TileDims::rows rows, both
// cut so that every block holds about the same number of entries (hot columns
// and long rows get narrower blocks, so tiles stay even on skewed matrices);
// tiles are ordered by (column block, row block), entries inside a tile in CSR
// order (stable sort):
//
//   phase 1  tiled_products_kernel   one workgroup per chunk of a column block:
//            the block's x slice (160 KiB) is copied to LDS, then the chunk's
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
//            phase takes without them.  A wave keeps 16 tiles in flight in a
//            ring of registers (loads issued unconditionally, so the counter of
//            outstanding loads lets it wait for the oldest tile only), 32 where
//            no tile holds more than one entry per lane.  The
//            kRedWaves waves of a workgroup own consecutive row blocks, whose
//            tiles are adjacent in memory.  Finally y = beta*y + alpha*acc, unit
//            stride.
//   phase 3  tiled_long_kernel       only if some tile holds more than kLongTile
//            entries (long rows, hot columns): those tiles are left out of phase
//            2; one workgroup per row block that has any deals them to its waves,
//            which add them into LDS accumulators of their own; the waves'
//            accumulators meet in wave order and are added to y.
//
// HBM traffic is 2*sizeof(T) + 4 bytes per entry more than plain CSR (the
// product round trip and the second index), all of it streamed.  The order of
// every addition is fixed by the layout (no floating-point atomics anywhere), so
// results are bit-reproducible.
// The reference has no counterpart; per-entry arithmetic is that of
// src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-54.
#pragma once

#include "device_utils.hpp"

namespace asamd {

constexpr int kLdsPerCu = 160 * 1024;   // LDS of one compute unit
constexpr int kTileBytes = 128 * 1024;  // LDS bytes of a workgroup's accumulators (phase 2), at most
// LDS bytes of an x slice (phase 1): the whole LDS of a compute unit.  Wider column blocks make fewer and
// longer tiles for phase 2 (16 M columns: 410 blocks instead of 512; 0.988 -> 0.979 ms on 2^24 rows x 16).
constexpr int kSliceBytes = kLdsPerCu;
constexpr int kProdThreads = 1024;      // phase-1 workgroup
constexpr int kRedWaves = 8;            // phase-2 workgroup: 8 waves = 8 consecutive row blocks, whose tiles are adjacent in memory
constexpr int kRedSlots = 16;
constexpr int kLongTile = 2 * kWave;     // phase 2 takes at most two entries per lane and tile; longer tiles go to phase 3
constexpr int kLongThreads = 512;  // phase 3: eight waves share the long tiles of one row block
constexpr int kLongPart = 32768;   // ... up to about this many entries; a row block with more gets several workgroups
constexpr int kLongNarrow = 256;   // row blocks of at most this many rows (hub rows) run with small accumulators
constexpr int kTiledMaxColBlocks = 2048;       // keeps the tile table small
constexpr int64_t kTiledMaxTiles = (int64_t)1 << 25;  // 12 bytes of tables per tile

constexpr int kColGroupLog2 = 8;        // column blocks are cut at multiples of 256 columns,
constexpr int kRowGroupLog2 = 6;        // row blocks at multiples of 64 rows

template <typename T>
struct TileDims {
  static constexpr int cols = kSliceBytes / (int)sizeof(T);           // widest column block: 40960 fp32, 20480 fp64
  // Phase 2 pays per TILE, so a row block keeps 2048 rows whatever the value size (1024 for 16-byte
  // values): 8 waves with 64 KiB of accumulators for 4-byte values, 128 KiB for wider ones.  (16 waves
  // with 128 KiB for 4-byte values -- runs of 16 adjacent tiles instead of 8 per column block -- were
  // measured no faster.)
  static constexpr int red_waves = kRedWaves;
  static constexpr int red_threads = red_waves * kWave;
  static constexpr int red_bytes = sizeof(T) >= 8 ? kTileBytes : kTileBytes / 2;
  static constexpr int rows = red_bytes / red_waves / (int)sizeof(T);  // tallest row block
  // every wave's accumulators are followed by one dummy row per lane, where lanes without an entry add their zero
  static constexpr int red_lds_bytes = red_bytes + red_waves * kWave * (int)sizeof(T);
  // tiles a wave keeps in flight in phase 2 when a tile may take two entries per lane (16 four-register
  // slots would not fit for 16-byte values); twice as many when every tile fits one entry per lane
  static constexpr int red_slots = sizeof(T) >= 16 ? kRedSlots / 2 : kRedSlots;
};

struct TiledChunk {
  int col0, ncols;  // the chunk's column block
  int begin;        // entry range [begin, end) in tile order
  int end;
};

struct TileRange {
  int begin, end;
};

struct LongTile {
  int begin, end;
  int row_block;
};

struct LongBlock {
  int first, count;  // long tiles of one row block, a run in the sorted list of long tiles
  int row0, nrows;   // the row block's rows
  int out;           // -1: the only part of its row block, adds to y itself; else where its sums go in the scratch
};

struct LongFinish {  // a row block whose long tiles were dealt to several workgroups
  int row0, nrows;
  int out0, parts;   // part p left its sums at scratch[out0 + p * nrows ...]
};

// ---- analysis ----------------------------------------------------------------
// Entries per group of 256 columns (for cutting equal-entry column blocks), counted on a sample:
// every stride-th run of kCountRun consecutive entries.  The counts only steer where the blocks are
// cut, so a few million samples are as good as all entries, and the atomics (which collide on hot
// columns) stay few.  Runs of consecutive entries hold whole rows, so the sample is not biased
// towards any position inside a row.
constexpr int kCountRun = 1024;
static __global__ __launch_bounds__(256) void col_group_count_kernel(int nnz, const int* __restrict__ col_ind,
                                                              int base, int stride, int* __restrict__ count) {
  const int64_t runs = ((int64_t)nnz + kCountRun - 1) / kCountRun;
  for (int64_t run = (int64_t)blockIdx.x * stride; run < runs; run += (int64_t)gridDim.x * stride) {
    const int64_t k0 = run * kCountRun;
    for (int i = threadIdx.x; i < kCountRun; i += 256) {
      const int64_t k = k0 + i;
      if (k < nnz) atomicAdd(&count[(col_ind[k] - base) >> kColGroupLog2], 1);
    }
  }
}

// out[g] = row_ptr[g * 64] for g in [0, groups], the last one clamped to row_ptr[m].
static __global__ __launch_bounds__(256) void row_group_offsets_kernel(int m, const int* __restrict__ row_ptr,
                                                                int groups, int* __restrict__ out) {
  const int g = blockIdx.x * blockDim.x + threadIdx.x;
  if (g > groups) return;
  int64_t r = (int64_t)g << kRowGroupLog2;
  if (r > m) r = m;
  out[g] = row_ptr[r];
}

// key[k] = col_block * row_blocks + row_block of entry k; idx[k] = k.
// coo_row holds the row of every entry in the matrix's index base; the block of
// a column / row is looked up through its group.
static __global__ __launch_bounds__(256) void tile_keys_kernel(int nnz, const int* __restrict__ coo_row,
                                                        const int* __restrict__ col_ind, int base,
                                                        const int* __restrict__ col_group_block,
                                                        const int* __restrict__ row_group_block,
                                                        int row_blocks, unsigned* __restrict__ key,
                                                        unsigned* __restrict__ idx) {
  for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz;
       k += (int64_t)gridDim.x * blockDim.x) {
    const unsigned cb = (unsigned)col_group_block[(col_ind[k] - base) >> kColGroupLog2];
    const unsigned rb = (unsigned)row_group_block[(coo_row[k] - base) >> kRowGroupLog2];
    key[k] = cb * (unsigned)row_blocks + rb;
    idx[k] = (unsigned)k;
  }
}

// For 4-byte values the entry's position and local indices travel with its key through the sort:
// payload = entry index (high word) | column local to its block << 16 | row local to its block.
// Gathering all three CSR streams through the sorted permutation afterwards moves a 128-byte line per
// entry and stream (18 ms for 2^28 entries, against 3 ms more in the sort and a streaming unpack); only
// the values are gathered that way (gather_values_kernel), and the permutation is kept so that they can
// be gathered again when the caller has changed them.
static __global__ __launch_bounds__(256) void tile_keys_payload_kernel(
    int nnz, const int* __restrict__ coo_row, const int* __restrict__ col_ind,
    int base, const int* __restrict__ col_group_block, const int* __restrict__ col_block_start,
    const int* __restrict__ row_group_block, const int* __restrict__ row_block_start, int row_blocks,
    unsigned* __restrict__ key, unsigned long long* __restrict__ payload) {
  for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz;
       k += (int64_t)gridDim.x * blockDim.x) {
    const int col = col_ind[k] - base, row = coo_row[k] - base;
    const unsigned cb = (unsigned)col_group_block[col >> kColGroupLog2];
    const unsigned rb = (unsigned)row_group_block[row >> kRowGroupLog2];
    key[k] = cb * (unsigned)row_blocks + rb;
    const unsigned lc = (unsigned)(col - col_block_start[cb]), lr = (unsigned)(row - row_block_start[rb]);
    payload[k] = ((unsigned long long)(unsigned)k << 32) | (lc << 16) | lr;
  }
}

static __global__ __launch_bounds__(256) void tile_unpack_kernel(int nnz, const unsigned long long* __restrict__ payload,
                                                          unsigned* __restrict__ t_perm,
                                                          unsigned short* __restrict__ t_col,
                                                          unsigned short* __restrict__ t_row) {
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < nnz;
       q += (int64_t)gridDim.x * blockDim.x) {
    const unsigned long long w = payload[q];
    t_perm[q] = (unsigned)(w >> 32);
    t_col[q] = (unsigned short)(w >> 16);
    t_row[q] = (unsigned short)w;
  }
}

// out[q] = val[perm[q]] (CONJ: conjugated): the values of a re-ordered copy, taken afresh from the
// caller's array.  Eight gathers in flight per lane.  gate: null, or a flag left by the value guard --
// zero means that the values have not changed, and the kernel returns at once.
template <typename T, bool CONJ>
__global__ __launch_bounds__(256) void gather_values_kernel(int nnz, const unsigned* __restrict__ perm,
                                                            const T* __restrict__ val, T* __restrict__ out,
                                                            const int* __restrict__ gate) {
  if (gate && *gate == 0) return;
  constexpr int kU = 8;
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; q + (kU - 1) * stride < nnz; q += kU * stride) {
    unsigned k[kU];
    T v[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) k[u] = nt_load(perm + q + u * stride);
#pragma unroll
    for (int u = 0; u < kU; ++u) v[u] = val[k[u]];
#pragma unroll
    for (int u = 0; u < kU; ++u) out[q + u * stride] = CONJ ? conj_t(v[u]) : v[u];
  }
  for (; q < nnz; q += stride) out[q] = CONJ ? conj_t(val[perm[q]]) : val[perm[q]];
}

// The same over a tiled layout, the tiles of ONE row block side by side on one XCD: the slots of a tile pick
// their values from the stretch of val that holds the row block's rows, one entry here and one there, and in slot
// order -- column block after column block -- every pass over the row blocks fetches that stretch again, a
// 128-byte line per entry (5.6 ms for 2^28 entries; 2.3 ms this way).  Tiles are short (a wave's worth or two of
// entries), so a wave takes eight of them at a time: the tiles (column blocks c .. c + 7, row block r), r = the
// workgroup's XCD (blockIdx.x % 8) + 8 i, consecutive waves taking consecutive c -- what an XCD works on at one
// time are a few whole row blocks.  gridDim.x: a multiple of 8.
template <typename T, bool CONJ>
__global__ __launch_bounds__(256) void gather_values_tiles_kernel(const unsigned* __restrict__ perm,
                                                                  const T* __restrict__ val, T* __restrict__ out,
                                                                  const int* __restrict__ tile_ptr, int col_blocks,
                                                                  int row_blocks, const int* __restrict__ gate) {
  if (gate && *gate == 0) return;
  constexpr int kU = 8;
  const int lane = threadIdx.x % kWave;
  const int xcd = blockIdx.x % 8;
  const int64_t waves_per_xcd = (int64_t)(gridDim.x / 8) * (256 / kWave);
  const int64_t col_groups = (col_blocks + kU - 1) / kU;
  const int64_t batches = (int64_t)((row_blocks - xcd + 7) / 8) * col_groups;  // row blocks xcd, xcd + 8, ...
  for (int64_t b = (int64_t)(blockIdx.x / 8) * (256 / kWave) + threadIdx.x / kWave; b < batches; b += waves_per_xcd) {
    const int64_t rb = xcd + 8 * (b / col_groups);
    const int c0 = (int)(b % col_groups) * kU;
    int my_lo = 0, my_hi = 0;  // lane u < 8: the slots of tile (c0 + u, rb)
    if (lane < kU && c0 + lane < col_blocks) {
      const int64_t tile = (int64_t)(c0 + lane) * row_blocks + rb;
      my_lo = tile_ptr[tile];
      my_hi = tile_ptr[tile + 1];
    }
    int lo[kU], len[kU], longest = 0;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      lo[u] = __builtin_amdgcn_readlane(my_lo, u);
      len[u] = __builtin_amdgcn_readlane(my_hi, u) - lo[u];
      longest = len[u] > longest ? len[u] : longest;
    }
    for (int at = 0; at < longest; at += kWave) {
      const int mine = at + lane;
      unsigned k[kU];
      T v[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) k[u] = mine < len[u] ? nt_load(perm + lo[u] + mine) : 0u;
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (mine < len[u]) v[u] = val[k[u]];
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (mine < len[u]) nt_store(CONJ ? conj_t(v[u]) : v[u], out + lo[u] + mine);
    }
  }
}

// Entries in sorted order: values, columns and rows local to their blocks.
template <typename T>
__global__ __launch_bounds__(256) void tile_gather_kernel(
    int nnz, const unsigned* __restrict__ perm, const int* __restrict__ coo_row,
    const int* __restrict__ col_ind, const T* __restrict__ val, int base,
    const int* __restrict__ col_group_block, const int* __restrict__ col_block_start,
    const int* __restrict__ row_group_block, const int* __restrict__ row_block_start,
    T* __restrict__ t_val, unsigned short* __restrict__ t_col, unsigned short* __restrict__ t_row) {
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < nnz;
       q += (int64_t)gridDim.x * blockDim.x) {
    const unsigned k = perm[q];
    const int col = col_ind[k] - base, row = coo_row[k] - base;
    t_val[q] = val[k];
    t_col[q] = (unsigned short)(col - col_block_start[col_group_block[col >> kColGroupLog2]]);
    t_row[q] = (unsigned short)(row - row_block_start[row_group_block[row >> kRowGroupLog2]]);
  }
}

// tile_ptr[t] = first position whose key is >= t, for t in [0, tiles].
static __global__ __launch_bounds__(256) void tile_bounds_kernel(int nnz, const unsigned* __restrict__ sorted_key,
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

// out[0] += entries held by tiles of more than kWave and at most kLongTile entries (one atomic per
// workgroup): phase 2 handles those only in its two-entries-per-lane form.
static __global__ __launch_bounds__(256) void tile_mid_entries_kernel(int64_t tiles, const int* __restrict__ tile_ptr,
                                                               unsigned long long* __restrict__ out) {
  __shared__ unsigned long long s_sum[256 / kWave];
  unsigned long long mine = 0;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < tiles; t += (int64_t)gridDim.x * blockDim.x) {
    const int len = tile_ptr[t + 1] - tile_ptr[t];
    if (len > kWave && len <= kLongTile) mine += (unsigned long long)len;
  }
  for (int d = kWave / 2; d > 0; d >>= 1) mine += __shfl_down(mine, d, kWave);
  if (threadIdx.x % kWave == 0) s_sum[threadIdx.x / kWave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long total = 0;
    for (int w = 0; w < 256 / kWave; ++w) total += s_sum[w];
    if (total) atomicAdd(out, total);
  }
}

// Phase 2 reads the tile table row block by row block:
// ranges[rb * col_blocks + cb] = {tile_ptr[cb*row_blocks + rb], tile_ptr[cb*row_blocks + rb + 1]}.
// Tiles longer than long_tile go to long_list instead (their range is left empty).
static __global__ __launch_bounds__(256) void tile_ranges_kernel(int row_blocks, int col_blocks, int long_tile,
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
  if (e - b > long_tile) {
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
// kPiece elements of T make one 128-bit access.
template <typename T>
struct alignas(16) Piece {
  static constexpr int n = 16 / (int)sizeof(T);
  T e[n];
};
// the same elements when only T's own alignment is known (x comes from the caller): the hardware takes
// unaligned wide global loads
template <typename T>
struct __attribute__((packed, aligned(alignof(T)))) LoosePiece {
  unsigned w[4];  // plain words: the piece is only moved, never computed with
};
// NTS: the products are stored non-temporally.  Worth it when they are far more than the 256 MiB memory-side
// cache holds (16 M x 16 M with 16 entries per row, 1 GiB of products: 0.907 -> 0.884 ms per multiply); products
// that fit are better left where the second phase finds them (2 M x 2 M: 0.159 -> 0.164 ms with NTS).
template <typename T, bool NTS>
__global__ __launch_bounds__(kProdThreads) void tiled_products_kernel(
    const TiledChunk* __restrict__ chunks, const T* __restrict__ t_val,
    const unsigned short* __restrict__ t_col, const T* __restrict__ x, T* __restrict__ prod) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* xs = reinterpret_cast<T*>(smem);
  const TiledChunk ch = chunks[blockIdx.x];
  {
    // x slice -> LDS: 128-bit pieces, all of a thread's loads issued before the first LDS write
    // (a load-wait-write loop pays the memory latency once per trip: 32 trips of it were a quarter
    // of this kernel's time)
    constexpr int kPer = Piece<T>::n;
    constexpr int kSlicePieces = TileDims<T>::cols / kPer / kProdThreads;  // pieces per thread in a full slice
    static_assert(kSlicePieces >= 1 && TileDims<T>::cols % (kPer * kProdThreads) == 0, "slice layout");
    const T* xsrc = x + (int64_t)ch.col0;
    const int whole = ch.ncols / kPer;
    LoosePiece<T> tmp[kSlicePieces];
#pragma unroll
    for (int u = 0; u < kSlicePieces; ++u) {
      const int q = threadIdx.x + u * kProdThreads;
      if (q < whole) tmp[u] = *reinterpret_cast<const LoosePiece<T>*>(xsrc + q * kPer);
    }
#pragma unroll
    for (int u = 0; u < kSlicePieces; ++u) {
      const int q = threadIdx.x + u * kProdThreads;
      if (q < whole) {
        unsigned* dst = reinterpret_cast<unsigned*>(xs + q * kPer);
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = tmp[u].w[i];
      }
    }
    const int rest = whole * kPer + threadIdx.x;  // fewer than kPer columns at the end of the last block
    if (rest < ch.ncols) xs[rest] = xsrc[rest];
  }
  __syncthreads();
  // Entries: a wave takes 1024 consecutive ones per trip (512 measured 2 % slower: fewer bytes in flight) as
  // 128-bit pieces of values, piece i*64 + lane in
  // instruction i, so every instruction moves 1 KiB of consecutive bytes; the lane's columns are the
  // matching Piece<T>::n 16-bit indices, its products go back the same way.  (A 2- or 4-byte access per
  // lane and entry issues four to eight times as many instructions; consecutive pieces per LANE instead of
  // per instruction touch every 128-byte line from several instructions.)  The arrays are the library's
  // own, 256-byte aligned; the chunk's first entries up to a multiple of 8 and what is left after the
  // last whole span are taken one by one.
  constexpr int kPer = Piece<T>::n;
  constexpr int kLaneEntries = 16;              // entries per lane and trip
  constexpr int kPieces = kLaneEntries / kPer;
  constexpr int kSpan = kLaneEntries * kWave;   // entries per wave and trip
  struct alignas(2 * kPer) ColPiece {
    unsigned short c[kPer];
  };
  const int lane = threadIdx.x % kWave;
  int head = (ch.begin + 7) & ~7;
  if (head > ch.end) head = ch.end;
  for (int k = ch.begin + threadIdx.x; k < head; k += kProdThreads) prod[k] = t_val[k] * xs[t_col[k]];
  const int spans = (ch.end - head) / kSpan;
  for (int g = threadIdx.x / kWave; g < spans; g += kProdThreads / kWave) {
    // at most four pieces (64 bytes per lane) in flight at a time: eight 16-byte values would spill
    constexpr int kFlight = kPieces < 4 ? kPieces : 4;
#pragma unroll
    for (int i0 = 0; i0 < kPieces; i0 += kFlight) {
      const int kb = head + g * kSpan + (i0 * kWave + lane) * kPer;
      Piece<T> v[kFlight];
      ColPiece c[kFlight];
#pragma unroll
      for (int i = 0; i < kFlight; ++i) {
        v[i] = *reinterpret_cast<const Piece<T>*>(t_val + kb + i * kWave * kPer);
        c[i] = *reinterpret_cast<const ColPiece*>(t_col + kb + i * kWave * kPer);
      }
#pragma unroll
      for (int i = 0; i < kFlight; ++i) {
#pragma unroll
        for (int j = 0; j < kPer; ++j) v[i].e[j] = v[i].e[j] * xs[c[i].c[j]];
        if constexpr (NTS) {
          typedef int V4 __attribute__((ext_vector_type(4)));
          __builtin_nontemporal_store(__builtin_bit_cast(V4, v[i]), reinterpret_cast<V4*>(prod + kb + i * kWave * kPer));
        } else {
          *reinterpret_cast<Piece<T>*>(prod + kb + i * kWave * kPer) = v[i];
        }
      }
    }
  }
  for (int k = head + spans * kSpan + threadIdx.x; k < ch.end; k += kProdThreads) prod[k] = t_val[k] * xs[t_col[k]];
}

// ---- phase 2 -------------------------------------------------------------------
// acc[r] += v for the valid lanes of one wave instruction.  acc is private to
// the wave.  Entries of one row are adjacent (a tile is
// stored in CSR order), so the lanes of a run of equal rows must not all do
// their read-modify-write at once.  From the ballot of "same row as the lane
// below" every lane knows its position in its run:
//   * only isolated pairs: the first lane of a pair takes its neighbour's value
//     through a DPP wave shift;
//   * runs of at most kMaxPasses lanes: pass p lets the p-th lane of every run
//     add, so the lanes of one pass always hold distinct rows;
//   * longer runs (long rows): a segmented suffix sum inside the wave leaves the
//     run's total in its first lane, which adds alone.
constexpr int kMaxPasses = 4;

// AllValid: every lane holds an entry or a private dummy row of acc (distinct per lane, so it never
// continues a run), and `valid` is not looked at: no masks around the read-modify-writes.
template <bool AllValid = false, typename T>
__device__ __forceinline__ void add_rows(T* acc, int r, T v, bool valid_arg) {
  const bool valid = AllValid ? true : valid_arg;
  const int lane = threadIdx.x % kWave;
  const int r_up = __builtin_amdgcn_update_dpp(-1, r, 0x138, 0xF, 0xF, false);  // wave_shr:1, lane 0 keeps -1
  // lanes without an entry carry a row of their own (a dummy row, or -2 - lane where acc has none):
  // distinct from each other and from the -1 that lane 0 sees below it, so the comparison alone
  // tells a continued run
  const bool same_as_prev = r_up == r;
  const uint64_t dup = __builtin_amdgcn_ballot_w64(same_as_prev);
  if (dup == 0) {
    if (valid) acc[r] += v;
    return;
  }
  if ((dup & (dup << 1)) == 0) {
    // runs of exactly two (the usual case on short rows): the first lane takes
    // its neighbour's value, three DPP wave shifts in all
    const T v_next = dpp_mov<0x130>(v);  // wave_shl:1: value of lane + 1 (0 past the end)
    if ((dup >> 1 >> lane) & 1) v += v_next;
    if (valid && !same_as_prev) acc[r] += v;
    return;
  }
  // first lane of my run: highest lane <= me whose dup bit is clear
  const uint64_t heads_below = ~dup & (((uint64_t)2 << lane) - 1);
  const int pos = lane - (63 - __builtin_clzll(heads_below));
  // a run longer than kMaxPasses shows as kMaxPasses consecutive dup bits
  uint64_t longrun = dup;
#pragma unroll
  for (int p = 1; p < kMaxPasses; ++p) longrun &= dup >> p;
  if (longrun == 0) {
#pragma unroll
    for (int p = 0; p < kMaxPasses; ++p) {
      if (p > 0 && __builtin_amdgcn_ballot_w64(valid && pos == p) == 0) break;
      if (valid && pos == p) acc[r] += v;
    }
    return;
  }
  // suffix sums inside every run; lane + d belongs to my run iff the d dup bits above me are all set
  const uint64_t above = dup >> 1 >> lane;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const T vd = lane_down(v, d);
    const uint64_t need = ((uint64_t)1 << d) - 1;
    if ((above & need) == need) v += vd;
  }
  if (valid && !same_as_prev) acc[r] += v;
}

// H = entries per lane and tile: 2 takes tiles of up to kLongTile entries with red_slots tiles in flight,
// 1 takes tiles of up to kWave entries with twice as many in flight (for the same number of outstanding
// loads: where tiles are short -- wide values make narrow column blocks -- the loads of the second half
// would all come back empty, and the bytes in flight, which bound the speed, would halve).
template <typename T, int H>
__global__ __launch_bounds__(TileDims<T>::red_threads) void tiled_reduce_kernel(
    int m, int row_blocks, int col_blocks, const int* __restrict__ row_block_start,
    const TileRange* __restrict__ ranges, const unsigned short* __restrict__ t_row,
    const T* __restrict__ prod, T alpha, T beta, T* __restrict__ y, const int* __restrict__ skip) {
  if (skip && *skip) return;  // the caller's guard found that the layout no longer describes the matrix
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_acc = reinterpret_cast<T*>(smem);
  constexpr int kTileRows = TileDims<T>::rows;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int rb = blockIdx.x * TileDims<T>::red_waves + wave;
  if (rb >= row_blocks) return;  // wave-uniform
  T* acc = s_acc + wave * (kTileRows + kWave);
  for (int i = lane; i < kTileRows + kWave; i += kWave) acc[i] = T(0);

  // Wave-private accumulators.  Every tile listed in `ranges` has at most H * 64 entries: H per lane.
  // The wave keeps kSlots tiles in flight in a ring of registers: step s adds the tile in slot s
  // and at once loads the tile kSlots further on into it, so the loads of the next kSlots - 1 tiles are
  // outstanding while one tile goes through its LDS read-modify-writes.  For the hardware counter of
  // outstanding loads to allow that, every load is issued unconditionally (the compiler can only
  // wait for "all but the N newest" when N is certain; lanes past the end of a tile are cut off by
  // the buffer range check and masked when the slot is used).  The waves of a workgroup
  // share no data and meet at no barrier: with one batch of 8 tiles in flight a barrier per batch kept
  // their reads on neighbouring tiles and doubled the speed, with the ring it measured no different.
  constexpr int kSlots = TileDims<T>::red_slots * (H == 1 ? 2 : 1);
  static_assert(H == 1 || H == 2, "one or two entries per lane");
  static_assert(kWave % kSlots == 0, "a group of tile ranges is a whole number of rings");
  T sv[kSlots][H];
  int sr[kSlots][H];
  int slen[kSlots];
  const TileRange* my = ranges + (int64_t)rb * col_blocks;
  auto load_ranges = [&](int group) {  // 64 tile ranges, one coalesced load
    // no select on the loaded value (it would wait for the load at once): tiles past col_blocks are
    // cut off in issue()
    const int cb = group * kWave + lane;
    return my[cb < col_blocks ? cb : 0];
  };
  const int r_none = kTileRows + lane;  // "no entry": the lane's dummy row behind the accumulators
  // the tile ranges of a group are loaded while the group before it is worked on
  TileRange tr = load_ranges(0);
  TileRange tr_next = load_ranges(1);
  // Buffer loads: the tile's two streams are described by resource words in scalar registers (base =
  // the tile's first entry, extent = the tile), the lane supplies a constant byte offset, and a
  // lane past the end of the tile gets zero from the hardware's range check without touching
  // memory: no address arithmetic and no masks in vector instructions.
  const int off_v = lane * (int)sizeof(T), off_r = lane * 2;
  auto issue = [&](int s, int ti) {  // tile ti (wave-uniform) -> slot s
    const int src = ti & (kWave - 1);
    const int b0 = __builtin_amdgcn_readlane(tr.begin, src);
    const int e0 = __builtin_amdgcn_readlane(tr.end, src);
    const int len = ti < col_blocks ? e0 - b0 : 0;
    slen[s] = len;
    const BufferRsrc rv = make_rsrc(prod + b0, len * (int)sizeof(T));
    const BufferRsrc rr = make_rsrc(t_row + b0, len * 2);
    sv[s][0] = buffer_load<T>(rv, off_v);
    sr[s][0] = buffer_load_u16(rr, off_r);
    if constexpr (H == 2) {
      sv[s][1] = buffer_load<T>(rv, off_v + kWave * (int)sizeof(T));
      sr[s][1] = buffer_load_u16(rr, off_r + kWave * 2);
    }
  };
  auto consume = [&](int s) {
    const int len = slen[s];
    // a lane without an entry holds value zero already; its row becomes the lane's dummy row
    add_rows<true>(acc, lane < len ? sr[s][0] : r_none, sv[s][0], true);
    if constexpr (H == 2) {
      if (len > kWave)  // wave-uniform
        add_rows<true>(acc, lane + kWave < len ? sr[s][1] : r_none, sv[s][1], true);
    }
  };
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    issue(s, s);
    // in slot order: the loop's first wait is for slot 0, and the count of loads that may stay
    // outstanding at that wait is the smaller of what the two ways into the loop guarantee
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int t0 = 0; t0 < col_blocks; t0 += kSlots) {
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      consume(s);
      const int ti = t0 + s + kSlots;
      if (s == 0 && (ti & (kWave - 1)) == 0) {  // ti is a multiple of kSlots here: groups change at s == 0 only
        tr = tr_next;
        tr_next = load_ranges(ti / kWave + 1);
      }
      issue(s, ti);
    }
  }
  const int64_t row0 = row_block_start[rb];
  const int nrows = row_block_start[rb + 1] - (int)row0;  // <= kTileRows
  for (int i = lane; i < nrows; i += kWave) store_axpby_nt(y, row0 + i, alpha, acc[i], beta);
}

// ---- phase 3 -------------------------------------------------------------------
// One workgroup per row block that has tiles too long for phase 2 (several, each with a run of the tiles,
// where the block has more than kLongPart such entries: a few hub rows can hold a good part of a power-law
// matrix).  The long tiles (in column block order) are dealt to the workgroup's waves in pieces of 256 entries; every wave
// streams its pieces and adds them into accumulators of its own in LDS (as phase 2 does: equal rows inside
// one instruction are combined first), then the waves' accumulators are added in wave order and
// y[row] += alpha * sum -- or, for a row block with several workgroups, the sums go to a scratch array and
// tiled_long_finish_kernel adds them up in part order.  Which wave takes which piece and the order of every
// addition are fixed by the layout: no atomics, results identical from run to run.  Runs after phase 2 has
// written y = beta*y + alpha*acc.
template <typename T>
__global__ __launch_bounds__(kLongThreads) void tiled_long_kernel(
    const LongBlock* __restrict__ blocks, const LongTile* __restrict__ tiles, const unsigned short* __restrict__ t_row,
    const T* __restrict__ prod, T alpha, T* __restrict__ y, T* __restrict__ scratch, int rows_cap,
    const int* __restrict__ skip) {
  if (skip && *skip) return;
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int kWaves = kLongThreads / kWave;
  // every wave's accumulators (rows_cap of them: no row block of this launch has more rows), then one dummy
  // row per lane
  const int kTileRows = rows_cap;
  const int kStride = kTileRows + kWave;
  T* s_acc = reinterpret_cast<T*>(smem);
  const LongBlock lb = blocks[blockIdx.x];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  T* acc = s_acc + wave * kStride;
  for (int i = lane; i < kStride; i += kWave) acc[i] = T(0);
  const int r_none = kTileRows + lane;
  constexpr int kU = 4;
  for (int t = lb.first; t < lb.first + lb.count; ++t) {
    const int begin = tiles[t].begin, end = tiles[t].end;
    // pieces of 64 * kU consecutive entries go to the waves in turn; the turn carries on from tile to tile
    // (tile t starts with wave t mod kWaves), so that short tiles do not all land on the first waves
    const int lead = (wave - (t - lb.first) % kWaves + kWaves) % kWaves;
    for (int k0 = begin + lead * (kWave * kU); k0 < end; k0 += kWaves * kWave * kU) {
      if (k0 + kWave * kU <= end) {
        T v[kU];
        int r[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          v[u] = prod[k0 + u * kWave + lane];
          r[u] = t_row[k0 + u * kWave + lane];
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) add_rows<true>(acc, r[u], v[u], true);
      } else {
        for (int k1 = k0; k1 < end; k1 += kWave) {  // wave-uniform trip count
          const int k = k1 + lane;
          const bool ok = k < end;
          add_rows<true>(acc, ok ? (int)t_row[k] : r_none, ok ? prod[k] : T(0), true);
        }
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < lb.nrows; i += kLongThreads) {
    T sum = s_acc[i];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += s_acc[w * kStride + i];
    if (lb.out < 0) y[(int64_t)lb.row0 + i] += alpha * sum;
    else scratch[(int64_t)lb.out + i] = sum;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void tiled_long_finish_kernel(const LongFinish* __restrict__ fin,
                                                                const T* __restrict__ scratch, T alpha,
                                                                T* __restrict__ y, const int* __restrict__ skip) {
  if (skip && *skip) return;
  const LongFinish f = fin[blockIdx.x];
  for (int i = threadIdx.x; i < f.nrows; i += 256) {
    T sum = scratch[(int64_t)f.out0 + i];
    for (int p = 1; p < f.parts; ++p) sum += scratch[(int64_t)f.out0 + (int64_t)p * f.nrows + i];
    y[(int64_t)f.row0 + i] += alpha * sum;
  }
}

}  // namespace asamd
