// The tiled two-phase layout of a CSR matrix and the launcher of its kernels (gfx950, wave64).
//
// asamd_tiled_build cuts the matrix into (column block x row block) tiles that hold about the same number
// of entries each, sorts the entries by tile (stable: CSR order inside a tile, so the layout and every sum
// formed from it are the same from run to run) and leaves the arrays of both phases in that order.  The
// reference has no counterpart: its analysis builds CSR-adaptive row blocks on the host
// (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267) that no kernel reads.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <vector>

#include "alsparse_amd_kernels.h"
#include "launch_utils.hpp"
#include "spmv_tiled.hpp"
#include "tile_sort.hpp"

using namespace asamd;

// dst[i] = src[i * stride]
__global__ __launch_bounds__(256) void strided_gather_kernel(int count, const int* __restrict__ src, int64_t stride,
                                                             int* __restrict__ dst) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < count) dst[i] = src[(int64_t)i * stride];
}

// Cuts groups [0, groups) with cumulative entry counts off[0..groups] into
// consecutive blocks of at most max_groups groups holding about `target`
// entries each.  group_block[g] = block of group g; returns the block starts
// (in groups), the last element being `groups`.
static std::vector<int> cut_blocks(const int* off, int groups, int max_groups, int64_t target,
                                   std::vector<int>& group_block) {
  std::vector<int> start;
  group_block.resize((size_t)groups);
  int g = 0;
  while (g < groups) {
    start.push_back(g);
    int e = g + 1;  // a block holds at least one group
    while (e < groups && e - g < max_groups && (int64_t)off[e + 1] - off[g] <= target) ++e;
    for (int i = g; i < e; ++i) group_block[(size_t)i] = (int)start.size() - 1;
    g = e;
  }
  start.push_back(groups);
  return start;
}

template <typename T>
static void launch_gather_tiles(hipStream_t s, const asamd_tiled_layout* L, const void* val, const int32_t* gate) {
  // eight tiles to a wave at a time, eight workgroups abreast (one per XCD), as many as the chip holds at once
  const int64_t per_xcd = ((int64_t)(L->row_blocks + 7) / 8) * ((L->col_blocks + 7) / 8);
  int64_t grid = (per_xcd + 3) / 4 * 8;
  if (grid > 8 * 512) grid = 8 * 512;
  gather_values_tiles_kernel<T, false><<<(unsigned)grid, 256, 0, s>>>(L->tperm, (const T*)val, (T*)L->tval, L->tile_ptr,
                                                                     L->col_blocks, L->row_blocks, gate);
}

// Equal-entry column / row blocks, stable sort of the entries by (column block,
// row block), then the arrays of both phases in that order and the tile tables.
template <typename T>
static hipError_t build_tiled(hipStream_t stream, asamd_tiled_layout* L, const int m, const int n, const int nnz_i,
                              const int base, const int max_len, const int force_halves, const int* row_ptr,
                              const int* col_ind, const T* val) {
  const size_t nnz = (size_t)nnz_i;
  const int col_groups = (int)(((int64_t)n + (1 << kColGroupLog2) - 1) >> kColGroupLog2);
  const int row_groups = (int)(((int64_t)m + (1 << kRowGroupLog2) - 1) >> kRowGroupLog2);

  int *d_coo = nullptr, *d_tile_ptr = nullptr, *d_long_count = nullptr, *d_cnt = nullptr;
  unsigned long long* d_mid = nullptr;
  // share of the entries that may sit in tiles of 65..128 entries for phase 2 to run one entry per lane
  // (every such tile then costs a phase-3 workgroup of its own)
  constexpr double kMidShare = 0.01;
  int *d_cgb = nullptr, *d_rgb = nullptr, *d_cbs = nullptr;
  LongTile* d_long_raw = nullptr;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr, *d_perm = nullptr;
  std::vector<int> h_off, cgb, rgb, cstart, rstart, h_colptr;
  int* h_cnt = nullptr;  // pinned
  char* d_arena = nullptr;
  std::vector<TiledChunk> h_chunks;
  int cb = 0, rb = 0, count_stride = 1;
  int64_t tiles = 0;

  // ---- 1. entry counts per column group and per row group -> block cuts ----------
  const size_t cnt_n = (size_t)(col_groups > row_groups ? col_groups : row_groups) + 1;
  hipError_t e = hipMalloc(&d_cnt, cnt_n * sizeof(int));
  if (e == hipSuccess) e = hipMemsetAsync(d_cnt, 0, cnt_n * sizeof(int), stream);
  if (e == hipSuccess) {
    // at least ~4 M sampled entries
    while (((int64_t)nnz_i >> 23) >= (int64_t)2 * count_stride) count_stride *= 2;
    col_group_count_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, col_ind, base, count_stride, d_cnt);
    h_off.resize(cnt_n + 1);
    // The counts travel to pinned host memory through a kernel that writes there: a device-to-host copy of
    // these 256 KB goes to the copy engine, and the first such copy after a pause took 6.4 ms here with the GPU
    // idle (the 1 MB copy right behind it 0.2 ms).
    e = hipHostMalloc((void**)&h_cnt, cnt_n * sizeof(int), hipHostMallocDefault);
    if (e == hipSuccess) {
      strided_gather_kernel<<<(unsigned)((col_groups + 255) / 256), 256, 0, stream>>>(col_groups, d_cnt, 1, h_cnt);
      e = hipGetLastError();
    }
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) {
    h_off[0] = 0;
    for (int g = 0; g < col_groups; ++g) h_off[(size_t)g + 1] = h_off[(size_t)g] + h_cnt[(size_t)g];
    // Width of a column block: at most TileDims<T>::cols (the x slice of phase 1).  A row block cannot be
    // shorter than one group of 64 rows, whose tiles hold 64 * entries per row / column blocks entries on
    // average: where the rows are so long that this exceeds 64 the column blocks are made narrower
    // (2 M x 2 M with 128 entries per row: 65 blocks -> 128).
    int col_max_groups = TileDims<T>::cols >> kColGroupLog2;
    int64_t full = ((int64_t)n + TileDims<T>::cols - 1) / TileDims<T>::cols;
    const double mean_len = (double)nnz_i / (double)(m > 0 ? m : 1);
    if (mean_len > (double)full) {
      const int64_t width = (int64_t)((double)n / mean_len);
      col_max_groups = width < (2 << kColGroupLog2) ? 1 : (int)(width >> kColGroupLog2);
      full = ((int64_t)n + ((int64_t)col_max_groups << kColGroupLog2) - 1) / ((int64_t)col_max_groups << kColGroupLog2);
    }
    cstart = cut_blocks(h_off.data(), col_groups, col_max_groups,
                        (int64_t)h_off[(size_t)col_groups] / full + 1, cgb);  // h_off: sampled entries
    cb = (int)cstart.size() - 1;
    row_group_offsets_kernel<<<(row_groups + 1 + 255) / 256, 256, 0, stream>>>(m, row_ptr, row_groups, d_cnt);
    strided_gather_kernel<<<(unsigned)((row_groups + 1 + 255) / 256), 256, 0, stream>>>(row_groups + 1, d_cnt, 1, h_cnt);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) {
    for (int g = 0; g <= row_groups; ++g) h_off[(size_t)g] = h_cnt[(size_t)g] - base;
    // Height of a row block: at most TileDims<T>::rows (the accumulators of a wave).  Phase 2 takes tiles
    // of up to 128 entries and longer ones go to the slow long-tile kernel: where the column blocks are
    // few (a narrow matrix) or the rows long, a full-height block would put more than that into most
    // tiles, so the height is cut to leave a tile about 64 entries on average (only if that takes a
    // quarter off or more: up to 85 entries on average still fit).
    // Phase 2 runs one row block per wave and the chip holds a fixed number of its waves at a time (the
    // accumulators fill the LDS): N blocks take ceil(N / slots) rounds, so 2.01 rounds of blocks cost three.
    // With even rows (the height decides every block, and a wave's time follows its entries) the blocks
    // are made just short enough to fill a whole number of rounds: 4-9 % on 5-10 M rows.  Not with skewed
    // rows: their waves are bound by the number of tiles they walk, and shorter blocks lost 20 % there.
    const int group_rows = 1 << kRowGroupLog2;
    int max_groups = TileDims<T>::rows >> kRowGroupLog2;
    const double per_row = (double)nnz_i / (double)(m > 0 ? m : 1);
    const double fit_rows = 64.0 * (double)cb / (per_row > 1e-9 ? per_row : 1e-9);
    if (fit_rows < 0.75 * max_groups * group_rows) max_groups = fit_rows < group_rows ? 1 : (int)(fit_rows / group_rows);
    int64_t full = ((int64_t)m + (int64_t)max_groups * group_rows - 1) / ((int64_t)max_groups * group_rows);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int64_t slots = (int64_t)cus * TileDims<T>::red_waves * (kLdsPerCu / TileDims<T>::red_lds_bytes);
    const bool even_rows = (double)max_len <= 3.0 * per_row + 16.0;
    if (even_rows && full > slots && full % slots != 0) {
      const int64_t want = (full + slots - 1) / slots * slots;
      const int64_t rows_each = ((int64_t)m + want - 1) / want;
      max_groups = (int)((rows_each + group_rows - 1) / group_rows);
      full = ((int64_t)m + (int64_t)max_groups * group_rows - 1) / ((int64_t)max_groups * group_rows);
    }
    // the entry limit is for skewed rows; with even rows the height decides: the mean content of a block
    // of full height plus 6 % always fits (random row lengths of mean 16 vary by 0.6 % per block, and every
    // block that the entry limit cuts short adds one to a count that otherwise fills whole rounds of waves)
    const int64_t even = (int64_t)((double)max_groups * group_rows * per_row * 1.0625) + 1;
    const int64_t row_target = std::max<int64_t>((int64_t)nnz_i / full + 1, even);
    rstart = cut_blocks(h_off.data(), row_groups, max_groups, row_target, rgb);
    rb = (int)rstart.size() - 1;
    tiles = (int64_t)cb * rb;
    if (cb > kTiledMaxColBlocks || tiles > kTiledMaxTiles) e = hipErrorNotSupported;  // "no tiled copy": not an error
  }
  L->col_blocks = cb;
  L->row_blocks = rb;
  unsigned key_bits = 1;
  while (((int64_t)1 << key_bits) < tiles) ++key_bits;

  // block starts in columns / rows
  std::vector<int> h_cbs((size_t)cb + 1), h_rbs((size_t)rb + 1);
  if (e == hipSuccess) {
    for (int c = 0; c <= cb; ++c) {
      const int64_t v = (int64_t)cstart[(size_t)c] << kColGroupLog2;
      h_cbs[(size_t)c] = (int)(v < n ? v : n);
    }
    for (int r = 0; r <= rb; ++r) {
      const int64_t v = (int64_t)rstart[(size_t)r] << kRowGroupLog2;
      h_rbs[(size_t)r] = (int)(v < m ? v : m);
    }
  }
  if (e == hipSuccess) e = hipMalloc(&d_cgb, (size_t)col_groups * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_rgb, (size_t)row_groups * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_cbs, ((size_t)cb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&L->row_block_start, ((size_t)rb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMemcpy(d_cgb, cgb.data(), (size_t)col_groups * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d_rgb, rgb.data(), (size_t)row_groups * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d_cbs, h_cbs.data(), ((size_t)cb + 1) * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess)
    e = hipMemcpy(L->row_block_start, h_rbs.data(), ((size_t)rb + 1) * sizeof(int), hipMemcpyHostToDevice);

  // ---- 2. sort the entries by tile, gather the tile-ordered arrays ---------------
  // 4-byte values: the local indices are sorted together with the keys (64-bit payloads that also carry
  // the entry's position); wider ones through a permutation alone
  constexpr bool kPayloadSort = sizeof(T) == 4;
  constexpr size_t kSortValBytes = kPayloadSort ? sizeof(unsigned long long) : sizeof(unsigned);
  const size_t long_cap = nnz / kWave + 1;  // a long tile holds more than kWave entries, at the least
  // (the pass's large temporaries in ONE allocation: an allocation of this size and its release cost 0.6 ms)
  if (e == hipSuccess) {
    const auto room = [](size_t bytes) { return (bytes + 255) / 256 * 256; };
    const size_t perm_bytes = kPayloadSort ? room(nnz * kSortValBytes) : 0;  // else it stays with the layout
    e = hipMalloc(&d_arena, 3 * room(nnz * sizeof(int)) + room(nnz * kSortValBytes) + perm_bytes +
                                room(long_cap * sizeof(LongTile)));
    if (e == hipSuccess) {
      char* at = d_arena;
      const auto take = [&](size_t bytes) {
        char* p = at;
        at += room(bytes);
        return (void*)p;
      };
      d_coo = (int*)take(nnz * sizeof(int));
      d_key = (unsigned*)take(nnz * sizeof(unsigned));
      d_key2 = (unsigned*)take(nnz * sizeof(unsigned));
      d_idx = (unsigned*)take(nnz * kSortValBytes);
      if (kPayloadSort) d_perm = (unsigned*)take(nnz * kSortValBytes);
      d_long_raw = (LongTile*)take(long_cap * sizeof(LongTile));
    }
  }
  if (e == hipSuccess && !kPayloadSort) e = hipMalloc(&d_perm, nnz * kSortValBytes);
  if (e == hipSuccess) e = hipMalloc(&d_tile_ptr, (size_t)(tiles + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&L->ranges, (size_t)tiles * sizeof(TileRange));
  if (e == hipSuccess) e = hipMalloc(&d_long_count, sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_mid, sizeof(unsigned long long));
  if (e == hipSuccess) e = hipMalloc(&L->tval, nnz * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&L->tcol, nnz * sizeof(unsigned short));
  if (e == hipSuccess) e = hipMalloc(&L->trow, nnz * sizeof(unsigned short));
  // d_key2 is free until the sort: it serves csr2coo as its table of chunk rows
  if (e == hipSuccess)
    e = (hipError_t)asamd_csr2coo_ws(stream, row_ptr, nnz_i, m, d_coo, base, d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    if constexpr (kPayloadSort) {
      tile_keys_payload_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, d_coo, col_ind, base, d_cgb,
                                                             d_cbs, d_rgb, L->row_block_start, rb, d_key,
                                                             (unsigned long long*)d_idx);
      e = sort_pairs_u32_u64(stream, d_key, d_key2, (unsigned long long*)d_idx, (unsigned long long*)d_perm, nnz, key_bits);
    } else {
      tile_keys_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, d_coo, col_ind, base, d_cgb, d_rgb, rb, d_key, d_idx);
      e = sort_pairs_u32(stream, d_key, d_key2, d_idx, d_perm, nnz, key_bits);
    }
  }
  if (e == hipSuccess && kPayloadSort) e = hipMalloc(&L->tperm, nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    if constexpr (kPayloadSort) {
      tile_unpack_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, (const unsigned long long*)d_perm, L->tperm,
                                                       L->tcol, L->trow);
    } else {
      tile_gather_kernel<T><<<256 * 32, 256, 0, stream>>>(nnz_i, d_perm, d_coo, col_ind, val, base, d_cgb, d_cbs,
                                                          d_rgb, L->row_block_start, (T*)L->tval,
                                                          L->tcol, L->trow);
      L->tperm = d_perm;  // the sorted permutation stays with the plan
      d_perm = nullptr;
    }
    tile_bounds_kernel<<<(unsigned)((tiles + 1 + 255) / 256), 256, 0, stream>>>(nnz_i, d_key2, tiles,
                                                                                d_tile_ptr);
    if constexpr (kPayloadSort) {
      L->tile_ptr = d_tile_ptr;  // stays with the layout: the values are gathered tile by tile, now and later
      launch_gather_tiles<T>(stream, L, val, nullptr);
    }
    // Entries in tiles of 65..128 entries: if they are few, phase 2 runs in its one-entry-per-lane form
    // (twice the tiles in flight) and leaves those tiles to phase 3.
    e = hipMemsetAsync(d_mid, 0, sizeof(unsigned long long), stream);
    tile_mid_entries_kernel<<<1024, 256, 0, stream>>>(tiles, d_tile_ptr, d_mid);
    unsigned long long h_mid = 0;
    if (e == hipSuccess) e = hipMemcpyAsync(&h_mid, d_mid, sizeof(h_mid), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    L->entries_per_lane = (double)h_mid <= kMidShare * (double)nnz_i ? 1 : 2;
    if (force_halves == 1 || force_halves == 2) L->entries_per_lane = force_halves;
    if (e == hipSuccess) e = hipMemsetAsync(d_long_count, 0, sizeof(int), stream);
    tile_ranges_kernel<<<(unsigned)((tiles + 255) / 256), 256, 0, stream>>>(
        rb, cb, L->entries_per_lane * kWave, d_tile_ptr, (TileRange*)L->ranges, d_long_raw, d_long_count);
    h_colptr.resize((size_t)cb + 1);
  }
  if (e == hipSuccess) {
    // column block c starts at tile_ptr[c * rb]: gathered on the device (d_cnt is free again and holds more
    // than cb + 1 ints), then one small copy -- a strided 2-D copy of these few hundred words took 22 ms
    strided_gather_kernel<<<(unsigned)((cb + 1 + 255) / 256), 256, 0, stream>>>(cb + 1, d_tile_ptr, (int64_t)rb, d_cnt);
    e = hipMemcpyAsync(h_colptr.data(), d_cnt, ((size_t)cb + 1) * sizeof(int), hipMemcpyDeviceToHost, stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);

  // ---- 3. tiles too long for phase 2: cut into phase-3 chunks ----------------------
  if (e == hipSuccess) {
    int n_long = 0;
    e = hipMemcpy(&n_long, d_long_count, sizeof(int), hipMemcpyDeviceToHost);
    std::vector<LongTile> h_long((size_t)(n_long > 0 ? n_long : 1));
    if (e == hipSuccess && n_long > 0)
      e = hipMemcpy(h_long.data(), d_long_raw, (size_t)n_long * sizeof(LongTile), hipMemcpyDeviceToHost);
    if (e == hipSuccess && n_long > 0) {
      // by row block; inside a row block by position, which is column block order
      std::sort(h_long.begin(), h_long.begin() + n_long, [](const LongTile& a, const LongTile& b) {
        return a.row_block != b.row_block ? a.row_block < b.row_block : a.begin < b.begin;
      });
      std::vector<LongBlock> h_lb;
      std::vector<LongFinish> h_fin;
      int64_t scratch_len = 0;
      int long_blocks = 0;
      for (int i = 0; i < n_long;) {
        int j = i;
        while (j < n_long && h_long[(size_t)j].row_block == h_long[(size_t)i].row_block) ++j;
        const int rbk = h_long[(size_t)i].row_block;
        const int row0 = h_rbs[(size_t)rbk], nrows = h_rbs[(size_t)rbk + 1] - h_rbs[(size_t)rbk];
        // runs of tiles with about kLongPart entries each
        const size_t first_part = h_lb.size();
        for (int t = i; t < j;) {
          int64_t entries = 0;
          int u = t;
          while (u < j && (u == t || entries + (h_long[(size_t)u].end - h_long[(size_t)u].begin) <= kLongPart)) {
            entries += h_long[(size_t)u].end - h_long[(size_t)u].begin;
            ++u;
          }
          h_lb.push_back(LongBlock{t, u - t, row0, nrows, -1});
          t = u;
        }
        const int parts = (int)(h_lb.size() - first_part);
        if (parts > 1) {
          h_fin.push_back(LongFinish{row0, nrows, (int)scratch_len, parts});
          for (int q = 0; q < parts; ++q) h_lb[first_part + (size_t)q].out = (int)(scratch_len + (int64_t)q * nrows);
          scratch_len += (int64_t)parts * nrows;
        }
        ++long_blocks;
        i = j;
      }
      // the narrow row blocks first: they are launched with small accumulators, so more of them share a compute unit
      std::stable_partition(h_lb.begin(), h_lb.end(), [](const LongBlock& b) { return b.nrows <= kLongNarrow; });
      L->n_long_narrow = 0;
      for (const LongBlock& b : h_lb) L->n_long_narrow += b.nrows <= kLongNarrow;
      if (scratch_len >= INT32_MAX) e = hipErrorOutOfMemory;
      L->n_long_chunks = (int)h_lb.size();
      L->n_long_finish = (int)h_fin.size();
      L->long_blocks = long_blocks;
      L->long_scratch_elems = scratch_len;  // the parts' sums meet in per-call scratch
      if (e == hipSuccess) e = hipMalloc(&L->long_list, h_lb.size() * sizeof(LongBlock));
      if (e == hipSuccess && !h_fin.empty()) {
        e = hipMalloc(&L->long_finish, h_fin.size() * sizeof(LongFinish));
        if (e == hipSuccess)
          e = hipMemcpy(L->long_finish, h_fin.data(), h_fin.size() * sizeof(LongFinish), hipMemcpyHostToDevice);
      }
      if (e == hipSuccess) e = hipMalloc(&L->long_tiles, (size_t)n_long * sizeof(LongTile));
      if (e == hipSuccess) e = hipMemcpy(L->long_list, h_lb.data(), h_lb.size() * sizeof(LongBlock), hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipMemcpy(L->long_tiles, h_long.data(), (size_t)n_long * sizeof(LongTile), hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)tiled_long_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (kLongThreads / kWave) * (TileDims<T>::rows + kWave) * (int)sizeof(T));
    }
  }
  // ---- 4. phase-1 work list: every column block cut into chunks of at most kChunk entries.  48 K entries
  // (the x slice, which neighbouring chunks find in the L2, is then loaded for every 288 KiB of fp32 streams)
  // measured best: 16 M x 16 M with 16 entries per row 0.553 ms with 128 K -> 0.511 ms, 2 M x 2 M 83 -> 69 us;
  // 32 K and 64 K were 3-4 % slower, equal shares for persistent workgroups no faster than 128 K.
  if (e == hipSuccess) {
    const int64_t kChunk = 48 * 1024;
    for (int c = 0; c < cb; ++c) {
      for (int64_t b = h_colptr[(size_t)c]; b < h_colptr[(size_t)c + 1]; b += kChunk) {
        TiledChunk ch;
        ch.col0 = h_cbs[(size_t)c];
        ch.ncols = h_cbs[(size_t)c + 1] - h_cbs[(size_t)c];
        ch.begin = (int)b;
        ch.end = (int)(b + kChunk < h_colptr[(size_t)c + 1] ? b + kChunk : h_colptr[(size_t)c + 1]);
        h_chunks.push_back(ch);
      }
    }
    L->n_chunks = (int)h_chunks.size();
    e = hipMalloc(&L->chunks, (h_chunks.size() ? h_chunks.size() : 1) * sizeof(TiledChunk));
    if (e == hipSuccess && !h_chunks.empty())
      e = hipMemcpy(L->chunks, h_chunks.data(), h_chunks.size() * sizeof(TiledChunk), hipMemcpyHostToDevice);
  }
  if (e == hipSuccess)  // both phases use more than the default 64 KiB of dynamic LDS
    e = hipFuncSetAttribute((const void*)tiled_products_kernel<T, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, kSliceBytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute((const void*)tiled_products_kernel<T, true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, kSliceBytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute((const void*)tiled_reduce_kernel<T, 1>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, TileDims<T>::red_lds_bytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute((const void*)tiled_reduce_kernel<T, 2>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, TileDims<T>::red_lds_bytes);
  if (h_cnt) (void)hipHostFree(h_cnt);
  if (L->tile_ptr == d_tile_ptr) d_tile_ptr = nullptr;
  if (kPayloadSort) d_perm = nullptr;  // part of the arena
  for (void* d : {(void*)d_arena, (void*)d_perm, (void*)d_tile_ptr, (void*)d_long_count, (void*)d_mid, (void*)d_cnt,
                  (void*)d_cgb, (void*)d_rgb, (void*)d_cbs})
    if (d) (void)hipFree(d);
  if (e != hipSuccess) {
    asamd_tiled_free(L);
    // too many blocks for the tile tables: the matrix simply gets no tiled copy (the record stays empty)
    return e == hipErrorNotSupported ? hipSuccess : e;
  }
  L->dtype = DtypeOf<T>::value;
  L->m = m;
  L->n = n;
  L->nnz = nnz_i;
  const int64_t tables = (int64_t)tiles * (int64_t)sizeof(TileRange) + ((int64_t)rb + 1) * 4 +
                         (L->tile_ptr ? ((int64_t)tiles + 1) * 4 : 0) +
                         (int64_t)L->n_chunks * (int64_t)sizeof(TiledChunk) +
                         (int64_t)L->n_long_chunks * (int64_t)sizeof(LongBlock) +
                         (int64_t)L->n_long_finish * (int64_t)sizeof(LongFinish);
  L->device_bytes = (int64_t)nnz * ((int64_t)sizeof(T) + 4 + 2 + 2) + tables;
  return hipSuccess;
}

extern "C" int asamd_tiled_fits(int32_t dtype, int32_t m, int32_t n, int32_t nnz) {
  return by_dtype(dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    // full-width block counts; the equal-entry cut (at most twice as many blocks per dimension) is checked
    // again once it is known
    const int64_t cb = ((int64_t)n + TileDims<T>::cols - 1) / TileDims<T>::cols;
    const int64_t rb = ((int64_t)m + TileDims<T>::rows - 1) / TileDims<T>::rows;
    if (m <= 0 || n <= 0 || 2 * cb > kTiledMaxColBlocks || cb * rb > kTiledMaxTiles / 2) return 0;
    // entry positions of the tiled copy are 32-bit and the kernels step past a range's end by up to
    // a workgroup's stride before they test it
    return (int64_t)nnz <= (int64_t)0x7fffffff - (1 << 16) && nnz > 0 ? 1 : 0;
  }) == 1;
}

extern "C" int asamd_tiled_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                                 const int32_t* row_ptr, const int32_t* col_ind, const void* val, int32_t max_len,
                                 int32_t entries_per_lane, asamd_tiled_layout* out) {
  if (!out) return hipErrorInvalidValue;
  *out = asamd_tiled_layout{};
  if (!row_ptr || !col_ind || !val || !asamd_tiled_fits(dtype, m, n, nnz)) return hipErrorInvalidValue;
  if ((uintptr_t)val % (size_t)dtype_size(dtype)) return hipErrorInvalidValue;
  return by_dtype(dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    return build_tiled<T>(stream, out, m, n, nnz, base, max_len, entries_per_lane, row_ptr, col_ind, (const T*)val);
  });
}

extern "C" void asamd_tiled_free(asamd_tiled_layout* L) {
  if (!L) return;
  free_all({L->tval, (void*)L->tperm, (void*)L->tcol, (void*)L->trow, (void*)L->row_block_start, (void*)L->tile_ptr,
            L->ranges, L->chunks,
            L->long_list, L->long_tiles, L->long_finish});
  *L = asamd_tiled_layout{};
}

// y = alpha*A*x + beta*y from the tiled arrays: phase 1 (products), phase 2 (per-wave row sums), phase 3
// (the tiles too long for phase 2) and its ordered finish.  The layout holds zero-based local indices and
// its own values.
extern "C" int asamd_spmv_tiled(hipStream_t s, const asamd_spmv_args* a, const asamd_tiled_layout* L, void* products,
                                void* long_scratch, const int32_t* skip) {
  if (!a || !L || !L->tval || !products || !a->alpha || !a->beta || !a->x || !a->y) return hipErrorInvalidValue;
  if (a->dtype != L->dtype || a->m != L->m || a->n != L->n || a->nnz != L->nnz) return hipErrorInvalidValue;
  if (L->n_long_finish > 0 && !long_scratch) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (((uintptr_t)a->x | (uintptr_t)a->y | (uintptr_t)products | (uintptr_t)long_scratch) % alignof(T))
      return hipErrorInvalidValue;
    const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
    const T* x = (const T*)a->x;
    T* y = (T*)a->y;
    T* prod = (T*)products;
    if (L->n_chunks > 0) {
      // products that the memory-side cache cannot hold anyway are stored past it
      if ((int64_t)L->nnz * (int64_t)sizeof(T) > ((int64_t)512 << 20))
        tiled_products_kernel<T, true><<<L->n_chunks, kProdThreads, kSliceBytes, s>>>(
            (const TiledChunk*)L->chunks, (const T*)L->tval, L->tcol, x, prod);
      else
        tiled_products_kernel<T, false><<<L->n_chunks, kProdThreads, kSliceBytes, s>>>(
            (const TiledChunk*)L->chunks, (const T*)L->tval, L->tcol, x, prod);
    }
    const unsigned red_grid = (unsigned)((L->row_blocks + TileDims<T>::red_waves - 1) / TileDims<T>::red_waves);
    if (L->entries_per_lane == 1)
      tiled_reduce_kernel<T, 1><<<red_grid, TileDims<T>::red_threads, TileDims<T>::red_lds_bytes, s>>>(
          L->m, L->row_blocks, L->col_blocks, L->row_block_start, (const TileRange*)L->ranges, L->trow, prod, alpha,
          beta, y, skip);
    else
      tiled_reduce_kernel<T, 2><<<red_grid, TileDims<T>::red_threads, TileDims<T>::red_lds_bytes, s>>>(
          L->m, L->row_blocks, L->col_blocks, L->row_block_start, (const TileRange*)L->ranges, L->trow, prod, alpha,
          beta, y, skip);
    if (L->n_long_chunks > 0) {
      const int waves = kLongThreads / kWave, narrow = L->n_long_narrow, wide = L->n_long_chunks - narrow;
      const LongBlock* list = (const LongBlock*)L->long_list;
      const LongTile* tiles = (const LongTile*)L->long_tiles;
      if (narrow > 0)
        tiled_long_kernel<T><<<narrow, kLongThreads, waves * (kLongNarrow + kWave) * (int)sizeof(T), s>>>(
            list, tiles, L->trow, prod, alpha, y, (T*)long_scratch, kLongNarrow, skip);
      if (wide > 0)
        tiled_long_kernel<T><<<wide, kLongThreads, waves * (TileDims<T>::rows + kWave) * (int)sizeof(T), s>>>(
            list + narrow, tiles, L->trow, prod, alpha, y, (T*)long_scratch, TileDims<T>::rows, skip);
    }
    if (L->n_long_finish > 0)
      tiled_long_finish_kernel<T><<<L->n_long_finish, 256, 0, s>>>((const LongFinish*)L->long_finish,
                                                                   (const T*)long_scratch, alpha, y, skip);
    return hipGetLastError();
  });
}

extern "C" int asamd_tiled_gather_values(hipStream_t s, const asamd_tiled_layout* L, const void* val,
                                         const int32_t* gate) {
  if (!L || !L->tval || !L->tperm || !val) return hipErrorInvalidValue;
  if (L->nnz == 0) return hipSuccess;
  if (!L->tile_ptr) return asamd_gather_values(s, L->dtype, 0, L->nnz, L->tperm, val, L->tval, gate);
  return by_dtype(L->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if ((uintptr_t)val % alignof(T)) return hipErrorInvalidValue;
    launch_gather_tiles<T>(s, L, val, gate);
    return hipGetLastError();
  });
}

// out[q] = val[perm[q]]: the values of a re-ordered copy taken afresh from the caller's array
extern "C" int asamd_gather_values(hipStream_t s, int32_t dtype, int32_t conj, int32_t nnz, const uint32_t* perm,
                                   const void* val, void* out, const int32_t* gate) {
  if (!perm || !val || !out || nnz < 0) return hipErrorInvalidValue;
  if (nnz == 0) return hipSuccess;
  return by_dtype(dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (((uintptr_t)val | (uintptr_t)out) % alignof(T)) return hipErrorInvalidValue;
    if (conj && kIsReal<T>) return hipErrorInvalidValue;
    int64_t grid = ((int64_t)nnz + 256 * 8 - 1) / (256 * 8);
    if (grid > 256 * 32) grid = 256 * 32;
    if constexpr (!kIsReal<T>) {
      if (conj) {
        gather_values_kernel<T, true><<<(unsigned)grid, 256, 0, s>>>(nnz, perm, (const T*)val, (T*)out, gate);
        return hipGetLastError();
      }
    }
    gather_values_kernel<T, false><<<(unsigned)grid, 256, 0, s>>>(nnz, perm, (const T*)val, (T*)out, gate);
    return hipGetLastError();
  });
}
