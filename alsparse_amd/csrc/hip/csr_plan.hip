// CSR analysis on the GPU and SpMV kernel dispatch for gfx950.
//
// asamd_csr_plan_create stands in for the reference's host-side, serial row
// block builder (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267 and
// its D2H/H2D round trip at :348-379): one pass over row_ptr on the device
// yields min/max row length and a log2 histogram, from which the kernel family
// is chosen; for the merge-path family the workgroup coordinates are computed
// by a second small kernel.  asamd_?_csrmv stands in for
// csr_gemv_vector_dispatch (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182).

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>

#include "alsparse_amd_kernels.h"
#include "spmv_ell.hpp"
#include "stream_policy.hpp"
#include "spmv_binned.hpp"
#include "spmv_hot.hpp"
#include "spmv_merge.hpp"
#include "spmv_rows.hpp"
#include "spmv_tiled.hpp"
#include "spmv_trans.hpp"
#include "tile_sort.hpp"

using namespace asamd;

// ---------------------------------------------------------------------------
// Row-length statistics.  out[0] = min, out[1] = max, out[2] = row_ptr[0],
// out[3 .. 3+2*33) = 64-bit histogram counters as (lo, hi) int pairs summed
// with 32-bit atomics on the low word only: a bin can hold at most m < 2^31.
// ---------------------------------------------------------------------------
constexpr int kStatWords = 3 + ASAMD_HIST_BINS;

__global__ __launch_bounds__(256) void row_stats_kernel(int m, const int* __restrict__ row_ptr,
                                                        int* __restrict__ out) {
  __shared__ int s_hist[ASAMD_HIST_BINS];
  __shared__ int s_min, s_max;
  if (threadIdx.x < ASAMD_HIST_BINS) s_hist[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    s_min = 0x7fffffff;
    s_max = 0;
  }
  __syncthreads();
  int lmin = 0x7fffffff, lmax = 0;
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < m;
       r += (int64_t)gridDim.x * blockDim.x) {
    int len = row_ptr[r + 1] - row_ptr[r];
    if (len < 0) len = 0;  // malformed offsets: counted as empty, never indexed with
    lmin = len < lmin ? len : lmin;
    lmax = len > lmax ? len : lmax;
    const int bin = len == 0 ? 0 : 32 - __builtin_clz((unsigned)len);
    atomicAdd(&s_hist[bin], 1);
  }
  atomicMin(&s_min, lmin);
  atomicMax(&s_max, lmax);
  __syncthreads();
  if (threadIdx.x < ASAMD_HIST_BINS && s_hist[threadIdx.x] != 0)
    atomicAdd(&out[3 + threadIdx.x], s_hist[threadIdx.x]);
  if (threadIdx.x == 0) {
    atomicMin(&out[0], s_min);
    atomicMax(&out[1], s_max);
    if (blockIdx.x == 0) out[2] = row_ptr[0];
  }
}

// dst[i] = src[i * stride]
__global__ __launch_bounds__(256) void strided_gather_kernel(int count, const int* __restrict__ src, int64_t stride,
                                                             int* __restrict__ dst) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < count) dst[i] = src[(int64_t)i * stride];
}

__global__ void stats_init_kernel(int* out) {
  const int t = threadIdx.x;
  if (t < kStatWords) out[t] = t == 0 ? 0x7fffffff : 0;
}

__global__ void warmup_kernel() {}

__global__ __launch_bounds__(256) void copy_bytes_kernel(Int4* __restrict__ dst,
                                                         const Int4* __restrict__ src, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// ---------------------------------------------------------------------------
struct asamd_csr_plan {
  asamd_csr_stats st;
  int auto_algo;
  int struct_algo = ASAMD_SPMV_MERGE;   // the choice from the row statistics alone (no copy involved)
  const void* copy_val_src = nullptr;   // the value array that the tiled / ELL copy was taken from
  int auto_width;
  int dtype;          // ASAMD_DTYPE_*: element type of the values
  int val_size;       // bytes per value
  int merge_ipt;      // items per thread of the merge-path kernel (4, 8 or 16)
  int* d_block_row;   // merge-path coordinates, merge_blocks + 1 ints
  int* d_carry_row;   // merge_blocks ints
  void* d_carry_val;  // merge_blocks values
  void* d_head_val;   // merge_blocks values: partial sum of each workgroup's first row
  bool coords_valid;  // d_block_row filled for a structure promised fixed
  // tiled two-phase copy (trusted plans only)
  int n_chunks;
  int* d_row_block_start;     // row_blocks + 1 first rows
  TileRange* d_ranges;        // row_blocks * col_blocks tile ranges, row block major
  LongBlock* d_long;          // phase-3 work list: the row blocks that have tiles too long for phase 2
  LongTile* d_long_tiles;     // ... and those tiles, sorted by row block, then by column block
  int n_long_chunks;          // workgroups of phase 3 (a row block with many long entries has several)
  int n_long_narrow;          // ... the first so many of them work on row blocks of at most kLongNarrow rows
  LongFinish* d_long_finish;  // the row blocks that have several, whose sums meet in d_long_scratch
  int n_long_finish;
  void* d_long_scratch;
  int tiled_halves;           // entries per lane and tile in phase 2: 2, or 1 where (nearly) all tiles are short
  void* d_tval;               // nnz values in tile order
  unsigned* d_tperm;          // nnz: CSR position of the entry in every tile-order slot (for refreshing d_tval)
  unsigned short* d_tcol;     // nnz local columns
  unsigned short* d_trow;     // nnz local rows
  void* d_tprod;              // nnz products (phase 1 -> phase 2)
  TiledChunk* d_chunks;       // phase-1 work list
  // hot-column copy (trusted plans of matrices whose entries crowd into few columns): structure only
  unsigned* d_pcol;           // nnz positions: rank of a hot column, or hot_cols + column
  int* d_hot_cols;            // hot_cols zero-based columns, most popular first
  void* d_xhot;               // their x, gathered by every multiply
  int hot_blocks;             // wave-sized merge blocks of the hot-column kernel, with their coordinates
  int* d_hot_block_row;       // hot_blocks + 1
  int* d_hot_carry_row;       // hot_blocks
  void* d_hot_carry_val;      // hot_blocks values
  void* d_hot_head_val;       // hot_blocks values
  // row-length bins (trusted plans of very uneven rows): structure only
  int* d_bin_rows;            // m row numbers sorted by length class, ascending inside a class
  int bin_count[kBinClasses]; // rows per class
  int bin_chunks;             // chunks that the rows of the last class are cut into
  BinChunk* d_bin_chunk;      // bin_chunks
  int* d_bin_first;           // bin_count[3] + 1: first chunk of every long row
  void* d_bin_partial;        // bin_chunks values
  // ELL copy (trusted plans of short, nearly equal rows)
  void* d_eval;               // ell_width * m values, column-major
  int* d_ecol;                // ... and zero-based columns
  // CSR copies of the transpose [0] and of the conjugate transpose [1] (trusted plans, on
  // request), each with a plan of its own
  struct TransCopy {
    asamd_csr_plan* plan;
    int* d_row_ptr;           // n + 1
    int* d_col;               // nnz zero-based rows of A
    void* d_val;              // nnz values (conjugated in copy [1])
    unsigned* d_perm;         // nnz: CSR position of every entry of the copy (for refreshing d_val)
    const void* val_src;      // the value array that d_val was gathered from
  } tr[2];
  bool lazy_transpose;        // build a copy on the first transposed multiply
};

// element type <-> tag
template <typename T> struct DtypeOf;
template <> struct DtypeOf<float> { static constexpr int value = ASAMD_DTYPE_FLOAT; };
template <> struct DtypeOf<double> { static constexpr int value = ASAMD_DTYPE_DOUBLE; };
template <> struct DtypeOf<Cx<float>> { static constexpr int value = ASAMD_DTYPE_FLOAT_COMPLEX; };
template <> struct DtypeOf<Cx<double>> { static constexpr int value = ASAMD_DTYPE_DOUBLE_COMPLEX; };
template <typename T>
constexpr bool kIsReal = std::is_floating_point<T>::value;

// calls f with a null pointer of the plan's element type: f's parameter type names T
template <typename F>
static hipError_t by_dtype(int dtype, F&& f) {
  switch (dtype) {
    case ASAMD_DTYPE_FLOAT: return f((float*)nullptr);
    case ASAMD_DTYPE_DOUBLE: return f((double*)nullptr);
    case ASAMD_DTYPE_FLOAT_COMPLEX: return f((Cx<float>*)nullptr);
    case ASAMD_DTYPE_DOUBLE_COMPLEX: return f((Cx<double>*)nullptr);
    default: return hipErrorInvalidValue;
  }
}

static bool is_complex(const asamd_csr_plan* p) { return p->dtype >= ASAMD_DTYPE_FLOAT_COMPLEX; }

static int width_for_mean(double mean) {
  // lanes per row from the mean row length; same break points as the
  // reference's dispatch (dcu_gemv_vector.h:77,94,111,128,145,162)
  if (mean < 4) return 2;
  if (mean < 8) return 4;
  if (mean < 16) return 8;
  if (mean < 32) return 16;
  if (mean < 64) return 32;
  return 64;
}

// rows plus entries below which one launch's latency outweighs the work
constexpr int64_t kSmallWork = 1 << 17;

static bool rowconst_ok(const asamd_csr_plan* p) {
  const asamd_csr_stats& st = p->st;
  const int L = st.const_len;
  // the kernel loads four values as 128-bit pieces: real element types only
  return !is_complex(p) && st.trusted && st.first_offset == 0 &&
         (L == 4 || L == 8 || L == 16 || L == 32 || L == 64 || L == 128 || L == 256);
}

// The LDS-staged row-block kernel sizes its staging area for rows of at most CAP * G entries (G lanes sum a
// row); the bound comes from the row statistics.  A workgroup whose rows hold more than that (the structure
// behind row_ptr changed under a plan that was not promised a fixed one) takes them straight from global
// memory, so the choice is safe for such plans too.  Returns G, or 0 when the
// kernel cannot take the matrix.  With `regular_only`, also 0 for G > 1 when the rows are so much shorter than
// the longest that a workgroup's 256 / G rows hold fewer than four entries per thread.
// 16 KiB of products per workgroup: 16 entries per thread for 4-byte values, 8 for 8-byte, 4 for 16-byte ones
// (measured on a 27-point stencil, fp64: 32 KiB per workgroup 317 us, 16 KiB 295 us)
static int stream_cap(const asamd_csr_plan* p) { return 64 / p->val_size; }
static int stream_group(const asamd_csr_plan* p, bool regular_only) {
  const asamd_csr_stats& st = p->st;
  if (st.max_len < 1) return 0;
  const int cap = stream_cap(p);
  if (st.max_len <= cap) return 1;
  int g = 2;
  while (g * cap < st.max_len && g <= kStreamMaxGroup) g *= 2;
  if (g > kStreamMaxGroup) return 0;
  // regular: the mean row is at least a quarter of the longest row the kernel is sized for
  if (regular_only && (double)st.nnz / (double)st.m < 0.25 * g * cap) return 0;
  return g;
}
static bool stream_ok(const asamd_csr_plan* p) { return stream_group(p, false) > 0; }

static void choose_algo(asamd_csr_plan* p) {
  asamd_csr_stats& st = p->st;
  const double mean = st.m > 0 ? (double)st.nnz / st.m : 0.0;
  const int w = width_for_mean(mean);
  p->auto_width = w;
  if (st.first_offset != 0) {
    // row_ptr points into the middle of a larger array: only the kernels that index with the absolute
    // offsets (as the reference's csr_gemv_vector does) see the right entries; merge-path and csr2coo,
    // the source of every re-ordered copy, count entries from position 0
    p->auto_algo = stream_group(p, true) > 0 ? ASAMD_SPMV_STREAM : ASAMD_SPMV_VECTOR;
  } else if (rowconst_ok(p)) {
    p->auto_algo = ASAMD_SPMV_ROWCONST;
  } else if (stream_group(p, true) > 0) {
    // short rows, or rows of some tens of entries of similar lengths
    p->auto_algo = ASAMD_SPMV_STREAM;
  } else if ((int64_t)st.max_len <= (int64_t)w * 16 && mean >= 6.0) {
    // regular rows: a lane group per row wastes little and needs no LDS
    p->auto_algo = ASAMD_SPMV_VECTOR;
  } else if ((int64_t)st.m + st.nnz <= kSmallWork && (int64_t)st.max_len <= (int64_t)w * 64) {
    // a matrix this small is over in the time of one launch: the single
    // kernel beats the balanced path's two or three
    p->auto_algo = ASAMD_SPMV_VECTOR;
  } else {
    p->auto_algo = ASAMD_SPMV_MERGE;
  }
  p->struct_algo = p->auto_algo;
  st.algo = p->auto_algo;
  st.vector_width = p->auto_width;
}

template <typename T>
static int csrmv_impl(hipStream_t s, asamd_csr_plan* p, T alpha, const T* val, const int* rp,
                      const int* ci, const T* x, T beta, T* y);

static void free_tiled(asamd_csr_plan* p) {
  if (p->d_ranges) (void)hipFree(p->d_ranges);
  if (p->d_row_block_start) (void)hipFree(p->d_row_block_start);
  p->d_row_block_start = nullptr;
  if (p->d_long) (void)hipFree(p->d_long);
  if (p->d_long_tiles) (void)hipFree(p->d_long_tiles);
  if (p->d_long_finish) (void)hipFree(p->d_long_finish);
  if (p->d_long_scratch) (void)hipFree(p->d_long_scratch);
  p->d_long = nullptr;
  p->d_long_tiles = nullptr;
  p->d_long_finish = nullptr;
  p->d_long_scratch = nullptr;
  p->n_long_finish = 0;
  p->st.tile_long_blocks = 0;
  p->n_long_chunks = 0;
  p->tiled_halves = 2;
  if (p->d_tval) (void)hipFree(p->d_tval);
  if (p->d_tperm) (void)hipFree(p->d_tperm);
  p->d_tperm = nullptr;
  if (p->d_tcol) (void)hipFree(p->d_tcol);
  if (p->d_trow) (void)hipFree(p->d_trow);
  if (p->d_tprod) (void)hipFree(p->d_tprod);
  if (p->d_chunks) (void)hipFree(p->d_chunks);
  p->d_ranges = nullptr;
  p->d_tval = p->d_tprod = nullptr;
  p->d_tcol = p->d_trow = nullptr;
  p->d_chunks = nullptr;
  p->st.tiled_built = 0;
  p->st.tile_entries_per_lane = 0;
}

static void free_ell(asamd_csr_plan* p) {
  if (p->d_eval) (void)hipFree(p->d_eval);
  if (p->d_ecol) (void)hipFree(p->d_ecol);
  p->d_eval = nullptr;
  p->d_ecol = nullptr;
  p->st.ell_built = 0;
}

static void free_hot(asamd_csr_plan* p) {
  for (void* d : {(void*)p->d_pcol, (void*)p->d_hot_cols, p->d_xhot, (void*)p->d_hot_block_row,
                  (void*)p->d_hot_carry_row, p->d_hot_carry_val, p->d_hot_head_val})
    if (d) (void)hipFree(d);
  p->d_pcol = nullptr;
  p->d_hot_cols = nullptr;
  p->d_xhot = nullptr;
  p->d_hot_block_row = nullptr;
  p->d_hot_carry_row = nullptr;
  p->d_hot_carry_val = nullptr;
  p->d_hot_head_val = nullptr;
  p->hot_blocks = 0;
  p->st.hot_built = 0;
}

static void free_binned(asamd_csr_plan* p) {
  for (void* d : {(void*)p->d_bin_rows, (void*)p->d_bin_chunk, (void*)p->d_bin_first, p->d_bin_partial})
    if (d) (void)hipFree(d);
  p->d_bin_rows = nullptr;
  p->d_bin_chunk = nullptr;
  p->d_bin_first = nullptr;
  p->d_bin_partial = nullptr;
  p->bin_chunks = 0;
  p->st.binned_built = 0;
}

static void free_transpose(asamd_csr_plan* p, int which) {
  asamd_csr_plan::TransCopy& t = p->tr[which];
  if (t.plan) asamd_csr_plan_destroy(t.plan);
  if (t.d_row_ptr) (void)hipFree(t.d_row_ptr);
  if (t.d_col) (void)hipFree(t.d_col);
  if (t.d_val) (void)hipFree(t.d_val);
  if (t.d_perm) (void)hipFree(t.d_perm);
  t = asamd_csr_plan::TransCopy{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  p->st.transpose_built &= ~(1 << which);
}

// An ELL copy pays when rows are short and padding them to the longest costs
// little: the kernel then streams 4 + sizeof(T) bytes per entry at full width
// with neither row_ptr nor LDS staging.
static bool ell_eligible(const asamd_csr_stats& st, bool force) {
  if (!st.trusted || st.first_offset != 0 || st.max_len < 1 || st.max_len > 32) return false;
  const int64_t slots = (int64_t)st.m * st.max_len;
  if (slots >= ((int64_t)1 << 31) || slots > (int64_t)st.nnz + st.nnz / 8) return false;
  return force || st.nnz >= (1 << 18);
}

template <typename T>
static hipError_t build_ell(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr, const int* col_ind,
                            const T* val) {
  asamd_csr_stats& st = p->st;
  const size_t slots = (size_t)st.m * (size_t)st.max_len;
  hipError_t e = hipMalloc(&p->d_eval, slots * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&p->d_ecol, slots * sizeof(int));
  if (e == hipSuccess) {
    // the conversion copies values bit for bit and pads with zero bits: only the element size matters
    if constexpr (sizeof(T) == 4)
      e = (hipError_t)asamd_s_csr2ell(stream, st.m, (const float*)val, row_ptr, col_ind, st.base, 0, st.max_len,
                                      (float*)p->d_eval, p->d_ecol);
    else if constexpr (sizeof(T) == 8)
      e = (hipError_t)asamd_d_csr2ell(stream, st.m, (const double*)val, row_ptr, col_ind, st.base, 0, st.max_len,
                                      (double*)p->d_eval, p->d_ecol);
    else
      e = (hipError_t)asamd_z_csr2ell(stream, st.m, (const asamd_complex16*)val, row_ptr, col_ind, st.base, 0,
                                      st.max_len, (asamd_complex16*)p->d_eval, p->d_ecol);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    free_ell(p);
    return e;
  }
  st.ell_built = 1;
  st.ell_width = st.max_len;
  return hipSuccess;
}

template <typename T>
static bool tiled_eligible(const asamd_csr_stats& st, bool force) {
  // full-width block counts; the equal-entry cut (at most twice as many blocks
  // per dimension) is checked again once it is known
  const int64_t cb = ((int64_t)st.n + TileDims<T>::cols - 1) / TileDims<T>::cols;
  const int64_t rb = ((int64_t)st.m + TileDims<T>::rows - 1) / TileDims<T>::rows;
  if (!st.trusted || st.first_offset != 0 || 2 * cb > kTiledMaxColBlocks || cb * rb > kTiledMaxTiles / 2) return false;
  // entry positions of the tiled copy are 32-bit and the kernels step past a range's end by up to
  // a workgroup's stride before they test it
  if ((int64_t)st.nnz > (int64_t)0x7fffffff - (1 << 16)) return false;
  // worth a try only when x fills an XCD's 4 MiB L2 (the matrix streams through the same cache; with
  // 2 MiB of x the tiled pair measured 0.43 ms against 0.34 ms, with 4 MiB 0.084 against 0.095) and the
  // matrix is large; the timing run of the analysis has the last word
  return force || ((int64_t)st.n * (int64_t)sizeof(T) >= ((int64_t)4 << 20) && st.nnz >= (1 << 22));
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

// Equal-entry column / row blocks, stable sort of the entries by (column block,
// row block), then the arrays of both phases in that order and the tile tables.
template <typename T>
static hipError_t build_tiled(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr,
                              const int* col_ind, const T* val) {
  asamd_csr_stats& st = p->st;
  const size_t nnz = (size_t)st.nnz;
  const int col_groups = (int)(((int64_t)st.n + (1 << kColGroupLog2) - 1) >> kColGroupLog2);
  const int row_groups = (int)(((int64_t)st.m + (1 << kRowGroupLog2) - 1) >> kRowGroupLog2);

  int *d_coo = nullptr, *d_tile_ptr = nullptr, *d_long_count = nullptr, *d_cnt = nullptr;
  unsigned long long* d_mid = nullptr;
  // share of the entries that may sit in tiles of 65..128 entries for phase 2 to run one entry per lane
  // (every such tile then costs a phase-3 workgroup of its own)
  constexpr double kMidShare = 0.01;
  int *d_cgb = nullptr, *d_rgb = nullptr, *d_cbs = nullptr;
  LongTile* d_long_raw = nullptr;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr, *d_perm = nullptr;
  std::vector<int> h_off, cgb, rgb, cstart, rstart, h_colptr;
  std::vector<TiledChunk> h_chunks;
  int cb = 0, rb = 0, count_stride = 1;
  int64_t tiles = 0;

  // ---- 1. entry counts per column group and per row group -> block cuts ----------
  const size_t cnt_n = (size_t)(col_groups > row_groups ? col_groups : row_groups) + 1;
  hipError_t e = hipMalloc(&d_cnt, cnt_n * sizeof(int));
  if (e == hipSuccess) e = hipMemsetAsync(d_cnt, 0, cnt_n * sizeof(int), stream);
  if (e == hipSuccess) {
    // at least ~4 M sampled entries
    while (((int64_t)st.nnz >> 23) >= (int64_t)2 * count_stride) count_stride *= 2;
    col_group_count_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, col_ind, st.base, count_stride, d_cnt);
    h_off.resize(cnt_n + 1);
    e = hipMemcpyAsync(h_off.data() + 1, d_cnt, (size_t)col_groups * sizeof(int), hipMemcpyDeviceToHost, stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) {
    h_off[0] = 0;
    for (int g = 0; g < col_groups; ++g) h_off[(size_t)g + 1] += h_off[(size_t)g];
    // Width of a column block: at most TileDims<T>::cols (the x slice of phase 1).  A row block cannot be
    // shorter than one group of 64 rows, whose tiles hold 64 * entries per row / column blocks entries on
    // average: where the rows are so long that this exceeds 64 the column blocks are made narrower
    // (2 M x 2 M with 128 entries per row: 65 blocks -> 128).
    int col_max_groups = TileDims<T>::cols >> kColGroupLog2;
    int64_t full = ((int64_t)st.n + TileDims<T>::cols - 1) / TileDims<T>::cols;
    const double mean_len = (double)st.nnz / (double)(st.m > 0 ? st.m : 1);
    if (mean_len > (double)full) {
      const int64_t width = (int64_t)((double)st.n / mean_len);
      col_max_groups = width < (2 << kColGroupLog2) ? 1 : (int)(width >> kColGroupLog2);
      full = ((int64_t)st.n + ((int64_t)col_max_groups << kColGroupLog2) - 1) / ((int64_t)col_max_groups << kColGroupLog2);
    }
    cstart = cut_blocks(h_off.data(), col_groups, col_max_groups,
                        (int64_t)h_off[(size_t)col_groups] / full + 1, cgb);  // h_off: sampled entries
    cb = (int)cstart.size() - 1;
    row_group_offsets_kernel<<<(row_groups + 1 + 255) / 256, 256, 0, stream>>>(st.m, row_ptr, row_groups, d_cnt);
    e = hipMemcpyAsync(h_off.data(), d_cnt, ((size_t)row_groups + 1) * sizeof(int), hipMemcpyDeviceToHost, stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) {
    for (int g = 0; g <= row_groups; ++g) h_off[(size_t)g] -= st.base;
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
    const double per_row = (double)st.nnz / (double)(st.m > 0 ? st.m : 1);
    const double fit_rows = 64.0 * (double)cb / (per_row > 1e-9 ? per_row : 1e-9);
    if (fit_rows < 0.75 * max_groups * group_rows) max_groups = fit_rows < group_rows ? 1 : (int)(fit_rows / group_rows);
    int64_t full = ((int64_t)st.m + (int64_t)max_groups * group_rows - 1) / ((int64_t)max_groups * group_rows);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int64_t slots = (int64_t)cus * TileDims<T>::red_waves * (kLdsPerCu / TileDims<T>::red_lds_bytes);
    const bool even_rows = (double)st.max_len <= 3.0 * per_row + 16.0;
    if (even_rows && full > slots && full % slots != 0) {
      const int64_t want = (full + slots - 1) / slots * slots;
      const int64_t rows_each = ((int64_t)st.m + want - 1) / want;
      max_groups = (int)((rows_each + group_rows - 1) / group_rows);
      full = ((int64_t)st.m + (int64_t)max_groups * group_rows - 1) / ((int64_t)max_groups * group_rows);
    }
    // the entry limit is for skewed rows; with even rows the height decides: the mean content of a block
    // of full height plus 6 % always fits (random row lengths of mean 16 vary by 0.6 % per block, and every
    // block that the entry limit cuts short adds one to a count that otherwise fills whole rounds of waves)
    const int64_t even = (int64_t)((double)max_groups * group_rows * per_row * 1.0625) + 1;
    const int64_t row_target = std::max<int64_t>((int64_t)st.nnz / full + 1, even);
    rstart = cut_blocks(h_off.data(), row_groups, max_groups, row_target, rgb);
    rb = (int)rstart.size() - 1;
    tiles = (int64_t)cb * rb;
    if (cb > kTiledMaxColBlocks || tiles > kTiledMaxTiles) e = hipErrorNotSupported;  // "no tiled copy": not an error
  }
  st.tile_col_blocks = cb;
  st.tile_row_blocks = rb;
  unsigned key_bits = 1;
  while (((int64_t)1 << key_bits) < tiles) ++key_bits;

  // block starts in columns / rows
  std::vector<int> h_cbs((size_t)cb + 1), h_rbs((size_t)rb + 1);
  if (e == hipSuccess) {
    for (int c = 0; c <= cb; ++c) {
      const int64_t v = (int64_t)cstart[(size_t)c] << kColGroupLog2;
      h_cbs[(size_t)c] = (int)(v < st.n ? v : st.n);
    }
    for (int r = 0; r <= rb; ++r) {
      const int64_t v = (int64_t)rstart[(size_t)r] << kRowGroupLog2;
      h_rbs[(size_t)r] = (int)(v < st.m ? v : st.m);
    }
  }
  if (e == hipSuccess) e = hipMalloc(&d_cgb, (size_t)col_groups * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_rgb, (size_t)row_groups * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_cbs, ((size_t)cb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_row_block_start, ((size_t)rb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMemcpy(d_cgb, cgb.data(), (size_t)col_groups * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d_rgb, rgb.data(), (size_t)row_groups * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d_cbs, h_cbs.data(), ((size_t)cb + 1) * sizeof(int), hipMemcpyHostToDevice);
  if (e == hipSuccess)
    e = hipMemcpy(p->d_row_block_start, h_rbs.data(), ((size_t)rb + 1) * sizeof(int), hipMemcpyHostToDevice);

  // ---- 2. sort the entries by tile, gather the tile-ordered arrays ---------------
  if (e == hipSuccess) e = hipMalloc(&d_coo, nnz * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_key, nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, nnz * sizeof(unsigned));
  // 4-byte values: the local indices are sorted together with the keys (64-bit payloads that also carry
  // the entry's position); wider ones through a permutation alone
  constexpr bool kPayloadSort = sizeof(T) == 4;
  constexpr size_t kSortValBytes = kPayloadSort ? sizeof(unsigned long long) : sizeof(unsigned);
  if (e == hipSuccess) e = hipMalloc(&d_idx, nnz * kSortValBytes);
  if (e == hipSuccess) e = hipMalloc(&d_perm, nnz * kSortValBytes);
  if (e == hipSuccess) e = hipMalloc(&d_tile_ptr, (size_t)(tiles + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_ranges, (size_t)tiles * sizeof(TileRange));
  const size_t long_cap = nnz / kWave + 1;  // a long tile holds more than kWave entries, at the least
  if (e == hipSuccess) e = hipMalloc(&d_long_raw, long_cap * sizeof(LongTile));
  if (e == hipSuccess) e = hipMalloc(&d_long_count, sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_mid, sizeof(unsigned long long));
  if (e == hipSuccess) e = hipMalloc(&p->d_tval, nnz * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&p->d_tcol, nnz * sizeof(unsigned short));
  if (e == hipSuccess) e = hipMalloc(&p->d_trow, nnz * sizeof(unsigned short));
  if (e == hipSuccess) e = hipMalloc(&p->d_tprod, nnz * sizeof(T));
  // d_key2 is free until the sort: it serves csr2coo as its table of chunk rows
  if (e == hipSuccess)
    e = (hipError_t)asamd_csr2coo_ws(stream, row_ptr, st.nnz, st.m, d_coo, st.base, d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    if constexpr (kPayloadSort) {
      tile_keys_payload_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, d_coo, col_ind, st.base, d_cgb,
                                                             d_cbs, d_rgb, p->d_row_block_start, rb, d_key,
                                                             (unsigned long long*)d_idx);
      e = sort_pairs_u32_u64(stream, d_key, d_key2, (unsigned long long*)d_idx, (unsigned long long*)d_perm, nnz, key_bits);
    } else {
      tile_keys_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, d_coo, col_ind, st.base, d_cgb, d_rgb, rb, d_key, d_idx);
      e = sort_pairs_u32(stream, d_key, d_key2, d_idx, d_perm, nnz, key_bits);
    }
  }
  if (e == hipSuccess && kPayloadSort) e = hipMalloc(&p->d_tperm, nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    if constexpr (kPayloadSort) {
      tile_unpack_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, (const unsigned long long*)d_perm, p->d_tperm,
                                                       p->d_tcol, p->d_trow);
      gather_values_kernel<T, false><<<256 * 32, 256, 0, stream>>>(st.nnz, p->d_tperm, val, (T*)p->d_tval);
    } else {
      tile_gather_kernel<T><<<256 * 32, 256, 0, stream>>>(st.nnz, d_perm, d_coo, col_ind, val, st.base, d_cgb, d_cbs,
                                                          d_rgb, p->d_row_block_start, (T*)p->d_tval,
                                                          p->d_tcol, p->d_trow);
      p->d_tperm = d_perm;  // the sorted permutation stays with the plan
      d_perm = nullptr;
    }
    tile_bounds_kernel<<<(unsigned)((tiles + 1 + 255) / 256), 256, 0, stream>>>(st.nnz, d_key2, tiles,
                                                                                d_tile_ptr);
    // Entries in tiles of 65..128 entries: if they are few, phase 2 runs in its one-entry-per-lane form
    // (twice the tiles in flight) and leaves those tiles to phase 3.
    e = hipMemsetAsync(d_mid, 0, sizeof(unsigned long long), stream);
    tile_mid_entries_kernel<<<1024, 256, 0, stream>>>(tiles, d_tile_ptr, d_mid);
    unsigned long long h_mid = 0;
    if (e == hipSuccess) e = hipMemcpyAsync(&h_mid, d_mid, sizeof(h_mid), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    p->tiled_halves = (double)h_mid <= kMidShare * (double)st.nnz ? 1 : 2;
    if (const char* ev = getenv("ALSPARSE_AMD_TILED_HALVES")) {
      const int v = atoi(ev);
      if (v == 1 || v == 2) p->tiled_halves = v;
    }
    p->st.tile_entries_per_lane = p->tiled_halves;
    if (e == hipSuccess) e = hipMemsetAsync(d_long_count, 0, sizeof(int), stream);
    tile_ranges_kernel<<<(unsigned)((tiles + 255) / 256), 256, 0, stream>>>(
        rb, cb, p->tiled_halves * kWave, d_tile_ptr, p->d_ranges, d_long_raw, d_long_count);
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
      p->n_long_narrow = 0;
      for (const LongBlock& b : h_lb) p->n_long_narrow += b.nrows <= kLongNarrow;
      if (scratch_len >= INT32_MAX) e = hipErrorOutOfMemory;
      p->n_long_chunks = (int)h_lb.size();
      p->n_long_finish = (int)h_fin.size();
      st.tile_long_blocks = long_blocks;
      if (e == hipSuccess) e = hipMalloc(&p->d_long, h_lb.size() * sizeof(LongBlock));
      if (e == hipSuccess && !h_fin.empty()) {
        e = hipMalloc(&p->d_long_finish, h_fin.size() * sizeof(LongFinish));
        if (e == hipSuccess) e = hipMalloc(&p->d_long_scratch, (size_t)scratch_len * sizeof(T));
        if (e == hipSuccess)
          e = hipMemcpy(p->d_long_finish, h_fin.data(), h_fin.size() * sizeof(LongFinish), hipMemcpyHostToDevice);
      }
      if (e == hipSuccess) e = hipMalloc(&p->d_long_tiles, (size_t)n_long * sizeof(LongTile));
      if (e == hipSuccess) e = hipMemcpy(p->d_long, h_lb.data(), h_lb.size() * sizeof(LongBlock), hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipMemcpy(p->d_long_tiles, h_long.data(), (size_t)n_long * sizeof(LongTile), hipMemcpyHostToDevice);
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
    p->n_chunks = (int)h_chunks.size();
    e = hipMalloc(&p->d_chunks, (h_chunks.size() ? h_chunks.size() : 1) * sizeof(TiledChunk));
    if (e == hipSuccess && !h_chunks.empty())
      e = hipMemcpy(p->d_chunks, h_chunks.data(), h_chunks.size() * sizeof(TiledChunk), hipMemcpyHostToDevice);
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
  for (void* d : {(void*)d_coo, (void*)d_key, (void*)d_key2, (void*)d_idx, (void*)d_perm, (void*)d_tile_ptr,
                  (void*)d_long_raw, (void*)d_long_count, (void*)d_mid, (void*)d_cnt, (void*)d_cgb, (void*)d_rgb, (void*)d_cbs})
    if (d) (void)hipFree(d);
  if (e != hipSuccess) {
    free_tiled(p);
    // too many blocks for the tile tables: the matrix simply gets no tiled copy (tiled_built stays 0)
    return e == hipErrorNotSupported ? hipSuccess : e;
  }
  st.tiled_built = 1;
  return hipSuccess;
}

// The hot-column kernel pays when x is far larger than an XCD's L2 and yet most entries fall into a few
// columns (power-law graphs).  Whether they do is only known after counting (build_hot).
constexpr int kHotFrontBytes = 1 << 20;  // of every XCD's 4 MiB L2, beside the streams passing through
template <typename T>
struct HotKernel {
  // 4-byte values: 8 items per lane and 16 waves; 8-byte values: 4 items per lane (the staging areas of
  // 16 waves must leave room for the table)
  static constexpr int ipt = sizeof(T) == 4 ? 8 : 4;
  static constexpr int nw = 16;
  using Dims = HotDims<T, ipt, nw>;
};
template <typename T>
static bool hot_eligible(const asamd_csr_plan* p, bool force) {
  const asamd_csr_stats& st = p->st;
  if (sizeof(T) > 8 || !st.trusted || st.first_offset != 0 || st.nnz < 1 || st.n < 1) return false;
  // positions are 32-bit words, x is addressed through a buffer resource with 32-bit byte offsets
  if (((int64_t)st.n + (int64_t)kHotFrontBytes) >= (int64_t)UINT32_MAX) return false;
  if ((int64_t)st.m + st.nnz >= (int64_t)INT32_MAX / 2) return false;
  if (force) return true;
  // Not tried unless asked for (ALSPARSE_AMD_TUNE_HOT=1): counting and ranking the columns costs several
  // multiplies, and on the power-law matrices it is meant for the kernel gained 4 % where a copy has to
  // gain 5 % to be kept.
  static const bool asked = [] {
    const char* a = getenv("ALSPARSE_AMD_TUNE_HOT");
    const char* b = getenv("ALSPARSE_AMD_TUNE_PICK");
    return (a && atoi(a) > 0) || (b && !strcmp(b, "hot"));
  }();
  return asked && (int64_t)st.n * (int64_t)sizeof(T) >= ((int64_t)8 << 20) && st.nnz >= (1 << 22);
}

// Counts the entries of every column, ranks the columns, rewrites the column stream as positions (LDS
// slot or column) and caches the merge coordinates of the wave-sized blocks.  Leaves hot_built = 0 (and
// no error) when the popular columns hold too few entries.
template <typename T>
static hipError_t build_hot(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr, const int* col_ind, bool force) {
  using HK = HotKernel<T>;
  asamd_csr_stats& st = p->st;
  const int n = st.n;
  const size_t nnz = (size_t)st.nnz;
  int h1 = HK::Dims::lds_cols;
  if (const char* ev = getenv("ALSPARSE_AMD_HOT_COLS")) {
    const int v = atoi(ev);
    if (v > 0 && v < h1) h1 = v;
  }
  if (h1 > n) h1 = n;
  // the compact front: the columns that share an XCD's L2 with the streams passing through
  int hc = (int)(((int64_t)kHotFrontBytes) / (int64_t)sizeof(T));
  if (const char* ev = getenv("ALSPARSE_AMD_HOT_FRONT")) {
    const int v = atoi(ev);
    if (v > 0) hc = v;
  }
  if (hc > n) hc = n;
  if (hc < h1) hc = h1;
  const int64_t nb = ((int64_t)st.m + st.nnz + HK::Dims::items - 1) / HK::Dims::items;
  unsigned *d_cnt = nullptr, *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr, *d_sorted = nullptr, *d_rank = nullptr;
  hipError_t e = hipMalloc(&d_cnt, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_sorted, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMemsetAsync(d_cnt, 0, (size_t)n * sizeof(unsigned), stream);
  std::vector<unsigned> h_key((size_t)h1);
  if (e == hipSuccess) {
    col_count_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, col_ind, st.base, d_cnt);
    col_rank_keys_kernel<<<(unsigned)(((int64_t)n + 255) / 256), 256, 0, stream>>>(n, d_cnt, d_key, d_idx);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, d_sorted, (size_t)n, 32);
  if (e == hipSuccess) e = hipMemcpy(h_key.data(), d_key2, (size_t)h1 * sizeof(unsigned), hipMemcpyDeviceToHost);
  if (e == hipSuccess) {
    double in_lds = 0.0;
    for (int i = 0; i < h1; ++i) in_lds += (double)(~h_key[(size_t)i]);
    st.hot_cols_lds = h1;
    st.hot_cols = hc;
    st.hot_share_lds = (float)(in_lds / (double)nnz);
    // worth laying out only if the LDS serves a good part of the gathers
    if (!force && st.hot_share_lds < 0.2f) e = hipErrorNotSupported;
  }
  if (e == hipSuccess) e = hipMalloc(&d_rank, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&p->d_pcol, nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&p->d_hot_cols, (size_t)hc * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_xhot, (size_t)hc * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&p->d_hot_block_row, ((size_t)nb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_hot_carry_row, (size_t)nb * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_hot_carry_val, (size_t)nb * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&p->d_hot_head_val, (size_t)nb * sizeof(T));
  if (e == hipSuccess) e = hipMemsetAsync(d_rank, 0xFF, (size_t)n * sizeof(unsigned), stream);
  if (e == hipSuccess) e = hipMemsetAsync(p->d_hot_head_val, 0, (size_t)nb * sizeof(T), stream);
  if (e == hipSuccess) {
    col_rank_scatter_kernel<<<(unsigned)((hc + 255) / 256), 256, 0, stream>>>(hc, d_sorted, d_rank, p->d_hot_cols);
    hot_pcol_kernel<<<256 * 32, 256, 0, stream>>>(st.nnz, col_ind, st.base, hc, d_rank, p->d_pcol);
    merge_partition_kernel<<<(unsigned)((nb + 1 + 255) / 256), 256, 0, stream>>>(st.m, st.nnz, row_ptr, st.base, (int)nb,
                                                                                HK::Dims::items, p->d_hot_block_row);
    e = hipGetLastError();
  }
  if (e == hipSuccess)
    e = hipFuncSetAttribute((const void*)spmv_merge_hot_kernel<T, HK::ipt, HK::nw>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, HK::Dims::table_bytes + HK::Dims::stage_bytes);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  for (void* d : {(void*)d_cnt, (void*)d_key, (void*)d_key2, (void*)d_idx, (void*)d_sorted, (void*)d_rank})
    if (d) (void)hipFree(d);
  if (e != hipSuccess) {
    free_hot(p);
    return e == hipErrorNotSupported ? hipSuccess : e;
  }
  p->hot_blocks = (int)nb;
  st.hot_built = 1;
  return hipSuccess;
}

// Row numbers sorted by length class and the chunk table of the longest rows.
template <typename T>
static bool binned_eligible(const asamd_csr_plan* p, bool force) {
  const asamd_csr_stats& st = p->st;
  if (!st.trusted || st.m < 1 || st.nnz < 1) return false;
  if (force) return true;
  if (st.nnz < (1 << 20) || st.max_len <= kBinShort) return false;
  // rows that differ enough in length for one mapping not to fit: the structural choice was merge-path, or
  // a lane group per row whose width (from the MEAN length) leaves three quarters of the lanes idle on a
  // quarter of the rows (row-length histogram: bin b holds the rows of 2^(b-1) .. 2^b - 1 entries)
  if (p->auto_algo == ASAMD_SPMV_MERGE) return st.max_len > kBinMid;
  if (p->auto_algo != ASAMD_SPMV_VECTOR) return false;
  int64_t short_rows = 0;
  for (int b = 0; b < ASAMD_HIST_BINS && ((int64_t)1 << b) <= p->auto_width / 4; ++b) short_rows += st.hist[b];
  return short_rows * 4 >= (int64_t)st.m;
}

template <typename T>
static hipError_t build_binned(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr) {
  asamd_csr_stats& st = p->st;
  const int m = st.m;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr;
  int *d_count = nullptr, *d_bounds = nullptr;
  int h_count[kBinClasses] = {0, 0, 0, 0};
  hipError_t e = hipMalloc(&d_key, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&p->d_bin_rows, (size_t)m * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_count, sizeof(h_count));
  if (e == hipSuccess) e = hipMemsetAsync(d_count, 0, sizeof(h_count), stream);
  if (e == hipSuccess) {
    bin_keys_kernel<<<(unsigned)(((int64_t)m + 255) / 256), 256, 0, stream>>>(m, row_ptr, d_key, d_idx, d_count);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, (unsigned*)p->d_bin_rows, (size_t)m, 2);
  if (e == hipSuccess) e = hipMemcpyAsync(h_count, d_count, sizeof(h_count), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  const int nlong = h_count[kBinClasses - 1];
  std::vector<int> bounds, first;
  std::vector<BinChunk> chunks;
  if (e == hipSuccess && nlong > 0) {
    // the long rows' offsets come to the host, which cuts them into chunks
    bounds.resize((size_t)nlong * 2);
    e = hipMalloc(&d_bounds, bounds.size() * sizeof(int));
    if (e == hipSuccess) {
      bin_row_bounds_kernel<<<(unsigned)((nlong + 255) / 256), 256, 0, stream>>>(nlong, p->d_bin_rows + (m - nlong), row_ptr,
                                                                               d_bounds);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(bounds.data(), d_bounds, bounds.size() * sizeof(int), hipMemcpyDeviceToHost);
    if (e == hipSuccess) {
      std::vector<int> rows((size_t)nlong);
      e = hipMemcpy(rows.data(), p->d_bin_rows + (m - nlong), rows.size() * sizeof(int), hipMemcpyDeviceToHost);
      first.resize((size_t)nlong + 1);
      for (int i = 0; i < nlong && e == hipSuccess; ++i) {
        first[(size_t)i] = (int)chunks.size();
        const int64_t b = (int64_t)bounds[2 * (size_t)i] - st.base, en = (int64_t)bounds[2 * (size_t)i + 1] - st.base;
        for (int64_t c = b; c < en; c += kBinChunk)
          chunks.push_back(BinChunk{rows[(size_t)i], (int)c, (int)(c + kBinChunk < en ? c + kBinChunk : en)});
      }
      first[(size_t)nlong] = (int)chunks.size();
    }
    if (e == hipSuccess) e = hipMalloc(&p->d_bin_chunk, chunks.size() * sizeof(BinChunk));
    if (e == hipSuccess) e = hipMalloc(&p->d_bin_first, first.size() * sizeof(int));
    if (e == hipSuccess) e = hipMalloc(&p->d_bin_partial, chunks.size() * sizeof(T));
    if (e == hipSuccess) e = hipMemcpy(p->d_bin_chunk, chunks.data(), chunks.size() * sizeof(BinChunk), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(p->d_bin_first, first.data(), first.size() * sizeof(int), hipMemcpyHostToDevice);
  }
  for (void* d : {(void*)d_key, (void*)d_key2, (void*)d_idx, (void*)d_count, (void*)d_bounds})
    if (d) (void)hipFree(d);
  if (e != hipSuccess) {
    free_binned(p);
    return e;
  }
  for (int c = 0; c < kBinClasses; ++c) {
    p->bin_count[c] = h_count[c];
    st.bin_rows[c] = h_count[c];
  }
  p->bin_chunks = (int)chunks.size();
  st.binned_built = 1;
  return hipSuccess;
}

// Whether the structural choice has rivals that need no copy either (merge-path, a lane group per row): it has
// when it is a lane group per row or a staged block with several lanes per row, merge-path can run (row_ptr
// starts at the base) and the matrix is not so small that one launch's latency is all there is to time.
static bool structural_alternatives(const asamd_csr_plan* p) {
  const asamd_csr_stats& st = p->st;
  if (st.first_offset != 0 || (int64_t)st.m + st.nnz <= kSmallWork) return false;
  return p->auto_algo == ASAMD_SPMV_VECTOR || (p->auto_algo == ASAMD_SPMV_STREAM && stream_group(p, false) > 1);
}

// Time the structural choice on scratch vectors, then the copies that the matrix is eligible for:
// the ELL copy (cheap to build), and the tiled copy only if the fastest so far is slower than the
// tiled pair could possibly be.  Keep the fastest and free the copies that lost.  A copy has to win
// by a margin to be worth its memory.
template <typename T>
static hipError_t tune_copies(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr,
                              const int* col_ind, const T* val, bool tiled_ok, bool ell_ok, bool hot_ok,
                              bool binned_ok) {
  asamd_csr_stats& st = p->st;
  T *x = nullptr, *y = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e = hipMalloc(&x, (size_t)st.n * sizeof(T));
  if (e == hipSuccess) e = hipMalloc(&y, (size_t)st.m * sizeof(T));
  if (e == hipSuccess) e = hipMemsetAsync(x, 0, (size_t)st.n * sizeof(T), stream);
  if (e == hipSuccess) e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  constexpr int kCand = 5;
  float best[kCand] = {0.f, 0.f, 0.f, 0.f, 0.f};
  int algos[kCand] = {p->auto_algo, ASAMD_SPMV_TILED, ASAMD_SPMV_ELL, ASAMD_SPMV_MERGE_HOT, ASAMD_SPMV_BINNED};
  auto time_algo = [&](int a) {
    st.algo = algos[a];
    // first run warms up; multiplies of a millisecond and more are timed once, shorter ones twice; a
    // first run of more than two milliseconds is its own measurement (cold caches are noise at that length)
    int reps = 3;
    for (int rep = 0; rep < reps && e == hipSuccess; ++rep) {
      e = hipEventRecord(e0, stream);
      if (e == hipSuccess)
        e = (hipError_t)csrmv_impl<T>(stream, p, T(1), val, row_ptr, col_ind, x, T(0), y);
      if (e == hipSuccess) e = hipEventRecord(e1, stream);
      if (e == hipSuccess) e = hipEventSynchronize(e1);
      float ms = 0.f;
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
      if (rep == 0 && ms > 1.0f) reps = ms > 2.0f ? 1 : 2;
      if ((rep > 0 || reps == 1) && (best[a] == 0.f || ms < best[a])) best[a] = ms;
    }
  };
  // The tiled pair streams about twice the algorithmic bytes (16 instead of 8 bytes per fp32 entry), so
  // it cannot finish before 2 * bytes / (the ~5 TB/s that streams reach).
  const double bytes = (double)st.nnz * (4.0 + sizeof(T)) + ((double)st.m + 1) * 4.0 +
                       ((double)st.n + (double)st.m) * sizeof(T);
  float tiled_floor_ms = (float)(2.0 * bytes / 5.0e9);
  // Heavy-tailed rows (power-law graphs) make uneven tiles: the in-wave combining of equal rows and the
  // long-tile phase then cost the tiled pair about 2.3 times its floor (measured 0.78 ms against 0.34 ms
  // on an 8 M-row R-MAT matrix whose longest row has 120 000 entries; 0.65 ms on its transpose).
  if ((double)st.max_len > 32.0 * ((double)st.nnz / (double)st.m) + 256.0) tiled_floor_ms *= 2.5f;
  if (e == hipSuccess) time_algo(0);
  // A lane group per row, or a staged block of rows with several lanes per row, was chosen from the mean and
  // the longest row alone.  Neither needs a copy, nor does merge-path, which takes any distribution: the
  // fastest of them stays.
  if (e == hipSuccess && structural_alternatives(p)) {
    int alts[2] = {ASAMD_SPMV_MERGE, p->auto_algo == ASAMD_SPMV_STREAM ? ASAMD_SPMV_VECTOR : -1};
    for (int alt : alts) {
      if (alt < 0 || e != hipSuccess) continue;
      const float first = best[0];
      const int kept = algos[0];
      best[0] = 0.f;
      algos[0] = alt;
      time_algo(0);
      if (e == hipSuccess && best[0] > 0.f && best[0] < 0.97f * first) {
        p->auto_algo = p->struct_algo = alt;
      } else {
        algos[0] = kept;
        best[0] = first;
      }
    }
  }
  // An ELL copy gathers x row by row like the kernel just timed; when that one is several times slower
  // than the tiled floor the gathers are the problem and the ELL copy (as large as the matrix) is not
  // worth building: the tiled copy is tried first, the ELL copy only if that does not win.
  const bool ell_first = !(tiled_ok && best[0] > 2.5f * tiled_floor_ms);
  auto try_ell = [&]() {
    if (e == hipSuccess && ell_ok) {
      e = build_ell<T>(stream, p, row_ptr, col_ind, val);
      if (e == hipSuccess) time_algo(2);
    }
  };
  if (ell_first) try_ell();
  if (e == hipSuccess && tiled_ok) {
    // A row kernel that is already as fast as the tiled floor (banded matrices, whose gathers stay in
    // the caches) makes the tiled copy pointless: its layout pass (a sort of all entries) and its
    // memory are saved.
    float fastest = best[0];
    if (best[2] > 0.f && best[2] < fastest) fastest = best[2];
    if (fastest > 1.1f * tiled_floor_ms) {
      e = build_tiled<T>(stream, p, row_ptr, col_ind, val);
      if (e == hipSuccess && st.tiled_built) time_algo(1);
    }
  }
  if (!ell_first && !(best[1] > 0.f && best[1] < 0.9f * best[0])) try_ell();
  // Skewed matrices on merge-path: count the entries per column and, if few columns hold most of them,
  // time the kernel that keeps those columns' x in LDS.
  if (e == hipSuccess && hot_ok && p->auto_algo == ASAMD_SPMV_MERGE) {
    e = build_hot<T>(stream, p, row_ptr, col_ind, false);
    if (e == hipSuccess && st.hot_built) time_algo(3);
  }
  // Very uneven rows: one launch per row-length class (cheap to lay out: a sort of the row numbers)
  if (e == hipSuccess && binned_ok) {
    e = build_binned<T>(stream, p, row_ptr);
    if (e == hipSuccess && st.binned_built) time_algo(4);
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (x) (void)hipFree(x);
  if (y) (void)hipFree(y);
  st.algo = p->auto_algo;
  if (e != hipSuccess) return e;
  st.tune_ms_binned = best[4];
  st.tune_ms_base = best[0];
  st.tune_ms_tiled = best[1];
  st.tune_ms_ell = best[2];
  st.tune_ms_hot = best[3];
  // a copy has to win by a margin to be worth its memory; among the winners the fastest is kept
  const float margin[kCand] = {1.f, 0.9f, 0.95f, 0.95f, 0.95f};
  int pick = 0;
  for (int a = 1; a < kCand; ++a)
    if (best[a] > 0.f && best[a] < margin[a] * best[0] && (pick == 0 || best[a] < best[pick])) pick = a;
  // ALSPARSE_AMD_TUNE_PICK = base | tiled | ell | hot | binned overrides the timing's verdict among the candidates
  // that were built (for profiling a kernel that lost)
  if (const char* ev = getenv("ALSPARSE_AMD_TUNE_PICK")) {
    const char* names[kCand] = {"base", "tiled", "ell", "hot", "binned"};
    for (int a = 0; a < kCand; ++a)
      if (!strcmp(ev, names[a]) && (a == 0 || best[a] > 0.f)) pick = a;
  }
  if (pick != 1) free_tiled(p);
  if (pick != 2) free_ell(p);
  if (pick != 3) free_hot(p);
  if (pick != 4) free_binned(p);
  if (pick != 0) {
    p->auto_algo = algos[pick];
    st.algo = algos[pick];
    if (pick != 3 && pick != 4) p->copy_val_src = val;  // the hot-column copy and the row bins hold no values
  }
  return hipSuccess;
}

static hipError_t plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, const int32_t* row_ptr,
                              const int32_t* col_ind, const void* val, int32_t base, int32_t dtype,
                              int32_t trusted, asamd_csr_plan** out) {
  if (!out || !row_ptr || m <= 0 || nnz < 0 || dtype < ASAMD_DTYPE_FLOAT || dtype > ASAMD_DTYPE_DOUBLE_COMPLEX)
    return hipErrorInvalidValue;
  static const int kValSize[4] = {4, 8, 8, 16};
  const int val_size = kValSize[dtype];
  if (val && (uintptr_t)val % (size_t)val_size) return hipErrorInvalidValue;
  asamd_csr_plan* p = new (std::nothrow) asamd_csr_plan();
  if (!p) return hipErrorOutOfMemory;
  p->st.m = m;
  p->st.n = n;
  p->st.nnz = nnz;
  p->st.base = base;
  p->st.trusted = trusted ? 1 : 0;
  p->dtype = dtype;
  p->val_size = val_size;

  int* d_stats = nullptr;
  hipError_t e = hipMalloc(&d_stats, kStatWords * sizeof(int));
  if (e != hipSuccess) {
    delete p;
    return e;
  }
  stats_init_kernel<<<1, 64, 0, stream>>>(d_stats);
  int64_t grid = ((int64_t)m + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;
  row_stats_kernel<<<(unsigned)grid, 256, 0, stream>>>(m, row_ptr, d_stats);
  int h[kStatWords];
  e = hipMemcpyAsync(h, d_stats, sizeof(h), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(d_stats);
  if (e != hipSuccess) {
    delete p;
    return e;
  }
  p->st.min_len = h[0];
  p->st.max_len = h[1];
  p->st.first_offset = h[2] - base;
  p->st.const_len = h[0] == h[1] ? h[0] : -1;
  for (int b = 0; b < ASAMD_HIST_BINS; ++b) p->st.hist[b] = h[3 + b];

  const int64_t total = (int64_t)m + nnz;
  // wider values take more LDS per item: fewer items keep more workgroups resident
  p->merge_ipt = val_size >= 8 ? 4 : 8;
  if (const char* ev = getenv("ALSPARSE_AMD_MERGE_IPT")) {
    const int v = atoi(ev);
    if (v == 4 || v == 8 || (v == 16 && dtype <= ASAMD_DTYPE_DOUBLE)) p->merge_ipt = v;
  }
  if (val_size == 16) p->merge_ipt = 4;  // the only instantiation for 16-byte values
  const int merge_items = kMergeThreads * p->merge_ipt;
  const int64_t nb = (total + merge_items - 1) / merge_items;
  p->st.merge_blocks = (int)nb;
  choose_algo(p);

  // merge-path buffers are sized by m + nnz only, so they stay valid even if
  // the structure behind row_ptr changes under an untrusted plan
  e = hipMalloc(&p->d_block_row, (nb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_carry_row, nb * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_carry_val, nb * (size_t)val_size);
  if (e == hipSuccess) e = hipMalloc(&p->d_head_val, nb * (size_t)val_size);
  if (e != hipSuccess) {
    asamd_csr_plan_destroy(p);
    return e;
  }
  if (p->st.trusted) {
    merge_partition_kernel<<<(int)((nb + 1 + 255) / 256), 256, 0, stream>>>(
        m, nnz, row_ptr, base, (int)nb, merge_items, p->d_block_row);
    e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
    p->coords_valid = true;
  }
  if (col_ind && val && nnz > 0) {
    // trusted == 2: build the tiled copy whatever the size and skip the timing
    // (lets small matrices exercise the tiled kernels)
    const bool force = trusted == 2;
    e = by_dtype(dtype, [&](auto* tag) -> hipError_t {
      using T = std::remove_pointer_t<decltype(tag)>;
      hipError_t err = hipSuccess;
      const bool tiled_ok = tiled_eligible<T>(p->st, force), ell_ok = ell_eligible(p->st, force);
      const bool hot_ok = hot_eligible<T>(p, force);
      const bool binned_ok = binned_eligible<T>(p, force);
      if (force) {
        if (binned_ok) err = build_binned<T>(stream, p, row_ptr);
        if (err != hipSuccess) return err;
        if (tiled_ok) err = build_tiled<T>(stream, p, row_ptr, col_ind, (const T*)val);
        if (err == hipSuccess && ell_ok) err = build_ell<T>(stream, p, row_ptr, col_ind, (const T*)val);
        if (err == hipSuccess && hot_ok) err = build_hot<T>(stream, p, row_ptr, col_ind, true);
        p->copy_val_src = val;
      } else if (tiled_ok || ell_ok || hot_ok || binned_ok || structural_alternatives(p)) {
        err = tune_copies<T>(stream, p, row_ptr, col_ind, (const T*)val, tiled_ok, ell_ok, hot_ok, binned_ok);
      }
      return err;
    });
    if (e == hipErrorOutOfMemory) {
      (void)hipGetLastError();  // the copies are optional: carry on without them
      free_tiled(p);
      free_ell(p);
      free_hot(p);
      free_binned(p);
      if (p->auto_algo == ASAMD_SPMV_TILED || p->auto_algo == ASAMD_SPMV_ELL || p->auto_algo == ASAMD_SPMV_MERGE_HOT ||
          p->auto_algo == ASAMD_SPMV_BINNED)
        p->auto_algo = p->struct_algo;
      p->st.algo = p->auto_algo;
      e = hipSuccess;
    }
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
  }
  *out = p;
  return hipSuccess;
}

extern "C" int asamd_csr_plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                                     const int32_t* row_ptr, const int32_t* col_ind,
                                     const void* val, int32_t base, int32_t val_size,
                                     int32_t trusted, asamd_csr_plan** out) {
  if (val_size != 4 && val_size != 8) return hipErrorInvalidValue;
  return plan_create(stream, m, n, nnz, row_ptr, col_ind, val, base,
                     val_size == 4 ? ASAMD_DTYPE_FLOAT : ASAMD_DTYPE_DOUBLE, trusted, out);
}

extern "C" int asamd_csr_plan_create_dtype(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                                           const int32_t* row_ptr, const int32_t* col_ind, const void* val,
                                           int32_t base, int32_t dtype, int32_t trusted, asamd_csr_plan** out) {
  return plan_create(stream, m, n, nnz, row_ptr, col_ind, val, base, dtype, trusted, out);
}

extern "C" void asamd_csr_plan_destroy(asamd_csr_plan* p) {
  if (!p) return;
  if (p->d_block_row) (void)hipFree(p->d_block_row);
  if (p->d_carry_row) (void)hipFree(p->d_carry_row);
  if (p->d_carry_val) (void)hipFree(p->d_carry_val);
  if (p->d_head_val) (void)hipFree(p->d_head_val);
  free_tiled(p);
  free_ell(p);
  free_hot(p);
  free_binned(p);
  free_transpose(p, 0);
  free_transpose(p, 1);
  delete p;
}

// CSR of A^T: sort (column, entry) pairs by column (stable: rows ascending inside
// a column), read the column offsets off the sorted keys, gather rows and values.
template <typename T>
static hipError_t build_transpose(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr, const int* col_ind,
                                  const T* val, int which) {
  asamd_csr_stats& st = p->st;
  asamd_csr_plan::TransCopy& t = p->tr[which];
  const int nnz = st.nnz, n = st.n;
  int* d_coo = nullptr;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr, *d_perm = nullptr;
  hipError_t e = hipMalloc(&d_coo, (size_t)nnz * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_key, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_perm, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&t.d_row_ptr, ((size_t)n + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&t.d_col, (size_t)nnz * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&t.d_val, (size_t)nnz * sizeof(T));
  if (e == hipSuccess)  // d_key2 is free until the sort
    e = (hipError_t)asamd_csr2coo_ws(stream, row_ptr, nnz, st.m, d_coo, st.base, d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    int64_t grid = ((int64_t)nnz + 255) / 256;
    if (grid > 256 * 32) grid = 256 * 32;
    transpose_keys_kernel<<<(unsigned)grid, 256, 0, stream>>>(nnz, col_ind, st.base, d_key, d_idx);
    e = hipGetLastError();
    unsigned bits = 1;
    while (bits < 32 && ((int64_t)1 << bits) < (int64_t)n) ++bits;
    if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, d_perm, (size_t)nnz, bits);
    if (e == hipSuccess) {
      tile_bounds_kernel<<<(unsigned)(((int64_t)n + 1 + 255) / 256), 256, 0, stream>>>(nnz, d_key2, (int64_t)n,
                                                                                      t.d_row_ptr);
      if (which == 1)
        transpose_gather_kernel<T, true><<<grid, 256, 0, stream>>>(nnz, d_perm, d_coo, val, st.base, t.d_col,
                                                                   (T*)t.d_val);
      else
        transpose_gather_kernel<T, false><<<grid, 256, 0, stream>>>(nnz, d_perm, d_coo, val, st.base, t.d_col,
                                                                    (T*)t.d_val);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
  }
  for (void* d : {(void*)d_coo, (void*)d_key, (void*)d_key2, (void*)d_idx})
    if (d) (void)hipFree(d);
  t.d_perm = d_perm;  // kept: the values of the copy can be gathered again through it
  if (e == hipSuccess)
    e = plan_create(stream, n, st.m, nnz, t.d_row_ptr, t.d_col, t.d_val, 0, DtypeOf<T>::value, /*trusted=*/1,
                    &t.plan);
  if (e != hipSuccess) {
    free_transpose(p, which);
    return e;
  }
  t.val_src = val;
  st.transpose_built |= 1 << which;
  return hipSuccess;
}

static int build_transpose_any(hipStream_t stream, asamd_csr_plan* p, const int32_t* row_ptr,
                               const int32_t* col_ind, const void* val, int which) {
  if (!p || !row_ptr || !col_ind || !val || !p->st.trusted || p->st.n <= 0) return hipErrorInvalidValue;
  if (which == 1 && !is_complex(p)) return hipErrorInvalidValue;
  if (p->st.transpose_built & (1 << which)) return hipSuccess;
  if (p->st.nnz == 0) return hipSuccess;  // the scatter route has nothing to add
  if (p->st.first_offset != 0) return hipSuccess;  // no copy (csr2coo counts from position 0): the scatter route serves
  return by_dtype(p->dtype, [&](auto* tag) -> hipError_t {
    using T = std::remove_pointer_t<decltype(tag)>;
    return build_transpose<T>(stream, p, row_ptr, col_ind, (const T*)val, which);
  });
}

extern "C" int asamd_csr_plan_build_transpose(hipStream_t stream, asamd_csr_plan* p, const int32_t* row_ptr,
                                              const int32_t* col_ind, const void* val) {
  return build_transpose_any(stream, p, row_ptr, col_ind, val, 0);
}

extern "C" int asamd_csr_plan_build_conj_transpose(hipStream_t stream, asamd_csr_plan* p, const int32_t* row_ptr,
                                                   const int32_t* col_ind, const void* val) {
  return build_transpose_any(stream, p, row_ptr, col_ind, val, 1);
}

extern "C" int asamd_csr_plan_set_lazy_transpose(asamd_csr_plan* p, int32_t on) {
  if (!p || !p->st.trusted) return hipErrorInvalidValue;
  p->lazy_transpose = on != 0;
  return hipSuccess;
}

extern "C" const asamd_csr_stats* asamd_csr_plan_transpose_stats(const asamd_csr_plan* p) {
  if (!p) return nullptr;
  if (p->tr[0].plan) return &p->tr[0].plan->st;
  return p->tr[1].plan ? &p->tr[1].plan->st : nullptr;
}

extern "C" int asamd_csr_plan_transpose_arrays(const asamd_csr_plan* p, int32_t conj, const int32_t** row_ptr,
                                               const int32_t** col_ind, const void** val) {
  if (!p || !row_ptr || !col_ind || !val) return hipErrorInvalidValue;
  const asamd_csr_plan::TransCopy& t = p->tr[conj ? 1 : 0];
  if (!t.plan) return hipErrorInvalidValue;
  *row_ptr = t.d_row_ptr;
  *col_ind = t.d_col;
  *val = t.d_val;
  return hipSuccess;
}

// The copies of a plan hold values: gather them again from `val` (the array the copies were laid out
// from, or one with the same structure).  Only kernels, on `stream`; nothing is allocated or waited for.
template <typename T>
static hipError_t refresh_values(hipStream_t stream, asamd_csr_plan* p, const int* row_ptr, const int* col_ind,
                                 const T* val) {
  const asamd_csr_stats& st = p->st;
  hipError_t e = hipSuccess;
  if (st.tiled_built) {
    if (!p->d_tperm) return hipErrorInvalidValue;
    gather_values_kernel<T, false><<<256 * 32, 256, 0, stream>>>(st.nnz, p->d_tperm, val, (T*)p->d_tval);
    e = hipGetLastError();
  }
  if (e == hipSuccess && st.ell_built) {
    if constexpr (sizeof(T) == 4)
      e = (hipError_t)asamd_s_csr2ell(stream, st.m, (const float*)val, row_ptr, col_ind, st.base, 0, st.ell_width,
                                      (float*)p->d_eval, p->d_ecol);
    else if constexpr (sizeof(T) == 8)
      e = (hipError_t)asamd_d_csr2ell(stream, st.m, (const double*)val, row_ptr, col_ind, st.base, 0, st.ell_width,
                                      (double*)p->d_eval, p->d_ecol);
    else
      e = (hipError_t)asamd_z_csr2ell(stream, st.m, (const asamd_complex16*)val, row_ptr, col_ind, st.base, 0,
                                      st.ell_width, (asamd_complex16*)p->d_eval, p->d_ecol);
  }
  if (e == hipSuccess && (st.tiled_built || st.ell_built)) p->copy_val_src = val;
  for (int which = 0; which < 2 && e == hipSuccess; ++which) {
    asamd_csr_plan::TransCopy& t = p->tr[which];
    if (!t.plan) continue;
    if (!t.d_perm) return hipErrorInvalidValue;
    if (which == 1)
      gather_values_kernel<T, true><<<256 * 32, 256, 0, stream>>>(st.nnz, t.d_perm, val, (T*)t.d_val);
    else
      gather_values_kernel<T, false><<<256 * 32, 256, 0, stream>>>(st.nnz, t.d_perm, val, (T*)t.d_val);
    e = hipGetLastError();
    t.val_src = val;
    // the transposed copy has a plan of its own, which may hold copies of the copy's values
    if (e == hipSuccess) e = refresh_values<T>(stream, t.plan, t.d_row_ptr, t.d_col, (const T*)t.d_val);
  }
  return e;
}

extern "C" int asamd_csr_plan_refresh_values(hipStream_t stream, asamd_csr_plan* p, const int32_t* row_ptr,
                                             const int32_t* col_ind, const void* val) {
  if (!p || !row_ptr || !col_ind || !val || !p->st.trusted) return hipErrorInvalidValue;
  if ((uintptr_t)val % (size_t)p->val_size) return hipErrorInvalidValue;
  return by_dtype(p->dtype, [&](auto* tag) -> hipError_t {
    using T = std::remove_pointer_t<decltype(tag)>;
    return refresh_values<T>(stream, p, row_ptr, col_ind, (const T*)val);
  });
}

extern "C" int asamd_csr_structure_hash(hipStream_t stream, int32_t m, int32_t nnz, const int32_t* row_ptr,
                                        const int32_t* col_ind, uint64_t* hash_host) {
  if (!row_ptr || !hash_host || m < 0 || nnz < 0 || (nnz > 0 && !col_ind)) return hipErrorInvalidValue;
  unsigned long long* d_hash = nullptr;
  hipError_t e = hipMalloc(&d_hash, sizeof(unsigned long long));
  if (e != hipSuccess) return e;
  e = hipMemsetAsync(d_hash, 0, sizeof(unsigned long long), stream);
  if (e == hipSuccess) {
    index_hash_kernel<<<256 * 8, 256, 0, stream>>>((int64_t)m + 1, row_ptr, 0x1234567ull, d_hash);
    if (nnz > 0) index_hash_kernel<<<256 * 16, 256, 0, stream>>>((int64_t)nnz, col_ind, 0xABCDEF01ull << 8, d_hash);
    e = hipGetLastError();
  }
  unsigned long long h = 0;
  if (e == hipSuccess) e = hipMemcpyAsync(&h, d_hash, sizeof(h), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(d_hash);
  *hash_host = (uint64_t)h;
  return e;
}

extern "C" const asamd_csr_stats* asamd_csr_plan_stats(const asamd_csr_plan* p) {
  return p ? &p->st : nullptr;
}

extern "C" int asamd_csr_plan_set_algo(asamd_csr_plan* p, int32_t algo) {
  if (!p) return hipErrorInvalidValue;
  switch (algo) {
    case ASAMD_SPMV_AUTO:
      p->st.algo = p->auto_algo;
      return hipSuccess;
    case ASAMD_SPMV_ROWCONST:
      if (!rowconst_ok(p)) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_TILED:
      if (!p->st.tiled_built) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_STREAM:
      if (!stream_ok(p)) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_ELL:
      if (!p->st.ell_built) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_MERGE_HOT:
      if (!p->st.hot_built) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_BINNED:
      if (!p->st.binned_built) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_MERGE:
      if (p->st.first_offset != 0) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_VECTOR:
    case ASAMD_SPMV_SCALAR:
      p->st.algo = algo;
      return hipSuccess;
    default:
      return hipErrorInvalidValue;
  }
}

// the cache policy of a CSR multiply's streams (stream_policy.hpp) from the plan's statistics
static int stream_policy(const asamd_csr_stats& st, size_t val_size, bool wide_both = false) {
  return asamd::stream_policy((double)st.nnz, val_size,
                              ((double)st.m + 1.0) * 4.0 + ((double)st.m + (double)st.n) * (double)val_size, wide_both);
}

// ---------------------------------------------------------------------------
template <typename T, int W>
static void launch_vector(hipStream_t s, const asamd_csr_stats& st, T alpha, const T* val,
                          const int* rp, const int* ci, const T* x, T beta, T* y) {
  constexpr int rows_per_block = kRowsBlock / W;
  const unsigned grid = (unsigned)(((int64_t)st.m + rows_per_block - 1) / rows_per_block);
  spmv_vector_kernel<T, W><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base);
}

template <typename T, int G>
static void launch_rowconst(hipStream_t s, const asamd_csr_stats& st, T alpha, const T* val,
                            const int* ci, const T* x, T beta, T* y) {
  constexpr int R = G >= 16 ? 1 : 2;
  constexpr int rows_per_block = (kRowsBlock / G) * R;
  const unsigned grid = (unsigned)(((int64_t)st.m + rows_per_block - 1) / rows_per_block);
  spmv_rowconst_kernel<T, G, R><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, ci, x, beta, y, st.base,
                                                            stream_policy(st, sizeof(T)));
}

template <typename T>
static int csrmv_impl(hipStream_t s, asamd_csr_plan* p, T alpha, const T* val, const int* rp,
                      const int* ci, const T* x, T beta, T* y) {
  if (!p || !val || !rp || !ci || !x || !y) return hipErrorInvalidValue;
  if (p->dtype != DtypeOf<T>::value) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % alignof(T)) return hipErrorInvalidValue;
  const asamd_csr_stats& st = p->st;
  int algo = st.algo;
  // The tiled and ELL copies hold the values of the array they were built from.  A multiply that
  // brings another value array (same structure, new numbers) must not see the old ones: it runs
  // the kernel that the row statistics alone would pick.  (Values changed IN PLACE cannot be seen
  // from here: that needs a new analysis.)
  if ((algo == ASAMD_SPMV_TILED || algo == ASAMD_SPMV_ELL) && p->copy_val_src && val != p->copy_val_src)
    algo = p->struct_algo;
  if (!kIsReal<T> && algo == ASAMD_SPMV_ROWCONST) algo = ASAMD_SPMV_VECTOR;
  if (algo == ASAMD_SPMV_ROWCONST) {
    // 128-bit loads need 16-byte aligned streams; fall back otherwise
    const bool aligned = (((uintptr_t)val | (uintptr_t)ci) & 15u) == 0;
    if (!aligned || !rowconst_ok(p)) algo = ASAMD_SPMV_VECTOR;
  }
  if (algo == ASAMD_SPMV_STREAM && !stream_ok(p)) algo = ASAMD_SPMV_MERGE;
  if (algo == ASAMD_SPMV_MERGE && st.first_offset != 0) algo = ASAMD_SPMV_VECTOR;
  if (algo == ASAMD_SPMV_TILED && !st.tiled_built) algo = p->auto_algo == ASAMD_SPMV_TILED ? ASAMD_SPMV_MERGE : p->auto_algo;
  if (algo == ASAMD_SPMV_ELL && !st.ell_built) algo = p->auto_algo == ASAMD_SPMV_ELL ? ASAMD_SPMV_MERGE : p->auto_algo;
  if (algo == ASAMD_SPMV_MERGE_HOT && !st.hot_built) algo = ASAMD_SPMV_MERGE;
  if (algo == ASAMD_SPMV_BINNED && !st.binned_built) algo = st.first_offset != 0 ? ASAMD_SPMV_VECTOR : ASAMD_SPMV_MERGE;
  switch (algo) {
    case ASAMD_SPMV_ELL: {
      // the ELL copy holds zero-based columns and its own values
      if constexpr (sizeof(T) <= 8) {
        if (st.m % 2 == 0) {  // the copy is the library's own (256-byte aligned): row pairs are aligned when m is even
          const unsigned grid2 = (unsigned)(((int64_t)st.m / 2 + kEllThreads - 1) / kEllThreads);
          // the ELL copy's streams: m * width slots of values and of indices
          const int policy = asamd::stream_policy((double)st.m * st.ell_width, sizeof(T),
                                                  ((double)st.m + (double)st.n) * (double)sizeof(T), true);
#define ASAMD_ELL_LAUNCH(NTV, NTC)                                                                                  \
  ellmv_multi_kernel<T, 2, NTV, NTC><<<grid2, kEllThreads, 0, s>>>(st.m, st.n, alpha, (const T*)p->d_eval, p->d_ecol, \
                                                                   st.ell_width, 0, x, beta, y)
          if (policy == 0) ASAMD_ELL_LAUNCH(false, false);
          else if (policy == kStreamNtValues) ASAMD_ELL_LAUNCH(true, false);
          else if (policy == kStreamNtIndices) ASAMD_ELL_LAUNCH(false, true);
          else ASAMD_ELL_LAUNCH(true, true);
#undef ASAMD_ELL_LAUNCH
          break;
        }
      }
      const unsigned grid = (unsigned)(((int64_t)st.m + kEllThreads - 1) / kEllThreads);
      ellmv_kernel<T><<<grid, kEllThreads, 0, s>>>(st.m, st.n, alpha, (const T*)p->d_eval, p->d_ecol, st.ell_width, 0,
                                                   x, beta, y);
      break;
    }
    case ASAMD_SPMV_TILED: {
      // the tiled copy holds zero-based local indices and its own values
      if (p->n_chunks > 0) {
        // products that the memory-side cache cannot hold anyway are stored past it
        if ((int64_t)st.nnz * (int64_t)sizeof(T) > ((int64_t)512 << 20))
          tiled_products_kernel<T, true><<<p->n_chunks, kProdThreads, kSliceBytes, s>>>(
              p->d_chunks, (const T*)p->d_tval, p->d_tcol, x, (T*)p->d_tprod);
        else
          tiled_products_kernel<T, false><<<p->n_chunks, kProdThreads, kSliceBytes, s>>>(
              p->d_chunks, (const T*)p->d_tval, p->d_tcol, x, (T*)p->d_tprod);
      }
      const unsigned red_grid = (unsigned)((st.tile_row_blocks + TileDims<T>::red_waves - 1) / TileDims<T>::red_waves);
      if (p->tiled_halves == 1)
        tiled_reduce_kernel<T, 1><<<red_grid, TileDims<T>::red_threads, TileDims<T>::red_lds_bytes, s>>>(
            st.m, st.tile_row_blocks, st.tile_col_blocks, p->d_row_block_start, p->d_ranges, p->d_trow,
            (const T*)p->d_tprod, alpha, beta, y);
      else
        tiled_reduce_kernel<T, 2><<<red_grid, TileDims<T>::red_threads, TileDims<T>::red_lds_bytes, s>>>(
            st.m, st.tile_row_blocks, st.tile_col_blocks, p->d_row_block_start, p->d_ranges, p->d_trow,
            (const T*)p->d_tprod, alpha, beta, y);
      if (p->n_long_chunks > 0)
        {
        const int waves = kLongThreads / kWave, narrow = p->n_long_narrow, wide = p->n_long_chunks - narrow;
        if (narrow > 0)
          tiled_long_kernel<T><<<narrow, kLongThreads, waves * (kLongNarrow + kWave) * (int)sizeof(T), s>>>(
              p->d_long, p->d_long_tiles, p->d_trow, (const T*)p->d_tprod, alpha, y, (T*)p->d_long_scratch, kLongNarrow);
        if (wide > 0)
          tiled_long_kernel<T><<<wide, kLongThreads, waves * (TileDims<T>::rows + kWave) * (int)sizeof(T), s>>>(
              p->d_long + narrow, p->d_long_tiles, p->d_trow, (const T*)p->d_tprod, alpha, y, (T*)p->d_long_scratch,
              TileDims<T>::rows);
        }
      if (p->n_long_finish > 0)
        tiled_long_finish_kernel<T><<<p->n_long_finish, 256, 0, s>>>(p->d_long_finish, (const T*)p->d_long_scratch, alpha, y);
      break;
    }
    case ASAMD_SPMV_ROWCONST: if constexpr (kIsReal<T>) {
      switch (st.const_len / 4) {
        case 1: launch_rowconst<T, 1>(s, st, alpha, val, ci, x, beta, y); break;
        case 2: launch_rowconst<T, 2>(s, st, alpha, val, ci, x, beta, y); break;
        case 4: launch_rowconst<T, 4>(s, st, alpha, val, ci, x, beta, y); break;
        case 8: launch_rowconst<T, 8>(s, st, alpha, val, ci, x, beta, y); break;
        case 16: launch_rowconst<T, 16>(s, st, alpha, val, ci, x, beta, y); break;
        case 32: launch_rowconst<T, 32>(s, st, alpha, val, ci, x, beta, y); break;
        default: launch_rowconst<T, 64>(s, st, alpha, val, ci, x, beta, y); break;
      }
      break;
    }
    case ASAMD_SPMV_STREAM: {
      const int g = stream_group(p, false);
      const unsigned grid = (unsigned)(((int64_t)st.m * g + kStreamRows - 1) / kStreamRows);
      constexpr int kCap = 64 / (int)sizeof(T);  // stream_cap(p)
      // 128-bit loads need 16-byte aligned streams
      const bool wide = (((uintptr_t)val | (uintptr_t)ci) & 15u) == 0;
      const int64_t limit = (int64_t)st.first_offset + st.nnz;
#define ASAMD_STREAM_LAUNCH(CAP, G)                                                                                      \
  do {                                                                                                                   \
    if (wide)                                                                                                            \
      spmv_stream_wide_kernel<T, CAP, G><<<grid, kStreamRows, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base,    \
                                                                      limit, stream_policy(st, sizeof(T)));             \
    else                                                                                                                 \
      spmv_stream_kernel<T, CAP, G><<<grid, kStreamRows, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base);        \
  } while (0)
      if (g == 1) {
        if (st.max_len <= 4) {
          ASAMD_STREAM_LAUNCH(4, 1);
        } else if constexpr (kCap >= 8) {
          if (st.max_len <= 8) {
            ASAMD_STREAM_LAUNCH(8, 1);
          } else if constexpr (kCap >= 16) {
            ASAMD_STREAM_LAUNCH(16, 1);
          }
        }
      } else if (g == 2) {
        ASAMD_STREAM_LAUNCH(kCap, 2);
      } else if (g == 4) {
        ASAMD_STREAM_LAUNCH(kCap, 4);
      } else if (g == 8) {
        ASAMD_STREAM_LAUNCH(kCap, 8);
      } else {
        ASAMD_STREAM_LAUNCH(kCap, 16);
      }
#undef ASAMD_STREAM_LAUNCH
      break;
    }
    case ASAMD_SPMV_SCALAR: {
      const unsigned grid = (unsigned)(((int64_t)st.m + kRowsBlock - 1) / kRowsBlock);
      spmv_scalar_kernel<T><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base);
      break;
    }
    case ASAMD_SPMV_BINNED: {
      // one launch per row-length class; the classes own disjoint rows, so the launches are independent
      const int* rows = p->d_bin_rows;
      const int n0 = p->bin_count[0], n1 = p->bin_count[1], n2 = p->bin_count[2], n3 = p->bin_count[3];
      auto blocks = [](int count, int w) { return (unsigned)(((int64_t)count * w + kRowsBlock - 1) / kRowsBlock); };
      if (n0 > 0)
        spmv_bin_rows_kernel<T, 4><<<blocks(n0, 4), kRowsBlock, 0, s>>>(n0, rows, alpha, val, rp, ci, x, beta, y, st.base);
      if (n1 > 0)
        spmv_bin_rows_kernel<T, 16><<<blocks(n1, 16), kRowsBlock, 0, s>>>(n1, rows + n0, alpha, val, rp, ci, x, beta, y,
                                                                        st.base);
      if (n2 > 0)
        spmv_bin_rows_kernel<T, 64><<<blocks(n2, 64), kRowsBlock, 0, s>>>(n2, rows + n0 + n1, alpha, val, rp, ci, x, beta,
                                                                        y, st.base);
      if (n3 > 0) {
        spmv_bin_chunk_kernel<T><<<(unsigned)p->bin_chunks, kRowsBlock, 0, s>>>(p->bin_chunks, p->d_bin_chunk, val, ci, x,
                                                                               st.base, (T*)p->d_bin_partial);
        spmv_bin_finish_kernel<T><<<(unsigned)((n3 + 255) / 256), 256, 0, s>>>(n3, rows + n0 + n1 + n2, p->d_bin_first,
                                                                              (const T*)p->d_bin_partial, alpha, beta, y);
      }
      break;
    }
    case ASAMD_SPMV_MERGE_HOT: {
      // x of the hot columns, then persistent workgroups, one per compute unit
      if constexpr (sizeof(T) <= 8) {
        using HK = HotKernel<T>;
        const int nb = p->hot_blocks;
        const int h1 = st.hot_cols_lds, hc = st.hot_cols;
        hot_prepare_kernel<T><<<(unsigned)((hc + 255) / 256), 256, 0, s>>>(hc, p->d_hot_cols, x, (T*)p->d_xhot);
        static const int cus = [] {
          int dev = 0, n_cu = 0;
          if (hipGetDevice(&dev) != hipSuccess ||
              hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
            n_cu = 256;
          return n_cu;
        }();
        const int per_wg = (nb + HK::nw - 1) / HK::nw;
        const int grid = per_wg < cus ? per_wg : cus;
        spmv_merge_hot_kernel<T, HK::ipt, HK::nw>
            <<<grid, HK::Dims::threads, HK::Dims::table_bytes + HK::Dims::stage_bytes, s>>>(
                st.m, st.nnz, alpha, val, rp, p->d_pcol, x, (const T*)p->d_xhot, h1, hc, beta, y, st.base, p->d_hot_block_row, p->d_hot_carry_row,
                (T*)p->d_hot_carry_val, (T*)p->d_hot_head_val, nb);
        if (nb > 1)
          merge_fixup_kernel<T><<<(nb + 255) / 256, 256, 0, s>>>(nb, st.m, alpha, beta, p->d_hot_carry_row,
                                                                 (const T*)p->d_hot_carry_val,
                                                                 (const T*)p->d_hot_head_val, y);
      }
      break;
    }
    case ASAMD_SPMV_MERGE: {
      const int nb = st.merge_blocks;
      if (!p->coords_valid) {
        merge_partition_kernel<<<(nb + 1 + 255) / 256, 256, 0, s>>>(
            st.m, st.nnz, rp, st.base, nb, kMergeThreads * p->merge_ipt, p->d_block_row);
      }
      // 128-bit loads of the streams need them 16-byte aligned
      const bool merge_wide = (((uintptr_t)val | (uintptr_t)ci) & 15u) == 0;
#define ASAMD_LAUNCH_MERGE(IPT)                                                                                  \
  do {                                                                                                           \
    if (merge_wide && (IPT) % 4 == 0)                                                                            \
      spmv_merge_kernel<T, IPT, true><<<nb, kMergeThreads, 0, s>>>(st.m, st.nnz, alpha, val, rp, ci, x, beta, y, \
                                                                   st.base, p->d_block_row, p->d_carry_row,      \
                                                                   (T*)p->d_carry_val, (T*)p->d_head_val,        \
                                                                   stream_policy(st, sizeof(T), true));          \
    else                                                                                                         \
      spmv_merge_kernel<T, IPT><<<nb, kMergeThreads, 0, s>>>(st.m, st.nnz, alpha, val, rp, ci, x, beta, y,       \
                                                             st.base, p->d_block_row, p->d_carry_row,            \
                                                             (T*)p->d_carry_val, (T*)p->d_head_val);             \
  } while (0)
      // LDS per workgroup grows with IPT * sizeof(T): 16-byte values run 4 items only, 8-byte ones up to 16
      if constexpr (sizeof(T) <= 8) {
        if (p->merge_ipt == 16 && kIsReal<T>) ASAMD_LAUNCH_MERGE(16);
        else if (p->merge_ipt == 8) ASAMD_LAUNCH_MERGE(8);
        else ASAMD_LAUNCH_MERGE(4);
      } else {
        ASAMD_LAUNCH_MERGE(4);
      }
#undef ASAMD_LAUNCH_MERGE
      if (nb > 1)
        merge_fixup_kernel<T><<<(nb + 255) / 256, 256, 0, s>>>(nb, st.m, alpha, beta, p->d_carry_row,
                                                               (const T*)p->d_carry_val,
                                                               (const T*)p->d_head_val, y);
      break;
    }
    case ASAMD_SPMV_VECTOR:
    default:
      switch (p->auto_width) {
        case 2: launch_vector<T, 2>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 4: launch_vector<T, 4>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 8: launch_vector<T, 8>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 16: launch_vector<T, 16>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 32: launch_vector<T, 32>(s, st, alpha, val, rp, ci, x, beta, y); break;
        default: launch_vector<T, 64>(s, st, alpha, val, rp, ci, x, beta, y); break;
      }
      break;
  }
  return hipGetLastError();
}

template <typename T, int W, bool CONJ>
static void launch_trans_scatter(hipStream_t s, const asamd_csr_stats& st, T alpha, const T* val, const int* rp,
                                 const int* ci, const T* x, T* y) {
  constexpr int rows_per_block = kTransThreads / W;
  const unsigned grid = (unsigned)(((int64_t)st.m + rows_per_block - 1) / rows_per_block);
  csrmv_trans_scatter_kernel<T, W, CONJ><<<grid, kTransThreads, 0, s>>>(st.m, st.n, alpha, val, rp, ci, x, y,
                                                                         st.base);
}

template <typename T, bool CONJ>
static void trans_scatter(hipStream_t s, const asamd_csr_plan* p, T alpha, const T* val, const int* rp,
                          const int* ci, const T* x, T* y) {
  const asamd_csr_stats& st = p->st;
  switch (p->auto_width) {
    case 2: launch_trans_scatter<T, 2, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
    case 4: launch_trans_scatter<T, 4, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
    case 8: launch_trans_scatter<T, 8, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
    case 16: launch_trans_scatter<T, 16, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
    case 32: launch_trans_scatter<T, 32, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
    default: launch_trans_scatter<T, 64, CONJ>(s, st, alpha, val, rp, ci, x, y); break;
  }
}

// which = 0: y = alpha*A^T*x + beta*y; which = 1 (complex element types): A^H in place of A^T
template <typename T>
static int csrmv_trans_impl(hipStream_t s, asamd_csr_plan* p, T alpha, const T* val, const int* rp, const int* ci,
                            const T* x, T beta, T* y, int which) {
  if (!p || !val || !rp || !ci || !x || !y) return hipErrorInvalidValue;
  if (p->dtype != DtypeOf<T>::value || (which == 1 && kIsReal<T>)) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % alignof(T)) return hipErrorInvalidValue;
  const asamd_csr_stats& st = p->st;
  asamd_csr_plan::TransCopy& t = p->tr[which];
  // A library-owned mirror lays out its copy of the transpose on the first transposed multiply: that
  // allocates and waits, which a stream under capture must not do -- such a call scatters instead, and
  // the copy is laid out by the first call outside a capture.
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (!t.plan && p->lazy_transpose && hipStreamIsCapturing(s, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    capturing = hipStreamCaptureStatusActive;  // unknown: do not risk it
  }
  if (!t.plan && p->lazy_transpose && st.trusted && st.nnz > 0 && st.first_offset == 0 &&
      capturing == hipStreamCaptureStatusNone) {
    const hipError_t e = build_transpose<T>(s, p, rp, ci, val, which);
    if (e == hipErrorOutOfMemory) {
      (void)hipGetLastError();  // no room for the copy: scatter instead, and do not try again
      p->lazy_transpose = false;
    } else if (e != hipSuccess) {
      return e;
    }
  }
  // the copy holds the values it was gathered from: another value array takes the scatter route below
  if (t.plan && val == t.val_src)
    return csrmv_impl<T>(s, t.plan, alpha, (const T*)t.d_val, t.d_row_ptr, t.d_col, x, beta, y);
  if (beta != T(1)) scale_vec_kernel<T><<<(unsigned)(((int64_t)st.n + 255) / 256), 256, 0, s>>>(st.n, beta, y);
  if constexpr (!kIsReal<T>) {
    if (which == 1) {
      trans_scatter<T, true>(s, p, alpha, val, rp, ci, x, y);
      return hipGetLastError();
    }
  }
  trans_scatter<T, false>(s, p, alpha, val, rp, ci, x, y);
  return hipGetLastError();
}

extern "C" int asamd_s_csrmv_trans(hipStream_t stream, asamd_csr_plan* plan, float alpha, const float* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, const float* x, float beta,
                                   float* y) {
  return csrmv_trans_impl<float>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y, 0);
}

extern "C" int asamd_d_csrmv_trans(hipStream_t stream, asamd_csr_plan* plan, double alpha, const double* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, const double* x, double beta,
                                   double* y) {
  return csrmv_trans_impl<double>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y, 0);
}

extern "C" int asamd_s_csrmv(hipStream_t stream, asamd_csr_plan* plan, float alpha,
                             const float* val, const int32_t* row_ptr, const int32_t* col_ind,
                             const float* x, float beta, float* y) {
  return csrmv_impl<float>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_d_csrmv(hipStream_t stream, asamd_csr_plan* plan, double alpha,
                             const double* val, const int32_t* row_ptr, const int32_t* col_ind,
                             const double* x, double beta, double* y) {
  return csrmv_impl<double>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

// complex element types: op = 0 (A), 1 (A^T), 2 (A^H), the values of alphasparse_operation_t
static_assert(sizeof(asamd_complex8) == sizeof(Cx<float>) && sizeof(asamd_complex16) == sizeof(Cx<double>),
              "complex layouts");

template <typename T, typename C>
static int csrmv_complex(hipStream_t stream, asamd_csr_plan* plan, int32_t op, C alpha, const C* val,
                         const int32_t* row_ptr, const int32_t* col_ind, const C* x, C beta, C* y) {
  const T a(alpha.real, alpha.imag), b(beta.real, beta.imag);
  if (op == 0) return csrmv_impl<T>(stream, plan, a, (const T*)val, row_ptr, col_ind, (const T*)x, b, (T*)y);
  if (op == 1 || op == 2)
    return csrmv_trans_impl<T>(stream, plan, a, (const T*)val, row_ptr, col_ind, (const T*)x, b, (T*)y, op - 1);
  return hipErrorInvalidValue;
}

extern "C" int asamd_c_csrmv_op(hipStream_t stream, asamd_csr_plan* plan, int32_t op, asamd_complex8 alpha,
                                const asamd_complex8* val, const int32_t* row_ptr, const int32_t* col_ind,
                                const asamd_complex8* x, asamd_complex8 beta, asamd_complex8* y) {
  return csrmv_complex<Cx<float>>(stream, plan, op, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_z_csrmv_op(hipStream_t stream, asamd_csr_plan* plan, int32_t op, asamd_complex16 alpha,
                                const asamd_complex16* val, const int32_t* row_ptr, const int32_t* col_ind,
                                const asamd_complex16* x, asamd_complex16 beta, asamd_complex16* y) {
  return csrmv_complex<Cx<double>>(stream, plan, op, alpha, val, row_ptr, col_ind, x, beta, y);
}

// ---- the unanalysed, one-lane-per-row path ("plain") ---------------------------------------------
// op 0: every row summed by one lane in storage order; op 1 / 2: y scaled by beta, then one lane per
// row scatters alpha*op(a)*x[row] with atomics, the traversal of the reference's own transposed kernels.
template <typename T>
static int csrmv_plain_impl(hipStream_t s, int32_t op, int32_t m, int32_t n, int32_t base, T alpha, const T* val,
                            const int* rp, const int* ci, const T* x, T beta, T* y) {
  if (!val || !rp || !ci || !x || !y || m <= 0 || n <= 0 || op < 0 || op > 2 || (op == 2 && kIsReal<T>))
    return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % alignof(T)) return hipErrorInvalidValue;
  if (op == 0) {
    const unsigned grid = (unsigned)(((int64_t)m + kRowsBlock - 1) / kRowsBlock);
    spmv_scalar_kernel<T><<<grid, kRowsBlock, 0, s>>>(m, alpha, val, rp, ci, x, beta, y, base);
    return hipGetLastError();
  }
  if (beta != T(1)) scale_vec_kernel<T><<<(unsigned)(((int64_t)n + 255) / 256), 256, 0, s>>>(n, beta, y);
  const unsigned grid = (unsigned)(((int64_t)m + kTransThreads - 1) / kTransThreads);
  if constexpr (!kIsReal<T>) {
    if (op == 2) {
      csrmv_trans_scatter_kernel<T, 1, true><<<grid, kTransThreads, 0, s>>>(m, n, alpha, val, rp, ci, x, y, base);
      return hipGetLastError();
    }
  }
  csrmv_trans_scatter_kernel<T, 1, false><<<grid, kTransThreads, 0, s>>>(m, n, alpha, val, rp, ci, x, y, base);
  return hipGetLastError();
}

extern "C" int asamd_s_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, float alpha,
                                   const float* val, const int32_t* row_ptr, const int32_t* col_ind, const float* x,
                                   float beta, float* y) {
  return csrmv_plain_impl<float>(stream, op, m, n, base, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_d_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, double alpha,
                                   const double* val, const int32_t* row_ptr, const int32_t* col_ind, const double* x,
                                   double beta, double* y) {
  return csrmv_plain_impl<double>(stream, op, m, n, base, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_c_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base,
                                   asamd_complex8 alpha, const asamd_complex8* val, const int32_t* row_ptr,
                                   const int32_t* col_ind, const asamd_complex8* x, asamd_complex8 beta,
                                   asamd_complex8* y) {
  using T = Cx<float>;
  return csrmv_plain_impl<T>(stream, op, m, n, base, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind,
                             (const T*)x, T(beta.real, beta.imag), (T*)y);
}

extern "C" int asamd_z_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base,
                                   asamd_complex16 alpha, const asamd_complex16* val, const int32_t* row_ptr,
                                   const int32_t* col_ind, const asamd_complex16* x, asamd_complex16 beta,
                                   asamd_complex16* y) {
  using T = Cx<double>;
  return csrmv_plain_impl<T>(stream, op, m, n, base, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind,
                             (const T*)x, T(beta.real, beta.imag), (T*)y);
}

extern "C" int asamd_copy_bytes(hipStream_t stream, void* dst, const void* src, size_t nbytes) {
  if (!dst || !src || (nbytes & 15u) || (((uintptr_t)dst | (uintptr_t)src) & 15u))
    return hipErrorInvalidValue;
  const size_t n16 = nbytes / 16;
  if (n16 == 0) return hipSuccess;
  size_t grid = (n16 + 255) / 256;
  if (grid > 256 * 64) grid = 256 * 64;
  copy_bytes_kernel<<<(unsigned)grid, 256, 0, stream>>>((Int4*)dst, (const Int4*)src, n16);
  return hipGetLastError();
}

// ---- the multiply that allocates nothing -----------------------------------------------------
// Merge-path SpMV (the kernels of spmv_merge.hpp, 8 items per thread) whose workgroup coordinates,
// carries and head sums live in a fixed device array instead of a plan's hipMalloc'ed buffers.
// The array has four equal quarters of kStaticSlots 4-byte slots: block_row | carry_row | carry_val |
// head_val.  Every slot that a call reads is written by that call first, so nothing has to be cleared
// between calls; two calls that overlap on one device share the array and race.
constexpr int kStaticIpt = 8;
constexpr int kStaticSlots = ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES / 16;
static_assert((int64_t)(kStaticSlots - 1) * kMergeThreads * kStaticIpt == ASAMD_CSRMV_NOALLOC_MAX_ITEMS,
              "the documented limit is what the array holds");
static __device__ __align__(256) unsigned char scratch[ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` per device: every GPU holds its own copy of the array.  In host code
// the array's name is only a handle for hipGetSymbolAddress, never a pointer a kernel can take.
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static hipError_t static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

extern "C" int asamd_s_csrmv_noalloc(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, int32_t base,
                                     float alpha, const float* val, const int32_t* row_ptr,
                                     const int32_t* col_ind, const float* x, float beta, float* y) {
  if (m <= 0 || n <= 0 || nnz < 0 || (base != 0 && base != 1) || !row_ptr || !x || !y) return hipErrorInvalidValue;
  if (nnz > 0 && (!val || !col_ind)) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % alignof(float)) return hipErrorInvalidValue;
  const int64_t total = (int64_t)m + nnz;
  // larger problems need more workgroup slots than the fixed array has, and this call may not allocate
  if (total > ASAMD_CSRMV_NOALLOC_MAX_ITEMS) return hipErrorOutOfMemory;
  if (nnz == 0) {  // y = beta*y
    scale_vec_kernel<float><<<(unsigned)(((int64_t)m + 255) / 256), 256, 0, stream>>>(m, beta, y);
    return hipGetLastError();
  }
  void* base_ptr = nullptr;
  const hipError_t e = static_scratch(&base_ptr);
  if (e != hipSuccess) return e;
  int* block_row = (int*)base_ptr;
  int* carry_row = block_row + kStaticSlots;
  float* carry_val = (float*)(carry_row + kStaticSlots);
  float* head_val = carry_val + kStaticSlots;
  constexpr int kItems = kMergeThreads * kStaticIpt;
  const int nb = (int)((total + kItems - 1) / kItems);
  merge_partition_kernel<<<(nb + 1 + 255) / 256, 256, 0, stream>>>(m, nnz, row_ptr, base, nb, kItems, block_row);
  spmv_merge_kernel<float, kStaticIpt><<<nb, kMergeThreads, 0, stream>>>(m, nnz, alpha, val, row_ptr, col_ind, x, beta,
                                                                         y, base, block_row, carry_row, carry_val,
                                                                         head_val);
  if (nb > 1)
    merge_fixup_kernel<float><<<(nb + 255) / 256, 256, 0, stream>>>(nb, m, alpha, beta, carry_row, carry_val, head_val,
                                                                    y);
  return hipGetLastError();
}

extern "C" int asamd_warmup(hipStream_t stream) {
  // the library's init call: also resolves, for the current device, the address of the fixed array that
  // asamd_s_csrmv_noalloc works in, so that its first call has nothing left to set up
  void* p = nullptr;
  const hipError_t e = static_scratch(&p);
  if (e != hipSuccess) return e;
  warmup_kernel<<<1, 1, 0, stream>>>();
  return hipGetLastError();
}

// Mean of the samples below twice the plain mean: src/util_cpp/handle.cpp:495-510.
#include <vector>
extern "C" double get_avg_time(std::vector<double> times) {
  if (times.empty()) return 0.0;
  double avg = 0.0;
  for (double t : times) avg += t;
  avg /= (double)times.size();
  double kept = 0.0;
  int cnt = 0;
  for (double t : times)
    if (t < 2 * avg) {
      kept += t;
      ++cnt;
    }
  return cnt ? kept / cnt : avg;
}
