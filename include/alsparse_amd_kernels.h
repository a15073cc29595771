/*
 * alsparse_amd_kernels.h -- the thin C-ABI layer between the C host library
 * and the hand-written HIP kernels (gfx950, wave64).
 *
 * Everything here takes plain device pointers, sizes and a stream; no C++
 * types cross the boundary.  Return value is a hipError_t cast to int
 * (0 == hipSuccess).  The functions enqueue work on `stream` and return
 * without synchronising unless stated otherwise.
 *
 * Each entry names the reference kernel or launch it stands in for
 * (paths relative to the AlphaSparse source tree).
 */
#ifndef ALSPARSE_AMD_KERNELS_H
#define ALSPARSE_AMD_KERNELS_H

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* SpMV kernel families.  The reference has exactly one: a sub-wavefront per
 * row (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57), chosen
 * unconditionally (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_x_csr.cpp:21-31). */
enum asamd_spmv_algo {
  ASAMD_SPMV_AUTO = 0,     /* pick from the analysis                                */
  ASAMD_SPMV_VECTOR = 1,   /* W lanes per row, W in {2..64} from the mean row length */
  ASAMD_SPMV_ROWCONST = 2, /* every row has the same length L = 4*G: no row_ptr read */
  ASAMD_SPMV_MERGE = 3,    /* merge-path split of (rows + nnz), LDS-staged products  */
  ASAMD_SPMV_SCALAR = 4,   /* one lane per row; diagnostic baseline                  */
  ASAMD_SPMV_TILED = 5,    /* two-phase, (column block x row block) tiles: every x
                              gather and y update in LDS, HBM sees only streams     */
  ASAMD_SPMV_STREAM = 6,   /* rows of similar lengths (<= 256 entries): a row block's
                              products staged in LDS, 1..16 lanes sum a row          */
  ASAMD_SPMV_ELL = 7,      /* short, nearly equal rows: a column-major ELL copy, one
                              lane per row                                          */
  ASAMD_SPMV_MERGE_HOT = 8, /* merge-path whose persistent workgroups keep x of the most
                              popular columns in LDS (power-law graphs); the copy it
                              needs is structure only: values come from the caller  */
  ASAMD_SPMV_BINNED = 9,   /* one launch per row-length class (4, 16, 64 lanes per row;
                              the longest rows in chunks, a workgroup each): for very
                              uneven rows; keeps a list of row numbers, no values   */
  ASAMD_SPMV_XLDS = 10     /* W lanes per row with x held in every compute unit's LDS:
                              matrices of few columns (x <= 160 KB); keeps nothing  */
};

#define ASAMD_HIST_BINS 33

/* Element types; the values are those of the reference's alphasparse_datatype_t
 * (include/alphasparse/spdef.h:137-143). */
enum asamd_dtype {
  ASAMD_DTYPE_FLOAT = 0,
  ASAMD_DTYPE_DOUBLE = 1,
  ASAMD_DTYPE_FLOAT_COMPLEX = 2,
  ASAMD_DTYPE_DOUBLE_COMPLEX = 3
};

/* Complex scalars with the memory layout of the reference's ALPHA_Complex8 /
 * ALPHA_Complex16 (include/alphasparse/types.h:42-56).  Device arrays of them
 * must be aligned to the element size (8 / 16 bytes), as hipMalloc'ed arrays are;
 * entry points return hipErrorInvalidValue otherwise. */
#ifndef ALPHA_COMPLEX_TYPES_DEFINED
#define ALPHA_COMPLEX_TYPES_DEFINED
typedef struct { float real, imag; } ALPHA_Complex8;
typedef struct { double real, imag; } ALPHA_Complex16;
#endif
typedef ALPHA_Complex8 asamd_complex8;
typedef ALPHA_Complex16 asamd_complex16;

/* ---- CSR SpMV launchers ---------------------------------------------------------------------
 * Stateless: each call enqueues the kernels of ONE family on `stream` and returns.  Nothing is
 * allocated, copied or waited for, so every one of them can be recorded into a HIP graph.  Whatever a
 * family needs beyond the CSR arrays -- coordinates, re-ordered copies, per-call scratch -- is passed in
 * by the caller (the host library's plan, include/alsparse_amd_plan.h, which decides the family and owns
 * the memory).  All of them stand in for csr_gemv_vector_dispatch,
 * src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182, the reference's only kernel. */
typedef struct {
  int32_t dtype;            /* enum asamd_dtype: element type of val, x, y, alpha, beta */
  int32_t m, n, nnz, base;
  const void *alpha, *beta; /* HOST scalars */
  const void *val;          /* nnz values                                              */
  const int32_t *row_ptr;   /* m + 1 offsets                                           */
  const int32_t *col_ind;   /* nnz columns                                             */
  const void *x;            /* n elements                                              */
  void *y;                  /* m elements; beta == 0 never reads it                    */
} asamd_spmv_args;

/* `width` in {2, 4, ..., 64} lanes sum a row (the reference's mapping, dcu_gemv_vector.h:14-57). */
int asamd_spmv_vector(hipStream_t stream, const asamd_spmv_args *a, int32_t width);
/* the same, launched whatever happens but returning at once unless the device word *run_if is non-zero
 * (NULL: always runs): the stand-in for a kernel that a device-side guard may turn away */
int asamd_spmv_vector_if(hipStream_t stream, const asamd_spmv_args *a, int32_t width, const int32_t *run_if);
/* x held in the LDS of every compute unit (one workgroup of 1 024 threads each), `width` lanes per row: for
 * matrices whose x is at most ASAMD_XLDS_MAX_BYTES (asamd_spmv_xlds_fits); reads the CSR arrays in place. */
#define ASAMD_XLDS_MAX_BYTES 163840 /* the LDS of a compute unit */
int asamd_spmv_xlds_fits(int32_t dtype, int32_t n);
int asamd_spmv_xlds(hipStream_t stream, const asamd_spmv_args *a, int32_t width);
/* The same with the column numbers read from a 16-bit copy (zero-based, nnz + 4 elements, made once by
 * asamd_narrow_columns for a structure that stays): 6 instead of 8 bytes per fp32 entry.  Real element types, at least
 * four entries per row on average, n <= 65536; a->col_ind is not read.  (No counterpart in the reference, whose one
 * kernel reads the caller's 32-bit columns: src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57.) */
int asamd_narrow_columns(hipStream_t stream, int32_t nnz, int32_t base, const int32_t *col_ind, uint16_t *col16);
int asamd_spmv_xlds_narrow(hipStream_t stream, const asamd_spmv_args *a, int32_t width, const uint16_t *col16);
/* The same for an x of several LDS fills (real element types): the matrix in `slices` slices of slice_cols columns,
 * a row of workgroups each.  With ascending columns inside the rows a row's entries of one slice are a contiguous
 * piece of the caller's arrays, so the layout is a table of offsets only -- seg[s * m + r], s = 0 .. slices: where
 * row r's piece of slice s begins (base included) -- and the values are read in place.  asamd_xlds_build leaves
 * the record EMPTY (seg NULL, not an error) if some row's columns do not ascend.  Per-call scratch: slices * m
 * elements of `partials`; `width` as for asamd_spmv_vector, from the pieces' mean length.
 * With `val` given, asamd_xlds_build also COPIES the entries slice by slice (every slice a CSR matrix of its own:
 * the pieces of consecutive rows consecutive in memory, 16-bit columns counted from the slice's first one, off[s * m
 * + r] the piece's place in the copy), which the multiply then reads instead of the caller's arrays; short pieces
 * scattered over the caller's arrays cost whole cache lines each.  asamd_xlds_refresh_values copies the values again
 * (gate: NULL, or a device word that is 0 when there is nothing to do).  (No counterpart in the reference, which keeps
 * no copy of a matrix: src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:269-391 records row blocks only.) */
typedef struct {
  int32_t *seg;  /* (slices + 1) * m offsets; NULL: no layout */
  int32_t slices, slice_cols, m;
  int64_t device_bytes;
  int32_t *off;  /* slices * m + 1 offsets into the copy; NULL: no copy */
  void *val;     /* nnz (+ 4 of padding) values, slice by slice */
  uint16_t *col; /* their columns, counted from the slice's first */
  int32_t dtype, nnz, base;
} asamd_xlds_layout;
int32_t asamd_xlds_slices(int32_t dtype, int32_t n); /* the slices asamd_xlds_build would cut n columns into */
int asamd_xlds_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                     const int32_t *row_ptr, const int32_t *col_ind, const void *val, asamd_xlds_layout *out);
int asamd_xlds_refresh_values(hipStream_t stream, const asamd_xlds_layout *layout, const void *val,
                              const int32_t *gate);
void asamd_xlds_free(asamd_xlds_layout *layout);
int asamd_spmv_xlds_sliced(hipStream_t stream, const asamd_spmv_args *a, int32_t width, const asamd_xlds_layout *layout,
                           void *partials);
/* One lane per row, entries in storage order (src/plain/kernel/level2/mv/gemv/gemv_x_csr_plain.c:11-22). */
int asamd_spmv_scalar(hipStream_t stream, const asamd_spmv_args *a);
/* Every row has row_len entries (4, 8, ..., 256): no row_ptr traffic.  Real element types, row_ptr[0] ==
 * base, val and col_ind 16-byte aligned; hipErrorInvalidValue otherwise. */
int asamd_spmv_rowconst(hipStream_t stream, const asamd_spmv_args *a, int32_t row_len);
/* Rows of at most max_len <= ASAMD_STREAM_MAX_GROUP * (64 / sizeof element) entries: 256 / group rows per
 * workgroup, their products staged in LDS, `group` lanes (1, 2, 4, 8, 16) sum a row.  A workgroup whose
 * rows hold more entries than its staging area takes them from global memory, so a max_len that has
 * gone stale costs speed, not correctness.  first_offset = row_ptr[0] - base. */
#define ASAMD_STREAM_MAX_GROUP 16
/* The same with the column numbers read as 16-bit signed distances from the first row of the entry's workgroup
 * (rel16: nnz + 4 elements, made once by asamd_narrow_rel_columns for a structure that stays and for THIS `group`;
 * *too_far, a device word the caller has cleared, is set if some entry lies further than 32 767 columns from that
 * row, and rel16 is then unusable): 10 instead of 12 bytes per fp64 entry.  Real element types, val 16-byte aligned,
 * row_ptr[0] == base.  (No counterpart in the reference: dcu_gemv_vector.h:14-57 reads 32-bit columns.) */
int asamd_narrow_rel_columns(hipStream_t stream, int32_t m, int32_t nnz, int32_t base, int32_t group,
                             const int32_t *row_ptr, const int32_t *col_ind, int16_t *rel16, int32_t *too_far);
int asamd_spmv_stream_rel16(hipStream_t stream, const asamd_spmv_args *a, int32_t group, int32_t max_len,
                            const int16_t *rel16);
int asamd_spmv_stream(hipStream_t stream, const asamd_spmv_args *a, int32_t group, int32_t max_len,
                      int32_t first_offset);

/* Merge-path: the (m + nnz) items are cut into blocks of ASAMD_MERGE_THREADS * ipt items (ipt: 4, 8, or
 * 16 for real types of at most 8 bytes; 4 only for 16-byte values).  block_row: blocks + 1 merge
 * coordinates from asamd_merge_partition (row_ptr[0] must equal base and nnz must be row_ptr[m] - base).
 * Per-call scratch: carry_row (blocks ints), carry_val and head_val (blocks elements each); every word
 * that a call reads it has written before, so the scratch needs no clearing, and two multiplies that
 * run at the same time need a scratch each.  No float atomics. */
#define ASAMD_MERGE_THREADS 256
int asamd_merge_partition(hipStream_t stream, int32_t m, int32_t nnz, const int32_t *row_ptr, int32_t base,
                          int32_t blocks, int32_t items_per_block, int32_t *block_row);
int asamd_spmv_merge(hipStream_t stream, const asamd_spmv_args *a, int32_t ipt, const int32_t *block_row,
                     int32_t *carry_row, void *carry_val, void *head_val);

/* Transposed / conjugate-transposed product without a copy: y (n elements) is scaled by beta, then
 * `width` lanes per row scatter alpha*op(a)*x[row] with hardware float atomics, the traversal of
 * src/kernel/dcu/level2/mv/csrmv/dcu_gemv_x_csr_trans.cpp:11-68 and dcu_gemv_c_csr_conj.cpp:22-75.
 * x has m elements.  conj != 0: complex types only. */
int asamd_spmv_trans_scatter(hipStream_t stream, const asamd_spmv_args *a, int32_t width, int32_t conj);
/* The same for a matrix of so few columns that y (n elements) fits a compute unit's LDS (asamd_spmv_xlds_fits):
 * every workgroup adds up its rows' contributions in LDS and the workgroups' sums are added in order.  partials:
 * asamd_spmv_trans_ylds_bytes(dtype, m, n) bytes of per-call scratch (0: the matrix does not suit). */
size_t asamd_spmv_trans_ylds_bytes(int32_t dtype, int32_t m, int32_t n);
int asamd_spmv_trans_ylds(hipStream_t stream, const asamd_spmv_args *a, int32_t width, int32_t conj, void *partials);

/* ---- re-ordered copies of a CSR matrix ("layouts") and the kernels that multiply with them ------
 * A layout is a plain record of device pointers and counts, filled by its *_build call (which
 * allocates, launches the layout kernels on `stream` and synchronises it) and released by *_free.
 * Builders return hipSuccess with an EMPTY record (first pointer NULL) when the matrix does not suit the
 * layout; that is not an error.  device_bytes: device memory the record holds. */

/* Tiled two-phase SpMV for x far larger than an XCD's L2: entries sorted by (column block, row block);
 * phase 1 multiplies against an x slice held in LDS and streams the products out, phase 2 adds them
 * up in per-wave LDS accumulators, phase 3 takes the tiles too long for phase 2.  Holds the VALUES in
 * tile order (tval) and the CSR position of every slot (tperm), through which asamd_gather_values
 * refreshes them.  Per-call scratch: nnz elements of products and long_scratch_elems elements. */
typedef struct {
  void *tval;                /* nnz values in tile order; NULL: no layout                      */
  uint32_t *tperm;           /* nnz: CSR position of the entry in every slot                   */
  uint16_t *tcol, *trow;     /* nnz columns / rows local to their blocks                       */
  int32_t *row_block_start;  /* row_blocks + 1                                                 */
  int32_t *tile_ptr;         /* col_blocks * row_blocks + 1: first slot of tile c * row_blocks + r */
  void *ranges, *chunks, *long_list, *long_tiles, *long_finish; /* tile tables and work lists  */
  int32_t dtype, m, n, nnz;
  int32_t col_blocks, row_blocks;
  int32_t entries_per_lane;  /* phase 2 takes 1 or 2 entries per lane and tile                 */
  int32_t n_chunks, n_long_chunks, n_long_narrow, n_long_finish, long_blocks;
  int64_t long_scratch_elems;
  int64_t device_bytes;
} asamd_tiled_layout;
/* 1 if the block counts that (dtype, m, n, nnz) give fit the tile tables */
int asamd_tiled_fits(int32_t dtype, int32_t m, int32_t n, int32_t nnz);
/* max_len: longest row (steers the block heights); entries_per_lane: 0 = choose from the tile lengths */
int asamd_tiled_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                      const int32_t *row_ptr, const int32_t *col_ind, const void *val, int32_t max_len,
                      int32_t entries_per_lane, asamd_tiled_layout *out);
void asamd_tiled_free(asamd_tiled_layout *layout);
/* layout->tval[q] = val[layout->tperm[q]] for every slot, the tiles taken row block by row block (each XCD its
 * own row blocks), so that the stretch of val a row block's tiles pick their values from is fetched from memory
 * once; gate as for asamd_gather_values */
int asamd_tiled_gather_values(hipStream_t stream, const asamd_tiled_layout *layout, const void *val,
                              const int32_t *gate);
/* y = alpha*A*x + beta*y from the layout (a->val, a->row_ptr, a->col_ind are not read).  skip: NULL, or a
 * device word; when it is non-zero the kernels that write y return at once (a guard found that the layout no
 * longer describes the caller's matrix, and asamd_spmv_vector_if on the same word computes y instead) */
int asamd_spmv_tiled(hipStream_t stream, const asamd_spmv_args *a, const asamd_tiled_layout *layout,
                     void *products, void *long_scratch, const int32_t *skip);

/* Hot-column merge-path for power-law columns: the column stream rewritten as ranks of the popular
 * columns (pcol), whose x sits in LDS (the cols_lds most popular) or in a compact front (cols_front).
 * Structure only: values come from the caller's array.  Per-call scratch: front (cols_front elements),
 * carry_row (blocks ints), carry_val and head_val (blocks elements each).  Element types of at most 8 bytes. */
typedef struct {
  uint32_t *pcol;            /* nnz positions; NULL: no layout */
  int32_t *hot_cols;         /* cols_front zero-based columns, most popular first */
  int32_t *block_row;        /* blocks + 1 merge coordinates of the wave-sized blocks */
  int32_t dtype, blocks, cols_lds, cols_front;
  float share_lds;           /* share of the entries whose column is one of the cols_lds */
  int64_t device_bytes;
} asamd_hot_layout;
/* force == 0: an empty record when the LDS columns hold less than a fifth of the entries;
 * cols_lds / cols_front: 0 = the kernel's capacity / what shares an L2 with the streams */
int asamd_hot_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                    const int32_t *row_ptr, const int32_t *col_ind, int32_t force, int32_t cols_lds,
                    int32_t cols_front, asamd_hot_layout *out);
void asamd_hot_free(asamd_hot_layout *layout);
int asamd_spmv_hot(hipStream_t stream, const asamd_spmv_args *a, const asamd_hot_layout *layout, void *front,
                   int32_t *carry_row, void *carry_val, void *head_val);

/* Row-length bins: the row numbers sorted by length class (<= 8, <= 64, <= 2 048 entries, longer), one
 * launch per class with 4 / 16 / 64 lanes per row, the longest rows in chunks of 4 096 entries whose
 * sums meet in chunk order.  Structure only.  Per-call scratch: `chunks` elements. */
typedef struct {
  int32_t *rows;             /* m row numbers by class, ascending inside a class; NULL: no layout */
  void *chunk_list;          /* chunks records */
  int32_t *chunk_first;      /* count[3] + 1: first chunk of every long row */
  int32_t count[4];          /* rows per class */
  int32_t chunks;
  int64_t device_bytes;
} asamd_binned_layout;
int asamd_binned_build(hipStream_t stream, int32_t m, int32_t base, const int32_t *row_ptr,
                       asamd_binned_layout *out);
void asamd_binned_free(asamd_binned_layout *layout);
int asamd_spmv_binned(hipStream_t stream, const asamd_spmv_args *a, const asamd_binned_layout *layout,
                      void *partial);

/* CSR copy of A^T (conj != 0: of A^H, complex types): n + 1 offsets, nnz zero-based columns (rows of
 * A, ascending inside a row of the copy), nnz values and the CSR position of every entry (perm),
 * through which asamd_gather_values refreshes the values.  The reference always scatters
 * (dcu_gemv_x_csr_trans.cpp:11-68); the ordinary kernels run on this copy instead. */
typedef struct {
  int32_t *row_ptr;          /* NULL: no copy */
  int32_t *col_ind;
  void *val;
  uint32_t *perm;
  int64_t device_bytes;
} asamd_transpose_layout;
int asamd_transpose_build(hipStream_t stream, int32_t dtype, int32_t conj, int32_t m, int32_t n, int32_t nnz,
                          int32_t base, const int32_t *row_ptr, const int32_t *col_ind, const void *val,
                          asamd_transpose_layout *out);
void asamd_transpose_free(asamd_transpose_layout *layout);

/* ---- analysis building blocks --------------------------------------------------------------- */
/* One pass over row_ptr: stats_host[0] = shortest row, [1] = longest, [2] = row_ptr[0], [3 + b] = rows
 * in bin b of the log2 histogram (bin 0: empty rows, bin b: 2^(b-1) .. 2^b - 1 entries).  d_scratch:
 * ASAMD_ROW_STATS_WORDS device ints.  Synchronises `stream`.  Replaces the host-side row walk of
 * src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267 and its round trip at :348-379. */
#define ASAMD_ROW_STATS_WORDS (3 + ASAMD_HIST_BINS)
int asamd_csr_row_stats(hipStream_t stream, int32_t m, const int32_t *row_ptr, int32_t *d_scratch,
                        int32_t *stats_host);
/* 64-bit fingerprint of the structure arrays (m + 1 offsets, nnz columns): equal arrays give equal
 * values.  d_scratch: 8 device bytes, 8-byte aligned.  Synchronises `stream`; *hash_host is a host word. */
int asamd_csr_structure_hash(hipStream_t stream, int32_t m, int32_t nnz, const int32_t *row_ptr,
                             const int32_t *col_ind, void *d_scratch, uint64_t *hash_host);
/* A deterministic look at where the columns of consecutive entries fall: `segments` runs of 32 768
 * consecutive entries spread evenly over the entry stream.  out_host[0] = distinct 128-byte lines of x per
 * entry among every 64 consecutive entries (1/64 .. 1: the requests that one gather instruction of a wave
 * sends to the L1), out_host[1] = distinct lines per entry within a whole run (reuse inside a compute unit's
 * neighbourhood of the stream counted once).  d_scratch: 24 device bytes, 8-byte aligned.  Synchronises
 * `stream`.  The same arrays always give the same two numbers. */
int asamd_csr_locality_probe(hipStream_t stream, int32_t nnz, int32_t base, int32_t elem_bytes,
                             const int32_t *col_ind, int32_t segments, void *d_scratch, float *out_host);

/* ---- values that change under a copy ---------------------------------------------------------
 * The reference's analysis keeps structure only (alphasparse_dcu_x_csrmv_analysis.cpp:382-388) and its
 * kernels read csr_val on every call (dcu_gemv_vector.h:43-46), so callers may rewrite the values in
 * place between multiplies.  A copy of the values is kept honest on the device, without a host
 * round trip and inside a HIP graph if need be:
 *   asamd_value_guard      fingerprints val (nbytes; every byte when nbytes <= ASAMD_GUARD_FULL_BYTES or
 *                          full != 0, otherwise 256 bytes at a varying position of every run of
 *                          asamd_value_guard_run(nbytes) bytes, 32 MiB in all), compares with the word
 *                          at `stored` and leaves the verdict in ws: a flag and the new fingerprint;
 *   gated kernels          (asamd_gather_values, asamd_csr2ell_gated) take the flag's address and return
 *                          at once when it is 0;
 *   asamd_value_guard_commit   stores the new fingerprint at `stored` if the flag is set -- AFTER the
 *                          gated kernels in stream order, so that another stream that finds the stored
 *                          word up to date also finds the copies refreshed.
 * stored == NULL in asamd_value_guard sets the flag whatever the values are (first fingerprint).
 * ws: ASAMD_GUARD_WS_BYTES of per-call device scratch, 8-byte aligned. */
#define ASAMD_GUARD_WS_BYTES (16384 + 64)
#define ASAMD_GUARD_FULL_BYTES ((size_t)32 << 20)
#define ASAMD_GUARD_FLAG(ws) ((const int32_t *)((const char *)(ws) + 16384 + 8))
size_t asamd_value_guard_run(size_t nbytes);
int asamd_value_guard(hipStream_t stream, const void *val, size_t nbytes, int32_t full, const uint64_t *stored,
                      void *ws);
int asamd_value_guard_commit(hipStream_t stream, const void *ws, uint64_t *stored);
/* *out = 1 if either of two guards' flags is set, else 0 (the guard works on any array of 4-byte words: the
 * structure arrays of a matrix that nobody promised to leave alone are watched with it too) */
int asamd_value_guard_any(hipStream_t stream, const void *ws_a, const void *ws_b, int32_t *out);
/* out[q] = val[perm[q]] (conj != 0: conjugated) for q < nnz; gate: NULL, or a device flag (0 = do nothing) */
int asamd_gather_values(hipStream_t stream, int32_t dtype, int32_t conj, int32_t nnz, const uint32_t *perm,
                        const void *val, void *out, const int32_t *gate);

/* y = alpha*op(A)*x + beta*y without any analysis, in the traversal of the reference's plain
 * kernels: op = 0 one lane per row summing its entries in storage order
 * (src/plain/kernel/level2/mv/gemv/gemv_x_csr_plain.c:11-22), op = 1 / 2 (2: complex types) one lane
 * per row scattering into y (gemv_x_csr_trans_plain.c:10-24, gemv_c_csr_conj_plain.c:10-27; atomics
 * make the order of those additions free).  Backs alphasparse_?_mv_plain. */
int asamd_s_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, float alpha,
                        const float *val, const int32_t *row_ptr, const int32_t *col_ind, const float *x,
                        float beta, float *y);
int asamd_d_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, double alpha,
                        const double *val, const int32_t *row_ptr, const int32_t *col_ind, const double *x,
                        double beta, double *y);
int asamd_c_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, asamd_complex8 alpha,
                        const asamd_complex8 *val, const int32_t *row_ptr, const int32_t *col_ind,
                        const asamd_complex8 *x, asamd_complex8 beta, asamd_complex8 *y);
int asamd_z_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, asamd_complex16 alpha,
                        const asamd_complex16 *val, const int32_t *row_ptr, const int32_t *col_ind,
                        const asamd_complex16 *x, asamd_complex16 beta, asamd_complex16 *y);

/* Dense operand addressing for SpMM: element (r, c) of B is
 * B[r*b_row_stride + c*b_col_stride], of C is C[r*c_row_stride + c*c_col_stride]. */
typedef struct {
  int64_t b_row_stride, b_col_stride;
  int64_t c_row_stride, c_col_stride;
} asamd_dense_strides;

/* C = alpha*A*B + beta*C, A m x k CSR, B k x n, C m x n.  Stands in for
 * dcu_gemm_?_csr_row (stub, src/kernel/dcu/level3/mm/csrmm/dcu_gemm_x_csr_row.cpp:15-36),
 * gemm_col_plain_dispatch (dcu_gemm_csr_col_plain.h:42-61) and
 * csrmmnt_general_device (dcu_gemm_x_csr_col_transB.cpp:39-108, :199-226). */
int asamd_s_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, float alpha,
                  const float *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                  const float *B, float beta, float *C,
                  const asamd_dense_strides *strides);
int asamd_d_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, double alpha,
                  const double *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                  const double *B, double beta, double *C,
                  const asamd_dense_strides *strides);

/* C = alpha*A*B + beta*C, one lane per element of C walking its row of A in storage order, any
 * strides (src/plain/kernel/level3/mm/gemm/gemm_x_csr_row_plain.c:6-21, gemm_x_csr_col_plain.c:6-19).
 * Backs alphasparse_?_mm_plain. */
int asamd_s_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, float alpha, const float *val,
                        const int32_t *row_ptr, const int32_t *col_ind, int32_t base, const float *B, float beta,
                        float *C, const asamd_dense_strides *strides);
int asamd_d_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, double alpha, const double *val,
                        const int32_t *row_ptr, const int32_t *col_ind, int32_t base, const double *B, double beta,
                        double *C, const asamd_dense_strides *strides);
int asamd_c_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex8 alpha, const asamd_complex8 *val,
                        const int32_t *row_ptr, const int32_t *col_ind, int32_t base, const asamd_complex8 *B,
                        asamd_complex8 beta, asamd_complex8 *C, const asamd_dense_strides *strides);
int asamd_z_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex16 alpha, const asamd_complex16 *val,
                        const int32_t *row_ptr, const int32_t *col_ind, int32_t base, const asamd_complex16 *B,
                        asamd_complex16 beta, asamd_complex16 *C, const asamd_dense_strides *strides);

/* Column-major B next to column-major C is multiplied from a row-major copy of B
 * (k*n elements) in a caller-provided device workspace; without one, or with too
 * small a one, the multiply falls back to gathering B element by element, which
 * is tens of times slower.  asamd_csrmm_workspace_bytes returns what those strides
 * need (0 for every other layout).  The workspace only has to live until the
 * call's kernels have run on `stream`. */
size_t asamd_csrmm_workspace_bytes(int32_t val_size, int32_t m, int32_t n, int32_t k,
                                   const asamd_dense_strides *strides);
int asamd_s_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, float alpha,
                     const float *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                     const float *B, float beta, float *C, const asamd_dense_strides *strides,
                     void *workspace, size_t workspace_bytes);
int asamd_d_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, double alpha,
                     const double *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                     const double *B, double beta, double *C, const asamd_dense_strides *strides,
                     void *workspace, size_t workspace_bytes);

int asamd_c_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, asamd_complex8 alpha,
                     const asamd_complex8 *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                     const asamd_complex8 *B, asamd_complex8 beta, asamd_complex8 *C,
                     const asamd_dense_strides *strides, void *workspace, size_t workspace_bytes);
int asamd_z_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, asamd_complex16 alpha,
                     const asamd_complex16 *val, const int32_t *row_ptr, const int32_t *col_ind, int32_t base,
                     const asamd_complex16 *B, asamd_complex16 beta, asamd_complex16 *C,
                     const asamd_dense_strides *strides, void *workspace, size_t workspace_bytes);

/* coo_row[k] = r + base for k in [row_ptr[r]-base, row_ptr[r+1]-base).
 * Defines on the GPU what src/core/format/convert_coo_x_csr.c:30-37 does on the host. */
int asamd_csr2coo(hipStream_t stream, const int32_t *row_ptr, int32_t nnz, int32_t m,
                  int32_t *coo_row, int32_t base);
/* The same with a device workspace of asamd_csr2coo_workspace_bytes(nnz) bytes (4 per 8192 entries):
 * the rows at the chunk boundaries are then found by a kernel of their own, all searches in flight
 * together, instead of by every workgroup for itself (2^28 entries: 0.39 ms -> 0.26 ms).  A null or
 * too small workspace gives the behaviour of asamd_csr2coo. */
size_t asamd_csr2coo_workspace_bytes(int32_t nnz);
int asamd_csr2coo_ws(hipStream_t stream, const int32_t *row_ptr, int32_t nnz, int32_t m,
                     int32_t *coo_row, int32_t base, void *workspace, size_t workspace_bytes);

/* Longest row.  Synchronises `stream`; *width_host is a host int.
 * src/core/format/convert_ell_x_coo.c:46-52. */
int asamd_csr2ell_width(hipStream_t stream, int32_t m, const int32_t *row_ptr,
                        int32_t *width_host);

/* Column-major ELL, padding (value 0, index ell_base).
 * src/core/format/convert_ell_x_coo.c:59-79. */
int asamd_s_csr2ell(hipStream_t stream, int32_t m, const float *val, const int32_t *row_ptr,
                    const int32_t *col_ind, int32_t csr_base, int32_t ell_base, int32_t width,
                    float *ell_val, int32_t *ell_col);
int asamd_d_csr2ell(hipStream_t stream, int32_t m, const double *val, const int32_t *row_ptr,
                    const int32_t *col_ind, int32_t csr_base, int32_t ell_base, int32_t width,
                    double *ell_val, int32_t *ell_col);
int asamd_c_csr2ell(hipStream_t stream, int32_t m, const asamd_complex8 *val, const int32_t *row_ptr,
                    const int32_t *col_ind, int32_t csr_base, int32_t ell_base, int32_t width,
                    asamd_complex8 *ell_val, int32_t *ell_col);
int asamd_z_csr2ell(hipStream_t stream, int32_t m, const asamd_complex16 *val, const int32_t *row_ptr,
                    const int32_t *col_ind, int32_t csr_base, int32_t ell_base, int32_t width,
                    asamd_complex16 *ell_val, int32_t *ell_col);
/* The same for elements of elem_bytes (4, 8 or 16) bytes, copied bit for bit, behind a gate: a device
 * flag left by asamd_value_guard (0 = the conversion does nothing), or NULL. */
int asamd_csr2ell_gated(hipStream_t stream, int32_t elem_bytes, int32_t m, const void *val, const int32_t *row_ptr,
                        const int32_t *col_ind, int32_t csr_base, int32_t ell_base, int32_t width, void *ell_val,
                        int32_t *ell_col, const int32_t *gate);

/* y = alpha*A*x + beta*y, A in column-major ELL (slot s of row r at [s*m + r]);
 * slots whose index (minus base) is outside [0, n) are skipped.  Stands in for
 * dcu_gemv_?_ell, src/kernel/dcu/level2/mv/dcu_gemv_x_ell.cpp:10-43, :48-69. */
int asamd_s_ellmv(hipStream_t stream, int32_t m, int32_t n, float alpha, const float *ell_val,
                  const int32_t *ell_col_ind, int32_t ell_width, int32_t base, const float *x,
                  float beta, float *y);
int asamd_d_ellmv(hipStream_t stream, int32_t m, int32_t n, double alpha, const double *ell_val,
                  const int32_t *ell_col_ind, int32_t ell_width, int32_t base, const double *x,
                  double beta, double *y);
int asamd_c_ellmv(hipStream_t stream, int32_t m, int32_t n, asamd_complex8 alpha, const asamd_complex8 *ell_val,
                  const int32_t *ell_col_ind, int32_t ell_width, int32_t base, const asamd_complex8 *x,
                  asamd_complex8 beta, asamd_complex8 *y);
int asamd_z_ellmv(hipStream_t stream, int32_t m, int32_t n, asamd_complex16 alpha, const asamd_complex16 *ell_val,
                  const int32_t *ell_col_ind, int32_t ell_width, int32_t base, const asamd_complex16 *x,
                  asamd_complex16 beta, asamd_complex16 *y);

/* y = alpha*A*x + beta*y, A in COO.  Fastest when entries are grouped by row
 * (as asamd_csr2coo leaves them) but correct for any order; entries whose row or
 * column (minus base) is out of range are skipped.  y must be ordinary device
 * memory (hardware float atomics).  workspace: device memory, 16-byte aligned, for two
 * (row, sum) slots per wave, where the first and last row segment of every wave meet
 * their neighbours' in wave order, so that entries grouped by row give the same y from
 * run to run; a small workspace makes the waves longer (1 MiB serves any size), NULL
 * sends every segment to y at once (rows shared by waves then add up in any order).
 * Stands in for dcu_gemv_?_coo,
 * src/kernel/dcu/level2/mv/dcu_gemv_x_coo.cpp:10-195. */
int asamd_s_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, float alpha,
                  const float *coo_val, const int32_t *coo_row_ind, const int32_t *coo_col_ind,
                  int32_t base, const float *x, float beta, float *y, void *workspace,
                  size_t workspace_bytes);
int asamd_d_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, double alpha,
                  const double *coo_val, const int32_t *coo_row_ind, const int32_t *coo_col_ind,
                  int32_t base, const double *x, double beta, double *y, void *workspace,
                  size_t workspace_bytes);
int asamd_c_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, asamd_complex8 alpha,
                  const asamd_complex8 *coo_val, const int32_t *coo_row_ind, const int32_t *coo_col_ind,
                  int32_t base, const asamd_complex8 *x, asamd_complex8 beta, asamd_complex8 *y, void *workspace,
                  size_t workspace_bytes);
int asamd_z_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, asamd_complex16 alpha,
                  const asamd_complex16 *coo_val, const int32_t *coo_row_ind, const int32_t *coo_col_ind,
                  int32_t base, const asamd_complex16 *x, asamd_complex16 beta, asamd_complex16 *y, void *workspace,
                  size_t workspace_bytes);

/* handle->stream for callers that cannot see the handle struct (language bindings); C callers assign
 * the field, as with the reference.  `handle` is an alphasparse_dcu_handle_t.  Every multiply that
 * runs from an explicit analysis only launches kernels on that stream, so it can be captured into
 * a HIP graph. */
int asamd_handle_set_stream(void *handle, hipStream_t stream);
hipStream_t asamd_handle_get_stream(void *handle);

/* Empty kernel; forces code-object load (src/util_cpp/handle.cpp:19, :113).  Also looks up, for the
 * current device, the address of the fixed array that asamd_s_csrmv_noalloc works in. */
int asamd_warmup(hipStream_t stream);

/* asamd_s_csrmv without a plan and without any allocation: for callers that cannot call hipMalloc
 * (code under HIP graph capture, tight serving loops, harnesses that forbid it).  No counterpart in
 * the reference.  Runs the merge-path kernels (any row-length distribution, no float atomics); their
 * workgroup coordinates, carries and head sums live in a fixed device array of
 * ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES that the library holds per GPU until the process ends.
 * m + nnz above ASAMD_CSRMV_NOALLOC_MAX_ITEMS returns hipErrorOutOfMemory (2) before anything is
 * launched; other bad arguments return hipErrorInvalidValue.  base is 0 or 1; nnz == 0 gives
 * y = beta*y.  Required and NOT checked (the check would need a look at device memory): row_ptr[0] ==
 * base and nnz == row_ptr[m] - base, i.e. row_ptr describes exactly the nnz entries passed -- a slice
 * of a larger matrix's row_ptr gives wrong results here.  Calls hipMalloc, hipFree or an allocating
 * library routine never; asamd_warmup (run by alphasparse_dcu_get_handle) resolves the array's address
 * for the current device; a first call on a device where that has not happened does so itself, which a
 * stream under capture may not allow: call asamd_warmup first.  All calls on one GPU share the array:
 * calls that overlap there (two streams, two threads) race; calls on one stream are ordered and safe. */
#define ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES (4 << 20)
#define ASAMD_CSRMV_NOALLOC_MAX_ITEMS 536868864LL /* (SCRATCH_BYTES / 16 - 1) workgroups x 2048 items */
int asamd_s_csrmv_noalloc(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, int32_t base, float alpha,
                          const float *val, const int32_t *row_ptr, const int32_t *col_ind, const float *x,
                          float beta, float *y);

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_KERNELS_H */
