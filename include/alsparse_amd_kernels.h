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
  ASAMD_SPMV_BINNED = 9    /* one launch per row-length class (4, 16, 64 lanes per row;
                              the longest rows in chunks, a workgroup each): for very
                              uneven rows; keeps a list of row numbers, no values   */
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

/* Row-length statistics gathered on the GPU.  hist[0] counts empty rows,
 * hist[b] rows whose length lies in [2^(b-1), 2^b). */
typedef struct {
  int32_t m, n, nnz, base;
  int32_t min_len, max_len;
  int32_t const_len;    /* common row length, or -1                          */
  int32_t first_offset; /* row_ptr[0] - base                                 */
  int32_t algo;         /* enum asamd_spmv_algo chosen for this structure     */
  int32_t vector_width; /* lanes per row when algo == VECTOR                  */
  int32_t merge_blocks; /* workgroups of the merge-path kernel                */
  int32_t trusted;      /* 1: structure promised fixed, coordinates cached    */
  int32_t tiled_built;  /* 1: a tiled copy exists (TILED can be selected)     */
  int32_t tile_col_blocks, tile_row_blocks;
  float tune_ms_base;   /* analysis-time timing of the non-tiled choice, or 0 */
  float tune_ms_tiled;  /* ... and of the tiled kernel pair, or 0             */
  float tune_ms_ell;    /* ... and of the ELL copy's kernel, or 0             */
  int32_t ell_built;    /* 1: an ELL copy exists (ELL can be selected)        */
  int32_t ell_width;    /* its slots per row                                  */
  int32_t transpose_built; /* bit 0: a CSR copy of the transpose exists, bit 1: of the
                              conjugate transpose                              */
  int32_t tile_entries_per_lane; /* tiled copy: entries per lane and tile in its second
                                    phase (1: twice the tiles in flight; tiles of more
                                    than 64 entries go to the long-tile kernel), or 0  */
  int64_t hist[ASAMD_HIST_BINS];
  int32_t hot_built;     /* 1: the hot-column copy exists (MERGE_HOT can be selected)        */
  int32_t hot_cols_lds;  /* columns whose x the kernel keeps in LDS                            */
  int32_t hot_cols;      /* most popular columns whose x every multiply gathers into a compact front */
  float hot_share_lds;   /* share of the entries that fall into the LDS columns               */
  float tune_ms_hot;     /* analysis-time timing of the hot-column kernel, or 0               */
  int32_t binned_built;  /* 1: the row numbers are sorted by length class (BINNED can be selected) */
  int32_t bin_rows[4];   /* rows of at most 8 / 64 / 2 048 entries / longer                   */
  float tune_ms_binned;  /* analysis-time timing of the per-class launches, or 0              */
  int32_t tile_long_blocks; /* tiled copy: row blocks with tiles too long for its second phase (its third
                               phase takes them), or 0                                           */
} asamd_csr_stats;

typedef struct asamd_csr_plan asamd_csr_plan;

/* Row-length histogram, kernel choice and (trusted != 0) cached merge-path
 * block coordinates.  Synchronises `stream` to read the statistics.
 * Replaces the host-side row-block builder
 * src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267, :348-379.
 * val_size is sizeof(value type): 4 (fp32) or 8 (fp64).
 * trusted != 0 promises that the structure behind row_ptr / col_ind and the
 * values behind val stay as they are for the life of the plan.  If in addition
 * col_ind and val are given (they may be NULL) and x is much larger than the L2,
 * a tiled copy of the matrix is built and the tiled two-phase kernel is timed
 * against the row / merge-path choice on scratch vectors; the faster one wins
 * (the reference's analysis record carries an `algo_tuning` flag for exactly
 * this, include/alphasparse/handle.h:120-123).  Likewise, when rows are short
 * (<= 32) and padding them to the longest adds at most 1/8 to the entry count,
 * a column-major ELL copy is built and timed.  Copies that lose are freed.
 * trusted == 2 builds both copies whatever the size and skips the timing (for
 * tests of those kernels); the kernel choice then stays the structural one. */
int asamd_csr_plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                          const int32_t *row_ptr, const int32_t *col_ind, const void *val,
                          int32_t base, int32_t val_size, int32_t trusted, asamd_csr_plan **plan);
/* The same for any element type (dtype: enum asamd_dtype).  Complex plans run every
 * kernel family (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57 is type-generic
 * through ALPHA_Number) except the constant-row-length one, whose 128-bit quads are
 * for real types. */
int asamd_csr_plan_create_dtype(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                                const int32_t *row_ptr, const int32_t *col_ind, const void *val,
                                int32_t base, int32_t dtype, int32_t trusted, asamd_csr_plan **plan);
void asamd_csr_plan_destroy(asamd_csr_plan *plan);
const asamd_csr_stats *asamd_csr_plan_stats(const asamd_csr_plan *plan);
/* Force a kernel family for later multiplies (AUTO restores the analysis'
 * own choice).  Returns hipErrorInvalidValue if the structure cannot run it. */
int asamd_csr_plan_set_algo(asamd_csr_plan *plan, int32_t algo);

/* y = alpha*A*x + beta*y.  Stands in for csr_gemv_vector_dispatch,
 * src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182.  `plan` must
 * describe (m, n, nnz, base); beta == 0 skips the read of y. */
int asamd_s_csrmv(hipStream_t stream, asamd_csr_plan *plan, float alpha, const float *val,
                  const int32_t *row_ptr, const int32_t *col_ind, const float *x, float beta,
                  float *y);
int asamd_d_csrmv(hipStream_t stream, asamd_csr_plan *plan, double alpha, const double *val,
                  const int32_t *row_ptr, const int32_t *col_ind, const double *x, double beta,
                  double *y);

/* asamd_s_csrmv without a plan and without any allocation: for callers that cannot call hipMalloc
 * (code under HIP graph capture, tight serving loops, harnesses that forbid it).  No counterpart in
 * the reference.  Runs the merge-path kernels (any row-length distribution, no float atomics); their
 * workgroup coordinates, carries and head sums live in a fixed device array of
 * ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES that the library holds per GPU until the process ends.
 * m + nnz above ASAMD_CSRMV_NOALLOC_MAX_ITEMS returns hipErrorOutOfMemory (2) before anything is
 * launched; other bad arguments return hipErrorInvalidValue.  base is 0 or 1; nnz == 0 gives
 * y = beta*y.  Calls hipMalloc, hipFree or an allocating library routine never; asamd_warmup (run by
 * alphasparse_dcu_get_handle) resolves the array's address for the current device, and the first
 * call on a device does so itself otherwise.  All calls on one GPU share the array: calls that
 * overlap there (two streams, two threads) race; calls on one stream are ordered and safe. */
#define ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES (4 << 20)
#define ASAMD_CSRMV_NOALLOC_MAX_ITEMS 536868864LL /* (SCRATCH_BYTES / 16 - 1) workgroups x 2048 items */
int asamd_s_csrmv_noalloc(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, int32_t base, float alpha,
                          const float *val, const int32_t *row_ptr, const int32_t *col_ind, const float *x,
                          float beta, float *y);

/* A trusted plan may hold re-ordered copies of the matrix VALUES (tiled, ELL, transposed); the
 * reference's analysis keeps structure only (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:382-388).
 * When the caller has changed the values behind `val` in place (same structure), this gathers every
 * copy again through the permutations that the plan kept: streaming kernels on `stream` only, no sort,
 * no allocation, no wait.  row_ptr / col_ind are the arrays the plan was created for. */
int asamd_csr_plan_refresh_values(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                  const int32_t *col_ind, const void *val);
/* 64-bit fingerprint of the structure arrays (m + 1 offsets, nnz column indices): equal arrays give equal
 * values; used to tell a changed structure from changed values when an analysis is repeated.
 * Synchronises `stream`; *hash_host is a host word. */
int asamd_csr_structure_hash(hipStream_t stream, int32_t m, int32_t nnz, const int32_t *row_ptr,
                             const int32_t *col_ind, uint64_t *hash_host);

/* CSR copy of the transpose, owned by the plan (trusted plans only; row_ptr,
 * col_ind, val are the arrays the plan was created for).  Later transposed
 * multiplies run the ordinary kernels on that copy (with an analysis of its
 * own: asamd_csr_plan_transpose_stats).  No reference counterpart: the
 * reference always scatters with atomics. */
int asamd_csr_plan_build_transpose(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                   const int32_t *col_ind, const void *val);
/* The same with conjugated values: a CSR copy of A^H (complex plans only). */
int asamd_csr_plan_build_conj_transpose(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                        const int32_t *col_ind, const void *val);
/* on != 0: the first transposed multiply builds that copy from the arrays it
 * is given (for matrices whose device arrays the library owns). */
int asamd_csr_plan_set_lazy_transpose(asamd_csr_plan *plan, int32_t on);
const asamd_csr_stats *asamd_csr_plan_transpose_stats(const asamd_csr_plan *plan);

/* y = alpha*A^T*x + beta*y: x has m entries, y has n.  Uses the transposed copy
 * when the plan has one; otherwise scales y and scatters with hardware float
 * atomics (y must be ordinary device memory), as
 * src/kernel/dcu/level2/mv/csrmv/dcu_gemv_x_csr_trans.cpp:11-45, :49-68 does. */
int asamd_s_csrmv_trans(hipStream_t stream, asamd_csr_plan *plan, float alpha, const float *val,
                        const int32_t *row_ptr, const int32_t *col_ind, const float *x, float beta,
                        float *y);
int asamd_d_csrmv_trans(hipStream_t stream, asamd_csr_plan *plan, double alpha, const double *val,
                        const int32_t *row_ptr, const int32_t *col_ind, const double *x, double beta,
                        double *y);

/* Complex element types: y = alpha*op(A)*x + beta*y with op = 0 (A), 1 (A^T), 2 (A^H), the
 * values of alphasparse_operation_t.  op = 0 stands in for csr_gemv_vector_dispatch as above,
 * op = 1 for dcu_gemv_x_csr_trans.cpp:11-68, op = 2 for csr_gemv_conj_scalar_atomicadd
 * (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_c_csr_conj.cpp:22-75); 1 and 2 use the plan's copy
 * of A^T / A^H when it has one and scatter with atomics otherwise. */
int asamd_c_csrmv_op(hipStream_t stream, asamd_csr_plan *plan, int32_t op, asamd_complex8 alpha,
                     const asamd_complex8 *val, const int32_t *row_ptr, const int32_t *col_ind,
                     const asamd_complex8 *x, asamd_complex8 beta, asamd_complex8 *y);
int asamd_z_csrmv_op(hipStream_t stream, asamd_csr_plan *plan, int32_t op, asamd_complex16 alpha,
                     const asamd_complex16 *val, const int32_t *row_ptr, const int32_t *col_ind,
                     const asamd_complex16 *x, asamd_complex16 beta, asamd_complex16 *y);

/* Arrays of the plan's CSR copy of A^T (conj == 0) or A^H (conj != 0): n + 1 row offsets, nnz
 * zero-based column indices (rows of A) and nnz values, owned by the plan.  hipErrorInvalidValue
 * if that copy has not been built. */
int asamd_csr_plan_transpose_arrays(const asamd_csr_plan *plan, int32_t conj, const int32_t **row_ptr,
                                    const int32_t **col_ind, const void **val);

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

/* Number of lazily made analyses (multiplies with info == NULL on arrays that no analysis or mirror
 * covers) that the library remembers at the moment: at most 64, the least recently used one makes room,
 * and a handle's own go with the handle.  For tests. */
int asamd_registry_lazy_count(void);

/* Introspection for benchmarks and tests: statistics of the analysis that a
 * multiply would use for `key`, where key is the alphasparse_dcu_mat_info_t of an
 * explicit analysis, or a device csr_row_ptr (library-built mirror or lazily
 * analysed array).  NULL if nothing is recorded.  Implemented by the host
 * library's registry; no reference counterpart. */
const asamd_csr_stats *asamd_analysis_stats(const void *key);
/* ... and of the analysis of the transposed copy, or NULL if there is none. */
const asamd_csr_stats *asamd_analysis_transpose_stats(const void *key);
/* Force a kernel family (enum asamd_spmv_algo) on the analysis recorded for
 * `key`; returns 0 on success, a hipError_t otherwise. */
int asamd_analysis_set_algo(const void *key, int32_t algo);

/* Plain 16-byte-per-lane copy of nbytes (a multiple of 16, both pointers 16-byte
 * aligned).  Exists to calibrate hardware byte counters against a transfer of
 * known size; no reference counterpart. */
int asamd_copy_bytes(hipStream_t stream, void *dst, const void *src, size_t nbytes);

/* Plain memory kernels that measure what the GPU sustains (the practical ceilings that the kernels'
 * roofline figures are read against); no reference counterpart.  kind: READ / WRITE / COPY stream nbytes
 * (a multiple of 16; 16 bytes per lane and access) from src / into dst; ROW_GATHER fetches `count`
 * 256-byte rows at random positions of the nbytes at src, one wave per row (what the row-major SpMM does
 * per entry of A with 64 dense columns); ELEM_GATHER fetches `count` single floats at random positions
 * (what a row SpMV kernel does per entry); RUN_GATHER / RUN_SCATTER copy nbytes in runs of `count` floats
 * (a multiple of 4) whose order differs between source and destination: the runs are contiguous on the
 * write side and scattered on the read side (what the second phase of the tiled SpMV reads), or the other
 * way round.  sink: 4 device bytes that are practically never written.
 * *bytes_moved receives the useful bytes of the launch (copy: read + written). */
enum asamd_ceiling_kind {
  ASAMD_CEILING_READ = 0,
  ASAMD_CEILING_WRITE = 1,
  ASAMD_CEILING_COPY = 2,
  ASAMD_CEILING_ROW_GATHER = 3,
  ASAMD_CEILING_ELEM_GATHER = 4,
  ASAMD_CEILING_READ_NT = 5, /* the same streams with non-temporal accesses */
  ASAMD_CEILING_COPY_NT = 6,
  ASAMD_CEILING_RUN_GATHER = 7,
  ASAMD_CEILING_RUN_SCATTER = 8
};
int asamd_ceiling_kernel(hipStream_t stream, int32_t kind, void *dst, const void *src, size_t nbytes,
                         int64_t count, void *sink, int64_t *bytes_moved);

/* handle->stream for callers that cannot see the handle struct (language bindings); C callers assign
 * the field, as with the reference.  `handle` is an alphasparse_dcu_handle_t.  Every multiply that
 * runs from an explicit analysis only launches kernels on that stream, so it can be captured into
 * a HIP graph. */
int asamd_handle_set_stream(void *handle, hipStream_t stream);
hipStream_t asamd_handle_get_stream(void *handle);

/* Empty kernel; forces code-object load (src/util_cpp/handle.cpp:19, :113).  Also looks up, for the
 * current device, the address of the fixed array that asamd_s_csrmv_noalloc works in. */
int asamd_warmup(hipStream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_KERNELS_H */
