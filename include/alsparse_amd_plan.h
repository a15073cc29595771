/*
 * alsparse_amd_plan.h -- the host library's CSR analysis object ("plan"): what
 * alphasparse_dcu_?_csrmv_analysis builds and alphasparse_dcu_?_csrmv multiplies with.
 *
 * A plan is host-side C.  It holds the row statistics, the kernel family chosen from them, and the
 * re-ordered copies ("layouts", include/alsparse_amd_kernels.h) that won the analysis; a multiply picks
 * the launcher of that family and hands it the CSR arrays, the layout and per-call scratch.  The plan
 * replaces the reference's _alphasparse_dcu_csrmv_info payload (include/alphasparse/handle.h:118-138) and
 * the row-block builder that fills it (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-391).
 *
 * Multiplies keep no state in the plan: everything a call writes besides y lives in the workspace that
 * the caller passes (alphasparse_dcu_?_csrmv passes the calling handle's buffer), so one plan may be
 * used from several handles and streams at once, like the reference's stateless kernels
 * (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57).
 *
 * Return values are hipError_t cast to int unless stated otherwise.
 */
#ifndef ALSPARSE_AMD_PLAN_H
#define ALSPARSE_AMD_PLAN_H

#include "alsparse_amd_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Row-length statistics gathered on the GPU and what the analysis made of them.  hist[0] counts empty
 * rows, hist[b] rows whose length lies in [2^(b-1), 2^b). */
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
  float tune_ms_base;   /* analysis-time timing (or model estimate) of the choice without a copy, or 0 */
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
  int32_t value_check;   /* how a multiply checks that csr_val still holds what the plan's copies were
                            taken from: 0 not at all, 1 a sample of 256-byte pieces, 2 every byte     */
  int32_t tune_mode;     /* 0: candidates were timed inside the analysis, 1: decided by the model alone */
  int64_t device_bytes;  /* device memory that the plan holds (layouts, copies, coordinates)            */
  int64_t workspace_bytes; /* per-call scratch that a multiply with this plan may ask for              */
  float lines_per_entry_wave;    /* locality probe (asamd_csr_locality_probe): distinct 128-byte lines of x
                                    per entry among 64 consecutive entries, or 0 if not probed          */
  float lines_per_entry_segment; /* ... and within runs of 32 768 consecutive entries                     */
  int32_t xlds_slices;   /* column slices of the kernel that holds x in LDS (a table of offsets exists), or 0   */
} asamd_csr_stats;

typedef struct asamd_csr_plan asamd_csr_plan;

/* Row-length histogram, kernel choice and (trusted != 0) cached merge-path block coordinates.
 * Synchronises `stream`.  val_size is sizeof(value type): 4 (fp32) or 8 (fp64).
 * trusted != 0 promises that the STRUCTURE behind row_ptr / col_ind stays as it is for the life of the
 * plan; the VALUES behind val may change at any time (see asamd_csr_plan_csrmv).  If in addition col_ind
 * and val are given (they may be NULL), the copies that the matrix is eligible for -- tiled, ELL, hot
 * columns, row-length bins -- are laid out and timed against the choice from the row statistics on
 * scratch vectors; the fastest is kept, the others are freed (the reference's analysis record carries an
 * `algo_tuning` flag for exactly this, include/alphasparse/handle.h:120-123).  ALSPARSE_AMD_TUNE=model
 * decides from the statistics and fixed constants instead of timings, so that the same matrix always gets
 * the same family.  trusted == 2 builds every copy whatever the size and skips the timing (for tests of
 * those kernels); the kernel choice then stays the structural one.  trusted == 3: as 1, with the tiled copy
 * as the only candidate (see asamd_csr_plan_csrmv_watched). */
int asamd_csr_plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                          const int32_t *row_ptr, const int32_t *col_ind, const void *val,
                          int32_t base, int32_t val_size, int32_t trusted, asamd_csr_plan **plan);
/* The same for any element type (dtype: enum asamd_dtype).  Complex plans run every kernel family
 * except the constant-row-length one, whose 128-bit quads are for real types. */
int asamd_csr_plan_create_dtype(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                                const int32_t *row_ptr, const int32_t *col_ind, const void *val,
                                int32_t base, int32_t dtype, int32_t trusted, asamd_csr_plan **plan);
void asamd_csr_plan_destroy(asamd_csr_plan *plan);
const asamd_csr_stats *asamd_csr_plan_stats(const asamd_csr_plan *plan);
/* Force a kernel family for later multiplies (AUTO restores the analysis' own choice).  Returns
 * hipErrorInvalidValue if the structure cannot run it. */
int asamd_csr_plan_set_algo(asamd_csr_plan *plan, int32_t algo);

/* Per-call scratch (device bytes) that asamd_csr_plan_csrmv may use with this plan, whatever the
 * operation: merge-path carries, the tiled kernels' product array, the value guard's words, ... */
size_t asamd_csr_plan_workspace_bytes(const asamd_csr_plan *plan);

/* y = alpha*op(A)*x + beta*y with op = 0 (A), 1 (A^T), 2 (A^H, complex types): the values of
 * alphasparse_operation_t.  Stands in for csr_gemv_vector_dispatch
 * (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182), dcu_gemv_x_csr_trans.cpp:11-68 and
 * dcu_gemv_c_csr_conj.cpp:22-75.  alpha, beta: HOST scalars of the plan's element type.  Only enqueues
 * kernels on `stream`: no allocation, copy or wait, so the call can be recorded into a HIP graph.
 *
 * workspace: device scratch of this call alone (two multiplies in flight at the same time need one
 * each; 256-byte aligned or aligned up here).  With less than asamd_csr_plan_workspace_bytes the
 * multiply still gives the right result through kernels that need no scratch (a lane group per row;
 * the atomic scatter for op != 0), slowly.
 *
 * Values changed in place: a plan's copies (tiled, ELL, A^T, A^H) hold the values that `val` held when
 * they were laid out.  Before such a copy is used, a guard kernel fingerprints val and compares with
 * the fingerprint of the values the copy was taken from; if they differ, the copy is gathered again
 * through the permutation the plan kept -- all on the device, in stream order, no host round trip.
 * By default the fingerprint covers every byte of arrays up to 32 MiB and, of larger ones, 256 bytes
 * at a varying position of every run of asamd_value_guard_run(bytes) bytes (8 KiB for a gigabyte): a
 * caller who rewrites the array, or any contiguous stretch of at least two runs, is always noticed; one who
 * pokes single entries of a large array is noticed with probability 256 / run and should call
 * asamd_csr_plan_refresh_values (or analyse again).  ALSPARSE_AMD_VALUE_CHECK=full fingerprints every
 * byte (one more pass over val per multiply), =off none (the caller then refreshes by hand).  A
 * multiply that passes ANOTHER value array than the copies were taken from runs on the caller's arrays. */
int asamd_csr_plan_csrmv(hipStream_t stream, asamd_csr_plan *plan, int32_t op, const void *alpha, const void *val,
                         const int32_t *row_ptr, const int32_t *col_ind, const void *x, const void *beta, void *y,
                         void *workspace, size_t workspace_bytes);

/* A matrix that is WATCHED instead of promised fixed -- what a caller who never analyses gets once the same
 * arrays have come back often enough.  The plan is one made with trusted == 3 (only the tiled copy is a
 * candidate) whose analysis kept that copy.  Every watched multiply fingerprints EVERY byte of row_ptr, col_ind
 * and val on the device, compares the first two with the words at watch[0..1] (set by asamd_csr_plan_watch_begin
 * when the plan was made) and the third with the plan's own, gathers the copy's values again if they moved, and
 * launches both the tiled kernels -- which return at once if the structure moved -- and a lane group per row on
 * the caller's arrays -- which returns at once if it did not.  The result is that of the arrays as they are,
 * whatever was done to them; nothing waits for the host.  *changed (if asked for) points at the device word
 * that says which of the two ran (non-zero: the structure moved), inside the workspace.
 * workspace: at least asamd_csr_plan_watched_workspace_bytes; hipErrorInvalidValue otherwise, or if the plan
 * did not keep a tiled copy of exactly this val. */
size_t asamd_csr_plan_watched_workspace_bytes(const asamd_csr_plan *plan);
int asamd_csr_plan_watch_begin(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                               const int32_t *col_ind, const void *val, uint64_t *watch, void *workspace,
                               size_t workspace_bytes);
int asamd_csr_plan_csrmv_watched(hipStream_t stream, asamd_csr_plan *plan, const void *alpha, const void *val,
                                 const int32_t *row_ptr, const int32_t *col_ind, const void *x, const void *beta,
                                 void *y, const uint64_t *watch, void *workspace, size_t workspace_bytes,
                                 const int32_t **changed);

/* Gathers every copy of the plan again from `val` (the array the copies were laid out from, or one
 * with the same structure) without looking whether anything changed: streaming kernels on `stream`
 * only, no sort, no allocation, no wait.  Not to be run while another stream multiplies with the plan. */
int asamd_csr_plan_refresh_values(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                  const int32_t *col_ind, const void *val);

/* CSR copy of the transpose, owned by the plan (trusted plans only; row_ptr, col_ind, val are the
 * arrays the plan was created for).  Later transposed multiplies run the ordinary kernels on that copy
 * (with an analysis of its own: asamd_csr_plan_transpose_stats).  No reference counterpart: the
 * reference always scatters with atomics. */
int asamd_csr_plan_build_transpose(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                   const int32_t *col_ind, const void *val);
/* The same with conjugated values: a CSR copy of A^H (complex plans only). */
int asamd_csr_plan_build_conj_transpose(hipStream_t stream, asamd_csr_plan *plan, const int32_t *row_ptr,
                                        const int32_t *col_ind, const void *val);
/* on != 0: the first transposed multiply outside a stream capture builds that copy from the arrays it
 * is given (for matrices whose device arrays the library owns). */
int asamd_csr_plan_set_lazy_transpose(asamd_csr_plan *plan, int32_t on);
const asamd_csr_stats *asamd_csr_plan_transpose_stats(const asamd_csr_plan *plan);
/* Arrays of the plan's CSR copy of A^T (conj == 0) or A^H (conj != 0): n + 1 row offsets, nnz
 * zero-based column indices (rows of A) and nnz values, owned by the plan.  hipErrorInvalidValue
 * if that copy has not been built. */
int asamd_csr_plan_transpose_arrays(const asamd_csr_plan *plan, int32_t conj, const int32_t **row_ptr,
                                    const int32_t **col_ind, const void **val);

/* Number of lazily made analyses (multiplies with info == NULL on arrays that no analysis or mirror
 * covers) that the library remembers at the moment: at most 64, the least recently used one makes room,
 * and a handle's own go with the handle.  For tests. */
int asamd_registry_lazy_count(void);
/* 1 if multiplies without analysis on `handle` with this device csr_row_ptr go through a watched tiled copy
 * at the moment (the same arrays came back often enough and the copy is expected to pay).  For tests. */
int asamd_registry_lazy_promoted(const void *handle, const void *row_ptr);

/* Introspection for benchmarks and tests: statistics of the analysis that a multiply would use for
 * `key`, where key is the alphasparse_dcu_mat_info_t of an explicit analysis, or a device csr_row_ptr
 * (library-built mirror or lazily analysed array).  NULL if nothing is recorded. */
const asamd_csr_stats *asamd_analysis_stats(const void *key);
/* ... and of the analysis of the transposed copy, or NULL if there is none. */
const asamd_csr_stats *asamd_analysis_transpose_stats(const void *key);
/* Force a kernel family (enum asamd_spmv_algo) on the analysis recorded for `key`; returns 0 on
 * success, a hipError_t otherwise.  The analysis' own choice may differ between two analyses of one
 * matrix when two candidates time within a few per cent of each other; a caller who needs the same
 * family (the same summation order, the same bits) every time pins it here, or sets
 * ALSPARSE_AMD_TUNE=model. */
int asamd_analysis_set_algo(const void *key, int32_t algo);

/* Makes sure the handle's scratch buffer (alphasparse_dcu_handle::buffer, src/util_cpp/handle.cpp:94-105)
 * holds at least `bytes`: a larger one replaces it after the handle's stream has drained.  Returns an
 * alphasparse_status_t.  Not to be called while the stream is being captured. */
int asamd_handle_reserve(void *handle, size_t bytes);

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_PLAN_H */
