/* The CSR analysis object: row statistics -> kernel family, the copies that win the analysis, and the
 * dispatch of a multiply to the launcher of its family (include/alsparse_amd_plan.h).
 *
 * Stands in for the reference's host-side analysis (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-391:
 * a serial walk over row_ptr that builds CSR-adaptive row blocks no kernel reads) and for
 * csr_gemv_vector_dispatch (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182: lanes per row from
 * the mean row length).  Everything that touches the GPU goes through the launchers and layout builders of
 * include/alsparse_amd_kernels.h; this file decides, owns memory and carves the per-call workspace. */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

typedef struct {
  asamd_transpose_layout t;
  asamd_csr_plan *plan;    /* the analysis of the copy */
  const void *val_src;     /* the value array that t.val was gathered from */
} asamd_trans_copy;

struct asamd_csr_plan {
  asamd_csr_stats st;
  int auto_algo;           /* the analysis' choice */
  int struct_algo;         /* the choice from the row statistics alone (no copy involved) */
  int plain_algo;          /* ... before x in LDS was considered */
  int auto_width;
  int dtype;               /* ASAMD_DTYPE_*: element type of the values */
  int val_size;            /* bytes per value */
  int merge_ipt;           /* items per thread of the merge-path kernel (4, 8 or 16) */
  int32_t *d_block_row;    /* merge-path coordinates of a structure promised fixed, merge_blocks + 1 ints */
  asamd_tiled_layout tiled;
  asamd_hot_layout hot;
  asamd_binned_layout binned;
  asamd_xlds_layout xlds;  /* column slices for the kernel that holds x in LDS (an x of several LDS fills) */
  int xlds_copy_wanted;    /* the slices are to come with a copy of the entries (known before they are laid out) */
  uint16_t *d_col16;       /* x in LDS, one slice: the column numbers as 16-bit words (structure promised fixed) */
  int16_t *d_rel16;        /* staged row blocks: the columns as 16-bit distances from the workgroup's first row */
  int rel16_group;         /* the lanes per row they were made for */
  int watched;             /* laid out for asamd_csr_plan_csrmv_watched: its fingerprints are the caller's account */
  void *d_eval;            /* ELL copy: ell_width * m values, column-major */
  int32_t *d_ecol;         /* ... and zero-based columns */
  const void *copy_val_src; /* the value array that the tiled / ELL copy was taken from */
  asamd_trans_copy tr[2];  /* CSR copies of the transpose [0] and of the conjugate transpose [1] */
  int lazy_transpose;      /* build a copy on the first transposed multiply */
  uint64_t *d_fp;          /* 3 device words: fingerprints of the values that the copies were taken from
                              (tiled / ELL, A^T, A^H) */
  void *d_setup;           /* device scratch of the plan's own set-up work (statistics, first fingerprints) */
};

#define SETUP_BYTES (ASAMD_GUARD_WS_BYTES + 1024)

static const int kValSize[4] = {4, 8, 8, 16};

/* rows plus entries below which one launch's latency outweighs the work */
#define SMALL_WORK ((int64_t)1 << 17)

static int is_complex(const asamd_csr_plan *p) { return p->dtype >= ASAMD_DTYPE_FLOAT_COMPLEX; }

/* ---- environment switches (read once) ------------------------------------------------------------ */
static int env_int(const char *name, int fallback) {
  const char *e = getenv(name);
  return e && *e ? atoi(e) : fallback;
}

static int env_value_check(void) {
  const char *e = getenv("ALSPARSE_AMD_VALUE_CHECK");
  if (e && !strcmp(e, "off")) return 0;
  if (e && !strcmp(e, "full")) return 2;
  return 1;
}

/* ALSPARSE_AMD_TUNE = model (default): the analysis decides from the row statistics, the locality probe and fixed
 * constants; timed: it times the candidates on scratch vectors, which follows the machine at hand more closely but
 * depends on whatever else the GPU is doing at that moment. */
static int env_tune_model(void) {
  const char *e = getenv("ALSPARSE_AMD_TUNE");
  return !(e && !strcmp(e, "timed"));
}

/* ---- kernel choice from the row statistics --------------------------------------------------------- */
static int width_for_mean(double mean) {
  /* lanes per row from the mean row length; same break points as the
   * reference's dispatch (dcu_gemv_vector.h:77,94,111,128,145,162) */
  if (mean < 4) return 2;
  if (mean < 8) return 4;
  if (mean < 16) return 8;
  if (mean < 32) return 16;
  if (mean < 64) return 32;
  return 64;
}

static int rowconst_ok(const asamd_csr_plan *p) {
  const asamd_csr_stats *st = &p->st;
  const int L = st->const_len;
  /* the kernel loads four values as 128-bit pieces: real element types only */
  return !is_complex(p) && st->trusted && st->first_offset == 0 &&
         (L == 4 || L == 8 || L == 16 || L == 32 || L == 64 || L == 128 || L == 256);
}

/* The LDS-staged row-block kernel sizes its staging area for rows of at most cap * G entries (G lanes sum a
 * row); the bound comes from the row statistics.  A workgroup whose rows hold more than that (the structure
 * behind row_ptr changed under a plan that was not promised a fixed one) takes them straight from global
 * memory, so the choice is safe for such plans too.  Returns G, or 0 when the kernel cannot take the matrix.
 * With `regular_only`, also 0 for G > 1 when the rows are so much shorter than the longest that a workgroup's
 * 256 / G rows hold fewer than four entries per thread.
 * 16 KiB of products per workgroup: 16 entries per thread for 4-byte values, 8 for 8-byte, 4 for 16-byte ones
 * (measured on a 27-point stencil, fp64: 32 KiB per workgroup 317 us, 16 KiB 295 us) */
static int stream_cap(const asamd_csr_plan *p) { return 64 / p->val_size; }
static int stream_group(const asamd_csr_plan *p, int regular_only) {
  const asamd_csr_stats *st = &p->st;
  if (st->max_len < 1) return 0;
  const int cap = stream_cap(p);
  if (st->max_len <= cap) return 1;
  int g = 2;
  while (g * cap < st->max_len && g <= ASAMD_STREAM_MAX_GROUP) g *= 2;
  if (g > ASAMD_STREAM_MAX_GROUP) return 0;
  /* regular: the mean row is at least a quarter of the longest row the kernel is sized for */
  if (regular_only && (double)st->nnz / (double)st->m < 0.25 * g * cap) return 0;
  return g;
}
static int stream_ok(const asamd_csr_plan *p) { return stream_group(p, 0) > 0; }

/* x in LDS: for an x that crowds the L1 (32 KB) and fits the LDS, on matrices large enough for 256 persistent
 * workgroups.  4 M x 16 entries, fp32: rowconst 0.105 / 0.125 / 0.20 / 0.25 / 0.29 ms with 4 / 16 / 32 / 64 / 128 KB of x,
 * this kernel 0.127 ms whatever x; fp64 with 128 KB of x 0.37 against 0.18 ms.  ALSPARSE_AMD_XLDS=0 leaves it out. */
/* The kernels that hold x in LDS give every row the lanes that fit the MEAN row, and a lane group walks a longer row
 * load by load while the wave's other groups wait: where rows of more than four times the mean hold more than a
 * tenth of the entries they lose to merge-path (rows of 4 and, every eighth, 256 entries, 4 M x 16 384: 0.84 against
 * 0.56 ms; rows of 2 and, every sixteenth, 2 000, in 32 slices: 1.49 against 0.65 for the tiled pair).  A few long
 * rows among regular ones go to whole waves and do not matter. */
static int xlds_rows_regular(const asamd_csr_stats *st) {
  if (st->m < 1 || st->nnz < 1) return 0;
  const double mean = (double)st->nnz / (double)st->m;
  double far = 0.0;
  for (int b = 2; b < ASAMD_HIST_BINS; ++b) /* bin b: rows of 2^(b-1) .. 2^b - 1 entries */
    if ((double)((int64_t)1 << (b - 1)) >= 4.0 * mean) far += (double)st->hist[b] * 0.75 * (double)((int64_t)1 << b);
  return far <= 0.1 * (double)st->nnz;
}

/* an x that crowds the L1 and fits a compute unit's LDS (4 M x 5 000 x 16, fp32, 20 KB of x: 0.108 ms against
 * rowconst's 0.138; with 16 KB the two are level) */
static int xlds_sized_x(const asamd_csr_plan *p) {
  const int64_t x_bytes = (int64_t)p->st.n * (int64_t)p->val_size;
  return x_bytes >= (18 << 10) && asamd_spmv_xlds_fits(p->dtype, p->st.n);
}
/* ... and enough rows of moderate length: a lane group takes four rows per trip and rows beyond 512 entries go to
 * single waves, so 2 048 rows of 2 048 entries keep 8 of the 256 workgroups busy (0.067 ms against merge-path's
 * 0.018; 8 192 x 1 024: 0.053 against 0.035; 32 768 x 256: 0.016 against rowconst's 0.033). */
static int xlds_rows_enough(const asamd_csr_stats *st, int slices) {
  return (int64_t)st->m * slices >= 32768 && (double)st->nnz <= 512.0 * (double)slices * (double)st->m;
}
/* Rows of fewer than four entries on average run the form with one entry per lane and two lanes per row, which pays
 * where all rows are equally long (8 M rows of 2 entries: 0.056 ms against the staged row blocks' 0.074; of 3: 0.073
 * against 0.102) and not otherwise (rows of 1 and 3 in turn: 0.091 against 0.073; one entry per row: 0.109 against 0.096). */
static int xlds_rows_not_too_short(const asamd_csr_stats *st) {
  return (int64_t)st->nnz >= 4 * (int64_t)st->m || st->const_len >= 2;
}
static int xlds_ok(const asamd_csr_plan *p) {
  const asamd_csr_stats *st = &p->st;
  return st->first_offset == 0 && st->m >= 1 && st->nnz >= (1 << 22) && xlds_sized_x(p) && xlds_rows_regular(st) &&
         xlds_rows_enough(st, 1) && xlds_rows_not_too_short(st) && env_int("ALSPARSE_AMD_XLDS", 1) > 0;
}

/* ... and slice by slice for an x of several LDS fills, where the rows are long enough for their pieces: a slice's
 * piece of a row should hold sixteen entries or more on average (262 144 x 262 144 x 400, fp32, 8 slices: merge-path
 * 0.51 ms, this 0.23 ms; 1 M x 131 072 x 128, 4 slices: 0.41 ms).  Needs ascending columns inside the rows (the
 * builder looks) and a structure that is promised fixed. */
static int xlds_slices_for(const asamd_csr_plan *p) { return asamd_xlds_slices(p->dtype, p->st.n); }
/* With a copy of the entries slice by slice the pieces of consecutive rows are neighbours in memory and a piece of
 * three entries is long enough for the estimate to decide (ALSPARSE_AMD_XLDS_COPY=0: never a copy). */
#define ALGO_XLDS_IN_PLACE 64 /* internal: the slices over the caller's arrays although the plan holds a copy */
static int xlds_sliced_ok(const asamd_csr_plan *p, int force, int copy) {
  const asamd_csr_stats *st = &p->st;
  if (!st->trusted || st->first_offset != 0 || st->m < 1 || st->nnz < 4) return 0;
  if (p->dtype != ASAMD_DTYPE_FLOAT && p->dtype != ASAMD_DTYPE_DOUBLE) return 0;
  const int slices = xlds_slices_for(p);
  if (slices < 2 || slices > 1024 || ((int64_t)slices + 1) * st->m >= (int64_t)INT32_MAX) return 0;
  if (force) return 1;
  return st->nnz >= (1 << 22) && xlds_rows_regular(st) && xlds_rows_enough(st, slices) &&
         (double)st->nnz >= (copy ? 3.0 : 16.0) * (double)slices * (double)st->m &&
         env_int("ALSPARSE_AMD_XLDS", 1) > 0;
}

static void choose_algo(asamd_csr_plan *p) {
  asamd_csr_stats *st = &p->st;
  const double mean = st->m > 0 ? (double)st->nnz / st->m : 0.0;
  const int w = width_for_mean(mean);
  p->auto_width = w;
  if (st->first_offset != 0) {
    /* row_ptr points into the middle of a larger array: only the kernels that index with the absolute
     * offsets (as the reference's csr_gemv_vector does) see the right entries; merge-path and csr2coo,
     * the source of every re-ordered copy, count entries from position 0 */
    p->auto_algo = stream_group(p, 1) > 0 ? ASAMD_SPMV_STREAM : ASAMD_SPMV_VECTOR;
  } else if (rowconst_ok(p)) {
    p->auto_algo = ASAMD_SPMV_ROWCONST;
  } else if (stream_group(p, 1) > 0) {
    /* short rows, or rows of some tens of entries of similar lengths */
    p->auto_algo = ASAMD_SPMV_STREAM;
  } else if ((int64_t)st->max_len <= (int64_t)w * 16 && mean >= 6.0) {
    /* regular rows: a lane group per row wastes little and needs no LDS */
    p->auto_algo = ASAMD_SPMV_VECTOR;
  } else if ((int64_t)st->m + st->nnz <= SMALL_WORK && (int64_t)st->max_len <= (int64_t)w * 64) {
    /* a matrix this small is over in the time of one launch: the single kernel beats the balanced
     * path's two or three */
    p->auto_algo = ASAMD_SPMV_VECTOR;
  } else {
    p->auto_algo = ASAMD_SPMV_MERGE;
  }
  p->plain_algo = p->auto_algo;
  if (xlds_ok(p)) p->auto_algo = ASAMD_SPMV_XLDS;
  p->struct_algo = p->auto_algo;
  st->algo = p->auto_algo;
  st->vector_width = p->auto_width;
}

/* ---- which copies a matrix is eligible for -------------------------------------------------------- */
/* An ELL copy pays when rows are short and padding them to the longest costs little: the kernel then
 * streams 4 + sizeof(T) bytes per entry at full width with neither row_ptr nor LDS staging. */
static int ell_eligible(const asamd_csr_stats *st, int force) {
  if (!st->trusted || st->first_offset != 0 || st->max_len < 1 || st->max_len > 32) return 0;
  const int64_t slots = (int64_t)st->m * st->max_len;
  if (slots >= ((int64_t)1 << 31) || slots > (int64_t)st->nnz + st->nnz / 8) return 0;
  return force || st->nnz >= (1 << 18);
}

static int tiled_eligible(const asamd_csr_plan *p, int force) {
  const asamd_csr_stats *st = &p->st;
  if (!st->trusted || st->first_offset != 0 || !asamd_tiled_fits(p->dtype, st->m, st->n, st->nnz)) return 0;
  /* worth a try only when x fills an XCD's 4 MiB L2 (the matrix streams through the same cache; with
   * 2 MiB of x the tiled pair measured 0.43 ms against 0.34 ms, with 4 MiB 0.084 against 0.095) and the
   * matrix is large; the comparison inside the analysis has the last word */
  return force || ((int64_t)st->n * (int64_t)p->val_size >= ((int64_t)4 << 20) && st->nnz >= (1 << 22));
}

static int hot_eligible(const asamd_csr_plan *p, int force) {
  const asamd_csr_stats *st = &p->st;
  if (p->val_size > 8 || !st->trusted || st->first_offset != 0 || st->nnz < 1 || st->n < 1) return 0;
  /* positions are 32-bit words, x is addressed through a buffer resource with 32-bit byte offsets */
  if (((int64_t)st->n + ((int64_t)1 << 20)) >= (int64_t)UINT32_MAX) return 0;
  if ((int64_t)st->m + st->nnz >= (int64_t)INT32_MAX / 2) return 0;
  if (force) return 1;
  /* An x that the L2 of one XCD holds is gathered fast enough as it is, and counting and ranking the columns
   * costs some twenty-five multiplies: large matrices only.  ALSPARSE_AMD_TUNE_HOT=0 leaves the copy out. */
  if (env_int("ALSPARSE_AMD_TUNE_HOT", 1) <= 0) return 0;
  /* ... and matrices of few columns whose row lengths keep them from the kernel that holds x in LDS: the table then
   * holds all of x, or most of it (see model_copies) */
  if (xlds_sized_x(p) && st->nnz >= (1 << 22) && !xlds_rows_regular(st)) return 1;
  return (int64_t)st->n * (int64_t)p->val_size >= ((int64_t)8 << 20) && st->nnz >= (1 << 22);
}

static int binned_eligible(const asamd_csr_plan *p, int force) {
  const asamd_csr_stats *st = &p->st;
  if (!st->trusted || st->m < 1 || st->nnz < 1) return 0;
  if (force) return 1;
  if (st->nnz < (1 << 20) || st->max_len <= 8) return 0;
  /* rows that differ enough in length for one mapping not to fit: the structural choice was merge-path, or
   * a lane group per row whose width (from the MEAN length) leaves three quarters of the lanes idle on a
   * quarter of the rows (row-length histogram: bin b holds the rows of 2^(b-1) .. 2^b - 1 entries) */
  if (p->auto_algo == ASAMD_SPMV_MERGE) return st->max_len > 64;
  if (p->auto_algo != ASAMD_SPMV_VECTOR) return 0;
  int64_t short_rows = 0;
  for (int b = 0; b < ASAMD_HIST_BINS && ((int64_t)1 << b) <= p->auto_width / 4; ++b) short_rows += st->hist[b];
  return short_rows * 4 >= (int64_t)st->m;
}

/* Whether the structural choice has rivals that need no copy either (merge-path, a lane group per row): it has
 * when it is a lane group per row or a staged block with several lanes per row, merge-path can run (row_ptr
 * starts at the base) and the matrix is not so small that one launch's latency is all there is to time. */
static int structural_alternatives(const asamd_csr_plan *p) {
  const asamd_csr_stats *st = &p->st;
  if (st->first_offset != 0 || (int64_t)st->m + st->nnz <= SMALL_WORK) return 0;
  return p->auto_algo == ASAMD_SPMV_VECTOR || (p->auto_algo == ASAMD_SPMV_STREAM && stream_group(p, 0) > 1);
}

/* ---- copies: lay out, free, account ------------------------------------------------------------------ */
static void free_tiled(asamd_csr_plan *p) {
  asamd_tiled_free(&p->tiled);
  p->st.tiled_built = 0;
  p->st.tile_entries_per_lane = 0;
  p->st.tile_long_blocks = 0;
}

static void free_ell(asamd_csr_plan *p) {
  if (p->d_eval) (void)hipFree(p->d_eval);
  if (p->d_ecol) (void)hipFree(p->d_ecol);
  p->d_eval = NULL;
  p->d_ecol = NULL;
  p->st.ell_built = 0;
}

static void free_hot(asamd_csr_plan *p) {
  asamd_hot_free(&p->hot);
  p->st.hot_built = 0;
}

static void free_binned(asamd_csr_plan *p) {
  asamd_binned_free(&p->binned);
  p->st.binned_built = 0;
}

static void free_transpose(asamd_csr_plan *p, int which) {
  asamd_trans_copy *t = &p->tr[which];
  if (t->plan) asamd_csr_plan_destroy(t->plan);
  asamd_transpose_free(&t->t);
  t->plan = NULL;
  t->val_src = NULL;
  p->st.transpose_built &= ~(1 << which);
}

static hipError_t build_tiled(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                              const void *val) {
  asamd_csr_stats *st = &p->st;
  /* ALSPARSE_AMD_TILED_HALVES = 1 | 2 forces the form of the second phase */
  int halves = env_int("ALSPARSE_AMD_TILED_HALVES", 0);
  if (halves != 1 && halves != 2) halves = 0;
  hipError_t e = (hipError_t)asamd_tiled_build(stream, p->dtype, st->m, st->n, st->nnz, st->base, row_ptr, col_ind, val,
                                               st->max_len, halves, &p->tiled);
  if (e != hipSuccess) return e;
  st->tile_col_blocks = p->tiled.col_blocks;
  st->tile_row_blocks = p->tiled.row_blocks;
  if (!p->tiled.tval) return hipSuccess; /* the matrix simply gets no tiled copy */
  st->tiled_built = 1;
  st->tile_entries_per_lane = p->tiled.entries_per_lane;
  st->tile_long_blocks = p->tiled.long_blocks;
  return hipSuccess;
}

static hipError_t build_ell(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                            const void *val) {
  asamd_csr_stats *st = &p->st;
  const size_t slots = (size_t)st->m * (size_t)st->max_len;
  hipError_t e = hipMalloc(&p->d_eval, slots * (size_t)p->val_size);
  if (e == hipSuccess) e = hipMalloc((void **)&p->d_ecol, slots * sizeof(int32_t));
  /* the conversion copies values bit for bit and pads with zero bits: only the element size matters */
  if (e == hipSuccess)
    e = (hipError_t)asamd_csr2ell_gated(stream, p->val_size, st->m, val, row_ptr, col_ind, st->base, 0, st->max_len,
                                        p->d_eval, p->d_ecol, NULL);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    free_ell(p);
    return e;
  }
  st->ell_built = 1;
  st->ell_width = st->max_len;
  return hipSuccess;
}

static hipError_t build_hot(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                            int force) {
  asamd_csr_stats *st = &p->st;
  /* ALSPARSE_AMD_HOT_COLS / ALSPARSE_AMD_HOT_FRONT size the LDS table and the compact front (columns) */
  hipError_t e = (hipError_t)asamd_hot_build(stream, p->dtype, st->m, st->n, st->nnz, st->base, row_ptr, col_ind, force,
                                             env_int("ALSPARSE_AMD_HOT_COLS", 0), env_int("ALSPARSE_AMD_HOT_FRONT", 0),
                                             &p->hot);
  if (e != hipSuccess) return e;
  st->hot_cols_lds = p->hot.cols_lds;
  st->hot_cols = p->hot.cols_front;
  st->hot_share_lds = p->hot.share_lds;
  st->hot_built = p->hot.pcol != NULL;
  return hipSuccess;
}

static hipError_t build_binned(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr) {
  hipError_t e = (hipError_t)asamd_binned_build(stream, p->st.m, p->st.base, row_ptr, &p->binned);
  if (e != hipSuccess) return e;
  for (int c = 0; c < 4; ++c) p->st.bin_rows[c] = p->binned.count[c];
  p->st.binned_built = p->binned.rows != NULL;
  return hipSuccess;
}

static size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

/* per-call scratch of one kernel family */
static size_t algo_scratch(const asamd_csr_plan *p, int algo) {
  const asamd_csr_stats *st = &p->st;
  const size_t vs = (size_t)p->val_size;
  switch (algo) {
    case ASAMD_SPMV_MERGE: {
      const size_t nb = (size_t)st->merge_blocks;
      return (p->d_block_row ? 0 : align256((nb + 1) * 4)) + align256(nb * 4) + 2 * align256(nb * vs);
    }
    case ASAMD_SPMV_TILED:
      if (!st->tiled_built) return 0;
      return align256((size_t)st->nnz * vs) + align256((size_t)p->tiled.long_scratch_elems * vs);
    case ASAMD_SPMV_MERGE_HOT:
      if (!st->hot_built) return 0;
      return align256((size_t)p->hot.cols_front * vs) + align256((size_t)p->hot.blocks * 4) +
             2 * align256((size_t)p->hot.blocks * vs);
    case ASAMD_SPMV_BINNED:
      return st->binned_built ? align256((size_t)p->binned.chunks * vs) : 0;
    case ASAMD_SPMV_XLDS:
      return p->xlds.seg ? align256((size_t)p->xlds.slices * (size_t)st->m * vs) : 0;
    default:
      return 0;
  }
}

static int has_value_copy(const asamd_csr_plan *p) {
  return p->st.tiled_built || p->st.ell_built || p->xlds.val != NULL;
}
/* the families whose kernels read values that the plan keeps */
static int holds_values(const asamd_csr_plan *p, int algo) {
  return algo == ASAMD_SPMV_TILED || algo == ASAMD_SPMV_ELL || (algo == ASAMD_SPMV_XLDS && p->xlds.val != NULL);
}

/* per-call scratch of the transposed multiply that keeps y in LDS, or 0 where the atomic scatter runs */
static size_t trans_ylds_scratch(const asamd_csr_plan *p) {
  const asamd_csr_stats *st = &p->st;
  if (st->nnz < (1 << 20) || st->first_offset != 0 || env_int("ALSPARSE_AMD_XLDS", 1) <= 0) return 0;
  return asamd_spmv_trans_ylds_bytes(p->dtype, st->m, st->n);
}

size_t asamd_csr_plan_workspace_bytes(const asamd_csr_plan *p) {
  if (!p) return 0;
  size_t need = 0;
  for (int a = ASAMD_SPMV_VECTOR; a <= ASAMD_SPMV_XLDS; ++a) {
    if (a == ASAMD_SPMV_MERGE && p->st.first_offset != 0) continue;
    const size_t s = algo_scratch(p, a);
    if (s > need) need = s;
  }
  if (has_value_copy(p)) need += align256(ASAMD_GUARD_WS_BYTES);
  {
    const size_t s = align256(ASAMD_GUARD_WS_BYTES) + align256(trans_ylds_scratch(p));
    if (trans_ylds_scratch(p) && s > need) need = s;
  }
  for (int w = 0; w < 2; ++w)
    if (p->tr[w].plan) {
      const size_t s = align256(ASAMD_GUARD_WS_BYTES) + asamd_csr_plan_workspace_bytes(p->tr[w].plan);
      if (s > need) need = s;
    }
  return need + 256; /* room for aligning the base up */
}

static void account(asamd_csr_plan *p) {
  asamd_csr_stats *st = &p->st;
  int64_t b = SETUP_BYTES + 3 * 8;
  if (p->d_block_row) b += ((int64_t)st->merge_blocks + 1) * 4;
  if (p->d_col16) b += ((int64_t)st->nnz + 4) * 2;
  if (p->d_rel16) b += ((int64_t)st->nnz + 4) * 2;
  b += p->tiled.device_bytes + p->hot.device_bytes + p->binned.device_bytes + p->xlds.device_bytes;
  if (st->ell_built) b += (int64_t)st->m * st->ell_width * ((int64_t)p->val_size + 4);
  for (int w = 0; w < 2; ++w)
    if (p->tr[w].plan) b += p->tr[w].t.device_bytes + p->tr[w].plan->st.device_bytes;
  st->device_bytes = b;
  st->workspace_bytes = (int64_t)asamd_csr_plan_workspace_bytes(p);
}

/* ---- the per-call workspace ----------------------------------------------------------------------- */
typedef struct {
  char *p;
  size_t left;
} ws_cursor;

static ws_cursor ws_open(void *ws, size_t bytes) {
  ws_cursor c = {NULL, 0};
  if (!ws) return c;
  const uintptr_t a = ((uintptr_t)ws + 255) & ~(uintptr_t)255;
  const size_t skip = (size_t)(a - (uintptr_t)ws);
  if (skip >= bytes) return c;
  c.p = (char *)a;
  c.left = bytes - skip;
  return c;
}

static void *ws_take(ws_cursor *c, size_t bytes) {
  const size_t need = align256(bytes ? bytes : 1);
  if (!c->p || c->left < need) return NULL;
  void *r = c->p;
  c->p += need;
  c->left -= need;
  return r;
}

/* ---- launching one family --------------------------------------------------------------------------- */
static int ellmv_any(hipStream_t s, int dtype, int32_t m, int32_t n, const void *alpha, const void *ev, const int32_t *ec,
                     int32_t width, const void *x, const void *beta, void *y) {
  switch (dtype) {
    case ASAMD_DTYPE_FLOAT:
      return asamd_s_ellmv(s, m, n, *(const float *)alpha, (const float *)ev, ec, width, 0, (const float *)x,
                           *(const float *)beta, (float *)y);
    case ASAMD_DTYPE_DOUBLE:
      return asamd_d_ellmv(s, m, n, *(const double *)alpha, (const double *)ev, ec, width, 0, (const double *)x,
                           *(const double *)beta, (double *)y);
    case ASAMD_DTYPE_FLOAT_COMPLEX:
      return asamd_c_ellmv(s, m, n, *(const asamd_complex8 *)alpha, (const asamd_complex8 *)ev, ec, width, 0,
                           (const asamd_complex8 *)x, *(const asamd_complex8 *)beta, (asamd_complex8 *)y);
    default:
      return asamd_z_ellmv(s, m, n, *(const asamd_complex16 *)alpha, (const asamd_complex16 *)ev, ec, width, 0,
                           (const asamd_complex16 *)x, *(const asamd_complex16 *)beta, (asamd_complex16 *)y);
  }
}

/* The family that actually runs for a wish: every step leads to a family that needs less. */
static int settle_algo(const asamd_csr_plan *p, int algo, const void *val, const int32_t *ci) {
  const asamd_csr_stats *st = &p->st;
  for (int pass = 0; pass < 6; ++pass) {
    int next = algo;
    if (algo == ASAMD_SPMV_AUTO) next = p->auto_algo;
    else if (algo == ASAMD_SPMV_TILED && !st->tiled_built) next = p->auto_algo == ASAMD_SPMV_TILED ? p->struct_algo : p->auto_algo;
    else if (algo == ASAMD_SPMV_ELL && !st->ell_built) next = p->auto_algo == ASAMD_SPMV_ELL ? p->struct_algo : p->auto_algo;
    else if (algo == ASAMD_SPMV_MERGE_HOT && !st->hot_built) next = ASAMD_SPMV_MERGE;
    else if (algo == ASAMD_SPMV_BINNED && !st->binned_built) next = ASAMD_SPMV_MERGE;
    else if (algo == ASAMD_SPMV_XLDS && !p->xlds.seg &&
             (!asamd_spmv_xlds_fits(p->dtype, st->n) || st->first_offset != 0 || st->nnz < 1 || st->m < 1))
      next = ASAMD_SPMV_VECTOR;
    else if (algo == ASAMD_SPMV_ROWCONST &&
             (!rowconst_ok(p) || (((uintptr_t)val | (uintptr_t)ci) & 15u) != 0)) /* 128-bit loads */
      next = ASAMD_SPMV_VECTOR;
    else if (algo == ASAMD_SPMV_STREAM && !stream_ok(p)) next = ASAMD_SPMV_MERGE;
    else if (algo == ASAMD_SPMV_MERGE && st->first_offset != 0) next = ASAMD_SPMV_VECTOR;
    if (next == algo) break;
    algo = next;
  }
  return algo;
}

static int run_algo(hipStream_t s, const asamd_csr_plan *p, int algo, const asamd_spmv_args *a, ws_cursor ws) {
  const asamd_csr_stats *st = &p->st;
  const size_t vs = (size_t)p->val_size;
  switch (algo) {
    case ASAMD_SPMV_ELL:
      /* the ELL copy holds zero-based columns and its own values */
      return ellmv_any(s, p->dtype, st->m, st->n, a->alpha, p->d_eval, p->d_ecol, st->ell_width, a->x, a->beta, a->y);
    case ASAMD_SPMV_TILED: {
      void *prod = ws_take(&ws, (size_t)st->nnz * vs);
      void *lscr = p->tiled.long_scratch_elems > 0 ? ws_take(&ws, (size_t)p->tiled.long_scratch_elems * vs) : NULL;
      if (!prod || (p->tiled.long_scratch_elems > 0 && !lscr)) return -1;
      return asamd_spmv_tiled(s, a, &p->tiled, prod, lscr, NULL);
    }
    case ASAMD_SPMV_ROWCONST:
      return asamd_spmv_rowconst(s, a, st->const_len);
    case ASAMD_SPMV_STREAM:
      if (p->d_rel16 && p->rel16_group == stream_group(p, 0) && ((uintptr_t)a->val & 15u) == 0)
        return asamd_spmv_stream_rel16(s, a, p->rel16_group, st->max_len, p->d_rel16);
      return asamd_spmv_stream(s, a, stream_group(p, 0), st->max_len, st->first_offset);
    case ASAMD_SPMV_SCALAR:
      return asamd_spmv_scalar(s, a);
    case ALGO_XLDS_IN_PLACE:
    case ASAMD_SPMV_XLDS:
      if (p->xlds.seg) {
        void *partials = ws_take(&ws, (size_t)p->xlds.slices * (size_t)st->m * vs);
        if (!partials) return -1;
        const double piece = (double)st->nnz / ((double)st->m * (double)p->xlds.slices);
        asamd_xlds_layout view = p->xlds;
        if (algo == ALGO_XLDS_IN_PLACE) view.val = NULL;
        if (view.val) {
          /* the copy's pieces: two loads for a piece of mean length beat one load with half of its lanes idle
           * (pieces of 8 / 12 / 32 / 37 / 50 entries: 8 / 8 / 16 / 32 / 32 entries per load measured best) */
          int width = 8;
          while (width < 64 && 2 * width <= 0.9 * piece) width *= 2;
          return asamd_spmv_xlds_sliced(s, a, width, &view, partials);
        }
        return asamd_spmv_xlds_sliced(s, a, width_for_mean(piece), &view, partials);
      }
      if (p->d_col16) return asamd_spmv_xlds_narrow(s, a, p->auto_width, p->d_col16);
      return asamd_spmv_xlds(s, a, p->auto_width);
    case ASAMD_SPMV_BINNED: {
      void *partial = p->binned.chunks > 0 ? ws_take(&ws, (size_t)p->binned.chunks * vs) : NULL;
      if (p->binned.chunks > 0 && !partial) return -1;
      return asamd_spmv_binned(s, a, &p->binned, partial);
    }
    case ASAMD_SPMV_MERGE_HOT: {
      void *front = ws_take(&ws, (size_t)p->hot.cols_front * vs);
      int32_t *carry_row = (int32_t *)ws_take(&ws, (size_t)p->hot.blocks * 4);
      void *carry_val = ws_take(&ws, (size_t)p->hot.blocks * vs);
      void *head_val = ws_take(&ws, (size_t)p->hot.blocks * vs);
      if (!head_val) return -1;
      return asamd_spmv_hot(s, a, &p->hot, front, carry_row, carry_val, head_val);
    }
    case ASAMD_SPMV_MERGE: {
      const size_t nb = (size_t)st->merge_blocks;
      const int32_t *block_row = p->d_block_row;
      if (!block_row) {
        /* structure not promised fixed: the coordinates are computed for this call */
        int32_t *fresh = (int32_t *)ws_take(&ws, (nb + 1) * 4);
        if (!fresh) return -1;
        const int e = asamd_merge_partition(s, st->m, st->nnz, a->row_ptr, st->base, st->merge_blocks,
                                            ASAMD_MERGE_THREADS * p->merge_ipt, fresh);
        if (e != hipSuccess) return e;
        block_row = fresh;
      }
      int32_t *carry_row = (int32_t *)ws_take(&ws, nb * 4);
      void *carry_val = ws_take(&ws, nb * vs);
      void *head_val = ws_take(&ws, nb * vs);
      if (!head_val) return -1;
      return asamd_spmv_merge(s, a, p->merge_ipt, block_row, carry_row, carry_val, head_val);
    }
    case ASAMD_SPMV_VECTOR:
    default:
      return asamd_spmv_vector(s, a, p->auto_width);
  }
}

/* Gathers the plan's tiled / ELL / slice-by-slice copy again from val; gate: NULL, or the value guard's flag. */
static hipError_t refresh_main(hipStream_t s, asamd_csr_plan *p, const int32_t *rp, const int32_t *ci, const void *val,
                               const int32_t *gate) {
  const asamd_csr_stats *st = &p->st;
  hipError_t e = hipSuccess;
  if (st->tiled_built)
    e = (hipError_t)asamd_tiled_gather_values(s, &p->tiled, val, gate);
  if (e == hipSuccess && st->ell_built)
    e = (hipError_t)asamd_csr2ell_gated(s, p->val_size, st->m, val, rp, ci, st->base, 0, st->ell_width, p->d_eval,
                                        p->d_ecol, gate);
  if (e == hipSuccess && p->xlds.val) e = (hipError_t)asamd_xlds_refresh_values(s, &p->xlds, val, gate);
  return e;
}

/* ... and one transposed copy with everything its own analysis keeps */
static hipError_t refresh_trans(hipStream_t s, asamd_csr_plan *p, int which, const void *val, const int32_t *gate) {
  asamd_trans_copy *t = &p->tr[which];
  hipError_t e = (hipError_t)asamd_gather_values(s, p->dtype, which == 1, p->st.nnz, t->t.perm, val, t->t.val, gate);
  if (e == hipSuccess) e = refresh_main(s, t->plan, t->t.row_ptr, t->t.col_ind, t->t.val, gate);
  return e;
}

static int csrmv_inner(hipStream_t s, asamd_csr_plan *p, const asamd_spmv_args *a, ws_cursor ws, int guard) {
  const asamd_csr_stats *st = &p->st;
  int algo = st->algo;
  /* The tiled, ELL and slice-by-slice copies hold the values of the array they were built from.  A multiply that
   * brings another value array (same structure, new numbers) must not see the old ones: it runs the kernel that
   * the row statistics alone would pick (the column slices: over the caller's arrays). */
  if (holds_values(p, algo) && p->copy_val_src && a->val != p->copy_val_src)
    algo = algo == ASAMD_SPMV_XLDS ? ALGO_XLDS_IN_PLACE : p->struct_algo;
  algo = settle_algo(p, algo, a->val, a->col_ind);
  if (holds_values(p, algo) && guard && st->value_check) {
    /* Values changed IN PLACE under the copy: fingerprint, compare, gather again if need be, and only
     * then record the new fingerprint -- a multiply on another stream that reads the recorded word
     * either finds the old one (and gathers the same values again itself) or finds the copy done. */
    void *g = ws_take(&ws, ASAMD_GUARD_WS_BYTES);
    if (!g) {
      /* no room to check the copy: do not use it */
      algo = algo == ASAMD_SPMV_XLDS ? ALGO_XLDS_IN_PLACE : settle_algo(p, p->struct_algo, a->val, a->col_ind);
    } else {
      int e = asamd_value_guard(s, a->val, (size_t)st->nnz * (size_t)p->val_size, st->value_check == 2, p->d_fp, g);
      if (e == hipSuccess) e = (int)refresh_main(s, p, a->row_ptr, a->col_ind, a->val, ASAMD_GUARD_FLAG(g));
      if (e == hipSuccess) e = asamd_value_guard_commit(s, g, p->d_fp);
      if (e != hipSuccess) return e;
    }
  }
  int e = run_algo(s, p, algo, a, ws);
  if (e == -1) {
    /* the workspace does not hold this family's scratch: a lane group per row needs none */
    e = asamd_spmv_vector(s, a, p->auto_width);
  }
  return e;
}

static void fill_args(asamd_spmv_args *a, const asamd_csr_plan *p, const void *alpha, const void *val,
                      const int32_t *rp, const int32_t *ci, const void *x, const void *beta, void *y) {
  a->dtype = p->dtype;
  a->m = p->st.m;
  a->n = p->st.n;
  a->nnz = p->st.nnz;
  a->base = p->st.base;
  a->alpha = alpha;
  a->beta = beta;
  a->val = val;
  a->row_ptr = rp;
  a->col_ind = ci;
  a->x = x;
  a->y = y;
}

static hipError_t build_transpose(hipStream_t stream, asamd_csr_plan *p, const int32_t *rp, const int32_t *ci,
                                  const void *val, int which);

int asamd_csr_plan_csrmv(hipStream_t s, asamd_csr_plan *p, int32_t op, const void *alpha, const void *val,
                         const int32_t *rp, const int32_t *ci, const void *x, const void *beta, void *y,
                         void *workspace, size_t workspace_bytes) {
  if (!p || !alpha || !beta || !val || !rp || !ci || !x || !y) return hipErrorInvalidValue;
  if (op < 0 || op > 2 || (op == 2 && !is_complex(p))) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % (size_t)p->val_size) return hipErrorInvalidValue;
  const asamd_csr_stats *st = &p->st;
  ws_cursor ws = ws_open(workspace, workspace_bytes);
  asamd_spmv_args a;
  fill_args(&a, p, alpha, val, rp, ci, x, beta, y);
  if (op == 0) return csrmv_inner(s, p, &a, ws, 1);

  const int which = op - 1;
  asamd_trans_copy *t = &p->tr[which];
  /* A library-owned mirror lays out its copy of the transpose on the first transposed multiply: that
   * allocates and waits, which a stream under capture must not do -- such a call scatters instead, and
   * the copy is laid out by the first call outside a capture. */
  if (!t->plan && p->lazy_transpose && st->trusted && st->nnz > 0 && st->first_offset == 0) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) {
      (void)hipGetLastError();
      capturing = hipStreamCaptureStatusActive; /* unknown: do not risk it */
    }
    if (capturing == hipStreamCaptureStatusNone) {
      const hipError_t e = build_transpose(s, p, rp, ci, val, which);
      if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError(); /* no room for the copy: scatter instead, and do not try again */
        p->lazy_transpose = 0;
      } else if (e != hipSuccess) {
        return e;
      }
    }
  }
  /* the copy holds the values it was gathered from: another value array takes the scatter route below */
  if (t->plan && val == t->val_src) {
    int usable = 1;
    if (st->value_check) {
      void *g = ws_take(&ws, ASAMD_GUARD_WS_BYTES);
      if (!g) {
        usable = 0; /* no room to check the copy: do not use it */
      } else {
        int e = asamd_value_guard(s, val, (size_t)st->nnz * (size_t)p->val_size, st->value_check == 2,
                                  p->d_fp + 1 + which, g);
        if (e == hipSuccess) e = (int)refresh_trans(s, p, which, val, ASAMD_GUARD_FLAG(g));
        if (e == hipSuccess) e = asamd_value_guard_commit(s, g, p->d_fp + 1 + which);
        if (e != hipSuccess) return e;
      }
    }
    if (usable) {
      asamd_spmv_args at;
      fill_args(&at, t->plan, alpha, t->t.val, t->t.row_ptr, t->t.col_ind, x, beta, y);
      return csrmv_inner(s, t->plan, &at, ws, 0);
    }
  }
  /* y in LDS where it fits and the matrix is large enough for a workgroup per compute unit to pay */
  const size_t ylds = trans_ylds_scratch(p);
  if (ylds) {
    void *partials = ws_take(&ws, ylds);
    if (partials) return asamd_spmv_trans_ylds(s, &a, p->auto_width, which == 1, partials);
  }
  return asamd_spmv_trans_scatter(s, &a, p->auto_width, which == 1);
}

/* ---- a matrix that nobody promised to leave alone ------------------------------------------------------ */
#define WATCH_FLAG_BYTES 256

size_t asamd_csr_plan_watched_workspace_bytes(const asamd_csr_plan *p) {
  if (!p) return 0;
  return asamd_csr_plan_workspace_bytes(p) + 3 * align256(ASAMD_GUARD_WS_BYTES) + WATCH_FLAG_BYTES;
}

int asamd_csr_plan_watch_begin(hipStream_t s, asamd_csr_plan *p, const int32_t *rp, const int32_t *ci, const void *val,
                               uint64_t *watch, void *workspace, size_t workspace_bytes) {
  if (!p || !rp || !ci || !val || !watch) return hipErrorInvalidValue;
  ws_cursor ws = ws_open(workspace, workspace_bytes);
  void *g = ws_take(&ws, ASAMD_GUARD_WS_BYTES);
  if (!g) return hipErrorInvalidValue;
  const asamd_csr_stats *st = &p->st;
  int e = asamd_value_guard(s, rp, ((size_t)st->m + 1) * 4, 1, NULL, g);
  if (e == hipSuccess) e = asamd_value_guard_commit(s, g, watch);
  if (e == hipSuccess) e = asamd_value_guard(s, ci, (size_t)st->nnz * 4, 1, NULL, g);
  if (e == hipSuccess) e = asamd_value_guard_commit(s, g, watch + 1);
  /* the values' fingerprint of the plan, which may be a sampled one, becomes one of every byte as well */
  if (e == hipSuccess) e = asamd_value_guard(s, val, (size_t)st->nnz * (size_t)p->val_size, 1, NULL, g);
  if (e == hipSuccess) e = asamd_value_guard_commit(s, g, p->d_fp);
  return e;
}

int asamd_csr_plan_csrmv_watched(hipStream_t s, asamd_csr_plan *p, const void *alpha, const void *val,
                                 const int32_t *rp, const int32_t *ci, const void *x, const void *beta, void *y,
                                 const uint64_t *watch, void *workspace, size_t workspace_bytes,
                                 const int32_t **changed) {
  if (!p || !alpha || !beta || !val || !rp || !ci || !x || !y || !watch) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % (size_t)p->val_size) return hipErrorInvalidValue;
  const asamd_csr_stats *st = &p->st;
  if (st->algo != ASAMD_SPMV_TILED || !st->tiled_built || val != p->copy_val_src) return hipErrorInvalidValue;
  if (workspace_bytes < asamd_csr_plan_watched_workspace_bytes(p)) return hipErrorInvalidValue;
  ws_cursor ws = ws_open(workspace, workspace_bytes);
  void *g_rp = ws_take(&ws, ASAMD_GUARD_WS_BYTES), *g_ci = ws_take(&ws, ASAMD_GUARD_WS_BYTES);
  void *g_val = ws_take(&ws, ASAMD_GUARD_WS_BYTES);
  int32_t *skip = (int32_t *)ws_take(&ws, WATCH_FLAG_BYTES);
  const size_t vs = (size_t)p->val_size;
  void *prod = ws_take(&ws, (size_t)st->nnz * vs);
  void *lscr = p->tiled.long_scratch_elems > 0 ? ws_take(&ws, (size_t)p->tiled.long_scratch_elems * vs) : NULL;
  if (!g_rp || !g_ci || !g_val || !skip || !prod || (p->tiled.long_scratch_elems > 0 && !lscr))
    return hipErrorInvalidValue;
  /* every byte of the three arrays is fingerprinted: a caller who made no promise gets no sampling */
  int e = asamd_value_guard(s, rp, ((size_t)st->m + 1) * 4, 1, watch, g_rp);
  if (e == hipSuccess) e = asamd_value_guard(s, ci, (size_t)st->nnz * 4, 1, watch + 1, g_ci);
  if (e == hipSuccess) e = asamd_value_guard_any(s, g_rp, g_ci, skip);
  if (e == hipSuccess) e = asamd_value_guard(s, val, (size_t)st->nnz * vs, 1, p->d_fp, g_val);
  if (e == hipSuccess) e = (int)refresh_main(s, p, rp, ci, val, ASAMD_GUARD_FLAG(g_val));
  if (e == hipSuccess) e = asamd_value_guard_commit(s, g_val, p->d_fp);
  asamd_spmv_args a;
  fill_args(&a, p, alpha, val, rp, ci, x, beta, y);
  /* the layout's kernels, which return at once if the structure has changed, and the stand-in on the caller's
   * arrays, which returns at once if it has not */
  if (e == hipSuccess) e = asamd_spmv_tiled(s, &a, &p->tiled, prod, lscr, skip);
  if (e == hipSuccess) e = asamd_spmv_vector_if(s, &a, p->auto_width, skip);
  if (changed) *changed = skip;
  return e;
}

/* ---- analysis: timing the candidates ----------------------------------------------------------------- */
enum { CAND_BASE = 0, CAND_TILED, CAND_ELL, CAND_HOT, CAND_BINNED, CAND_COUNT };

typedef struct {
  hipStream_t stream;
  asamd_csr_plan *p;
  const int32_t *row_ptr, *col_ind;
  const void *val;
  void *x, *y, *ws;
  size_t ws_bytes;
  hipEvent_t e0, e1;
  float best[CAND_COUNT];
  int algos[CAND_COUNT];
  hipError_t err;
} tune_ctx;

/* the candidates' scratch comes from a buffer of the analysis' own, grown as the candidates ask */
static void tune_reserve(tune_ctx *t, size_t bytes) {
  if (t->err != hipSuccess || bytes <= t->ws_bytes) return;
  if (t->ws) (void)hipFree(t->ws);
  t->ws = NULL;
  t->ws_bytes = 0;
  t->err = hipMalloc(&t->ws, bytes);
  if (t->err == hipSuccess) t->ws_bytes = bytes;
}

static void time_algo(tune_ctx *t, int cand) {
  asamd_csr_plan *p = t->p;
  p->st.algo = t->algos[cand];
  tune_reserve(t, algo_scratch(p, t->algos[cand]) + 512);
  static const double one[2] = {1.0, 0.0}, zero[2] = {0.0, 0.0};
  static const float onef[2] = {1.0f, 0.0f}, zerof[2] = {0.0f, 0.0f};
  const int wide = p->dtype == ASAMD_DTYPE_DOUBLE || p->dtype == ASAMD_DTYPE_DOUBLE_COMPLEX;
  const void *alpha = wide ? (const void *)one : (const void *)onef;
  const void *beta = wide ? (const void *)zero : (const void *)zerof;
  asamd_spmv_args a;
  fill_args(&a, p, alpha, t->val, t->row_ptr, t->col_ind, t->x, beta, t->y);
  /* first run warms up; multiplies of a millisecond and more are timed once, shorter ones twice; a
   * first run of more than two milliseconds is its own measurement (cold caches are noise at that length) */
  int reps = 3;
  for (int rep = 0; rep < reps && t->err == hipSuccess; ++rep) {
    t->err = hipEventRecord(t->e0, t->stream);
    if (t->err == hipSuccess) t->err = (hipError_t)csrmv_inner(t->stream, p, &a, ws_open(t->ws, t->ws_bytes), 0);
    if (t->err == hipSuccess) t->err = hipEventRecord(t->e1, t->stream);
    if (t->err == hipSuccess) t->err = hipEventSynchronize(t->e1);
    float ms = 0.f;
    if (t->err == hipSuccess) t->err = hipEventElapsedTime(&ms, t->e0, t->e1);
    if (rep == 0 && ms > 1.0f) reps = ms > 2.0f ? 1 : 2;
    if ((rep > 0 || reps == 1) && (t->best[cand] == 0.f || ms < t->best[cand])) t->best[cand] = ms;
  }
}

/* Time the structural choice on scratch vectors, then the copies that the matrix is eligible for:
 * the ELL copy (cheap to build), and the tiled copy only if the fastest so far is slower than the
 * tiled pair could possibly be.  Keep the fastest and free the copies that lost.  A copy has to win
 * by a margin to be worth its memory. */
static hipError_t tune_copies(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                              const void *val, int tiled_ok, int ell_ok, int hot_ok, int binned_ok) {
  asamd_csr_stats *st = &p->st;
  const size_t vs = (size_t)p->val_size;
  tune_ctx t;
  memset(&t, 0, sizeof t);
  t.stream = stream;
  t.p = p;
  t.row_ptr = row_ptr;
  t.col_ind = col_ind;
  t.val = val;
  t.err = hipMalloc(&t.x, (size_t)st->n * vs);
  if (t.err == hipSuccess) t.err = hipMalloc(&t.y, (size_t)st->m * vs);
  if (t.err == hipSuccess) t.err = hipMemsetAsync(t.x, 0, (size_t)st->n * vs, stream);
  if (t.err == hipSuccess) t.err = hipEventCreate(&t.e0);
  if (t.err == hipSuccess) t.err = hipEventCreate(&t.e1);
  t.algos[CAND_BASE] = p->auto_algo;
  t.algos[CAND_TILED] = ASAMD_SPMV_TILED;
  t.algos[CAND_ELL] = ASAMD_SPMV_ELL;
  t.algos[CAND_HOT] = ASAMD_SPMV_MERGE_HOT;
  t.algos[CAND_BINNED] = ASAMD_SPMV_BINNED;
  /* The tiled pair streams about twice the algorithmic bytes (16 instead of 8 bytes per fp32 entry), so
   * it cannot finish before 2 * bytes / (the ~5 TB/s that streams reach). */
  const double bytes = (double)st->nnz * (4.0 + (double)vs) + ((double)st->m + 1) * 4.0 +
                       ((double)st->n + (double)st->m) * (double)vs;
  float tiled_floor_ms = (float)(2.0 * bytes / 5.0e9);
  /* Heavy-tailed rows (power-law graphs) make uneven tiles: the in-wave combining of equal rows and the
   * long-tile phase then cost the tiled pair about 2.3 times its floor (measured 0.78 ms against 0.34 ms
   * on an 8 M-row R-MAT matrix whose longest row has 120 000 entries; 0.65 ms on its transpose). */
  if ((double)st->max_len > 32.0 * ((double)st->nnz / (double)st->m) + 256.0) tiled_floor_ms *= 2.5f;
  if (t.err == hipSuccess) time_algo(&t, CAND_BASE);
  /* A lane group per row, or a staged block of rows with several lanes per row, was chosen from the mean and
   * the longest row alone.  Neither needs a copy, nor does merge-path, which takes any distribution: the
   * fastest of them stays. */
  if (t.err == hipSuccess && structural_alternatives(p)) {
    const int alts[2] = {ASAMD_SPMV_MERGE, p->auto_algo == ASAMD_SPMV_STREAM ? ASAMD_SPMV_VECTOR : -1};
    for (int i = 0; i < 2; ++i) {
      const int alt = alts[i];
      if (alt < 0 || t.err != hipSuccess) continue;
      const float first = t.best[CAND_BASE];
      const int kept = t.algos[CAND_BASE];
      t.best[CAND_BASE] = 0.f;
      t.algos[CAND_BASE] = alt;
      time_algo(&t, CAND_BASE);
      if (t.err == hipSuccess && t.best[CAND_BASE] > 0.f && t.best[CAND_BASE] < 0.97f * first) {
        p->auto_algo = p->struct_algo = alt;
      } else {
        t.algos[CAND_BASE] = kept;
        t.best[CAND_BASE] = first;
      }
    }
  }
  /* An ELL copy gathers x row by row like the kernel just timed; when that one is several times slower
   * than the tiled floor the gathers are the problem and the ELL copy (as large as the matrix) is not
   * worth building: the tiled copy is tried first, the ELL copy only if that does not win. */
  const int ell_first = !(tiled_ok && t.best[CAND_BASE] > 2.5f * tiled_floor_ms);
  if (ell_first && t.err == hipSuccess && ell_ok) {
    t.err = build_ell(stream, p, row_ptr, col_ind, val);
    if (t.err == hipSuccess) time_algo(&t, CAND_ELL);
  }
  if (t.err == hipSuccess && tiled_ok) {
    /* A row kernel that is already as fast as the tiled floor (banded matrices, whose gathers stay in
     * the caches) makes the tiled copy pointless: its layout pass (a sort of all entries) and its
     * memory are saved. */
    float fastest = t.best[CAND_BASE];
    if (t.best[CAND_ELL] > 0.f && t.best[CAND_ELL] < fastest) fastest = t.best[CAND_ELL];
    if (fastest > 1.1f * tiled_floor_ms) {
      t.err = build_tiled(stream, p, row_ptr, col_ind, val);
      if (t.err == hipSuccess && st->tiled_built) time_algo(&t, CAND_TILED);
    }
  }
  if (!ell_first && !(t.best[CAND_TILED] > 0.f && t.best[CAND_TILED] < 0.9f * t.best[CAND_BASE]) &&
      t.err == hipSuccess && ell_ok) {
    t.err = build_ell(stream, p, row_ptr, col_ind, val);
    if (t.err == hipSuccess) time_algo(&t, CAND_ELL);
  }
  /* Skewed matrices on merge-path: count the entries per column and, if few columns hold most of them,
   * time the kernel that keeps those columns' x in LDS. */
  if (t.err == hipSuccess && hot_ok && p->auto_algo == ASAMD_SPMV_MERGE) {
    t.err = build_hot(stream, p, row_ptr, col_ind, 0);
    if (t.err == hipSuccess && st->hot_built) time_algo(&t, CAND_HOT);
  }
  /* Very uneven rows: one launch per row-length class (cheap to lay out: a sort of the row numbers) */
  if (t.err == hipSuccess && binned_ok) {
    t.err = build_binned(stream, p, row_ptr);
    if (t.err == hipSuccess && st->binned_built) time_algo(&t, CAND_BINNED);
  }
  if (t.e0) (void)hipEventDestroy(t.e0);
  if (t.e1) (void)hipEventDestroy(t.e1);
  if (t.x) (void)hipFree(t.x);
  if (t.y) (void)hipFree(t.y);
  if (t.ws) (void)hipFree(t.ws);
  st->algo = p->auto_algo;
  if (t.err != hipSuccess) return t.err;
  st->tune_ms_binned = t.best[CAND_BINNED];
  st->tune_ms_base = t.best[CAND_BASE];
  st->tune_ms_tiled = t.best[CAND_TILED];
  st->tune_ms_ell = t.best[CAND_ELL];
  st->tune_ms_hot = t.best[CAND_HOT];
  /* a copy has to win by a margin to be worth its memory; among the winners the fastest is kept */
  const float margin[CAND_COUNT] = {1.f, 0.9f, 0.95f, 0.95f, 0.95f};
  /* (the timing runs launch the kernels alone: a copy that holds values is multiplied behind the value guard's four
   * small launches later on, and is compared with them counted) */
  float cost[CAND_COUNT];
  for (int c = 0; c < CAND_COUNT; ++c)
    cost[c] = t.best[c] + (t.best[c] > 0.f && (c == CAND_TILED || c == CAND_ELL) && st->value_check && !p->watched ? 0.022f : 0.f);
  int pick = 0;
  for (int c = 1; c < CAND_COUNT; ++c)
    if (cost[c] > 0.f && cost[c] < margin[c] * cost[CAND_BASE] && (pick == 0 || cost[c] < cost[pick])) pick = c;
  /* ALSPARSE_AMD_TUNE_PICK = base | tiled | ell | hot | binned overrides the timing's verdict among the
   * candidates that were built (for profiling a kernel that lost) */
  const char *ev = getenv("ALSPARSE_AMD_TUNE_PICK");
  if (ev) {
    static const char *names[CAND_COUNT] = {"base", "tiled", "ell", "hot", "binned"};
    for (int c = 0; c < CAND_COUNT; ++c)
      if (!strcmp(ev, names[c]) && (c == 0 || t.best[c] > 0.f)) pick = c;
  }
  if (pick != CAND_TILED) free_tiled(p);
  if (pick != CAND_ELL) free_ell(p);
  if (pick != CAND_HOT) free_hot(p);
  if (pick != CAND_BINNED) free_binned(p);
  if (pick != CAND_BASE) {
    p->auto_algo = t.algos[pick];
    st->algo = t.algos[pick];
  }
  return hipSuccess;
}

/* ---- analysis: deciding from a model ---------------------------------------------------------------
 * The same decisions without a single timing run, so that one matrix always gets one family whatever else
 * the GPU is doing while it is analysed.  A multiply is modelled as its matrix streams and its gathers of x,
 *     t = sqrt(t_stream^2 + t_gather^2),   t_stream = algorithmic bytes / the family's streaming rate,
 *                                          t_gather = entries * w * T(s),
 * with the two numbers of the locality probe: w, the distinct 128-byte lines of x per entry among 64
 * consecutive entries (how many requests a gather instruction sends to the L1), and s, the distinct lines per
 * entry within 32 768 consecutive entries, which orders matrices by how far their gathers reach (uniform
 * columns over 2 / 4 / 8 / 16 / 64 MiB of x: s = 0.43 / 0.63 / 0.79 / 0.89 / 0.94; a power-law graph with 32 MiB
 * of x: 0.45; a stencil: 0.005).  T(s) and the rates are measurements of these kernels on an MI355X:
 *     s      0     0.25   0.45   0.63   0.68   0.79   0.885   0.94   1      (entries whose line must come from
 *     T ps   3.6   4.7    5.6    5.9    10.5   10.5   13.5    17.8   19      beyond an XCD's L2 wait 3 x longer)
 *     TB/s   constant row length 6.0, staged row block 6.6 (one lane per row) / 5.2 (several), lane group per
 *            row 2.4 x the share of its lanes that hold an entry, merge-path 2.9, ELL copy 6.1 (of its padded
 *            streams); tiled pair: 0.015 .. 0.045 ms (small matrices less) + 2 x bytes / 5.6 TB/s (8-byte values and wider: their 28 / 52 bytes per
 *            entry at 4.6 TB/s), x 1 .. 1.5 with the spread of the row lengths, x 2.5 for heavy-tailed rows.
 * The estimates are within about 10 % of the timings on the shapes they were read from (5-point and 27-point
 * stencils, uniform rows over 0.25 - 64 MiB of x, two row lengths, power-law rows and columns, fp32 / fp64). */
static double gather_ps(double s) {
  static const double xs[9] = {0.0, 0.25, 0.45, 0.63, 0.68, 0.79, 0.885, 0.94, 1.0};
  static const double ys[9] = {3.6, 4.7, 5.6, 5.9, 10.5, 10.5, 13.5, 17.8, 19.0};
  if (s <= xs[0]) return ys[0];
  for (int i = 1; i < 9; ++i)
    if (s <= xs[i]) return ys[i - 1] + (ys[i] - ys[i - 1]) * (s - xs[i - 1]) / (xs[i] - xs[i - 1]);
  return ys[8];
}

static double hypot2(double a, double b) {
  /* sqrt(a^2 + b^2) without libm: the larger of the two scaled by a few Newton steps */
  const double big = a > b ? a : b, small = a > b ? b : a;
  if (big <= 0.0) return 0.0;
  const double q = small / big, v = 1.0 + q * q;
  double r = 1.0 + 0.5 * q * q; /* sqrt(v) for v in [1, 2] */
  for (int i = 0; i < 4; ++i) r = 0.5 * (r + v / r);
  return big * r;
}

/* share of the lanes of a W-lane group that hold an entry, over the rows of the log2 histogram */
static double vector_utilisation(const asamd_csr_stats *st, int w) {
  double used = 0.0, slots = 0.0;
  for (int b = 1; b < ASAMD_HIST_BINS; ++b) {
    if (!st->hist[b]) continue;
    const double len = b == 1 ? 1.0 : 0.75 * (double)((int64_t)1 << b); /* middle of [2^(b-1), 2^b) */
    const double trips = (double)(int64_t)((len + w - 1) / w);
    used += (double)st->hist[b] * len;
    slots += (double)st->hist[b] * trips * w;
  }
  return slots > 0.0 ? used / slots : 1.0;
}

static double model_ms(const asamd_csr_plan *p, int algo) {
  const asamd_csr_stats *st = &p->st;
  const double vs = (double)p->val_size, nnz = (double)st->nnz, m = (double)st->m, n = (double)st->n;
  const double bytes = nnz * (4.0 + vs) + (m + 1.0) * 4.0 + (n + m) * vs;
  const double gather = nnz * (double)st->lines_per_entry_wave * gather_ps((double)st->lines_per_entry_segment) * 1e-9;
  const double mean = nnz / (m > 0 ? m : 1);
  double rate = 2.9; /* TB/s */
  switch (algo) {
    case ASAMD_SPMV_ROWCONST: rate = 6.0; break;
    case ASAMD_SPMV_STREAM:
      rate = stream_group(p, 0) > 1 ? 5.2 : 6.6;
      /* 16-byte values (four per lane, so two lanes per row of five): 5-point Laplacian of 4 M rows, complex128
       * (570 MB), 0.139 ms */
      if (vs >= 16.0 && rate > 4.2) rate = 4.2;
      /* 16-bit distances for columns: half of the bytes they save shows (27-point stencil, 160^3 points: 0.204 ->
       * 0.181 ms with 4-byte values, 0.300 -> 0.274 with 8-byte ones) */
      if (p->d_rel16) return hypot2((bytes - 1.0 * nnz) / (rate * 1e9), gather);
      break;
    case ASAMD_SPMV_VECTOR: rate = 2.4 * vector_utilisation(st, p->auto_width); break;
    case ASAMD_SPMV_MERGE: rate = 2.9; break;
    case ASAMD_SPMV_XLDS: {
      /* measured: 1.9 ps per fp32 entry, 2.65 per fp64; in slices the pieces of the rows start anywhere in their
       * cache lines (pieces of 50 / 36 / 32 entries: 1.14 / 1.57 / 1.6 times that) and the slices' sums travel */
      const double one = nnz * (1.15 + 0.1875 * vs) * 1e-9;
      const int slices = p->xlds.seg ? p->xlds.slices : (asamd_spmv_xlds_fits(p->dtype, st->n) ? 1 : xlds_slices_for(p));
      if (slices < 2) return one;
      const double sums = (double)slices * m * 3.0 * vs / 4.0e9;
      if (p->xlds.seg ? p->xlds.val != NULL : p->xlds_copy_wanted) {
        /* the copy (16-bit columns, neighbouring pieces), measured with pieces of 50 / 32 / 12.5 / 8 entries, fp32:
         * 1.91 / 1.92 / 2.20 / 2.54 ps per entry, the slices' sums included; 37 entries, fp64: 2.82 */
        /* (65 536 x 65 536 x 64, 4 M entries: 0.029 ms, of which the value guard's launches, the slices' sums and 256
         * workgroups' fills of LDS are 0.02) */
        return 0.02 + 0.94 * one + (double)slices * m * 6.0e-9;
      }
      return one * (1.0 + 22.0 * (double)slices / mean) + sums;
    }
    case ASAMD_SPMV_ELL: {
      const double ell_bytes = m * (double)st->max_len * (4.0 + vs) + (n + m) * vs;
      /* The lanes of one ELL gather hold the SAME position of 64 neighbouring rows; with ascending columns those
       * fall into a narrower window of x than the positions of one row, which pays once x outgrows an XCD's L2:
       * 1 M x 1 M x 16 / x 32, fp64 (8 MB of x): 0.143 / 0.261 ms against rowconst's 0.186 / 0.355 (more rows in
       * flight per lane group do not help rowconst: 0.357); fp32 (4 MB): 0.100 / 0.196 against 0.095 / 0.196 */
      /* (rows of 16 and more; with few entries per row one position's columns spread as far as a row's: 2 M x 2 M x 4,
       * fp64, 0.130 ms against rowconst's 0.128; 1 M x 1 M x 8: 0.086 against 0.096) */
      double narrow = 1.0;
      if (vs >= 8.0 && mean > 8.0) narrow = mean >= 16.0 ? 0.72 : 1.0 - 0.28 * (mean - 8.0) / 8.0;
      return hypot2(ell_bytes / 6.1e9, narrow * gather);
    }
    case ASAMD_SPMV_TILED: {
      double skew = 1.0 + 0.5 * ((double)st->max_len / mean - 1.0) / 8.0;
      if (skew > 1.5) skew = 1.5;
      if ((double)st->max_len > 32.0 * mean + 256.0) skew = 2.5; /* heavy tail: long tiles, uneven waves */
      /* 4-byte values: twice the CSR bytes at 5.6 TB/s; wider ones move 3 values + 4 index bytes per entry
       * through both phases and their second phase (shorter row blocks) reaches 4.6 TB/s */
      const double stream = vs >= 8.0 ? (nnz * (3.0 * vs + 4.0) + (n + m) * vs) / 4.6e9 : 2.0 * bytes / 5.6e9;
      /* rows that all hold 64 entries and more make short row blocks (a tile holds 128 entries at most) and ran 1.37-1.64 times
       * the estimate that fits rows of 16 (1 M x 1 M x 64: 0.346 ms, 2 M x 2 M x 64: 0.657, 1 M x 1 M x 128: 0.607) */
      const double usual = mean < 4.0 * (st->min_len + 1.0) ? mean : 4.0 * (st->min_len + 1.0); /* (not a few long rows) */
      /* (8-byte values: 1 M x 1 M x 64 measured 0.587 ms, 1.30 times the estimate for rows of 16) */
      const double most = vs >= 8.0 ? 0.30 : 0.45;
      double long_rows = 1.0 + most * (usual - 16.0) / 48.0;
      if (long_rows < 1.0) long_rows = 1.0;
      if (long_rows > 1.0 + most) long_rows = 1.0 + most;
      /* short rows on matrices of up to 16 M entries ran below the estimate that fits rows of 16 (8-byte values,
       * 2 M x 2 M x 4: 0.073 against 0.095 ms, 4 M x 4 M x 4: 0.125 / 0.162, 1 M x 1 M x 8: 0.079 / 0.088; 4-byte ones,
       * 2 M x 2 M x 4: 0.050 / 0.062, 4 M x 4 M x 2: 0.056 / 0.075, 2 M x 2 M x 8: 0.089 / 0.100); with 32 M entries and
       * more they do not (8 M x 8 M x 4, 8-byte values: 0.301 / 0.278) */
      if (usual < 16.0 && nnz < 33.5e6) {
        double cut = 0.22 * (16.0 - usual) / 12.0;
        if (cut > 0.22) cut = 0.22;
        const double fade = nnz <= 16.8e6 ? 1.0 : (33.5e6 - nnz) / 16.7e6;
        long_rows = 1.0 - cut * fade;
      }
      /* the fixed part: 0.045 ms from about 200 MB of CSR bytes on; a matrix of a few tens of MB has fewer tiles than
       * the two phases keep in flight and runs them in less (4 M x 4 M x 2, 118 MB: 0.057 ms measured, 2 M x 2 M x 8,
       * 158 MB: 0.089) */
      const double fixed = 0.015 + 0.03 * (bytes < 200.0e6 ? bytes / 200.0e6 : 1.0);
      return (fixed + stream) * skew * long_rows;
    }
    default: break;
  }
  return hypot2(bytes / (rate * 1e9), gather);
}

static hipError_t model_copies(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                               const void *val, int tiled_ok, int ell_ok, int hot_ok, int binned_ok) {
  asamd_csr_stats *st = &p->st;
  if (st->lines_per_entry_wave <= 0.f) return hipSuccess; /* not probed (a tiny matrix): the structural choice stays */
  double base = model_ms(p, p->auto_algo);
  if (p->auto_algo == ASAMD_SPMV_XLDS && !p->xlds.seg) {
    /* columns that neighbouring entries share are cheap to gather from the caches too */
    const double plain = model_ms(p, p->plain_algo);
    if (base > 0.95 * plain) {
      p->auto_algo = p->struct_algo = p->plain_algo;
      base = plain;
    }
  }
  if (structural_alternatives(p)) {
    const int alts[2] = {ASAMD_SPMV_MERGE, p->auto_algo == ASAMD_SPMV_STREAM ? ASAMD_SPMV_VECTOR : -1};
    for (int i = 0; i < 2; ++i) {
      if (alts[i] < 0) continue;
      const double alt = model_ms(p, alts[i]);
      if (alt < 0.97 * base) {
        p->auto_algo = p->struct_algo = alts[i];
        base = alt;
      }
    }
  }
  st->algo = p->auto_algo;
  st->tune_ms_base = (float)base;
  /* the copies in the order of their estimates; each is laid out only if it is the best one left */
  /* a copy that holds values is multiplied behind the value guard: four small launches, 22-30 us (27-point stencil
   * on 128 x 128 x 64 points: the ELL kernel 0.041 ms, the guarded multiply 0.057, the staged row blocks 0.046) */
  const double guard_ms = st->value_check && !p->watched ? 0.022 : 0.0;
  const double est_tiled = tiled_ok ? model_ms(p, ASAMD_SPMV_TILED) + guard_ms : 0.0;
  const double est_ell = ell_ok ? model_ms(p, ASAMD_SPMV_ELL) + guard_ms : 0.0;
  st->tune_ms_tiled = (float)est_tiled;
  st->tune_ms_ell = (float)est_ell;
  /* The per-class launches read short rows in pieces of a few bytes; they win where the long rows hold nearly
   * all the entries and the gathers are cheap (x stays in the caches, neighbouring lanes share lines). */
  int want_binned = 0;
  if (binned_ok && p->auto_algo == ASAMD_SPMV_MERGE && st->lines_per_entry_wave <= 0.25f) {
    /* rows of fewer than 128 entries hold at most this many entries (bin b: up to 2^b - 1 each) */
    double short_entries = 0.0;
    for (int b = 1; b < 8; ++b) short_entries += (double)st->hist[b] * (double)(((int64_t)1 << b) - 1);
    want_binned = short_entries <= 0.1 * (double)st->nnz;
  }
  /* Popular columns in LDS: where merge-path runs, the gathers weigh as much as the streams and reach beyond
   * what the L2s hold, and (the count decides, below) the columns that fit the table hold three entries in ten.
   * Power-law rows x R-MAT columns, fp32, 2.1 / 4.2 / 8.4 M rows (s = 0.30 / 0.38 / 0.45): 0.122 ms against
   * 0.117 ms for merge-path, 0.247 against 0.254, 0.526 against 0.580 (37.6 % of the entries from LDS). */
  int want_hot = 0;
  if (hot_ok && p->auto_algo == ASAMD_SPMV_MERGE) {
    const double vs = (double)p->val_size, nnz = (double)st->nnz;
    const double stream_ms = (nnz * (4.0 + vs) + ((double)st->m + 1.0) * 4.0 + ((double)st->n + (double)st->m) * vs) / 2.9e9;
    const double gather_ms = nnz * (double)st->lines_per_entry_wave * gather_ps((double)st->lines_per_entry_segment) * 1e-9;
    want_hot = gather_ms >= 0.5 * stream_ms && st->lines_per_entry_segment >= 0.42f;
    /* Few columns under rows of very different lengths: x is too large for the L1 and the kernel that holds it in
     * LDS walks long rows load by load; merge-path with its table holding all of x (or the better part) balances
     * them.  Rows of 4 and, every eighth, 256 entries, 4 M x 16 384: 0.57 -> 0.43 ms; 1 and, every 64th, 4 000,
     * 2 M x 16 384: 0.39 -> 0.25. */
    if (xlds_sized_x(p) && st->nnz >= (1 << 22) && !xlds_rows_regular(st)) want_hot = 1;
  }
  const char *ev = getenv("ALSPARSE_AMD_TUNE_PICK");
  int forced = -1;
  if (ev) {
    static const char *names[CAND_COUNT] = {"base", "tiled", "ell", "hot", "binned"};
    for (int c = 0; c < CAND_COUNT; ++c)
      if (!strcmp(ev, names[c])) forced = c;
  }
  int order[4] = {CAND_BASE, CAND_BASE, CAND_BASE, CAND_BASE};
  const int tiled_wins = tiled_ok && est_tiled < 0.9 * base, ell_wins = ell_ok && est_ell < 0.95 * base;
  int k = 0;
  if (forced > 0) {
    order[k++] = forced;
  } else if (forced < 0) {
    if (want_binned) order[k++] = CAND_BINNED;
    if (want_hot && !tiled_wins && !ell_wins) order[k++] = CAND_HOT;
    if (tiled_wins && ell_wins) {
      order[k++] = est_tiled < est_ell ? CAND_TILED : CAND_ELL;
      order[k++] = est_tiled < est_ell ? CAND_ELL : CAND_TILED;
    } else if (tiled_wins) {
      order[k++] = CAND_TILED;
    } else if (ell_wins) {
      order[k++] = CAND_ELL;
    }
  }
  hipError_t e = hipSuccess;
  for (int i = 0; i < k && e == hipSuccess; ++i) {
    int built = 0, algo = p->auto_algo;
    switch (order[i]) {
      case CAND_TILED:
        if (tiled_ok) e = build_tiled(stream, p, row_ptr, col_ind, val);
        built = st->tiled_built;
        algo = ASAMD_SPMV_TILED;
        break;
      case CAND_ELL:
        if (ell_ok) e = build_ell(stream, p, row_ptr, col_ind, val);
        built = st->ell_built;
        algo = ASAMD_SPMV_ELL;
        break;
      case CAND_HOT:
        if (hot_ok) e = build_hot(stream, p, row_ptr, col_ind, forced == CAND_HOT);
        built = st->hot_built;
        algo = ASAMD_SPMV_MERGE_HOT;
        break;
      case CAND_BINNED:
        if (binned_ok) e = build_binned(stream, p, row_ptr);
        built = st->binned_built;
        algo = ASAMD_SPMV_BINNED;
        break;
      default: break;
    }
    if (e == hipSuccess && built) {
      p->auto_algo = algo;
      st->algo = algo;
      break;
    }
  }
  return e;
}

/* the fingerprint of the values a copy set was taken from (set-up work: plan-owned scratch, not concurrent) */
static hipError_t first_fingerprint(hipStream_t stream, asamd_csr_plan *p, const void *val, int slot) {
  if (!p->st.value_check) return hipSuccess;
  hipError_t e = (hipError_t)asamd_value_guard(stream, val, (size_t)p->st.nnz * (size_t)p->val_size,
                                               p->st.value_check == 2, NULL, p->d_setup);
  if (e == hipSuccess) e = (hipError_t)asamd_value_guard_commit(stream, p->d_setup, p->d_fp + slot);
  return e;
}

static hipError_t plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, const int32_t *row_ptr,
                              const int32_t *col_ind, const void *val, int32_t base, int32_t dtype, int32_t trusted,
                              asamd_csr_plan **out) {
  if (!out || !row_ptr || m <= 0 || nnz < 0 || dtype < ASAMD_DTYPE_FLOAT || dtype > ASAMD_DTYPE_DOUBLE_COMPLEX)
    return hipErrorInvalidValue;
  const int val_size = kValSize[dtype];
  if (val && (uintptr_t)val % (size_t)val_size) return hipErrorInvalidValue;
  asamd_csr_plan *p = (asamd_csr_plan *)calloc(1, sizeof(*p));
  if (!p) return hipErrorOutOfMemory;
  asamd_csr_stats *st = &p->st;
  st->m = m;
  st->n = n;
  st->nnz = nnz;
  st->base = base;
  st->trusted = trusted ? 1 : 0;
  st->value_check = env_value_check();
  st->tune_mode = env_tune_model();
  p->dtype = dtype;
  p->val_size = val_size;
  p->watched = trusted == 3;

  hipError_t e = hipMalloc(&p->d_setup, SETUP_BYTES);
  if (e == hipSuccess) e = hipMalloc((void **)&p->d_fp, 3 * sizeof(uint64_t));
  int32_t h[ASAMD_ROW_STATS_WORDS];
  if (e == hipSuccess) e = (hipError_t)asamd_csr_row_stats(stream, m, row_ptr, (int32_t *)p->d_setup, h);
  if (e != hipSuccess) {
    asamd_csr_plan_destroy(p);
    return e;
  }
  st->min_len = h[0];
  st->max_len = h[1];
  st->first_offset = h[2] - base;
  st->const_len = h[0] == h[1] ? h[0] : -1;
  for (int b = 0; b < ASAMD_HIST_BINS; ++b) st->hist[b] = h[3 + b];

  const int64_t total = (int64_t)m + nnz;
  /* wider values take more LDS per item: fewer items keep more workgroups resident */
  p->merge_ipt = val_size >= 8 ? 4 : 8;
  const int want_ipt = env_int("ALSPARSE_AMD_MERGE_IPT", 0);
  if (want_ipt == 4 || want_ipt == 8 || (want_ipt == 16 && dtype <= ASAMD_DTYPE_DOUBLE)) p->merge_ipt = want_ipt;
  if (val_size == 16) p->merge_ipt = 4; /* the only instantiation for 16-byte values */
  const int merge_items = ASAMD_MERGE_THREADS * p->merge_ipt;
  const int64_t nb = (total + merge_items - 1) / merge_items;
  st->merge_blocks = (int)nb;
  choose_algo(p);

  if (st->trusted && st->first_offset == 0) {
    /* the structure is promised fixed: the merge-path coordinates are computed once */
    e = hipMalloc((void **)&p->d_block_row, ((size_t)nb + 1) * sizeof(int32_t));
    if (e == hipSuccess)
      e = (hipError_t)asamd_merge_partition(stream, m, nnz, row_ptr, base, (int)nb, merge_items, p->d_block_row);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
  }
  if (col_ind && nnz >= 4096 && st->trusted) {
    /* where the columns of neighbouring entries fall: two numbers for the record and for the model */
    float probe[2] = {0.f, 0.f};
    e = (hipError_t)asamd_csr_locality_probe(stream, nnz, base, val_size, col_ind, 64, p->d_setup, probe);
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
    st->lines_per_entry_wave = probe[0];
    st->lines_per_entry_segment = probe[1];
  }
  p->xlds_copy_wanted = val != NULL && env_int("ALSPARSE_AMD_XLDS_COPY", 1) > 0;
  if (col_ind && nnz > 0 && trusted != 3 && xlds_sliced_ok(p, trusted == 2, p->xlds_copy_wanted)) {
    /* x in LDS slice by slice, if the model expects it to beat the structural choice by a fifth (no probe: no
     * estimate of that choice, and no slices) */
    const int wanted = trusted == 2 || (st->lines_per_entry_wave > 0.f &&
                                        model_ms(p, ASAMD_SPMV_XLDS) < 0.9 * model_ms(p, p->auto_algo));
    if (wanted) {
      e = (hipError_t)asamd_xlds_build(stream, p->dtype, m, n, nnz, base, row_ptr, col_ind,
                                       p->xlds_copy_wanted ? val : NULL, &p->xlds);
      if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        e = hipSuccess;
      }
      if (e != hipSuccess) {
        asamd_csr_plan_destroy(p);
        return e;
      }
      if (p->xlds.seg && !p->xlds.val && p->xlds_copy_wanted && trusted != 2) {
        /* no room for the copy: the table alone, if it still pays */
        p->xlds_copy_wanted = 0;
        if (!xlds_sliced_ok(p, 0, 0) || !(model_ms(p, ASAMD_SPMV_XLDS) < 0.9 * model_ms(p, p->auto_algo)))
          asamd_xlds_free(&p->xlds);
      }
      st->xlds_slices = p->xlds.seg ? p->xlds.slices : 0;
      if (p->xlds.seg && trusted != 2) {
        p->auto_algo = p->struct_algo = ASAMD_SPMV_XLDS;
        st->algo = p->auto_algo;
      }
    }
  }
  if (col_ind && st->trusted && trusted != 3 && (p->auto_algo == ASAMD_SPMV_STREAM || (trusted == 2 && stream_ok(p))) &&
      (p->dtype == ASAMD_DTYPE_FLOAT || p->dtype == ASAMD_DTYPE_DOUBLE) && nnz >= 1 && st->first_offset == 0 &&
      (trusted == 2 || (double)nnz * (4.0 + val_size) + ((double)m + n) * val_size > 400.0e6) &&
      env_int("ALSPARSE_AMD_STREAM_NARROW", 1) > 0) {
    /* staged row blocks and a structure that stays: where every entry lies within 32 767 columns of its workgroup's
     * first row (a discretisation, a band) the kernel reads 16-bit distances instead of the column numbers.  Pays
     * on matrices well beyond the memory-side cache (256 MB): 27-point stencil on 160^3 points 0.204 -> 0.177 ms,
     * nothing on the 5-point Laplacian on 2048^2 (336 MB). */
    int32_t *too_far = (int32_t *)p->d_setup;
    int32_t h_far = 1;
    p->rel16_group = stream_group(p, 0);
    e = hipMalloc((void **)&p->d_rel16, ((size_t)nnz + 4) * sizeof(int16_t));
    if (e == hipSuccess) e = hipMemsetAsync(too_far, 0, sizeof(int32_t), stream);
    if (e == hipSuccess)
      e = (hipError_t)asamd_narrow_rel_columns(stream, m, nnz, base, p->rel16_group, row_ptr, col_ind, p->d_rel16, too_far);
    if (e == hipSuccess) e = hipMemcpyAsync(&h_far, too_far, sizeof(int32_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e == hipErrorOutOfMemory) (void)hipGetLastError();
    if (e == hipErrorOutOfMemory || (e == hipSuccess && h_far != 0)) {
      if (p->d_rel16) (void)hipFree(p->d_rel16);
      p->d_rel16 = NULL;
      e = hipSuccess;
    }
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
  }
  if (col_ind && val && nnz > 0) {
    /* trusted == 2: build every copy whatever the size and skip the timing
     * (lets small matrices exercise those kernels) */
    const int force = trusted == 2;
    /* trusted == 3: for a matrix that is WATCHED rather than promised fixed (asamd_csr_plan_csrmv_watched): the
     * tiled copy is the only one whose kernels a watcher can turn away */
    const int only_tiled = trusted == 3;
    const int tiled_ok = tiled_eligible(p, force), ell_ok = !only_tiled && ell_eligible(st, force);
    const int hot_ok = !only_tiled && hot_eligible(p, force), binned_ok = !only_tiled && binned_eligible(p, force);
    if (force) {
      if (binned_ok) e = build_binned(stream, p, row_ptr);
      if (e == hipSuccess && tiled_ok) e = build_tiled(stream, p, row_ptr, col_ind, val);
      if (e == hipSuccess && ell_ok) e = build_ell(stream, p, row_ptr, col_ind, val);
      if (e == hipSuccess && hot_ok) e = build_hot(stream, p, row_ptr, col_ind, 1);
    } else if (tiled_ok || ell_ok || hot_ok || binned_ok || structural_alternatives(p) ||
               p->auto_algo == ASAMD_SPMV_XLDS) {
      e = st->tune_mode ? model_copies(stream, p, row_ptr, col_ind, val, tiled_ok, ell_ok, hot_ok, binned_ok)
                        : tune_copies(stream, p, row_ptr, col_ind, val, tiled_ok, ell_ok, hot_ok, binned_ok);
    }
    if (e == hipErrorOutOfMemory) {
      (void)hipGetLastError(); /* the copies are optional: carry on without them */
      free_tiled(p);
      free_ell(p);
      free_hot(p);
      free_binned(p);
      if (p->auto_algo == ASAMD_SPMV_TILED || p->auto_algo == ASAMD_SPMV_ELL || p->auto_algo == ASAMD_SPMV_MERGE_HOT ||
          p->auto_algo == ASAMD_SPMV_BINNED)
        p->auto_algo = p->struct_algo;
      st->algo = p->auto_algo;
      e = hipSuccess;
    }
    if (e == hipSuccess && !force && p->xlds.seg && p->auto_algo != ASAMD_SPMV_XLDS) {
      /* another copy won against the column slices: their table and copy are not kept beside it */
      asamd_xlds_free(&p->xlds);
      st->xlds_slices = 0;
      if (p->struct_algo == ASAMD_SPMV_XLDS) p->struct_algo = p->plain_algo;
    }
    if (e == hipSuccess && has_value_copy(p)) {
      p->copy_val_src = val;
      e = first_fingerprint(stream, p, val, 0);
      if (e == hipSuccess) e = hipStreamSynchronize(stream);
    }
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
  }
  if (col_ind && st->trusted && trusted != 3 && (p->auto_algo == ASAMD_SPMV_XLDS || trusted == 2) && !p->xlds.seg &&
      n <= 65536 &&
      (p->dtype == ASAMD_DTYPE_FLOAT || p->dtype == ASAMD_DTYPE_DOUBLE) && nnz >= 4 && (int64_t)nnz >= 4 * (int64_t)m &&
      asamd_spmv_xlds_fits(p->dtype, n) && st->first_offset == 0 && env_int("ALSPARSE_AMD_XLDS_NARROW", 1) > 0) {
    /* x in LDS and a structure that stays: the kernel reads 16-bit column numbers (a quarter of an fp32 entry's
     * bytes less; 4 M x 32 768 x 16: 0.123 -> 0.109 ms, 262 144 x 30 000 x 400: 0.153 -> 0.137).  No room for them: the caller's columns serve. */
    e = hipMalloc((void **)&p->d_col16, ((size_t)nnz + 4) * sizeof(uint16_t));
    if (e == hipSuccess) e = (hipError_t)asamd_narrow_columns(stream, nnz, base, col_ind, p->d_col16);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e == hipErrorOutOfMemory) {
      (void)hipGetLastError();
      p->d_col16 = NULL;
      e = hipSuccess;
    }
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
  }
  if (p->d_rel16 && p->auto_algo != ASAMD_SPMV_STREAM && trusted != 2) {
    (void)hipFree(p->d_rel16); /* another family was kept */
    p->d_rel16 = NULL;
  }
  account(p);
  *out = p;
  return hipSuccess;
}

int asamd_csr_plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, const int32_t *row_ptr,
                          const int32_t *col_ind, const void *val, int32_t base, int32_t val_size, int32_t trusted,
                          asamd_csr_plan **out) {
  if (val_size != 4 && val_size != 8) return hipErrorInvalidValue;
  return plan_create(stream, m, n, nnz, row_ptr, col_ind, val, base,
                     val_size == 4 ? ASAMD_DTYPE_FLOAT : ASAMD_DTYPE_DOUBLE, trusted, out);
}

int asamd_csr_plan_create_dtype(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, const int32_t *row_ptr,
                                const int32_t *col_ind, const void *val, int32_t base, int32_t dtype, int32_t trusted,
                                asamd_csr_plan **out) {
  return plan_create(stream, m, n, nnz, row_ptr, col_ind, val, base, dtype, trusted, out);
}

void asamd_csr_plan_destroy(asamd_csr_plan *p) {
  if (!p) return;
  if (p->d_block_row) (void)hipFree(p->d_block_row);
  if (p->d_col16) (void)hipFree(p->d_col16);
  if (p->d_rel16) (void)hipFree(p->d_rel16);
  if (p->d_setup) (void)hipFree(p->d_setup);
  if (p->d_fp) (void)hipFree(p->d_fp);
  free_tiled(p);
  free_ell(p);
  free_hot(p);
  free_binned(p);
  asamd_xlds_free(&p->xlds);
  free_transpose(p, 0);
  free_transpose(p, 1);
  free(p);
}

/* CSR of A^T (which = 1: of A^H) with an analysis of its own. */
static hipError_t build_transpose(hipStream_t stream, asamd_csr_plan *p, const int32_t *rp, const int32_t *ci,
                                  const void *val, int which) {
  asamd_csr_stats *st = &p->st;
  asamd_trans_copy *t = &p->tr[which];
  hipError_t e = (hipError_t)asamd_transpose_build(stream, p->dtype, which == 1, st->m, st->n, st->nnz, st->base, rp, ci,
                                                   val, &t->t);
  if (e == hipSuccess)
    e = plan_create(stream, st->n, st->m, st->nnz, t->t.row_ptr, t->t.col_ind, t->t.val, 0, p->dtype, /*trusted=*/1,
                    &t->plan);
  if (e == hipSuccess) e = first_fingerprint(stream, p, val, 1 + which);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    free_transpose(p, which);
    return e;
  }
  t->val_src = val;
  st->transpose_built |= 1 << which;
  account(p);
  return hipSuccess;
}

static int build_transpose_any(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr, const int32_t *col_ind,
                               const void *val, int which) {
  if (!p || !row_ptr || !col_ind || !val || !p->st.trusted || p->st.n <= 0) return hipErrorInvalidValue;
  if (which == 1 && !is_complex(p)) return hipErrorInvalidValue;
  if (p->st.transpose_built & (1 << which)) return hipSuccess;
  if (p->st.nnz == 0) return hipSuccess;          /* the scatter route has nothing to add */
  if (p->st.first_offset != 0) return hipSuccess; /* no copy (csr2coo counts from position 0): the scatter route serves */
  return build_transpose(stream, p, row_ptr, col_ind, val, which);
}

int asamd_csr_plan_build_transpose(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr,
                                   const int32_t *col_ind, const void *val) {
  return build_transpose_any(stream, p, row_ptr, col_ind, val, 0);
}

int asamd_csr_plan_build_conj_transpose(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr,
                                        const int32_t *col_ind, const void *val) {
  return build_transpose_any(stream, p, row_ptr, col_ind, val, 1);
}

int asamd_csr_plan_set_lazy_transpose(asamd_csr_plan *p, int32_t on) {
  if (!p || !p->st.trusted) return hipErrorInvalidValue;
  p->lazy_transpose = on != 0;
  return hipSuccess;
}

const asamd_csr_stats *asamd_csr_plan_transpose_stats(const asamd_csr_plan *p) {
  if (!p) return NULL;
  if (p->tr[0].plan) return &p->tr[0].plan->st;
  return p->tr[1].plan ? &p->tr[1].plan->st : NULL;
}

int asamd_csr_plan_transpose_arrays(const asamd_csr_plan *p, int32_t conj, const int32_t **row_ptr,
                                    const int32_t **col_ind, const void **val) {
  if (!p || !row_ptr || !col_ind || !val) return hipErrorInvalidValue;
  const asamd_trans_copy *t = &p->tr[conj ? 1 : 0];
  if (!t->plan) return hipErrorInvalidValue;
  *row_ptr = t->t.row_ptr;
  *col_ind = t->t.col_ind;
  *val = t->t.val;
  return hipSuccess;
}

int asamd_csr_plan_refresh_values(hipStream_t stream, asamd_csr_plan *p, const int32_t *row_ptr,
                                  const int32_t *col_ind, const void *val) {
  if (!p || !row_ptr || !col_ind || !val || !p->st.trusted) return hipErrorInvalidValue;
  if ((uintptr_t)val % (size_t)p->val_size) return hipErrorInvalidValue;
  hipError_t e = refresh_main(stream, p, row_ptr, col_ind, val, NULL);
  if (e == hipSuccess && has_value_copy(p)) {
    p->copy_val_src = val;
    e = first_fingerprint(stream, p, val, 0);
  }
  for (int which = 0; which < 2 && e == hipSuccess; ++which) {
    if (!p->tr[which].plan) continue;
    e = refresh_trans(stream, p, which, val, NULL);
    p->tr[which].val_src = val;
    if (e == hipSuccess) e = first_fingerprint(stream, p, val, 1 + which);
  }
  return e;
}

const asamd_csr_stats *asamd_csr_plan_stats(const asamd_csr_plan *p) { return p ? &p->st : NULL; }

int asamd_csr_plan_set_algo(asamd_csr_plan *p, int32_t algo) {
  if (!p) return hipErrorInvalidValue;
  switch (algo) {
    case ASAMD_SPMV_AUTO:
      p->st.algo = p->auto_algo;
      return hipSuccess;
    case ASAMD_SPMV_ROWCONST:
      if (!rowconst_ok(p)) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_TILED:
      if (!p->st.tiled_built) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_STREAM:
      if (!stream_ok(p)) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_ELL:
      if (!p->st.ell_built) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_MERGE_HOT:
      if (!p->st.hot_built) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_BINNED:
      if (!p->st.binned_built) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_MERGE:
      if (p->st.first_offset != 0) return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_XLDS:
      if (!p->xlds.seg && (!asamd_spmv_xlds_fits(p->dtype, p->st.n) || p->st.first_offset != 0))
        return hipErrorInvalidValue;
      break;
    case ASAMD_SPMV_VECTOR:
    case ASAMD_SPMV_SCALAR:
      break;
    default:
      return hipErrorInvalidValue;
  }
  p->st.algo = algo;
  return hipSuccess;
}
