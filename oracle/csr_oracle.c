/* TEST INFRASTRUCTURE -- not part of the product.
 *
 * CPU restatement of the reference's algorithms for the CSR SpMV / SpMM path,
 * used only by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * as the checker / reported baseline.  libalpha_spblas.so never links, loads
 * or calls anything in this directory.
 *
 * Each function cites the reference file:line it follows (paths relative to
 * the AlphaSparse source tree).  Compiled twice:
 *   liboracle.so       -O2 -ffp-contract=off   reproducible rounding: the parity oracle
 *   liboracle_fast.so  -Ofast -fopenmp         how the reference builds its CPU kernels
 *                                              (Makefile:53,56,86): the timed baseline
 *
 * Pinning (tests/test_oracle_*.py): brute-force dense products in fp64 on tiny
 * matrices, scipy.sparse as an independent library routine, closed forms
 * (identity, diagonal, Laplacian times ones, alpha = 0, beta = 1), linearity
 * and row-splitting invariants, and -- where it builds -- bit-for-bit agreement
 * with the reference's own sources compiled into oracle/_ref/.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- *
 * Plain (serial) SpMV: src/plain/kernel/level2/mv/gemv/gemv_x_csr_plain.c:11-22
 *   y[r] *= beta; tmp = sum_{ai} val[ai]*x[col[ai]] left to right in type T;
 *   y[r] += alpha*tmp.   (madde is d += a*b, include/alphasparse/real_compute.h:41-42)
 * ------------------------------------------------------------------------- */
#define ORACLE_MV_PLAIN(NAME, T)                                                              \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const T *values, T alpha, const T *x, T beta, T *y) {   \
    for (int32_t r = 0; r < m; r++) {                                                         \
      y[r] *= beta;                                                                           \
      T tmp = 0;                                                                              \
      for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++) tmp += values[ai] * x[col_indx[ai]]; \
      y[r] += alpha * tmp;                                                                    \
    }                                                                                         \
  }
ORACLE_MV_PLAIN(oracle_s_csrmv_plain, float)
ORACLE_MV_PLAIN(oracle_d_csrmv_plain, double)

/* ------------------------------------------------------------------------- *
 * Plain transposed SpMV, y = alpha*A^T*x + beta*y (x has m entries, y has n):
 * src/plain/kernel/level2/mv/gemv/gemv_x_csr_trans_plain.c:10-24
 *   y[j] *= beta for j < n; per entry, row by row: val = alpha*values[ai];
 *   y[col] += val*x[row].
 * ------------------------------------------------------------------------- */
#define ORACLE_MV_TRANS_PLAIN(NAME, T)                                                        \
  void NAME(int32_t m, int32_t n, const int32_t *rows_start, const int32_t *rows_end,        \
            const int32_t *col_indx, const T *values, T alpha, const T *x, T beta, T *y) {   \
    for (int32_t j = 0; j < n; ++j) y[j] *= beta;                                             \
    for (int32_t i = 0; i < m; i++) {                                                         \
      for (int32_t ai = rows_start[i]; ai < rows_end[i]; ai++) {                              \
        T val = alpha * values[ai];                                                           \
        y[col_indx[ai]] += val * x[i];                                                        \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_MV_TRANS_PLAIN(oracle_s_csrmv_trans_plain, float)
ORACLE_MV_TRANS_PLAIN(oracle_d_csrmv_trans_plain, double)

/* Same product with every row accumulated in fp64 whatever T is: separates the
 * oracle's own rounding noise from a real error on long rows.  Not a
 * restatement of reference code. */
#define ORACLE_MV_F64ACC(NAME, T)                                                             \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const T *values, double alpha, const T *x, double beta, \
            const T *y_in, double *y_out) {                                                   \
    _Pragma("omp parallel for schedule(dynamic, 1024)")                                       \
    for (int32_t r = 0; r < m; r++) {                                                         \
      double tmp = 0;                                                                         \
      for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++)                                \
        tmp += (double)values[ai] * (double)x[col_indx[ai]];                                  \
      y_out[r] = beta * (double)y_in[r] + alpha * tmp;                                        \
    }                                                                                         \
  }
ORACLE_MV_F64ACC(oracle_s_csrmv_f64acc, float)
ORACLE_MV_F64ACC(oracle_d_csrmv_f64acc, double)

/* ------------------------------------------------------------------------- *
 * nnz-balanced row partition: src/util/partition.c:46-61 (lower_bound_int) and
 * :79-92 (balanced_partition_row_by_nnz).  acc is rows_end (inclusive prefix).
 * ------------------------------------------------------------------------- */
static int32_t oracle_lower_bound(const int32_t *t, int32_t l, int32_t r, int32_t value) {
  while (r > l) {
    int32_t m = (l + r) / 2;
    if (t[m] < value) l = m + 1;
    else r = m;
  }
  return l;
}

void oracle_partition_rows_by_nnz(const int32_t *acc, int32_t rows, int32_t num_threads,
                                  int32_t *partition) {
  int32_t nnz = acc[rows - 1];
  int32_t ave = nnz / num_threads;
  partition[0] = 0;
  for (int32_t i = 1; i < num_threads; i++)
    partition[i] = oracle_lower_bound(acc, 0, rows - 1, ave * i);
  partition[num_threads] = rows;
}

/* ------------------------------------------------------------------------- *
 * OpenMP SpMV: src/kernel/x86_64/level2/mv/gemv/gemv_x_csr.c
 *   :129-153 four partial sums over i mod 4, tail into the first, combined as
 *            (t0+t1)+(t2+t3);
 *   :155-182 per row: y *= beta; y += alpha*tmp;
 *   :184-208 rows split across threads by nnz.
 * num_threads <= 0 means all cores (src/util/thread.c:31-38).
 * ------------------------------------------------------------------------- */
#define ORACLE_MV_OMP(NAME, T)                                                                \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const T *values, T alpha, const T *x, T beta, T *y,     \
            int32_t num_threads) {                                                            \
    if (num_threads <= 0) num_threads = oracle_num_procs();                                   \
    int32_t *partition = (int32_t *)malloc(sizeof(int32_t) * (size_t)(num_threads + 1));      \
    oracle_partition_rows_by_nnz(rows_end, m, num_threads, partition);                        \
    _Pragma("omp parallel num_threads(num_threads)")                                          \
    {                                                                                         \
      int tid = oracle_thread_id();                                                           \
      for (int32_t i = partition[tid]; i < partition[tid + 1]; i++) {                         \
        const int32_t pks = rows_start[i], pkl = rows_end[i] - pks;                           \
        const T *v = values + pks;                                                            \
        const int32_t *ix = col_indx + pks;                                                   \
        const int32_t ns4 = (pkl >> 2) << 2;                                                  \
        T t0 = 0, t1 = 0, t2 = 0, t3 = 0;                                                     \
        int32_t k;                                                                            \
        for (k = 0; k < ns4; k += 4) {                                                        \
          t0 += v[k] * x[ix[k]];                                                              \
          t1 += v[k + 1] * x[ix[k + 1]];                                                      \
          t2 += v[k + 2] * x[ix[k + 2]];                                                      \
          t3 += v[k + 3] * x[ix[k + 3]];                                                      \
        }                                                                                     \
        for (; k < pkl; ++k) t0 += v[k] * x[ix[k]];                                           \
        t0 += t1;                                                                             \
        t2 += t3;                                                                             \
        t0 += t2;                                                                             \
        y[i] *= beta;                                                                         \
        y[i] += alpha * t0;                                                                   \
      }                                                                                       \
    }                                                                                         \
    free(partition);                                                                          \
  }

int32_t oracle_num_procs(void) {
#ifdef _OPENMP
  return omp_get_num_procs();
#else
  return 1;
#endif
}
static int oracle_thread_id(void) {
#ifdef _OPENMP
  return omp_get_thread_num();
#else
  return 0;
#endif
}
ORACLE_MV_OMP(oracle_s_csrmv_omp, float)
ORACLE_MV_OMP(oracle_d_csrmv_omp, double)

/* ------------------------------------------------------------------------- *
 * Plain SpMM, row-major dense operands:
 *   src/plain/kernel/level3/mm/gemm/gemm_x_csr_row_plain.c:6-21
 *   Y[r,:] *= beta; per entry v = alpha*val; Y[r,c] += v*X[col,c].
 * Plain SpMM, column-major dense operands:
 *   src/plain/kernel/level3/mm/gemm/gemm_x_csr_col_plain.c:6-19
 *   ctmp = sum val*X[col,cc]; Y[cr,cc] *= beta; Y[cr,cc] += alpha*ctmp.
 * index2(y, x, ld) = x + ld*y (include/alphasparse/util/...): row-major (r,c)
 * is c + ld*r, column-major (r,c) is r + ld*c.
 * ------------------------------------------------------------------------- */
#define ORACLE_MM_ROW(NAME, T, PRAGMA)                                                        \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const T *values, T alpha, const T *x, int32_t columns,  \
            int32_t ldx, T beta, T *y, int32_t ldy) {                                         \
    PRAGMA                                                                                    \
    for (int32_t r = 0; r < m; ++r) {                                                         \
      T *Y = &y[(size_t)r * ldy];                                                             \
      for (int32_t c = 0; c < columns; c++) Y[c] *= beta;                                     \
      for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++) {                              \
        T val = alpha * values[ai];                                                           \
        const T *X = &x[(size_t)col_indx[ai] * ldx];                                          \
        for (int32_t c = 0; c < columns; ++c) Y[c] += val * X[c];                             \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_MM_ROW(oracle_s_csrmm_row_plain, float, )
ORACLE_MM_ROW(oracle_d_csrmm_row_plain, double, )
/* OpenMP variant: src/kernel/x86_64/level3/mm/gemm/gemm_x_csr_row.c:6-26
 * (omp parallel for over rows, default static schedule) */
ORACLE_MM_ROW(oracle_s_csrmm_row_omp, float, _Pragma("omp parallel for"))
ORACLE_MM_ROW(oracle_d_csrmm_row_omp, double, _Pragma("omp parallel for"))

#define ORACLE_MM_COL(NAME, T)                                                                \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const T *values, T alpha, const T *x, int32_t columns,  \
            int32_t ldx, T beta, T *y, int32_t ldy) {                                         \
    for (int32_t cc = 0; cc < columns; ++cc) {                                                \
      for (int32_t cr = 0; cr < m; ++cr) {                                                    \
        T ctmp = 0;                                                                           \
        for (int32_t ai = rows_start[cr]; ai < rows_end[cr]; ++ai)                            \
          ctmp += values[ai] * x[(size_t)cc * ldx + col_indx[ai]];                            \
        y[(size_t)cc * ldy + cr] *= beta;                                                     \
        y[(size_t)cc * ldy + cr] += alpha * ctmp;                                             \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_MM_COL(oracle_s_csrmm_col_plain, float)
ORACLE_MM_COL(oracle_d_csrmm_col_plain, double)

/* ------------------------------------------------------------------------- *
 * CSR -> COO row indices: src/core/format/convert_coo_x_csr.c:30-37
 * ------------------------------------------------------------------------- */
void oracle_csr2coo(int32_t m, const int32_t *row_ptr, int32_t base, int32_t *coo_row) {
  for (int32_t r = 0; r < m; r++)
    for (int32_t ai = row_ptr[r] - base; ai < row_ptr[r + 1] - base; ai++) coo_row[ai] = r + base;
}

/* ------------------------------------------------------------------------- *
 * CSR -> ELL: src/core/format/convert_ell_x_coo.c
 *   :46-52 width = longest row; :53-56 width*m >= 2^31 is fatal (-1 here);
 *   :59-60 arrays zero-filled; :67-79 slot i of row j at [i*m + j].
 * ------------------------------------------------------------------------- */
int32_t oracle_csr2ell_width(int32_t m, const int32_t *row_ptr) {
  int32_t ld = 0;
  for (int32_t i = 0; i < m; i++) {
    int32_t n = row_ptr[i + 1] - row_ptr[i];
    ld = ld > n ? ld : n;
  }
  return ld;
}

#define ORACLE_CSR2ELL(NAME, T)                                                               \
  int32_t NAME(int32_t m, const int32_t *row_ptr, const int32_t *col_indx, const T *values,  \
               int32_t csr_base, int32_t ell_base, int32_t ld, T *ell_val, int32_t *ell_col) { \
    if ((uint64_t)ld * (uint64_t)m >= ((uint64_t)1 << 31)) return -1;                         \
    for (size_t k = 0; k < (size_t)ld * m; ++k) {                                             \
      ell_val[k] = 0;                                                                         \
      ell_col[k] = ell_base;                                                                  \
    }                                                                                         \
    for (int32_t i = 0; i < ld; i++) {                                                        \
      for (int32_t j = 0; j < m; j++) {                                                       \
        int32_t rs = row_ptr[j] - csr_base, re = row_ptr[j + 1] - csr_base;                   \
        if (rs + i < re) {                                                                    \
          ell_val[(size_t)i * m + j] = values[rs + i];                                        \
          ell_col[(size_t)i * m + j] = col_indx[rs + i] - csr_base + ell_base;                \
        }                                                                                     \
      }                                                                                       \
    }                                                                                         \
    return 0;                                                                                 \
  }
ORACLE_CSR2ELL(oracle_s_csr2ell, float)
ORACLE_CSR2ELL(oracle_d_csr2ell, double)

/* ------------------------------------------------------------------------- *
 * COO SpMV: src/plain/kernel/level2/mv/gemv/gemv_x_coo_plain.c:11-24
 *   y[i] *= beta for all i; then per entry, in storage order,
 *   v = val*x[col]; y[row] += alpha*v.   Indices zero-based.
 * ------------------------------------------------------------------------- */
#define ORACLE_COOMV(NAME, T)                                                                 \
  void NAME(int32_t m, int32_t nnz, const int32_t *row_indx, const int32_t *col_indx,        \
            const T *values, T alpha, const T *x, T beta, T *y) {                            \
    for (int32_t i = 0; i < m; i++) y[i] *= beta;                                             \
    for (int32_t i = 0; i < nnz; i++) {                                                       \
      T v = values[i] * x[col_indx[i]];                                                       \
      y[row_indx[i]] += alpha * v;                                                            \
    }                                                                                         \
  }
ORACLE_COOMV(oracle_s_coomv_plain, float)
ORACLE_COOMV(oracle_d_coomv_plain, double)

/* ------------------------------------------------------------------------- *
 * ELL SpMV: src/kernel/dcu/level2/mv/dcu_gemv_x_ell.cpp:22-42 (the reference has
 * no CPU kernel for this format; this follows its device kernel).  Per row ar:
 *   sum = 0; for slot i: idx = m*i + ar, col = ell_col[idx]; if (col < n)
 *   sum = fma(ell_val[idx], x[col], sum)   (device madde is an fma,
 *   include/alphasparse/real_compute.h:37-39); y[ar] = beta*y[ar] + alpha*sum.
 * Indices zero-based; a negative index is not guarded in the reference and is
 * skipped here.
 * ------------------------------------------------------------------------- */
#define ORACLE_ELLMV(NAME, T, FMA)                                                            \
  void NAME(int32_t m, int32_t n, T alpha, const T *ell_val, const int32_t *ell_col,         \
            int32_t width, const T *x, T beta, T *y) {                                        \
    for (int32_t ar = 0; ar < m; ar++) {                                                      \
      T sum = 0;                                                                              \
      for (int32_t i = 0; i < width; i++) {                                                   \
        size_t idx = (size_t)m * i + ar;                                                      \
        int32_t col = ell_col[idx];                                                           \
        if (col >= 0 && col < n) sum = FMA(ell_val[idx], x[col], sum);                        \
      }                                                                                       \
      T left = beta * y[ar], right = alpha * sum;                                             \
      y[ar] = left + right;                                                                   \
    }                                                                                         \
  }
ORACLE_ELLMV(oracle_s_ellmv, float, fmaf)
ORACLE_ELLMV(oracle_d_ellmv, double, fma)

/* ------------------------------------------------------------------------- *
 * Parity metric.  For every row i, with all sums accumulated in fp64,
 *     strict_i = |y_test[i] - y_ref[i]| / (|alpha| * sum_j |a_ij * x_j|)
 *     full_i   = |y_test[i] - y_ref[i]| / (|alpha| * sum_j |a_ij * x_j| + |beta * y0[i]|)
 * `strict` is the criterion as stated for the benchmark configurations; `full`
 * adds the magnitude of the beta*y term, whose rounding (in the reference's
 * kernels as much as in any other) is relative to |beta*y| and not to the
 * products, so that it stays meaningful for rows whose products are tiny next
 * to beta*y.  With beta == 0 (or y0 == NULL) the two coincide.  Rows whose
 * strict denominator is 0 must match y_ref exactly.
 * Returns the worst full_i; *worst_strict the worst strict_i, *worst_row the
 * row of the worst full_i, *zero_den_mismatch the number of zero-denominator
 * rows that differ.  *ref_check_ratio is the reference's own statistic,
 * src/util/check.c:701-737 (check_s) / :739-776 (check_d): max|a-b| / max|b|.
 * ------------------------------------------------------------------------- */
#define ORACLE_MV_ERR(NAME, T)                                                                \
  double NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                 \
              const int32_t *col_indx, const T *values, double alpha, const T *x,            \
              double beta, const T *y0, const T *y_test, const T *y_ref, int64_t *worst_row, \
              int64_t *zero_den_mismatch, double *ref_check_ratio, double *worst_strict) {    \
    double worst = 0, wstrict = 0, maxdiff = 0, maxref = 0;                                   \
    int64_t wrow = -1, zbad = 0;                                                              \
    _Pragma("omp parallel")                                                                   \
    {                                                                                         \
      double lw = 0, ls = 0, ld = 0, lr = 0;                                                  \
      int64_t lrow = -1, lz = 0;                                                              \
      _Pragma("omp for schedule(dynamic, 4096)")                                              \
      for (int32_t r = 0; r < m; r++) {                                                       \
        double den = 0;                                                                       \
        for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++)                              \
          den += fabs((double)values[ai] * (double)x[col_indx[ai]]);                          \
        den *= fabs(alpha);                                                                   \
        const double diff = fabs((double)y_test[r] - (double)y_ref[r]);                       \
        if (diff > ld) ld = diff;                                                             \
        if (fabs((double)y_ref[r]) > lr) lr = fabs((double)y_ref[r]);                         \
        if (den == 0) {                                                                       \
          if (!(diff == 0)) lz++;                                                             \
        } else {                                                                              \
          double e = diff / den;                                                              \
          if (e != e) e = INFINITY;                                                           \
          if (e > ls) ls = e;                                                                 \
          const double full = den + (y0 ? fabs(beta * (double)y0[r]) : 0.0);                  \
          e = diff / full;                                                                    \
          if (e != e) e = INFINITY;                                                           \
          if (e > lw) {                                                                       \
            lw = e;                                                                           \
            lrow = r;                                                                         \
          }                                                                                   \
        }                                                                                     \
      }                                                                                       \
      _Pragma("omp critical")                                                                 \
      {                                                                                       \
        if (lw > worst) { worst = lw; wrow = lrow; }                                          \
        if (ls > wstrict) wstrict = ls;                                                       \
        if (ld > maxdiff) maxdiff = ld;                                                       \
        if (lr > maxref) maxref = lr;                                                         \
        zbad += lz;                                                                           \
      }                                                                                       \
    }                                                                                         \
    if (worst_row) *worst_row = wrow;                                                         \
    if (zero_den_mismatch) *zero_den_mismatch = zbad;                                         \
    if (ref_check_ratio) *ref_check_ratio = maxref > 0 ? maxdiff / maxref : maxdiff;          \
    if (worst_strict) *worst_strict = wstrict;                                                \
    return worst;                                                                             \
  }
ORACLE_MV_ERR(oracle_s_csrmv_err, float)
ORACLE_MV_ERR(oracle_d_csrmv_err, double)

/* Same two metrics per element (i, c) of C for SpMM with strided dense
 * operands: element (r, c) of B at B[r*sbr + c*sbc], of C (c0, c_test, c_ref
 * alike) at [r*scr + c*scc]. */
#define ORACLE_MM_ERR(NAME, T)                                                                \
  double NAME(int32_t m, int32_t n, const int32_t *rows_start, const int32_t *rows_end,      \
              const int32_t *col_indx, const T *values, double alpha, const T *B, int64_t sbr, \
              int64_t sbc, double beta, const T *c0, const T *c_test, const T *c_ref,        \
              int64_t scr, int64_t scc, int64_t *zero_den_mismatch, double *worst_strict) {   \
    double worst = 0, wstrict = 0;                                                            \
    int64_t zbad = 0;                                                                         \
    _Pragma("omp parallel for schedule(dynamic, 256) reduction(max : worst, wstrict) reduction(+ : zbad)") \
    for (int32_t r = 0; r < m; r++) {                                                         \
      for (int32_t c = 0; c < n; c++) {                                                       \
        double den = 0;                                                                       \
        for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++)                              \
          den += fabs((double)values[ai] * (double)B[(int64_t)col_indx[ai] * sbr + c * sbc]); \
        den *= fabs(alpha);                                                                   \
        const int64_t o = (int64_t)r * scr + (int64_t)c * scc;                                \
        const double diff = fabs((double)c_test[o] - (double)c_ref[o]);                       \
        if (den == 0) {                                                                       \
          if (!(diff == 0)) zbad++;                                                           \
        } else {                                                                              \
          double e = diff / den;                                                              \
          if (e != e) e = INFINITY;                                                           \
          if (e > wstrict) wstrict = e;                                                       \
          e = diff / (den + (c0 ? fabs(beta * (double)c0[o]) : 0.0));                         \
          if (e != e) e = INFINITY;                                                           \
          if (e > worst) worst = e;                                                           \
        }                                                                                     \
      }                                                                                       \
    }                                                                                         \
    if (zero_den_mismatch) *zero_den_mismatch = zbad;                                         \
    if (worst_strict) *worst_strict = wstrict;                                                \
    return worst;                                                                             \
  }
ORACLE_MM_ERR(oracle_s_csrmm_err, float)
ORACLE_MM_ERR(oracle_d_csrmm_err, double)
