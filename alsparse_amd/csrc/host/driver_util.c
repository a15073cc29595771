/* Helpers that the reference's CPU test programs (test/arm/mv_?_csr_arm_test.c and their kin) call
 * around alphasparse_?_mv / _mm and their _plain variants: wall-clock timers, operation counts and the
 * norm-scaled residual checks.  Own text after the behaviour of src/util/timer.c, src/util/analysis.c,
 * src/util/check.c:7-57, :218-345 and src/util/norm.c of the reference. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/time.h>

#include "internal.h"

/* ---- timers: src/util/timer.c:14-58 ------------------------------------------------------------ */
double alpha_timing_wtime(void) {
  struct timeval t;
  gettimeofday(&t, NULL);
  return (double)t.tv_sec + (double)t.tv_usec / 1e6;
}

void alpha_timing_start(alpha_timer_t *timer) { timer->start = alpha_timing_wtime(); }

void alpha_timing_end(alpha_timer_t *timer) { timer->end = alpha_timing_wtime(); }

double alpha_timing_elapsed_time(const alpha_timer_t *timer) { return timer->end - timer->start; }

double alpha_timing_gflops(const alpha_timer_t *timer, int64_t operations) {
  return (double)operations * 1e-9 / alpha_timing_elapsed_time(timer);
}

void alpha_timing_elaped_time_print(const alpha_timer_t *timer, const char *name) {
  printf("%s elasped time : %lf[sec]\n", name, alpha_timing_elapsed_time(timer));
}

void alpha_timing_gflops_print(const alpha_timer_t *timer, int64_t operations, const char *name) {
  printf("%s gflops : %lf\n", name, alpha_timing_gflops(timer, operations));
}

/* src/util/malloc.c:50-61 sweeps a buffer larger than the CPU's last-level cache; the multiplies of
 * this library run on the GPU, whose caches a host sweep does not reach: nothing to do. */
void alpha_clear_cache(void) {}

/* ---- operation counts: src/util/analysis.c:8-56, :58-153 --------------------------------------- */
void alphasparse_nnz_counter_coo(const ALPHA_INT *row_indx, const ALPHA_INT *col_indx, const ALPHA_INT nnz,
                                 ALPHA_INT *lo_p, ALPHA_INT *diag_p, ALPHA_INT *hi_p) {
  ALPHA_INT lo = 0, diag = 0, hi = 0;
  for (ALPHA_INT i = 0; i < nnz; ++i) {
    if (row_indx[i] < col_indx[i]) ++hi;
    else if (row_indx[i] > col_indx[i]) ++lo;
    else ++diag;
  }
  *lo_p = lo;
  *diag_p = diag;
  *hi_p = hi;
}

/* entries that take part in the product for the descriptor's matrix type */
static int64_t counted_entries(ALPHA_INT rows, ALPHA_INT lo, ALPHA_INT diag, ALPHA_INT hi,
                               alphasparse_operation_t operation, struct alpha_matrix_descr descr) {
  const int64_t d = descr.diag == ALPHA_SPARSE_DIAG_UNIT ? rows : diag;
  switch (descr.type) {
    case ALPHA_SPARSE_MATRIX_TYPE_GENERAL:
      return (int64_t)lo + diag + hi;
    case ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC:
    case ALPHA_SPARSE_MATRIX_TYPE_HERMITIAN:
      return (descr.mode == ALPHA_SPARSE_FILL_MODE_LOWER ? lo : hi) + d;
    case ALPHA_SPARSE_MATRIX_TYPE_TRIANGULAR: {
      const int lower = (descr.mode == ALPHA_SPARSE_FILL_MODE_LOWER) ==
                        (operation == ALPHA_SPARSE_OPERATION_NON_TRANSPOSE);
      return (lower ? lo : hi) + d;
    }
    case ALPHA_SPARSE_MATRIX_TYPE_DIAGONAL:
      return d;
    default:
      return 0;
  }
}

ALPHA_INT64 alphasparse_operations_mm(const ALPHA_INT rows, const ALPHA_INT cols, const ALPHA_INT lo,
                                      const ALPHA_INT diag, const ALPHA_INT hi,
                                      const alphasparse_operation_t operation,
                                      const struct alpha_matrix_descr descr, const ALPHA_INT columns,
                                      const alphasparse_datatype_t datatype) {
  (void)cols;
  const int cx = datatype == ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX || datatype == ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX;
  const int64_t mul = cx ? 7 : 1, add = cx ? 2 : 1, madd = cx ? 9 : 2; /* as the reference weighs them */
  const int64_t nnz = counted_entries(rows, lo, diag, hi, operation, descr);
  return (nnz * madd + (int64_t)rows * (2 * mul + add)) * columns;
}

ALPHA_INT64 alphasparse_operations_mv(const ALPHA_INT rows, const ALPHA_INT cols, const ALPHA_INT lo,
                                      const ALPHA_INT diag, const ALPHA_INT hi,
                                      const alphasparse_operation_t operation,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_datatype_t datatype) {
  return alphasparse_operations_mm(rows, cols, lo, diag, hi, operation, descr, 1, datatype);
}

/* ---- residual checks ------------------------------------------------------------------------------
 * resid = ||answer - result|| / (max(||A||_1, 1) max(||x||, 1) max(||result||, 1) eps max(m, k[, columns]))
 * must not exceed 50 (THRESH, include/alphasparse/util/check.h:39); eps is ten times the machine
 * epsilon found by halving (src/util/norm.c:20-32); vectors in the max norm, dense matrices in the
 * 1-norm, complex numbers as |re| + |im|; ||x|| and ||result|| are scaled by alpha / beta (their real
 * parts for complex types) when those exceed 1 in magnitude.  The matrix is read again from
 * --data-file.  Matrix types other than GENERAL are weighed with the general 1-norm here. */
static double ten_eps(int is_double) { return is_double ? 10.0 * 0x1p-53 : 10.0 * 0x1p-24; }

/* components per value: 1 for real types, 2 for complex ones; all data viewed as arrays of reals */
static double get(const void *p, size_t i, int is_double) {
  return is_double ? ((const double *)p)[i] : (double)((const float *)p)[i];
}

static double elem_abs(const void *p, size_t i, int comps, int is_double) {
  double s = 0;
  for (int c = 0; c < comps; ++c) s += fabs(get(p, i * comps + c, is_double));
  return s;
}

static double elem_diff(const void *a, const void *b, size_t ia, size_t ib, int comps, int is_double) {
  double s = 0;
  for (int c = 0; c < comps; ++c) s += fabs(get(a, ia * comps + c, is_double) - get(b, ib * comps + c, is_double));
  return s;
}

static double matrix_norm1(ALPHA_INT cols, ALPHA_INT nnz, const ALPHA_INT *col_indx, const void *val, int comps,
                           int is_double) {
  double *sum = (double *)calloc((size_t)(cols > 0 ? cols : 1), sizeof(double));
  double best = 0;
  if (!sum) return 0;
  for (ALPHA_INT i = 0; i < nnz; ++i) sum[col_indx[i]] += elem_abs(val, (size_t)i, comps, is_double);
  for (ALPHA_INT c = 0; c < cols; ++c)
    if (sum[c] > best) best = sum[c];
  free(sum);
  return best;
}

/* the matrix named by --data-file in the given value type: 1-norm and shape */
static double file_norm1(int argc, const char *argv[], int comps, int is_double, ALPHA_INT *m, ALPHA_INT *k,
                         ALPHA_INT *nnz) {
  const char *file = args_get_data_file(argc, argv);
  ALPHA_INT *ri = NULL, *ci = NULL;
  void *val = NULL;
  if (comps == 1 && !is_double) alpha_read_coo(file, m, k, nnz, &ri, &ci, (float **)&val);
  else if (comps == 1) alpha_read_coo_d(file, m, k, nnz, &ri, &ci, (double **)&val);
  else if (!is_double) alpha_read_coo_c(file, m, k, nnz, &ri, &ci, (ALPHA_Complex8 **)&val);
  else alpha_read_coo_z(file, m, k, nnz, &ri, &ci, (ALPHA_Complex16 **)&val);
  const double n1 = matrix_norm1(*k, *nnz, ci, val, comps, is_double);
  alpha_free(ri);
  alpha_free(ci);
  alpha_free(val);
  return n1;
}

static int verdict(double normD, double normX, double normY, double normA, double eps, ALPHA_INT nnz, ALPHA_INT m,
                   ALPHA_INT k, double size) {
  const double one = 1.0;
  const double resid = normD / (fmax(normA, one) * fmax(normX, one) * fmax(normY, one) * eps * size);
  printf("normD : %.16f, normX : %.16f, normY : %.16f, normA : %.16f, episilon : %.16f, nnz : %d, row : %d, col : %d\n",
         normD, normX, normY, normA, eps, nnz, m, k);
  if (!(resid <= 50.0)) {
    printf("error,%.16f\n", resid);
    return -1;
  }
  printf("correct,%.16f\n", resid);
  return 0;
}

static int check_l2(const void *answer, size_t answer_size, const void *result, size_t result_size, const void *x,
                    double alpha_re, double beta_re, int argc, const char *argv[], int comps, int is_double) {
  if (answer_size != result_size) {
    printf("answer_size ans result_size is not equal (%zu %zu)\n", answer_size, result_size);
    return -1;
  }
  ALPHA_INT m = 0, k = 0, nnz = 0;
  const double normA = file_norm1(argc, argv, comps, is_double, &m, &k, &nnz);
  const alphasparse_operation_t transA = alpha_args_get_transA(argc, argv);
  const size_t size_x = transA == ALPHA_SPARSE_OPERATION_NON_TRANSPOSE ? (size_t)k : (size_t)m;
  double normD = 0, normX = 0, normY = 0;
  for (size_t i = 0; i < answer_size; ++i) {
    normD = fmax(normD, elem_diff(answer, result, i, i, comps, is_double));
    normY = fmax(normY, elem_abs(result, i, comps, is_double));
  }
  for (size_t i = 0; i < size_x; ++i) normX = fmax(normX, elem_abs(x, i, comps, is_double));
  if (fabs(alpha_re) > 1.0) normX *= alpha_re;
  if (fabs(beta_re) > 1.0) normY *= beta_re;
  return verdict(normD, normX, normY, normA, ten_eps(is_double), nnz, m, k, (double)(m > k ? m : k));
}

/* column sums of |.| over a rows x cols dense matrix with leading dimension ld, largest one */
static double dense_norm1(ALPHA_INT rows, ALPHA_INT cols, const void *a, ALPHA_INT lda, const void *b, ALPHA_INT ldb,
                          alphasparse_layout_t layout, int comps, int is_double) {
  double best = 0;
  const int rm = layout == ALPHA_SPARSE_LAYOUT_ROW_MAJOR;
  for (ALPHA_INT c = 0; c < cols; ++c) {
    double t = 0;
    for (ALPHA_INT r = 0; r < rows; ++r) {
      const size_t ia = rm ? (size_t)r * lda + c : (size_t)c * lda + r;
      const size_t ib = rm ? (size_t)r * ldb + c : (size_t)c * ldb + r;
      t += b ? elem_diff(a, b, ia, ib, comps, is_double) : elem_abs(a, ia, comps, is_double);
    }
    if (t > best) best = t;
  }
  return best;
}

static int check_l3(const void *answer, ALPHA_INT ldans, size_t answer_size, const void *result, ALPHA_INT ldres,
                    size_t result_size, const void *x, ALPHA_INT ldx, ALPHA_INT ldy, int argc, const char *argv[],
                    int comps, int is_double) {
  if (answer_size != result_size) {
    printf("answer_size ans result_size is not equal (%zu %zu)\n", answer_size, result_size);
    return -1;
  }
  if (args_get_data_file(argc, argv)[0] == '\0') {
    printf("check: only the --data-file form (sparse times dense) is supported\n");
    return -1;
  }
  ALPHA_INT m = 0, k = 0, nnz = 0;
  const double normA = file_norm1(argc, argv, comps, is_double, &m, &k, &nnz);
  const alphasparse_operation_t transA = alpha_args_get_transA(argc, argv);
  const alphasparse_layout_t layout = alpha_args_get_layout(argc, argv);
  const ALPHA_INT columns = args_get_columns(argc, argv, k);
  const int tr = transA != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
  const ALPHA_INT rowsx = tr ? m : k, rowsy = tr ? k : m;
  const double normD = dense_norm1(rowsy, columns, answer, ldans, result, ldres, layout, comps, is_double);
  const double normX = dense_norm1(rowsx, columns, x, ldx, NULL, 0, layout, comps, is_double);
  const double normY = dense_norm1(rowsy, columns, result, ldy, NULL, 0, layout, comps, is_double);
  const ALPHA_INT mk = m > k ? m : k;
  return verdict(normD, normX, normY, normA, ten_eps(is_double), nnz, m, k, (double)(mk > columns ? mk : columns));
}

#define ASAMD_CHECKS(S, T, COMPS, IS_DOUBLE, RE)                                                              \
  int check_##S##_l2(const T *answer_data, size_t answer_size, const T *result_data, size_t result_size,     \
                     const T *x, const T *y, const T alpha, const T beta, int argc, const char *argv[]) {     \
    (void)y;                                                                                                  \
    return check_l2(answer_data, answer_size, result_data, result_size, x, RE(alpha), RE(beta), argc, argv,   \
                    COMPS, IS_DOUBLE);                                                                        \
  }                                                                                                           \
  int check_##S##_l3(const T *answer_data, const ALPHA_INT ldans, size_t answer_size, const T *result_data,  \
                     const ALPHA_INT ldres, size_t result_size, const ALPHA_INT *res_col_indx, const T *x,    \
                     const ALPHA_INT ldx, const T *y, const ALPHA_INT ldy, const T alpha, const T beta,       \
                     int argc, const char *argv[]) {                                                          \
    (void)res_col_indx;                                                                                       \
    (void)y;                                                                                                  \
    (void)alpha;                                                                                              \
    (void)beta;                                                                                               \
    return check_l3(answer_data, ldans, answer_size, result_data, ldres, result_size, x, ldx, ldy, argc,      \
                    argv, COMPS, IS_DOUBLE);                                                                  \
  }
#define ASAMD_RE_REAL(v) ((double)(v))
#define ASAMD_RE_CX(v) ((double)(v).real)
ASAMD_CHECKS(s, float, 1, 0, ASAMD_RE_REAL)
ASAMD_CHECKS(d, double, 1, 1, ASAMD_RE_REAL)
ASAMD_CHECKS(c, ALPHA_Complex8, 2, 0, ASAMD_RE_CX)
ASAMD_CHECKS(z, ALPHA_Complex16, 2, 1, ASAMD_RE_CX)
