/* Helpers that the reference's test drivers call next to the sparse API: matrix
 * files, command-line flags, allocation, random fill, result comparison, timing.
 * Own text; each declaration cites the reference declaration it stands in for
 * (paths relative to the AlphaSparse tree).  Included by alphasparse.h inside
 * its extern "C" block. */
#ifndef ALSPARSE_AMD_ALPHASPARSE_UTIL_H
#define ALSPARSE_AMD_ALPHASPARSE_UTIL_H

#include <stdbool.h>
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>

/* include/alphasparse/util/malloc.h:13-17, :37-38.  alpha_free releases the
 * block (the reference's frees only NULL pointers, src/util/malloc.c:45-48). */
#ifndef DEFAULT_ALIGNMENT
#define DEFAULT_ALIGNMENT 32 /* include/alphasparse/util/malloc.h:11 */
#endif
void *alpha_malloc(size_t bytes);
void *alpha_memalign(size_t bytes, size_t alignment);
void alpha_free(void *point);
/* uniform values from rand() after srand(seed); seed 0 takes the clock */
void alpha_fill_random_s(float *arr, unsigned int seed, const size_t size);
void alpha_fill_random_d(double *arr, unsigned int seed, const size_t size);
/* include/alphasparse/util/malloc.h:39-41; src/util/malloc.c:104-112: 2*size reals */
void alpha_fill_random_c(ALPHA_Complex8 *arr, unsigned int seed, const size_t size);
void alpha_fill_random_z(ALPHA_Complex16 *arr, unsigned int seed, const size_t size);

/* include/alphasparse/util/thread.h:10-14; src/util/thread.c:11-38.  The reference's CPU kernels take
 * their OpenMP thread count from here; this library multiplies on the GPU, so the number is only kept
 * (0 means "all cores", as there) for programs that set it before alphasparse_?_mv / _mm. */
int alpha_get_core_num(void);
void alpha_set_thread_num(const int thread_num);
int alpha_get_thread_num(void);

/* include/alphasparse/util/io.h:19-20; src/util/io.c:39-114: Matrix Market
 * coordinate text ("%%MatrixMarket matrix coordinate <field> <symmetry>"):
 * one-based "row col [value]" lines become zero-based triplets, a missing value
 * reads as 1, a "symmetric" header mirrors every off-diagonal entry.  The
 * arrays are allocated with alpha_malloc. */
void alpha_read_coo(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                    ALPHA_INT **row_index, ALPHA_INT **col_index, float **values);
void alpha_read_coo_d(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, double **values);
/* include/alphasparse/util/io.h:21-22; src/util/io.c:193-345: the value of a line is
 * taken as both the real and the imaginary part */
void alpha_read_coo_c(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, ALPHA_Complex8 **values);
void alpha_read_coo_z(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, ALPHA_Complex16 **values);

/* include/alphasparse/util/check.h:45-46; src/util/check.c:701-776:
 * max|answer - result| / max|result|, printed as "correct,<ratio>" (return 0)
 * or "error,<ratio>" (return -1) against 2e-5 (fp32) / 1e-10 (fp64). */
int check_s(const float *answer_data, size_t answer_size, const float *result_data, size_t result_size);
int check_d(const double *answer_data, size_t answer_size, const double *result_data, size_t result_size);
/* include/alphasparse/util/check.h:47-48; src/util/check.c:778-786: as 2*size reals */
int check_c(const ALPHA_Complex8 *answer_data, size_t answer_size, const ALPHA_Complex8 *result_data,
            size_t result_size);
int check_z(const ALPHA_Complex16 *answer_data, size_t answer_size, const ALPHA_Complex16 *result_data,
            size_t result_size);

/* include/alphasparse/types.h:67-69 */
#ifndef ALPHA_INT64
#define ALPHA_INT64 int64_t
#endif

/* include/alphasparse/util/timing.h:7-20; src/util/timer.c: wall-clock timers of the CPU test programs */
typedef struct {
  double start;
  double end;
} alpha_timer_t;
double alpha_timing_wtime(void);
void alpha_timing_start(alpha_timer_t *timer);
void alpha_timing_end(alpha_timer_t *timer);
double alpha_timing_elapsed_time(const alpha_timer_t *timer);
double alpha_timing_gflops(const alpha_timer_t *timer, int64_t operations);
void alpha_timing_elaped_time_print(const alpha_timer_t *timer, const char *name);
void alpha_timing_gflops_print(const alpha_timer_t *timer, int64_t operations, const char *name);
/* include/alphasparse/util/malloc.h:23: flushes the CPU caches in the reference; no effect here */
void alpha_clear_cache(void);

/* include/alphasparse/util/analysis.h:6-8; src/util/analysis.c: entries below / on / above the
 * diagonal, and the operation count the reference's programs divide their times by */
void alphasparse_nnz_counter_coo(const ALPHA_INT *row_indx, const ALPHA_INT *col_indx, const ALPHA_INT nnz,
                                 ALPHA_INT *lo_p, ALPHA_INT *diag_p, ALPHA_INT *hi_p);
ALPHA_INT64 alphasparse_operations_mm(const ALPHA_INT rows, const ALPHA_INT cols, const ALPHA_INT lo,
                                      const ALPHA_INT diag, const ALPHA_INT hi,
                                      const alphasparse_operation_t operation,
                                      const struct alpha_matrix_descr descr, const ALPHA_INT columns,
                                      const alphasparse_datatype_t datatype);
ALPHA_INT64 alphasparse_operations_mv(const ALPHA_INT rows, const ALPHA_INT cols, const ALPHA_INT lo,
                                      const ALPHA_INT diag, const ALPHA_INT hi,
                                      const alphasparse_operation_t operation,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_datatype_t datatype);

/* include/alphasparse/util/check.h:50-57; src/util/check.c:7-57 (level 2), :218-345 (level 3): the
 * residual ||answer - result|| / (max(||A||_1,1) max(||x||,1) max(||result||,1) 10 eps max(m,k[,columns]))
 * against 50, with A read again from --data-file; prints "correct,<resid>" (0) or "error,<resid>" (-1).
 * Level 3 is served in its --data-file form (sparse times dense). */
int check_s_l2(const float *answer_data, size_t answer_size, const float *result_data, size_t result_size,
               const float *x, const float *y, const float alpha, const float beta, int argc, const char *argv[]);
int check_d_l2(const double *answer_data, size_t answer_size, const double *result_data, size_t result_size,
               const double *x, const double *y, const double alpha, const double beta, int argc,
               const char *argv[]);
int check_c_l2(const ALPHA_Complex8 *answer_data, size_t answer_size, const ALPHA_Complex8 *result_data,
               size_t result_size, const ALPHA_Complex8 *x, const ALPHA_Complex8 *y, const ALPHA_Complex8 alpha,
               const ALPHA_Complex8 beta, int argc, const char *argv[]);
int check_z_l2(const ALPHA_Complex16 *answer_data, size_t answer_size, const ALPHA_Complex16 *result_data,
               size_t result_size, const ALPHA_Complex16 *x, const ALPHA_Complex16 *y, const ALPHA_Complex16 alpha,
               const ALPHA_Complex16 beta, int argc, const char *argv[]);
int check_s_l3(const float *answer_data, const ALPHA_INT ldans, size_t answer_size, const float *result_data,
               const ALPHA_INT ldres, size_t result_size, const ALPHA_INT *res_col_indx, const float *x,
               const ALPHA_INT ldx, const float *y, const ALPHA_INT ldy, const float alpha, const float beta,
               int argc, const char *argv[]);
int check_d_l3(const double *answer_data, const ALPHA_INT ldans, size_t answer_size, const double *result_data,
               const ALPHA_INT ldres, size_t result_size, const ALPHA_INT *res_col_indx, const double *x,
               const ALPHA_INT ldx, const double *y, const ALPHA_INT ldy, const double alpha, const double beta,
               int argc, const char *argv[]);
int check_c_l3(const ALPHA_Complex8 *answer_data, const ALPHA_INT ldans, size_t answer_size,
               const ALPHA_Complex8 *result_data, const ALPHA_INT ldres, size_t result_size,
               const ALPHA_INT *res_col_indx, const ALPHA_Complex8 *x, const ALPHA_INT ldx, const ALPHA_Complex8 *y,
               const ALPHA_INT ldy, const ALPHA_Complex8 alpha, const ALPHA_Complex8 beta, int argc,
               const char *argv[]);
int check_z_l3(const ALPHA_Complex16 *answer_data, const ALPHA_INT ldans, size_t answer_size,
               const ALPHA_Complex16 *result_data, const ALPHA_INT ldres, size_t result_size,
               const ALPHA_INT *res_col_indx, const ALPHA_Complex16 *x, const ALPHA_INT ldx,
               const ALPHA_Complex16 *y, const ALPHA_INT ldy, const ALPHA_Complex16 alpha,
               const ALPHA_Complex16 beta, int argc, const char *argv[]);

/* include/alphasparse/util/args.h:16-44; src/util/args.c: GNU long options
 * --help --check --thread-num= --transA= --transB= --typeA= --fillA= --diagA=
 * --typeB= --fillB= --diagB= --data-file= --data-fileA= --data-fileB= --layout=
 * --layoutB= --layoutC= --columns= --iter= --formatA= --formatB= --data-type= */
void args_help(const int argc, const char *argv[]);
bool args_get_if_check(const int argc, const char *argv[]);
int args_get_thread_num(const int argc, const char *argv[]);
int args_get_columns(const int argc, const char *argv[], int k);
int args_get_iter(const int argc, const char *argv[]);
const char *args_get_data_file(const int argc, const char *argv[]);
const char *args_get_data_fileA(const int argc, const char *argv[]);
const char *args_get_data_fileB(const int argc, const char *argv[]);
alphasparse_layout_t alpha_args_get_layout(const int argc, const char *argv[]);
alphasparse_layout_t alpha_args_get_layoutB(const int argc, const char *argv[]);
alphasparse_layout_t alpha_args_get_layoutC(const int argc, const char *argv[]);
struct alpha_matrix_descr alpha_args_get_matrix_descrA(const int argc, const char *argv[]);
struct alpha_matrix_descr alpha_args_get_matrix_descrB(const int argc, const char *argv[]);
alphasparse_operation_t alpha_args_get_transA(const int argc, const char *argv[]);
alphasparse_operation_t alpha_args_get_transB(const int argc, const char *argv[]);

/* include/alphasparse/handle.h:334; src/util_cpp/handle.cpp:487-493:
 * wall clock in microseconds after a device synchronisation. */
double get_time_us(void);

#ifdef __cplusplus
/* include/alphasparse/handle.h:336; src/util_cpp/handle.cpp:495-510: mean of the
 * samples below twice the plain mean (drops warm-up outliers).  C++ callers only. */
extern "C++" {
#include <vector>
}
double get_avg_time(std::vector<double> times);
#endif

/* include/alphasparse/util/error.h:9-45 and :139-150 */
#define alpha_call_exit(func, message)                                      \
  do {                                                                      \
    alphasparse_status_t alpha_status_ = (func);                            \
    if (alpha_status_ != ALPHA_SPARSE_STATUS_SUCCESS) {                     \
      printf("%s\nstatus : %d\n", (message), (int)alpha_status_);           \
      exit(-1);                                                             \
    }                                                                       \
  } while (0)

#define roc_call_exit(func, message)                                        \
  do {                                                                      \
    int roc_status_ = (int)(func);                                          \
    if (roc_status_ != 0) {                                                 \
      printf("%s\nstatus : %d\n", (message), roc_status_);                  \
      exit(-1);                                                             \
    }                                                                       \
  } while (0)

#define PRINT_IF_HIP_ERROR(INPUT_STATUS_FOR_CHECK)                                            \
  {                                                                                           \
    int TMP_STATUS_FOR_CHECK = (int)(INPUT_STATUS_FOR_CHECK);                                 \
    if (TMP_STATUS_FOR_CHECK != 0) {                                                          \
      fprintf(stderr, "hip error code: %d at %s:%d\n", TMP_STATUS_FOR_CHECK, __FILE__, __LINE__); \
    }                                                                                         \
  }

#endif /* ALSPARSE_AMD_ALPHASPARSE_UTIL_H */
