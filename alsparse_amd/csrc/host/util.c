/* Driver-side helpers: allocation, random fill, Matrix Market reader, result
 * check, command-line flags, timer.  Behaviour follows src/util/malloc.c,
 * src/util/io.c:39-114, src/util/check.c:701-776, src/util/args.c and
 * src/util_cpp/handle.cpp:487-493 of the reference. */
#define _GNU_SOURCE
#include <getopt.h>
#include <math.h>
#include <string.h>
#include <unistd.h>
#include <sys/time.h>
#include <time.h>

#include "internal.h"

void *alpha_malloc(size_t bytes) {
  void *p = malloc(bytes ? bytes : 1);
  if (!p) {
    fprintf(stderr, "alpha_malloc: no memory for %zu bytes\n", bytes);
    exit(-1);
  }
  return p;
}

void *alpha_memalign(size_t bytes, size_t alignment) {
  void *p = NULL;
  if (alignment < sizeof(void *)) alignment = sizeof(void *);
  if (posix_memalign(&p, alignment, bytes ? bytes : 1) != 0) {
    fprintf(stderr, "alpha_memalign: no memory for %zu bytes\n", bytes);
    exit(-1);
  }
  return p;
}

void alpha_free(void *point) { free(point); }

static unsigned int seed_or_clock(unsigned int seed) { return seed ? seed : (unsigned int)time(NULL); }

void alpha_fill_random_s(float *arr, unsigned int seed, const size_t size) {
  srand(seed_or_clock(seed));
  for (size_t i = 0; i < size; ++i) arr[i] = (float)rand() / (float)RAND_MAX;
}

void alpha_fill_random_d(double *arr, unsigned int seed, const size_t size) {
  srand(seed_or_clock(seed));
  for (size_t i = 0; i < size; ++i) arr[i] = (double)rand() / (double)RAND_MAX;
}

/* ---- thread count of the reference's CPU kernels (kept, not used: the GPU multiplies) ---------- */
static int g_thread_num;

int alpha_get_core_num(void) {
  const long n = sysconf(_SC_NPROCESSORS_ONLN);
  return n > 0 ? (int)n : 1;
}

void alpha_set_thread_num(const int thread_num) { g_thread_num = thread_num; }

int alpha_get_thread_num(void) { return g_thread_num == 0 ? alpha_get_core_num() : g_thread_num; }

/* src/util/malloc.c:104-112: a complex array is filled as twice as many reals */
void alpha_fill_random_c(ALPHA_Complex8 *arr, unsigned int seed, const size_t size) {
  alpha_fill_random_s((float *)arr, seed, size * 2);
}

void alpha_fill_random_z(ALPHA_Complex16 *arr, unsigned int seed, const size_t size) {
  alpha_fill_random_d((double *)arr, seed, size * 2);
}

/* ---- Matrix Market coordinate reader ------------------------------------- */
typedef struct {
  ALPHA_INT m, n, nnz;
  ALPHA_INT *row, *col;
  double *val;
} coo_triplets;

static void read_coo_triplets(const char *file, coo_triplets *out) {
  FILE *fp = fopen(file, "r");
  if (!fp) {
    printf("file is not exist!!!\n");
    exit(-1);
  }
  char line[1024];
  int symmetric = 0, first = 1, have_size = 0;
  while (fgets(line, sizeof line, fp)) {
    if (line[0] == '%') {
      if (first && strstr(line, "symmetric")) symmetric = 1;
      first = 0;
      continue;
    }
    have_size = 1;
    break;
  }
  long long m = 0, n = 0, nnz = 0;
  if (!have_size || sscanf(line, "%lld %lld %lld", &m, &n, &nnz) != 3 || m < 0 || n < 0 || nnz < 0 ||
      m > 0x7fffffffLL || n > 0x7fffffffLL || nnz > 0x3fffffffLL) {
    printf("bad size line in %s\n", file);
    exit(-1);
  }
  const size_t cap = (size_t)nnz * (symmetric ? 2 : 1);
  ALPHA_INT *row = (ALPHA_INT *)alpha_malloc(cap * sizeof(ALPHA_INT));
  ALPHA_INT *col = (ALPHA_INT *)alpha_malloc(cap * sizeof(ALPHA_INT));
  double *val = (double *)alpha_malloc(cap * sizeof(double));
  size_t real = 0;
  for (long long i = 0; i < nnz; ++i) {
    if (!fgets(line, sizeof line, fp)) {
      printf("%s ends after %lld of %lld entries\n", file, i, nnz);
      exit(-1);
    }
    long long r = 0, c = 0;
    double v = 1.0; /* pattern files carry no value */
    const int got = sscanf(line, "%lld %lld %lf", &r, &c, &v);
    if (got < 2 || r < 1 || c < 1 || r > m || c > n) {
      printf("bad entry line %lld in %s\n", i + 1, file);
      exit(-1);
    }
    row[real] = (ALPHA_INT)(r - 1);
    col[real] = (ALPHA_INT)(c - 1);
    val[real] = v;
    ++real;
    if (symmetric && r != c) {
      row[real] = (ALPHA_INT)(c - 1);
      col[real] = (ALPHA_INT)(r - 1);
      val[real] = v;
      ++real;
    }
  }
  fclose(fp);
  out->m = (ALPHA_INT)m;
  out->n = (ALPHA_INT)n;
  out->nnz = (ALPHA_INT)real;
  out->row = row;
  out->col = col;
  out->val = val;
}

void alpha_read_coo(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                    ALPHA_INT **row_index, ALPHA_INT **col_index, float **values) {
  coo_triplets t;
  read_coo_triplets(file, &t);
  float *v = (float *)alpha_malloc((size_t)t.nnz * sizeof(float));
  for (ALPHA_INT i = 0; i < t.nnz; ++i) v[i] = (float)t.val[i];
  alpha_free(t.val);
  *m_p = t.m;
  *n_p = t.n;
  *nnz_p = t.nnz;
  *row_index = t.row;
  *col_index = t.col;
  *values = v;
}

void alpha_read_coo_d(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, double **values) {
  coo_triplets t;
  read_coo_triplets(file, &t);
  *m_p = t.m;
  *n_p = t.n;
  *nnz_p = t.nnz;
  *row_index = t.row;
  *col_index = t.col;
  *values = t.val;
}

/* src/util/io.c:193-268, :270-345: the one value of a line becomes both the real and the
 * imaginary part (a line without a value reads as 1 + 1i) */
void alpha_read_coo_c(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, ALPHA_Complex8 **values) {
  coo_triplets t;
  read_coo_triplets(file, &t);
  ALPHA_Complex8 *v = (ALPHA_Complex8 *)alpha_malloc((size_t)t.nnz * sizeof(ALPHA_Complex8));
  for (ALPHA_INT i = 0; i < t.nnz; ++i) v[i].real = v[i].imag = (float)t.val[i];
  alpha_free(t.val);
  *m_p = t.m;
  *n_p = t.n;
  *nnz_p = t.nnz;
  *row_index = t.row;
  *col_index = t.col;
  *values = v;
}

void alpha_read_coo_z(const char *file, ALPHA_INT *m_p, ALPHA_INT *n_p, ALPHA_INT *nnz_p,
                      ALPHA_INT **row_index, ALPHA_INT **col_index, ALPHA_Complex16 **values) {
  coo_triplets t;
  read_coo_triplets(file, &t);
  ALPHA_Complex16 *v = (ALPHA_Complex16 *)alpha_malloc((size_t)t.nnz * sizeof(ALPHA_Complex16));
  for (ALPHA_INT i = 0; i < t.nnz; ++i) v[i].real = v[i].imag = t.val[i];
  alpha_free(t.val);
  *m_p = t.m;
  *n_p = t.n;
  *nnz_p = t.nnz;
  *row_index = t.row;
  *col_index = t.col;
  *values = v;
}

/* ---- result check ---------------------------------------------------------- */
#define ASAMD_CHECK(NAME, T, FABS, TOL)                                                          \
  int NAME(const T *answer_data, size_t answer_size, const T *result_data, size_t result_size) { \
    if (answer_size != result_size) {                                                            \
      printf("answer_size ans result_size is not equal (%zu %zu)\n", answer_size, result_size);  \
      return -1;                                                                                 \
    }                                                                                            \
    if (answer_size == 0) {                                                                      \
      printf("answer_size ans result_size is less than 0\n");                                    \
      return -1;                                                                                 \
    }                                                                                            \
    T max_error = 0, max_result = 0;                                                             \
    for (size_t i = 0; i < answer_size; i++) {                                                   \
      const T err = FABS(answer_data[i] - result_data[i]);                                       \
      if (err > max_error || err != err) max_error = err;                                        \
      if (FABS(result_data[i]) > max_result) max_result = FABS(result_data[i]);                  \
    }                                                                                            \
    const T relative_error = max_error / max_result;                                             \
    if (!(relative_error <= (T)(TOL))) {                                                         \
      printf("error,%.10f\n", (double)relative_error);                                           \
      return -1;                                                                                 \
    }                                                                                            \
    printf("correct,%.10f\n", (double)relative_error);                                           \
    return 0;                                                                                    \
  }
ASAMD_CHECK(check_s, float, fabsf, 2e-5)
ASAMD_CHECK(check_d, double, fabs, 1e-10)

/* src/util/check.c:778-786: complex arrays are compared as twice as many reals */
int check_c(const ALPHA_Complex8 *answer_data, size_t answer_size, const ALPHA_Complex8 *result_data,
            size_t result_size) {
  return check_s((const float *)answer_data, answer_size * 2, (const float *)result_data, result_size * 2);
}

int check_z(const ALPHA_Complex16 *answer_data, size_t answer_size, const ALPHA_Complex16 *result_data,
            size_t result_size) {
  return check_d((const double *)answer_data, answer_size * 2, (const double *)result_data, result_size * 2);
}

/* ---- command line ---------------------------------------------------------- */
enum {
  OPT_HELP = 1, OPT_CHECK, OPT_THREADS, OPT_TRANSA, OPT_TRANSB, OPT_TYPEA, OPT_FILLA, OPT_DIAGA, OPT_TYPEB,
  OPT_FILLB, OPT_DIAGB, OPT_FILE, OPT_FILEA, OPT_FILEB, OPT_LAYOUT, OPT_LAYOUTB, OPT_LAYOUTC, OPT_COLUMNS,
  OPT_ITER, OPT_FORMATA, OPT_FORMATB, OPT_DATATYPE
};
static const struct option k_options[] = {
    {"help", no_argument, NULL, OPT_HELP},           {"check", no_argument, NULL, OPT_CHECK},
    {"thread-num", optional_argument, NULL, OPT_THREADS}, {"transA", optional_argument, NULL, OPT_TRANSA},
    {"transB", optional_argument, NULL, OPT_TRANSB}, {"typeA", optional_argument, NULL, OPT_TYPEA},
    {"fillA", optional_argument, NULL, OPT_FILLA},   {"diagA", optional_argument, NULL, OPT_DIAGA},
    {"typeB", optional_argument, NULL, OPT_TYPEB},   {"fillB", optional_argument, NULL, OPT_FILLB},
    {"diagB", optional_argument, NULL, OPT_DIAGB},   {"data-file", optional_argument, NULL, OPT_FILE},
    {"data-fileA", optional_argument, NULL, OPT_FILEA}, {"data-fileB", optional_argument, NULL, OPT_FILEB},
    {"layout", optional_argument, NULL, OPT_LAYOUT}, {"layoutB", optional_argument, NULL, OPT_LAYOUTB},
    {"layoutC", optional_argument, NULL, OPT_LAYOUTC}, {"columns", optional_argument, NULL, OPT_COLUMNS},
    {"iter", optional_argument, NULL, OPT_ITER},     {"formatA", optional_argument, NULL, OPT_FORMATA},
    {"formatB", optional_argument, NULL, OPT_FORMATB}, {"data-type", optional_argument, NULL, OPT_DATATYPE},
    {NULL, 0, NULL, 0}};

/* value of the first occurrence of `which`, "" for a flag without value, NULL if absent */
static const char *find_option(const int argc, const char *argv[], int which) {
  optind = 0;
  opterr = 0; /* each driver only asks for the flags it knows */
  int opt, index;
  while ((opt = getopt_long_only(argc, (char *const *)argv, "", k_options, &index)) != -1)
    if (opt == which) return optarg ? optarg : "";
  return NULL;
}

static void bad_value(const char *what, const char *arg) {
  printf("invalid %s value!!! %s\n", what, arg);
  exit(-1);
}

static int is_one_of(const char *arg, const char *a, const char *b) { return !strcmp(arg, a) || !strcmp(arg, b); }

void args_help(const int argc, const char *argv[]) {
  if (!find_option(argc, argv, OPT_HELP)) return;
  printf("--help\n--check\n\tcompare with the reference result, default: no check\n"
         "--thread-num=<int>\n--data-file=<file>\n--data-fileA=<file>\n--data-fileB=<file>\n"
         "--columns=<int>\n\tdense matrix columns, default: k\n--iter=<int>\n\ttest iterations, default: 1\n"
         "--layout=<R|C>\n\tdense matrix layout, default: R\n--transA=<N|T|H>\n--transB=<N|T|H>\n"
         "--typeA=<G|S|H|T|D|BT|BD>\n--fillA=<L|U>\n--diagA=<N|U>\n--typeB=...\n--fillB=...\n--diagB=...\n");
  exit(-1);
}

bool args_get_if_check(const int argc, const char *argv[]) { return find_option(argc, argv, OPT_CHECK) != NULL; }

static int int_option(const int argc, const char *argv[], int which, int fallback) {
  const char *v = find_option(argc, argv, which);
  return v && *v ? atoi(v) : fallback;
}
int args_get_thread_num(const int argc, const char *argv[]) { return int_option(argc, argv, OPT_THREADS, 1); }
int args_get_columns(const int argc, const char *argv[], int k) { return int_option(argc, argv, OPT_COLUMNS, k); }
int args_get_iter(const int argc, const char *argv[]) { return int_option(argc, argv, OPT_ITER, 1); }

static const char *string_option(const int argc, const char *argv[], int which) {
  const char *v = find_option(argc, argv, which);
  return v ? v : "";
}
const char *args_get_data_file(const int argc, const char *argv[]) { return string_option(argc, argv, OPT_FILE); }
const char *args_get_data_fileA(const int argc, const char *argv[]) { return string_option(argc, argv, OPT_FILEA); }
const char *args_get_data_fileB(const int argc, const char *argv[]) { return string_option(argc, argv, OPT_FILEB); }

static alphasparse_layout_t layout_option(const int argc, const char *argv[], int which) {
  const char *v = find_option(argc, argv, which);
  if (!v || !*v) return ALPHA_SPARSE_LAYOUT_ROW_MAJOR;
  if (is_one_of(v, "R", "ROW")) return ALPHA_SPARSE_LAYOUT_ROW_MAJOR;
  if (is_one_of(v, "C", "COL") || !strcmp(v, "COLUMN")) return ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR;
  bad_value("layout", v);
  return ALPHA_SPARSE_LAYOUT_ROW_MAJOR;
}
alphasparse_layout_t alpha_args_get_layout(const int argc, const char *argv[]) { return layout_option(argc, argv, OPT_LAYOUT); }
alphasparse_layout_t alpha_args_get_layoutB(const int argc, const char *argv[]) { return layout_option(argc, argv, OPT_LAYOUTB); }
alphasparse_layout_t alpha_args_get_layoutC(const int argc, const char *argv[]) { return layout_option(argc, argv, OPT_LAYOUTC); }

static alphasparse_operation_t trans_option(const int argc, const char *argv[], int which) {
  const char *v = find_option(argc, argv, which);
  if (!v || !*v) return ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
  if (is_one_of(v, "N", "NON_TRANSPOSE")) return ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
  if (is_one_of(v, "T", "TRANSPOSE")) return ALPHA_SPARSE_OPERATION_TRANSPOSE;
  if (is_one_of(v, "H", "CONJUGATE_TRANSPOSE")) return ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE;
  bad_value("operation", v);
  return ALPHA_SPARSE_OPERATION_NON_TRANSPOSE;
}
alphasparse_operation_t alpha_args_get_transA(const int argc, const char *argv[]) { return trans_option(argc, argv, OPT_TRANSA); }
alphasparse_operation_t alpha_args_get_transB(const int argc, const char *argv[]) { return trans_option(argc, argv, OPT_TRANSB); }

static struct alpha_matrix_descr descr_option(const int argc, const char *argv[], int type_opt, int fill_opt,
                                              int diag_opt) {
  struct alpha_matrix_descr d = {ALPHA_SPARSE_MATRIX_TYPE_GENERAL, ALPHA_SPARSE_FILL_MODE_LOWER,
                                 ALPHA_SPARSE_DIAG_NON_UNIT};
  const char *v = find_option(argc, argv, type_opt);
  if (v && *v) {
    if (is_one_of(v, "G", "GENERAL")) d.type = ALPHA_SPARSE_MATRIX_TYPE_GENERAL;
    else if (is_one_of(v, "S", "SYMMETRIC")) d.type = ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC;
    else if (is_one_of(v, "H", "HERMITIAN")) d.type = ALPHA_SPARSE_MATRIX_TYPE_HERMITIAN;
    else if (is_one_of(v, "T", "TRIANGULAR")) d.type = ALPHA_SPARSE_MATRIX_TYPE_TRIANGULAR;
    else if (is_one_of(v, "D", "DIAGONAL")) d.type = ALPHA_SPARSE_MATRIX_TYPE_DIAGONAL;
    else if (is_one_of(v, "BT", "BLOCK_TRIANGULAR")) d.type = ALPHA_SPARSE_MATRIX_TYPE_BLOCK_TRIANGULAR;
    else if (is_one_of(v, "BD", "BLOCK_DIAGONAL")) d.type = ALPHA_SPARSE_MATRIX_TYPE_BLOCK_DIAGONAL;
    else bad_value("type", v);
  }
  v = find_option(argc, argv, fill_opt);
  if (v && *v) {
    if (is_one_of(v, "L", "LOWER")) d.mode = ALPHA_SPARSE_FILL_MODE_LOWER;
    else if (is_one_of(v, "U", "UPPER")) d.mode = ALPHA_SPARSE_FILL_MODE_UPPER;
    else bad_value("fill", v);
  }
  v = find_option(argc, argv, diag_opt);
  if (v && *v) {
    if (is_one_of(v, "N", "NON_UNIT")) d.diag = ALPHA_SPARSE_DIAG_NON_UNIT;
    else if (is_one_of(v, "U", "UNIT")) d.diag = ALPHA_SPARSE_DIAG_UNIT;
    else bad_value("diag", v);
  }
  return d;
}
struct alpha_matrix_descr alpha_args_get_matrix_descrA(const int argc, const char *argv[]) {
  return descr_option(argc, argv, OPT_TYPEA, OPT_FILLA, OPT_DIAGA);
}
struct alpha_matrix_descr alpha_args_get_matrix_descrB(const int argc, const char *argv[]) {
  return descr_option(argc, argv, OPT_TYPEB, OPT_FILLB, OPT_DIAGB);
}

double get_time_us(void) {
  (void)hipDeviceSynchronize();
  struct timeval tv;
  gettimeofday(&tv, NULL);
  return (double)tv.tv_sec * 1e6 + (double)tv.tv_usec;
}
