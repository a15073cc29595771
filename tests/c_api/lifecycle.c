/* A C program against the public headers, as a user of the library would write it: handles and
 * descriptors through their whole lifecycle (CSR / COO / ELL handles, device mirrors, analysis,
 * clear, re-analysis, hand-made info bundles, freed and reallocated device arrays under stale
 * analysis records, a second handle on its own stream, the generic descriptor call), all four
 * element types, every result compared with a double-precision loop on the CPU.  Prints
 * "lifecycle: all passed".  Built by tests/c_api/Makefile, plain or with the host-side sanitizers
 * (`make asan`: ASan + UBSan on the library's host code and on this program; device code is not
 * instrumented). */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include "alphasparse.h"
#include "alpha_spblas_dcu.h"

#define OK(call)                                                                   \
  do {                                                                             \
    int st_ = (int)(call);                                                         \
    if (st_ != 0) {                                                                \
      fprintf(stderr, "%s:%d: %s -> %d\n", __FILE__, __LINE__, #call, st_);        \
      exit(2);                                                                     \
    }                                                                              \
  } while (0)
#define EXPECT(call, want)                                                                    \
  do {                                                                                        \
    int st_ = (int)(call);                                                                    \
    if (st_ != (int)(want)) {                                                                 \
      fprintf(stderr, "%s:%d: %s -> %d, expected %d\n", __FILE__, __LINE__, #call, st_, (int)(want)); \
      exit(2);                                                                                \
    }                                                                                         \
  } while (0)

static unsigned long long rng_state = 88172645463325252ull;
static unsigned rnd(void) {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (unsigned)(rng_state >> 16);
}
static double urand(void) { return (double)(rnd() % 2000001) / 1000000.0 - 1.0; }

typedef struct {
  int m, n, nnz;
  int *rp, *ci;
  double *v;
} csr_t;

/* rows of skewed length, some empty, columns sorted without repeats */
static csr_t make_csr(int m, int n, int max_len) {
  csr_t a = {m, n, 0, (int *)malloc(sizeof(int) * (size_t)(m + 1)), NULL, NULL};
  int *len = (int *)malloc(sizeof(int) * (size_t)m);
  long total = 0;
  for (int r = 0; r < m; ++r) {
    unsigned u = rnd() % 100;
    int l = u < 10 ? 0 : (u < 90 ? 1 + (int)(rnd() % 12) : 1 + (int)(rnd() % (unsigned)max_len));
    if (l > n) l = n;
    len[r] = l;
    total += l;
  }
  a.nnz = (int)total;
  a.ci = (int *)malloc(sizeof(int) * (size_t)(total ? total : 1));
  a.v = (double *)malloc(sizeof(double) * (size_t)(total ? total : 1));
  char *used = (char *)calloc((size_t)n, 1);
  int p = 0;
  for (int r = 0; r < m; ++r) {
    a.rp[r] = p;
    for (int k = 0; k < len[r];) {
      int c = (int)(rnd() % (unsigned)n);
      if (used[c]) continue;
      used[c] = 1;
      ++k;
    }
    for (int c = 0; c < n; ++c)
      if (used[c]) {
        used[c] = 0;
        a.ci[p] = c;
        a.v[p] = urand();
        ++p;
      }
  }
  a.rp[m] = p;
  free(used);
  free(len);
  return a;
}
static void free_csr(csr_t *a) {
  free(a->rp);
  free(a->ci);
  free(a->v);
}

static void *dev_copy(const void *h, size_t bytes) {
  void *d = NULL;
  OK(hipMalloc(&d, bytes ? bytes : 4));
  if (bytes) OK(hipMemcpy(d, h, bytes, hipMemcpyHostToDevice));
  return d;
}

/* ---- real types ---------------------------------------------------------------------------- */
#define REAL_SUITE(S, T, TOL)                                                                                  \
  static void ref_mv_##S(const csr_t *a, int trans, double alpha, const T *x, double beta, const T *y0, double *y) { \
    int ylen = trans ? a->n : a->m;                                                                            \
    for (int i = 0; i < ylen; ++i) y[i] = beta * (double)y0[i];                                                \
    for (int r = 0; r < a->m; ++r)                                                                             \
      for (int j = a->rp[r]; j < a->rp[r + 1]; ++j) {                                                          \
        if (trans) y[a->ci[j]] += alpha * (double)(T)a->v[j] * (double)x[r];                                   \
        else y[r] += alpha * (double)(T)a->v[j] * (double)x[a->ci[j]];                                         \
      }                                                                                                        \
  }                                                                                                            \
  static void cmp_##S(const char *what, const double *ref, const T *got, int len) {                            \
    double worst = 0;                                                                                          \
    for (int i = 0; i < len; ++i) {                                                                            \
      double e = fabs(ref[i] - (double)got[i]) / (1.0 + fabs(ref[i]));                                         \
      if (e > worst) worst = e;                                                                                \
    }                                                                                                          \
    if (!(worst <= TOL)) {                                                                                     \
      fprintf(stderr, "MISMATCH %s: %g\n", what, worst);                                                       \
      exit(3);                                                                                                 \
    }                                                                                                          \
  }                                                                                                            \
  static void suite_##S(alphasparse_dcu_handle_t h, const csr_t *a) {                                          \
    const int m = a->m, n = a->n, nnz = a->nnz;                                                                \
    T *val = (T *)malloc(sizeof(T) * (size_t)(nnz ? nnz : 1));                                                 \
    for (int i = 0; i < nnz; ++i) val[i] = (T)a->v[i];                                                         \
    int big = m > n ? m : n;                                                                                   \
    T *x = (T *)malloc(sizeof(T) * (size_t)big), *y0 = (T *)malloc(sizeof(T) * (size_t)big);                   \
    T *y = (T *)malloc(sizeof(T) * (size_t)big);                                                               \
    double *ref = (double *)malloc(sizeof(double) * (size_t)big);                                              \
    for (int i = 0; i < big; ++i) { x[i] = (T)urand(); y0[i] = (T)urand(); }                                   \
    struct alpha_matrix_descr hd = {ALPHA_SPARSE_MATRIX_TYPE_GENERAL, ALPHA_SPARSE_FILL_MODE_LOWER, ALPHA_SPARSE_DIAG_NON_UNIT}; \
    /* host handles: CSR, COO -> CSR, COO -> ELL */                                                            \
    alphasparse_matrix_t A = NULL;                                                                             \
    OK(alphasparse_##S##_create_csr(&A, ALPHA_SPARSE_INDEX_BASE_ZERO, m, n, a->rp, a->rp + 1, a->ci, val));    \
    for (int trans = 0; trans < 2; ++trans) {                                                                  \
      int ylen = trans ? n : m;                                                                                \
      memcpy(y, y0, sizeof(T) * (size_t)ylen);                                                                 \
      OK(alphasparse_##S##_mv((alphasparse_operation_t)trans, (T)1.5, A, hd, x, (T)0.5, y));                   \
      ref_mv_##S(a, trans, 1.5, x, 0.5, y0, ref);                                                              \
      cmp_##S("mv", ref, y, ylen);                                                                             \
      memcpy(y, y0, sizeof(T) * (size_t)ylen);                                                                 \
      OK(alphasparse_##S##_mv_plain((alphasparse_operation_t)trans, (T)1.5, A, hd, x, (T)0.5, y));             \
      cmp_##S("mv_plain", ref, y, ylen);                                                                       \
    }                                                                                                          \
    {                                                                                                          \
      const int cols = 5;                                                                                      \
      T *B = (T *)malloc(sizeof(T) * (size_t)big * cols), *C = (T *)malloc(sizeof(T) * (size_t)big * cols);    \
      for (int i = 0; i < big * cols; ++i) { B[i] = (T)urand(); C[i] = (T)urand(); }                           \
      OK(alphasparse_##S##_mm(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, (T)1.0, A, hd, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, B, cols, cols, (T)0.0, C, cols)); \
      OK(alphasparse_##S##_mm(ALPHA_SPARSE_OPERATION_TRANSPOSE, (T)1.0, A, hd, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, B, cols, cols, (T)2.0, C, cols)); \
      OK(alphasparse_##S##_mm(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, (T)1.0, A, hd, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, B, cols, n, (T)1.0, C, m)); \
      OK(alphasparse_##S##_mm_plain(ALPHA_SPARSE_OPERATION_TRANSPOSE, (T)1.0, A, hd, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, B, cols, m, (T)1.0, C, n)); \
      free(B);                                                                                                 \
      free(C);                                                                                                 \
    }                                                                                                          \
    OK(alphasparse_destroy(A));                                                                                \
    if (nnz > 0) {                                                                                             \
      int *ri = (int *)malloc(sizeof(int) * (size_t)nnz);                                                      \
      for (int r = 0; r < m; ++r)                                                                              \
        for (int j = a->rp[r]; j < a->rp[r + 1]; ++j) ri[j] = r + 1;                                           \
      int *c1 = (int *)malloc(sizeof(int) * (size_t)nnz);                                                      \
      for (int j = 0; j < nnz; ++j) c1[j] = a->ci[j] + 1;                                                      \
      alphasparse_matrix_t coo = NULL, csr = NULL, ell = NULL;                                                 \
      OK(alphasparse_##S##_create_coo(&coo, ALPHA_SPARSE_INDEX_BASE_ONE, m, n, nnz, ri, c1, val));             \
      OK(alphasparse_convert_csr(coo, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, &csr));                            \
      OK(alphasparse_convert_ell(coo, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, &ell));                            \
      OK(host2device_##S##_coo(coo));                                                                          \
      OK(host2device_##S##_ell(ell));                                                                          \
      OK(host2device_##S##_csr(csr));                                                                          \
      OK(host2device_##S##_csr(csr)); /* replaces the mirror */                                                \
      T *dx = (T *)dev_copy(x, sizeof(T) * (size_t)big), *dy = (T *)dev_copy(y0, sizeof(T) * (size_t)big);     \
      alpha_dcu_matrix_descr_t dd;                                                                             \
      OK(alphasparse_dcu_create_mat_descr(&dd));                                                               \
      T al = (T)1.5, be = (T)0.5;                                                                              \
      ref_mv_##S(a, 0, 1.5, x, 0.5, y0, ref);                                                                  \
      alphasparse_matrix_t hs[3] = {coo, ell, csr};                                                            \
      for (int k = 0; k < 3; ++k) {                                                                            \
        OK(hipMemcpy(dy, y0, sizeof(T) * (size_t)m, hipMemcpyHostToDevice));                                   \
        OK(alphasparse_##S##_mv_dcu(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, &al, hs[k], dd, dx, &be, dy));    \
        OK(hipDeviceSynchronize());                                                                            \
        OK(hipMemcpy(y, dy, sizeof(T) * (size_t)m, hipMemcpyDeviceToHost));                                    \
        cmp_##S("mv_dcu", ref, y, m);                                                                          \
      }                                                                                                        \
      ALPHA_INT er, ec, ew, *eci;                                                                              \
      T *ev;                                                                                                   \
      alphasparse_index_base_t eb;                                                                             \
      OK(alphasparse_##S##_export_ell(ell, &eb, &er, &ec, &ew, &eci, &ev));                                    \
      OK(alphasparse_destroy(coo));                                                                            \
      OK(alphasparse_destroy(ell));                                                                            \
      OK(alphasparse_destroy(csr));                                                                            \
      OK(alphasparse_dcu_destroy_mat_descr(dd));                                                               \
      OK(hipFree(dx));                                                                                         \
      OK(hipFree(dy));                                                                                         \
      free(ri);                                                                                                \
      free(c1);                                                                                                \
    }                                                                                                          \
    /* raw device pointers */                                                                                  \
    if (nnz > 0) {                                                                                             \
      int *drp = (int *)dev_copy(a->rp, sizeof(int) * (size_t)(m + 1));                                        \
      int *dci = (int *)dev_copy(a->ci, sizeof(int) * (size_t)nnz);                                            \
      T *dv = (T *)dev_copy(val, sizeof(T) * (size_t)nnz);                                                     \
      T *dx = (T *)dev_copy(x, sizeof(T) * (size_t)big), *dy = (T *)dev_copy(y0, sizeof(T) * (size_t)big);     \
      alpha_dcu_matrix_descr_t dd;                                                                             \
      OK(alphasparse_dcu_create_mat_descr(&dd));                                                               \
      T al = (T)1.5, be = (T)0.5;                                                                              \
      alphasparse_dcu_mat_info_t info = NULL;                                                                  \
      OK(alphasparse_dcu_create_mat_info(&info));                                                              \
      for (int round = 0; round < 3; ++round) {                                                                \
        for (int trans = 0; trans < 2; ++trans) {                                                              \
          int ylen = trans ? n : m;                                                                            \
          alphasparse_dcu_mat_info_t use = round == 1 ? NULL : info;                                           \
          if (use) OK(alphasparse_dcu_##S##_csrmv_analysis(h, (alphasparse_operation_t)trans, m, n, nnz, dd, dv, drp, dci, use)); \
          OK(hipMemcpy(dy, y0, sizeof(T) * (size_t)ylen, hipMemcpyHostToDevice));                              \
          OK(alphasparse_dcu_##S##_csrmv(h, (alphasparse_operation_t)trans, m, n, nnz, &al, dd, dv, drp, dci, use, dx, &be, dy)); \
          OK(hipDeviceSynchronize());                                                                          \
          OK(hipMemcpy(y, dy, sizeof(T) * (size_t)ylen, hipMemcpyDeviceToHost));                               \
          ref_mv_##S(a, trans, 1.5, x, 0.5, y0, ref);                                                          \
          cmp_##S("csrmv", ref, y, ylen);                                                                      \
        }                                                                                                      \
        if (round == 0) OK(alphasparse_dcu_csrmv_clear(h, info));                                              \
      }                                                                                                        \
      /* a bundle the caller made by hand, mostly garbage */                                                   \
      {                                                                                                        \
        struct _alphasparse_dcu_mat_info *junk = (struct _alphasparse_dcu_mat_info *)malloc(sizeof(*junk));    \
        memset(junk, 0x5a, sizeof(*junk));                                                                     \
        junk->csrmv_info = (alphasparse_dcu_csrmv_info_t)malloc(sizeof(*junk->csrmv_info));                    \
        memset(junk->csrmv_info, 0xa5, sizeof(*junk->csrmv_info));                                             \
        junk->csrmv_info->csr_adaptive_has_tuned = false;                                                      \
        OK(hipMemcpy(dy, y0, sizeof(T) * (size_t)m, hipMemcpyHostToDevice));                                   \
        OK(alphasparse_dcu_##S##_csrmv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, m, n, nnz, &al, dd, dv, drp, dci, junk, dx, &be, dy)); \
        OK(hipDeviceSynchronize());                                                                            \
        OK(hipMemcpy(y, dy, sizeof(T) * (size_t)m, hipMemcpyDeviceToHost));                                    \
        ref_mv_##S(a, 0, 1.5, x, 0.5, y0, ref);                                                                \
        cmp_##S("csrmv junk info", ref, y, m);                                                                 \
        free(junk->csrmv_info);                                                                                \
        free(junk);                                                                                            \
      }                                                                                                        \
      /* conversions + ellmv + coomv */                                                                        \
      int *dri = (int *)dev_copy(NULL, 0);                                                                     \
      OK(hipFree(dri));                                                                                        \
      OK(hipMalloc((void **)&dri, sizeof(int) * (size_t)nnz));                                                 \
      OK(alphasparse_dcu_csr2coo(h, drp, nnz, m, dri, ALPHA_SPARSE_INDEX_BASE_ZERO));                          \
      OK(hipMemcpy(dy, y0, sizeof(T) * (size_t)m, hipMemcpyHostToDevice));                                     \
      OK(alphasparse_dcu_##S##_coomv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, m, n, nnz, &al, dd, dv, dri, dci, dx, &be, dy)); \
      OK(hipDeviceSynchronize());                                                                              \
      OK(hipMemcpy(y, dy, sizeof(T) * (size_t)m, hipMemcpyDeviceToHost));                                      \
      cmp_##S("coomv", ref, y, m);                                                                             \
      ALPHA_INT width = 0;                                                                                     \
      OK(alphasparse_dcu_csr2ell_width(h, m, dd, drp, dd, &width));                                            \
      if (width > 0 && (long)width * m < (1l << 27)) {                                                         \
        T *dev = NULL;                                                                                         \
        int *dec = NULL;                                                                                       \
        OK(hipMalloc((void **)&dev, sizeof(T) * (size_t)width * (size_t)m));                                   \
        OK(hipMalloc((void **)&dec, sizeof(int) * (size_t)width * (size_t)m));                                 \
        OK(alphasparse_dcu_##S##csr2ell(h, m, dd, dv, drp, dci, dd, width, dev, dec));                         \
        OK(hipMemcpy(dy, y0, sizeof(T) * (size_t)m, hipMemcpyHostToDevice));                                   \
        OK(alphasparse_dcu_##S##_ellmv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, m, n, &al, dd, dev, dec, width, dx, &be, dy)); \
        OK(hipDeviceSynchronize());                                                                            \
        OK(hipMemcpy(y, dy, sizeof(T) * (size_t)m, hipMemcpyDeviceToHost));                                    \
        cmp_##S("ellmv", ref, y, m);                                                                           \
        OK(hipFree(dev));                                                                                      \
        OK(hipFree(dec));                                                                                      \
      }                                                                                                        \
      /* csrmm: row-major, column-major N/N with a workspace beyond the handle's first MiB, N/T */             \
      {                                                                                                        \
        const int cols = 300;                                                                                  \
        T *dB = NULL, *dC = NULL;                                                                              \
        OK(hipMalloc((void **)&dB, sizeof(T) * (size_t)big * cols));                                           \
        OK(hipMalloc((void **)&dC, sizeof(T) * (size_t)big * cols));                                           \
        OK(hipMemset(dB, 0, sizeof(T) * (size_t)big * cols));                                                  \
        OK(hipMemset(dC, 0, sizeof(T) * (size_t)big * cols));                                                  \
        OK(alphasparse_dcu_##S##_csrmm(h, 0, 0, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, m, cols, n, nnz, &al, dd, dv, drp, dci, dB, cols, &be, dC, cols)); \
        OK(alphasparse_dcu_##S##_csrmm(h, 0, 0, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, m, cols, n, nnz, &al, dd, dv, drp, dci, dB, n, &be, dC, m)); \
        OK(alphasparse_dcu_##S##_csrmm(h, 0, 1, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, m, cols, n, nnz, &al, dd, dv, drp, dci, dB, cols, &be, dC, m)); \
        OK(alphasparse_dcu_##S##_csrmm(h, 0, 0, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, m, 24, n, nnz, &al, dd, dv, drp, dci, dB, 24, &be, dC, 24)); \
        OK(alphasparse_dcu_##S##_csrmm(h, 0, 0, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, m, 4, n, nnz, &al, dd, dv, drp, dci, dB, n, &be, dC, m)); \
        OK(hipDeviceSynchronize());                                                                            \
        OK(hipFree(dB));                                                                                       \
        OK(hipFree(dC));                                                                                       \
      }                                                                                                        \
      OK(alphasparse_dcu_destroy_mat_info(info));                                                              \
      OK(alphasparse_dcu_destroy_mat_descr(dd));                                                               \
      OK(hipFree(dri));                                                                                        \
      OK(hipFree(drp));                                                                                        \
      OK(hipFree(dci));                                                                                        \
      OK(hipFree(dv));                                                                                         \
      OK(hipFree(dx));                                                                                         \
      OK(hipFree(dy));                                                                                         \
    }                                                                                                          \
    free(val);                                                                                                 \
    free(x);                                                                                                   \
    free(y0);                                                                                                  \
    free(y);                                                                                                   \
    free(ref);                                                                                                 \
  }

REAL_SUITE(s, float, 2e-4)
REAL_SUITE(d, double, 1e-11)

/* ---- complex: host handles and the lazy raw-pointer path ------------------------------------- */
#define CX_SUITE(S, T, R)                                                                                      \
  static void suite_##S(alphasparse_dcu_handle_t h, const csr_t *a) {                                          \
    const int m = a->m, n = a->n, nnz = a->nnz;                                                                \
    if (nnz == 0) return;                                                                                      \
    T *val = (T *)malloc(sizeof(T) * (size_t)nnz);                                                             \
    for (int i = 0; i < nnz; ++i) { val[i].real = (R)a->v[i]; val[i].imag = (R)(0.5 * a->v[i]); }              \
    int big = m > n ? m : n;                                                                                   \
    T *x = (T *)malloc(sizeof(T) * (size_t)big * 4), *y = (T *)malloc(sizeof(T) * (size_t)big * 4);            \
    for (int i = 0; i < big * 4; ++i) { x[i].real = (R)urand(); x[i].imag = (R)urand(); y[i] = x[i]; }         \
    struct alpha_matrix_descr hd = {ALPHA_SPARSE_MATRIX_TYPE_GENERAL, ALPHA_SPARSE_FILL_MODE_LOWER, ALPHA_SPARSE_DIAG_NON_UNIT}; \
    T al = {(R)1.5, (R)-0.5}, be = {(R)0.5, (R)0.25};                                                          \
    alphasparse_matrix_t A = NULL;                                                                             \
    OK(alphasparse_##S##_create_csr(&A, ALPHA_SPARSE_INDEX_BASE_ZERO, m, n, a->rp, a->rp + 1, a->ci, val));    \
    for (int op = 0; op < 3; ++op) {                                                                           \
      OK(alphasparse_##S##_mv((alphasparse_operation_t)op, al, A, hd, x, be, y));                              \
      OK(alphasparse_##S##_mv_plain((alphasparse_operation_t)op, al, A, hd, x, be, y));                        \
      OK(alphasparse_##S##_mm((alphasparse_operation_t)op, al, A, hd, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, x, 4, 4, be, y, 4)); \
      OK(alphasparse_##S##_mm_plain((alphasparse_operation_t)op, al, A, hd, ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, x, 4, big, be, y, big)); \
    }                                                                                                          \
    OK(alphasparse_destroy(A));                                                                                \
    int *drp = (int *)dev_copy(a->rp, sizeof(int) * (size_t)(m + 1));                                          \
    int *dci = (int *)dev_copy(a->ci, sizeof(int) * (size_t)nnz);                                              \
    T *dv = (T *)dev_copy(val, sizeof(T) * (size_t)nnz);                                                       \
    T *dx = (T *)dev_copy(x, sizeof(T) * (size_t)big), *dy = (T *)dev_copy(y, sizeof(T) * (size_t)big);        \
    alpha_dcu_matrix_descr_t dd;                                                                               \
    OK(alphasparse_dcu_create_mat_descr(&dd));                                                                 \
    alphasparse_dcu_mat_info_t info = NULL;                                                                    \
    OK(alphasparse_dcu_create_mat_info(&info));                                                                \
    for (int op = 0; op < 3; ++op) {                                                                           \
      OK(alphasparse_dcu_##S##_csrmv(h, (alphasparse_operation_t)op, m, n, nnz, &al, dd, dv, drp, dci, NULL, dx, &be, dy)); \
      OK(alphasparse_dcu_##S##_csrmv_analysis(h, (alphasparse_operation_t)op, m, n, nnz, dd, dv, drp, dci, info)); \
      OK(alphasparse_dcu_##S##_csrmv(h, (alphasparse_operation_t)op, m, n, nnz, &al, dd, dv, drp, dci, info, dx, &be, dy)); \
    }                                                                                                          \
    OK(hipDeviceSynchronize());                                                                                \
    OK(alphasparse_dcu_destroy_mat_info(info));                                                                \
    OK(alphasparse_dcu_destroy_mat_descr(dd));                                                                 \
    OK(hipFree(drp));                                                                                          \
    OK(hipFree(dci));                                                                                          \
    OK(hipFree(dv));                                                                                           \
    OK(hipFree(dx));                                                                                           \
    OK(hipFree(dy));                                                                                           \
    free(val);                                                                                                 \
    free(x);                                                                                                   \
    free(y);                                                                                                   \
  }

CX_SUITE(c, ALPHA_Complex8, float)
CX_SUITE(z, ALPHA_Complex16, double)

/* device arrays that are freed and reallocated under the library's feet: stale records must not be used */
static void churn(alphasparse_dcu_handle_t h) {
  alpha_dcu_matrix_descr_t dd;
  OK(alphasparse_dcu_create_mat_descr(&dd));
  for (int it = 0; it < 40; ++it) {
    csr_t a = make_csr(200 + (int)(rnd() % 3000), 100 + (int)(rnd() % 3000), 1 + (int)(rnd() % 500));
    if (a.nnz == 0) {
      free_csr(&a);
      continue;
    }
    float *val = (float *)malloc(sizeof(float) * (size_t)a.nnz);
    for (int i = 0; i < a.nnz; ++i) val[i] = (float)a.v[i];
    float *x = (float *)malloc(sizeof(float) * (size_t)a.n), *y = (float *)calloc((size_t)a.m, sizeof(float));
    for (int i = 0; i < a.n; ++i) x[i] = (float)urand();
    int *drp = (int *)dev_copy(a.rp, sizeof(int) * (size_t)(a.m + 1));
    int *dci = (int *)dev_copy(a.ci, sizeof(int) * (size_t)a.nnz);
    float *dv = (float *)dev_copy(val, sizeof(float) * (size_t)a.nnz);
    float *dx = (float *)dev_copy(x, sizeof(float) * (size_t)a.n), *dy = (float *)dev_copy(y, sizeof(float) * (size_t)a.m);
    float al = 1.0f, be = 0.0f;
    alphasparse_dcu_mat_info_t info = NULL;
    if (it % 3 == 0) {
      OK(alphasparse_dcu_create_mat_info(&info));
      OK(alphasparse_dcu_s_csrmv_analysis(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, a.m, a.n, a.nnz, dd, dv, drp, dci, info));
    }
    OK(alphasparse_dcu_s_csrmv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, a.m, a.n, a.nnz, &al, dd, dv, drp, dci, info, dx, &be, dy));
    OK(hipDeviceSynchronize());
    OK(hipMemcpy(y, dy, sizeof(float) * (size_t)a.m, hipMemcpyDeviceToHost));
    double *ref = (double *)malloc(sizeof(double) * (size_t)a.m);
    float *zero = (float *)calloc((size_t)a.m, sizeof(float));
    ref_mv_s(&a, 0, 1.0, x, 0.0, zero, ref);
    cmp_s("churn csrmv", ref, y, a.m);
    /* every third analysed bundle is destroyed, the others leak their record on purpose (callers do) */
    if (info && it % 2 == 0) OK(alphasparse_dcu_destroy_mat_info(info));
    OK(hipFree(drp));
    OK(hipFree(dci));
    OK(hipFree(dv));
    OK(hipFree(dx));
    OK(hipFree(dy));
    free(ref);
    free(zero);
    free(val);
    free(x);
    free(y);
    free_csr(&a);
  }
  OK(alphasparse_dcu_destroy_mat_descr(dd));
}

static void generic(alphasparse_dcu_handle_t h, const csr_t *a) {
  if (a->nnz == 0) return;
  double *x = (double *)malloc(sizeof(double) * (size_t)a->n), *y0 = (double *)calloc((size_t)a->m, sizeof(double));
  double *y = (double *)malloc(sizeof(double) * (size_t)a->m), *ref = (double *)malloc(sizeof(double) * (size_t)a->m);
  for (int i = 0; i < a->n; ++i) x[i] = urand();
  int *drp = (int *)dev_copy(a->rp, sizeof(int) * (size_t)(a->m + 1));
  int *dci = (int *)dev_copy(a->ci, sizeof(int) * (size_t)a->nnz);
  double *dv = (double *)dev_copy(a->v, sizeof(double) * (size_t)a->nnz);
  double *dx = (double *)dev_copy(x, sizeof(double) * (size_t)a->n), *dy = (double *)dev_copy(y0, sizeof(double) * (size_t)a->m);
  struct alpha_dcu_matrix_descr dd = {ALPHA_SPARSE_MATRIX_TYPE_GENERAL, ALPHA_SPARSE_FILL_MODE_LOWER, ALPHA_SPARSE_DIAG_NON_UNIT, ALPHA_SPARSE_INDEX_BASE_ZERO};
  alphasparse_dcu_mat_info_t info = NULL;
  OK(alphasparse_dcu_create_mat_info(&info));
  struct _alphasparse_dcu_spmat_descr mat;
  memset(&mat, 0, sizeof mat);
  mat.init = true;
  mat.rows = a->m;
  mat.cols = a->n;
  mat.nnz = a->nnz;
  mat.row_data = drp;
  mat.col_data = dci;
  mat.val_data = dv;
  mat.row_type = mat.col_type = ALPHA_SPARSE_DCU_INDEXTYPE_I32;
  mat.data_type = ALPHA_SPARSE_DATATYPE_DOUBLE;
  mat.idx_base = ALPHA_SPARSE_INDEX_BASE_ZERO;
  mat.format = ALPHA_SPARSE_FORMAT_CSR;
  mat.descr = &dd;
  mat.info = info;
  struct _alphasparse_dcu_dnvec_descr vx = {true, a->n, dx, ALPHA_SPARSE_DATATYPE_DOUBLE}, vy = {true, a->m, dy, ALPHA_SPARSE_DATATYPE_DOUBLE};
  double al = 1.5, be = 0.0;
  size_t bs = 0;
  OK(alphasparse_dcu_spmv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, &al, &mat, &vx, &be, &vy, ALPHA_SPARSE_DATATYPE_DOUBLE, ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, &bs, NULL));
  void *buf = NULL;
  OK(hipMalloc(&buf, bs ? bs : 4));
  OK(alphasparse_dcu_spmv(h, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, &al, &mat, &vx, &be, &vy, ALPHA_SPARSE_DATATYPE_DOUBLE, ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, &bs, buf));
  OK(hipDeviceSynchronize());
  OK(hipMemcpy(y, dy, sizeof(double) * (size_t)a->m, hipMemcpyDeviceToHost));
  ref_mv_d(a, 0, 1.5, x, 0.0, y0, ref);
  cmp_d("generic spmv", ref, y, a->m);
  OK(alphasparse_dcu_destroy_mat_info(info));
  OK(hipFree(buf));
  OK(hipFree(drp));
  OK(hipFree(dci));
  OK(hipFree(dv));
  OK(hipFree(dx));
  OK(hipFree(dy));
  free(x);
  free(y0);
  free(y);
  free(ref);
}

/* base-one arrays, a second handle with its own stream, clears and destroys in odd orders */
static void odd_orders(const csr_t *a) {
  if (a->nnz == 0) return;
  alphasparse_dcu_handle_t h2 = NULL;
  OK(alphasparse_dcu_get_handle(&h2));
  hipStream_t st = NULL;
  OK(hipStreamCreate(&st));
  h2->stream = st;
  int *rp1 = (int *)malloc(sizeof(int) * (size_t)(a->m + 1)), *ci1 = (int *)malloc(sizeof(int) * (size_t)a->nnz);
  for (int i = 0; i <= a->m; ++i) rp1[i] = a->rp[i] + 1;
  for (int i = 0; i < a->nnz; ++i) ci1[i] = a->ci[i] + 1;
  /* both vectors hold max(m, n) entries: the transposed multiply below reads m of x and writes n of y */
  const size_t big = (size_t)(a->m > a->n ? a->m : a->n);
  double *x = (double *)malloc(sizeof(double) * big), *y0 = (double *)calloc(big, sizeof(double));
  double *y = (double *)malloc(sizeof(double) * big), *ref = (double *)malloc(sizeof(double) * big);
  for (size_t i = 0; i < big; ++i) x[i] = urand();
  int *drp = (int *)dev_copy(rp1, sizeof(int) * (size_t)(a->m + 1));
  int *dci = (int *)dev_copy(ci1, sizeof(int) * (size_t)a->nnz);
  double *dv = (double *)dev_copy(a->v, sizeof(double) * (size_t)a->nnz);
  double *dx = (double *)dev_copy(x, sizeof(double) * big), *dy = (double *)dev_copy(y0, sizeof(double) * big);
  alpha_dcu_matrix_descr_t dd;
  OK(alphasparse_dcu_create_mat_descr(&dd));
  dd->base = ALPHA_SPARSE_INDEX_BASE_ONE;
  alphasparse_dcu_mat_info_t never = NULL, info = NULL;
  OK(alphasparse_dcu_create_mat_info(&never));
  OK(alphasparse_dcu_csrmv_clear(h2, never));
  OK(alphasparse_dcu_destroy_mat_info(never));
  OK(alphasparse_dcu_create_mat_info(&info));
  double al = 1.5, be = 0.0;
  ref_mv_d(a, 0, 1.5, x, 0.0, y0, ref);
  for (int k = 0; k < 3; ++k) {
    OK(alphasparse_dcu_d_csrmv_analysis(h2, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, a->m, a->n, a->nnz, dd, dv, drp, dci, info));
    OK(alphasparse_dcu_d_csrmv_analysis(h2, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, a->m, a->n, a->nnz, dd, dv, drp, dci, info));
    OK(alphasparse_dcu_d_csrmv(h2, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, a->m, a->n, a->nnz, &al, dd, dv, drp, dci, info, dx, &be, dy));
    OK(hipStreamSynchronize(st));
    OK(hipMemcpy(y, dy, sizeof(double) * (size_t)a->m, hipMemcpyDeviceToHost));
    cmp_d("base one", ref, y, a->m);
    OK(alphasparse_dcu_csrmv_clear(h2, info));
    OK(alphasparse_dcu_csrmv_clear(h2, info));
  }
  /* multiply after the clear: falls back to the unanalysed route */
  OK(alphasparse_dcu_d_csrmv(h2, ALPHA_SPARSE_OPERATION_TRANSPOSE, a->m, a->n, a->nnz, &al, dd, dv, drp, dci, info, dx, &be, dy));
  OK(hipStreamSynchronize(st));
  OK(hipMemcpy(y, dy, sizeof(double) * (size_t)a->n, hipMemcpyDeviceToHost));
  ref_mv_d(a, 1, 1.5, x, 0.0, y0, ref);
  cmp_d("transposed after clear", ref, y, a->n);
  /* empty shapes return before anything is dereferenced */
  OK(alphasparse_dcu_d_csrmv(h2, ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, 0, a->n, 0, &al, dd, dv, drp, dci, info, dx, &be, dy));
  OK(alphasparse_dcu_d_csrmm(h2, 0, 0, ALPHA_SPARSE_LAYOUT_ROW_MAJOR, a->m, 0, a->n, a->nnz, &al, dd, dv, drp, dci, dx, 1, &be, dy, 1));
  OK(alphasparse_dcu_destroy_mat_info(info));
  OK(alphasparse_dcu_destroy_mat_descr(dd));
  OK(alphasparse_dcu_destory_handle(h2));
  free(h2);
  OK(hipStreamDestroy(st));
  OK(hipFree(drp));
  OK(hipFree(dci));
  OK(hipFree(dv));
  OK(hipFree(dx));
  OK(hipFree(dy));
  free(rp1);
  free(ci1);
  free(x);
  free(y0);
  free(y);
  free(ref);
}

int main(void) {
  alphasparse_dcu_handle_t h = NULL;
  OK(alphasparse_dcu_get_handle(&h));
  /* status paths that touch no device memory */
  EXPECT(alphasparse_dcu_s_csrmv(NULL, 0, 1, 1, 1, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL), ALPHA_SPARSE_STATUS_INVALID_HANDLE);
  EXPECT(alphasparse_destroy(NULL), ALPHA_SPARSE_STATUS_SUCCESS);
  const int shapes[][3] = {{2000, 1500, 300}, {64, 64, 64}, {1, 1, 1}, {5000, 7000, 3000}, {300, 40000, 20}, {40000, 300, 200}};
  for (unsigned s = 0; s < sizeof shapes / sizeof shapes[0]; ++s) {
    csr_t a = make_csr(shapes[s][0], shapes[s][1], shapes[s][2]);
    printf("shape %d x %d, %d entries\n", a.m, a.n, a.nnz);
    fflush(stdout);
    suite_s(h, &a);
    suite_d(h, &a);
    suite_c(h, &a);
    suite_z(h, &a);
    generic(h, &a);
    odd_orders(&a);
    free_csr(&a);
  }
  printf("churn\n");
  fflush(stdout);
  churn(h);
  printf("churn done\n");
  fflush(stdout);
  OK(alphasparse_dcu_destory_handle(h));
  free(h);
  printf("lifecycle: all passed\n");
  fflush(stdout);
#if defined(__has_feature)
#if __has_feature(address_sanitizer)
  _exit(0); /* the sanitizer runtime's own device allocator asserts while the GPU runtime unloads at exit */
#endif
#endif
  return 0;
}
