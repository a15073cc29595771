/* TEST INFRASTRUCTURE -- not part of the product.
 *
 * CPU restatement of the reference's complex-valued kernels on the CSR SpMV /
 * SpMM path (element types ALPHA_Complex8 / ALPHA_Complex16,
 * include/alphasparse/types.h:42-56).  Same rules as csr_oracle.c: used only by
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; compiled into
 * liboracle.so with -O2 -ffp-contract=off so that every operation below is
 * rounded on its own, in the order written.
 *
 * The complex arithmetic follows include/alphasparse/complex_compute.h as the
 * host compiler sees it (no __DCU__):
 *   cmp_mul    :76-82    z = x*y, four multiplications
 *   cmp_mule   :103      z = x*z
 *   cmp_madde  :158-164  d += a*b in the three-multiplication form
 *                        re += (a.re+a.im)*(b.re-b.im) + B - C,  im += B + C,
 *                        B = a.re*b.im, C = a.im*b.re
 *   cmp_conj   :22-26
 *
 * Pinning (tests/test_oracle_complex.py): numpy / scipy complex products in
 * higher precision on tiny and seeded matrices, closed forms (identity, alpha = 0,
 * real-valued inputs reduce to the real oracle's result pattern, conjugation
 * identities), and -- where it builds -- bit-for-bit agreement with the
 * reference's own sources compiled with -DCOMPLEX into oracle/_ref/.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

typedef struct { float real, imag; } oracle_c8;
typedef struct { double real, imag; } oracle_c16;

#define CX_FUNCS(C, R, S)                                                                     \
  static inline C S##_mul(C x, C y) {                                                         \
    R re = x.real * y.real - x.imag * y.imag;                                                 \
    R im = x.imag * y.real + x.real * y.imag;                                                 \
    C z = {re, im};                                                                           \
    return z;                                                                                 \
  }                                                                                           \
  static inline void S##_madde(C *d, C a, C b) {                                              \
    R B_ = a.real * b.imag;                                                                   \
    R C_ = a.imag * b.real;                                                                   \
    d->real += (a.real + a.imag) * (b.real - b.imag) + B_ - C_;                               \
    d->imag += B_ + C_;                                                                       \
  }                                                                                           \
  static inline C S##_conj(C a) {                                                             \
    C z = {a.real, -a.imag};                                                                  \
    return z;                                                                                 \
  }                                                                                           \
  /* device form of madde, complex_compute.h:139-146: two chained fmas per component */      \
  static inline void S##_madde_fma(C *d, C a, C b) {                                          \
    R re = FMA_##S(-a.imag, b.imag, FMA_##S(a.real, b.real, d->real));                        \
    R im = FMA_##S(a.real, b.imag, FMA_##S(a.imag, b.real, d->imag));                         \
    d->real = re;                                                                             \
    d->imag = im;                                                                             \
  }
#define FMA_c fmaf
#define FMA_z fma
CX_FUNCS(oracle_c8, float, c)
CX_FUNCS(oracle_c16, double, z)

/* src/plain/kernel/level2/mv/gemv/gemv_x_csr_plain.c:11-22 with ALPHA_Number complex:
 *   y[r] = beta*y[r] (mule); tmp = 0; tmp += val*x (madde) left to right; y[r] += alpha*tmp (madde) */
#define ORACLE_CX_MV_PLAIN(NAME, C, S)                                                        \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const C *values, C alpha, const C *x, C beta, C *y) {   \
    for (int32_t r = 0; r < m; r++) {                                                         \
      y[r] = S##_mul(beta, y[r]);                                                             \
      C tmp = {0, 0};                                                                         \
      for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++)                                \
        S##_madde(&tmp, values[ai], x[col_indx[ai]]);                                         \
      S##_madde(&y[r], alpha, tmp);                                                           \
    }                                                                                         \
  }
ORACLE_CX_MV_PLAIN(oracle_c_csrmv_plain, oracle_c8, c)
ORACLE_CX_MV_PLAIN(oracle_z_csrmv_plain, oracle_c16, z)

/* op(A) = A^T: src/plain/kernel/level2/mv/gemv/gemv_x_csr_trans_plain.c:10-24
 *   y[j] = beta*y[j]; per entry val = alpha*values[ai] (mul); y[col] += val*x[row] (madde)
 * op(A) = A^H: src/plain/kernel/level2/mv/gemv/gemv_c_csr_conj_plain.c:10-27
 *   the same with val = alpha*conj(values[ai]) */
#define ORACLE_CX_MV_TRANS(NAME, C, S, CONJ)                                                  \
  void NAME(int32_t m, int32_t n, const int32_t *rows_start, const int32_t *rows_end,        \
            const int32_t *col_indx, const C *values, C alpha, const C *x, C beta, C *y) {   \
    for (int32_t j = 0; j < n; ++j) y[j] = S##_mul(beta, y[j]);                               \
    for (int32_t i = 0; i < m; i++) {                                                         \
      for (int32_t ai = rows_start[i]; ai < rows_end[i]; ai++) {                              \
        C val = CONJ ? S##_conj(values[ai]) : values[ai];                                     \
        val = S##_mul(alpha, val);                                                            \
        S##_madde(&y[col_indx[ai]], val, x[i]);                                               \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_CX_MV_TRANS(oracle_c_csrmv_trans_plain, oracle_c8, c, 0)
ORACLE_CX_MV_TRANS(oracle_z_csrmv_trans_plain, oracle_c16, z, 0)
ORACLE_CX_MV_TRANS(oracle_c_csrmv_conj_plain, oracle_c8, c, 1)
ORACLE_CX_MV_TRANS(oracle_z_csrmv_conj_plain, oracle_c16, z, 1)

/* src/plain/kernel/level3/mm/gemm/gemm_x_csr_row_plain.c:6-21 (row-major dense operands):
 *   Y[r,:] = beta*Y[r,:]; per entry val = alpha*values[ai]; Y[r,c] += val*X[col,c] */
#define ORACLE_CX_MM_ROW(NAME, C, S)                                                          \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const C *values, C alpha, const C *x, int32_t columns,  \
            int32_t ldx, C beta, C *y, int32_t ldy) {                                         \
    for (int32_t r = 0; r < m; ++r) {                                                         \
      C *Y = &y[(size_t)r * ldy];                                                             \
      for (int32_t c = 0; c < columns; c++) Y[c] = S##_mul(beta, Y[c]);                       \
      for (int32_t ai = rows_start[r]; ai < rows_end[r]; ai++) {                              \
        C val = S##_mul(alpha, values[ai]);                                                   \
        const C *X = &x[(size_t)col_indx[ai] * ldx];                                          \
        for (int32_t c = 0; c < columns; ++c) S##_madde(&Y[c], val, X[c]);                    \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_CX_MM_ROW(oracle_c_csrmm_row_plain, oracle_c8, c)
ORACLE_CX_MM_ROW(oracle_z_csrmm_row_plain, oracle_c16, z)

/* src/plain/kernel/level3/mm/gemm/gemm_x_csr_col_plain.c:6-19 (column-major dense operands):
 *   ctmp = sum values[ai]*X[col,cc] (madde); Y[cr,cc] = beta*Y[cr,cc]; Y[cr,cc] += alpha*ctmp */
#define ORACLE_CX_MM_COL(NAME, C, S)                                                          \
  void NAME(int32_t m, const int32_t *rows_start, const int32_t *rows_end,                   \
            const int32_t *col_indx, const C *values, C alpha, const C *x, int32_t columns,  \
            int32_t ldx, C beta, C *y, int32_t ldy) {                                         \
    for (int32_t cc = 0; cc < columns; ++cc) {                                                \
      for (int32_t cr = 0; cr < m; ++cr) {                                                    \
        C ctmp = {0, 0};                                                                      \
        for (int32_t ai = rows_start[cr]; ai < rows_end[cr]; ++ai)                            \
          S##_madde(&ctmp, values[ai], x[(size_t)cc * ldx + col_indx[ai]]);                   \
        C *out = &y[(size_t)cc * ldy + cr];                                                   \
        *out = S##_mul(beta, *out);                                                           \
        S##_madde(out, alpha, ctmp);                                                          \
      }                                                                                       \
    }                                                                                         \
  }
ORACLE_CX_MM_COL(oracle_c_csrmm_col_plain, oracle_c8, c)
ORACLE_CX_MM_COL(oracle_z_csrmm_col_plain, oracle_c16, z)

/* src/plain/kernel/level2/mv/gemv/gemv_x_coo_plain.c:11-24: y[i] = beta*y[i]; per entry in
 * storage order v = val*x[col] (mul); y[row] += alpha*v (madde).  Indices zero-based. */
#define ORACLE_CX_COOMV(NAME, C, S)                                                           \
  void NAME(int32_t m, int32_t nnz, const int32_t *row_indx, const int32_t *col_indx,        \
            const C *values, C alpha, const C *x, C beta, C *y) {                            \
    for (int32_t i = 0; i < m; i++) y[i] = S##_mul(beta, y[i]);                               \
    for (int32_t i = 0; i < nnz; i++) {                                                       \
      C v = S##_mul(values[i], x[col_indx[i]]);                                               \
      S##_madde(&y[row_indx[i]], alpha, v);                                                   \
    }                                                                                         \
  }
ORACLE_CX_COOMV(oracle_c_coomv_plain, oracle_c8, c)
ORACLE_CX_COOMV(oracle_z_coomv_plain, oracle_c16, z)

/* ELL SpMV after the reference's device kernel, src/kernel/dcu/level2/mv/dcu_gemv_x_ell.cpp:22-42
 * (there is no CPU kernel for this format): sum = 0; per slot with col < n:
 * sum = madde(sum, val, x[col]) in the device's fma form; y = beta*y + alpha*sum (mul, mul, add). */
#define ORACLE_CX_ELLMV(NAME, C, S)                                                           \
  void NAME(int32_t m, int32_t n, C alpha, const C *ell_val, const int32_t *ell_col,         \
            int32_t width, const C *x, C beta, C *y) {                                        \
    for (int32_t ar = 0; ar < m; ar++) {                                                      \
      C sum = {0, 0};                                                                         \
      for (int32_t i = 0; i < width; i++) {                                                   \
        size_t idx = (size_t)m * i + ar;                                                      \
        int32_t col = ell_col[idx];                                                           \
        if (col >= 0 && col < n) S##_madde_fma(&sum, ell_val[idx], x[col]);                   \
      }                                                                                       \
      C left = S##_mul(beta, y[ar]), right = S##_mul(alpha, sum);                             \
      y[ar].real = left.real + right.real;                                                    \
      y[ar].imag = left.imag + right.imag;                                                    \
    }                                                                                         \
  }
ORACLE_CX_ELLMV(oracle_c_ellmv, oracle_c8, c)
ORACLE_CX_ELLMV(oracle_z_ellmv, oracle_c16, z)

/* CSR -> ELL for complex values: src/core/format/convert_ell_x_coo.c:46-79 (zero-filled
 * arrays, slot i of row j at [i*m + j]); returns -1 where the reference aborts (:53-56). */
#define ORACLE_CX_CSR2ELL(NAME, C)                                                            \
  int32_t NAME(int32_t m, const int32_t *row_ptr, const int32_t *col_indx, const C *values,  \
               int32_t csr_base, int32_t ell_base, int32_t ld, C *ell_val, int32_t *ell_col) { \
    if ((uint64_t)ld * (uint64_t)m >= ((uint64_t)1 << 31)) return -1;                         \
    const C zero = {0, 0};                                                                    \
    for (size_t k = 0; k < (size_t)ld * m; ++k) {                                             \
      ell_val[k] = zero;                                                                      \
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
ORACLE_CX_CSR2ELL(oracle_c_csr2ell, oracle_c8)
ORACLE_CX_CSR2ELL(oracle_z_csr2ell, oracle_c16)
