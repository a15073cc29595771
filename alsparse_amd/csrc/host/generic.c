/* Generic (descriptor-based) SpMV: a dispatcher over the typed entry points.
 * Check order of src/core/op_dcu/generic/alphasparse_dcu_spmv.cpp:30-56. */
#include "internal.h"

alphasparse_status_t alphasparse_dcu_spmv(alphasparse_dcu_handle_t handle, alphasparse_operation_t trans,
                                          const void *alpha, const alphasparse_dcu_spmat_descr_t mat,
                                          const alphasparse_dcu_dnvec_descr_t x, const void *beta,
                                          const alphasparse_dcu_dnvec_descr_t y,
                                          alphasparse_datatype_t compute_type,
                                          alphasparse_dcu_spmv_alg_t alg, size_t *buffer_size,
                                          void *temp_buffer) {
  if (handle == NULL) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  if (x == NULL || y == NULL || mat == NULL || alpha == NULL || beta == NULL)
    return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (!mat->init || !x->init || !y->init) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  /* no mixed precision */
  if (compute_type != mat->data_type || compute_type != x->data_type || compute_type != y->data_type)
    return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  if (mat->row_type != mat->col_type || mat->row_type != ALPHA_SPARSE_DCU_INDEXTYPE_I32)
    return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  if (mat->data_type < ALPHA_SPARSE_DATATYPE_FLOAT || mat->data_type > ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX)
    return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  /* dimensions travel as 64-bit in the descriptor and as ALPHA_INT in the typed calls */
  if (mat->rows < 0 || mat->cols < 0 || mat->nnz < 0 || mat->rows > 0x7fffffff || mat->cols > 0x7fffffff ||
      mat->nnz > 0x7fffffff)
    return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  const ALPHA_INT m = (ALPHA_INT)mat->rows, n = (ALPHA_INT)mat->cols, nnz = (ALPHA_INT)mat->nnz;
  const ALPHA_INT *rows = (const ALPHA_INT *)mat->row_data, *cols = (const ALPHA_INT *)mat->col_data;

  if (temp_buffer == NULL) {
    /* size query; the analysis rides on it (reference :58-76) */
    if (buffer_size == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    *buffer_size = 4;
    if (mat->format == ALPHA_SPARSE_FORMAT_CSR &&
        (alg == ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT || alg == ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE) &&
        !mat->analysed) {
      alphasparse_status_t st;
      switch (mat->data_type) {
#define ASAMD_ANALYSE(S, T)                                                                                  \
  st = alphasparse_dcu_##S##_csrmv_analysis(handle, trans, m, n, nnz, mat->descr, (const T *)mat->val_data, \
                                            rows, cols, mat->info)
        case ALPHA_SPARSE_DATATYPE_FLOAT: ASAMD_ANALYSE(s, float); break;
        case ALPHA_SPARSE_DATATYPE_DOUBLE: ASAMD_ANALYSE(d, double); break;
        case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX: ASAMD_ANALYSE(c, ALPHA_Complex8); break;
        default: ASAMD_ANALYSE(z, ALPHA_Complex16); break;
#undef ASAMD_ANALYSE
      }
      if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
      mat->analysed = true;
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
  }

  /* COO / CSR / ELL multiply in the matrix's value type; for ELL the descriptor's nnz field carries
   * the width (reference :226); the info bundle of a CSR matrix is only honoured if the analysis
   * above filled it; COO_AOS and the rest are not supported, as in the reference (:143-147, :274) */
#define ASAMD_MULTIPLY(S, T)                                                                                   \
  switch (mat->format) {                                                                                       \
    case ALPHA_SPARSE_FORMAT_COO:                                                                              \
      return alphasparse_dcu_##S##_coomv(handle, trans, m, n, nnz, (const T *)alpha, mat->descr,               \
                                         (const T *)mat->val_data, rows, cols, (const T *)x->values,           \
                                         (const T *)beta, (T *)y->values);                                     \
    case ALPHA_SPARSE_FORMAT_CSR:                                                                              \
      return alphasparse_dcu_##S##_csrmv(handle, trans, m, n, nnz, (const T *)alpha, mat->descr,               \
                                         (const T *)mat->val_data, rows, cols, mat->info,                      \
                                         (const T *)x->values, (const T *)beta, (T *)y->values);               \
    case ALPHA_SPARSE_FORMAT_ELL:                                                                              \
      return alphasparse_dcu_##S##_ellmv(handle, trans, m, n, (const T *)alpha, mat->descr,                    \
                                         (const T *)mat->val_data, cols, nnz, (const T *)x->values,            \
                                         (const T *)beta, (T *)y->values);                                     \
    default:                                                                                                   \
      return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;                                                                \
  }
  switch (mat->data_type) {
    case ALPHA_SPARSE_DATATYPE_FLOAT: ASAMD_MULTIPLY(s, float)
    case ALPHA_SPARSE_DATATYPE_DOUBLE: ASAMD_MULTIPLY(d, double)
    case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX: ASAMD_MULTIPLY(c, ALPHA_Complex8)
    default: ASAMD_MULTIPLY(z, ALPHA_Complex16)
  }
#undef ASAMD_MULTIPLY
}
