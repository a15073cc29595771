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
  const int is_s = mat->data_type == ALPHA_SPARSE_DATATYPE_FLOAT;
  const int is_d = mat->data_type == ALPHA_SPARSE_DATATYPE_DOUBLE;
  /* dimensions travel as 64-bit in the descriptor and as ALPHA_INT in the typed calls */
  if (mat->rows < 0 || mat->cols < 0 || mat->nnz < 0 || mat->rows > 0x7fffffff || mat->cols > 0x7fffffff ||
      mat->nnz > 0x7fffffff)
    return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  const ALPHA_INT m = (ALPHA_INT)mat->rows, n = (ALPHA_INT)mat->cols, nnz = (ALPHA_INT)mat->nnz;

  if (temp_buffer == NULL) {
    /* size query; the analysis rides on it (reference :58-76) */
    if (buffer_size == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    *buffer_size = 4;
    if (mat->format == ALPHA_SPARSE_FORMAT_CSR &&
        (alg == ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT || alg == ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE) &&
        !mat->analysed && (is_s || is_d)) {
      alphasparse_status_t st =
          is_s ? alphasparse_dcu_s_csrmv_analysis(handle, trans, m, n, nnz, mat->descr, (const float *)mat->val_data,
                                                  (const ALPHA_INT *)mat->row_data,
                                                  (const ALPHA_INT *)mat->col_data, mat->info)
               : alphasparse_dcu_d_csrmv_analysis(handle, trans, m, n, nnz, mat->descr, (const double *)mat->val_data,
                                                  (const ALPHA_INT *)mat->row_data,
                                                  (const ALPHA_INT *)mat->col_data, mat->info);
      if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
      mat->analysed = true;
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
  }

  if (!is_s && !is_d) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED; /* complex types are not built */
  switch (mat->format) {
    case ALPHA_SPARSE_FORMAT_COO:
      return is_s ? alphasparse_dcu_s_coomv(handle, trans, m, n, nnz, (const float *)alpha, mat->descr,
                                            (const float *)mat->val_data, (const ALPHA_INT *)mat->row_data,
                                            (const ALPHA_INT *)mat->col_data, (const float *)x->values,
                                            (const float *)beta, (float *)y->values)
                  : alphasparse_dcu_d_coomv(handle, trans, m, n, nnz, (const double *)alpha, mat->descr,
                                            (const double *)mat->val_data, (const ALPHA_INT *)mat->row_data,
                                            (const ALPHA_INT *)mat->col_data, (const double *)x->values,
                                            (const double *)beta, (double *)y->values);
    case ALPHA_SPARSE_FORMAT_CSR:
      /* the info bundle is only honoured if the analysis above filled it */
      return is_s ? alphasparse_dcu_s_csrmv(handle, trans, m, n, nnz, (const float *)alpha, mat->descr,
                                            (const float *)mat->val_data, (const ALPHA_INT *)mat->row_data,
                                            (const ALPHA_INT *)mat->col_data, mat->info,
                                            (const float *)x->values, (const float *)beta, (float *)y->values)
                  : alphasparse_dcu_d_csrmv(handle, trans, m, n, nnz, (const double *)alpha, mat->descr,
                                            (const double *)mat->val_data, (const ALPHA_INT *)mat->row_data,
                                            (const ALPHA_INT *)mat->col_data, mat->info,
                                            (const double *)x->values, (const double *)beta, (double *)y->values);
    case ALPHA_SPARSE_FORMAT_ELL:
      /* the descriptor's nnz field carries the ELL width (reference :226) */
      return is_s ? alphasparse_dcu_s_ellmv(handle, trans, m, n, (const float *)alpha, mat->descr,
                                            (const float *)mat->val_data, (const ALPHA_INT *)mat->col_data, nnz,
                                            (const float *)x->values, (const float *)beta, (float *)y->values)
                  : alphasparse_dcu_d_ellmv(handle, trans, m, n, (const double *)alpha, mat->descr,
                                            (const double *)mat->val_data, (const ALPHA_INT *)mat->col_data, nnz,
                                            (const double *)x->values, (const double *)beta, (double *)y->values);
    default:
      return ALPHA_SPARSE_STATUS_NOT_SUPPORTED; /* COO_AOS and the rest, as in the reference (:143-147, :274) */
  }
}
