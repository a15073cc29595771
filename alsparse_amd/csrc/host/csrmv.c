/* Device SpMV entry points: analysis, clear, raw-pointer csrmv, handle-based
 * mv_dcu.  Argument validation reproduces the reference's order so that every
 * status code is the one a caller of the reference would get. */
#include <stdlib.h>

#include "internal.h"

/* op = 0: A, 1: A^T (the values of alphasparse_operation_t); real types have no third operation */
static int asamd_s_csrmv_op(hipStream_t stream, asamd_csr_plan *plan, int32_t op, float alpha, const float *val,
                            const int32_t *row_ptr, const int32_t *col_ind, const float *x, float beta, float *y) {
  return op == 1 ? asamd_s_csrmv_trans(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y)
                 : asamd_s_csrmv(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

static int asamd_d_csrmv_op(hipStream_t stream, asamd_csr_plan *plan, int32_t op, double alpha, const double *val,
                            const int32_t *row_ptr, const int32_t *col_ind, const double *x, double beta,
                            double *y) {
  return op == 1 ? asamd_d_csrmv_trans(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y)
                 : asamd_d_csrmv(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_CSR spmat_csr_s_t
#define ASAMD_COO spmat_coo_s_t
#define ASAMD_ELL spmat_ell_s_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT
#define ASAMD_IS_COMPLEX 0
#define ASAMD_KERNEL_CSRMV_OP asamd_s_csrmv_op
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_KERNEL_CSRMV_OP

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_CSR spmat_csr_d_t
#define ASAMD_COO spmat_coo_d_t
#define ASAMD_ELL spmat_ell_d_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE
#define ASAMD_IS_COMPLEX 0
#define ASAMD_KERNEL_CSRMV_OP asamd_d_csrmv_op
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_KERNEL_CSRMV_OP

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_CSR spmat_csr_c_t
#define ASAMD_COO spmat_coo_c_t
#define ASAMD_ELL spmat_ell_c_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX
#define ASAMD_IS_COMPLEX 1
#define ASAMD_KERNEL_CSRMV_OP asamd_c_csrmv_op
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_KERNEL_CSRMV_OP

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_CSR spmat_csr_z_t
#define ASAMD_COO spmat_coo_z_t
#define ASAMD_ELL spmat_ell_z_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX
#define ASAMD_IS_COMPLEX 1
#define ASAMD_KERNEL_CSRMV_OP asamd_z_csrmv_op
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_KERNEL_CSRMV_OP

/* Declared at include/alphasparse/spapi_dcu.h:573 and never defined in the
 * reference; semantics taken from the declaration's rocSPARSE namesake:
 * forget the analysis attached to `info`. */
alphasparse_status_t alphasparse_dcu_csrmv_clear(alphasparse_dcu_handle_t handle,
                                                 alphasparse_dcu_mat_info_t info) {
  if (handle == NULL) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  if (info == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (asamd_registry_find(ASAMD_KEY_INFO, info)) {
    alphasparse_dcu_destroy_csrmv_info(info->csrmv_info);
    info->csrmv_info = NULL;
    asamd_registry_erase(ASAMD_KEY_INFO, info);
  }
  return ALPHA_SPARSE_STATUS_SUCCESS;
}
