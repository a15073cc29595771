/* Device SpMV entry points: analysis, clear, raw-pointer csrmv, handle-based
 * mv_dcu.  Argument validation reproduces the reference's order so that every
 * status code is the one a caller of the reference would get. */
#include <stdlib.h>

#include "internal.h"

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_CSR spmat_csr_s_t
#define ASAMD_COO spmat_coo_s_t
#define ASAMD_ELL spmat_ell_s_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT
#define ASAMD_IS_COMPLEX 0
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_CSR spmat_csr_d_t
#define ASAMD_COO spmat_coo_d_t
#define ASAMD_ELL spmat_ell_d_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE
#define ASAMD_IS_COMPLEX 0
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_CSR spmat_csr_c_t
#define ASAMD_COO spmat_coo_c_t
#define ASAMD_ELL spmat_ell_c_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX
#define ASAMD_IS_COMPLEX 1
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_CSR spmat_csr_z_t
#define ASAMD_COO spmat_coo_z_t
#define ASAMD_ELL spmat_ell_z_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX
#define ASAMD_IS_COMPLEX 1
#include "csrmv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_COO
#undef ASAMD_ELL
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX

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
