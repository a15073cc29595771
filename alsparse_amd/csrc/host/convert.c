/* Device format conversions CSR -> COO and CSR -> ELL.  The reference only
 * declares these (include/alphasparse/spapi_dcu.h:3113-3118, :3303-3332);
 * argument checks follow the pattern of its other device entry points
 * (handle, then descriptors, then sizes, quick return, then pointers). */
#include <stdint.h>

#include "internal.h"

alphasparse_status_t alphasparse_dcu_csr2coo(alphasparse_dcu_handle_t handle,
                                             const ALPHA_INT *csr_row_ptr, ALPHA_INT nnz,
                                             ALPHA_INT m, ALPHA_INT *coo_row_ind,
                                             alphasparse_index_base_t idx_base) {
  if (handle == NULL) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  if (idx_base != ALPHA_SPARSE_INDEX_BASE_ZERO && idx_base != ALPHA_SPARSE_INDEX_BASE_ONE)
    return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (nnz < 0 || m < 0) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (nnz == 0 || m == 0) return ALPHA_SPARSE_STATUS_SUCCESS;
  if (csr_row_ptr == NULL || coo_row_ind == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  /* the handle's scratch holds the table of chunk rows whenever it is large enough (1 MiB: up to 2^31 entries) */
  ASAMD_HIP_STATUS(asamd_csr2coo_ws(handle->stream, csr_row_ptr, nnz, m, coo_row_ind, (int32_t)idx_base,
                                    handle->buffer, handle->buffer_size));
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

static int descr_ok(const alpha_dcu_matrix_descr_t d) {
  return d->base == ALPHA_SPARSE_INDEX_BASE_ZERO || d->base == ALPHA_SPARSE_INDEX_BASE_ONE;
}

alphasparse_status_t alphasparse_dcu_csr2ell_width(alphasparse_dcu_handle_t handle, ALPHA_INT m,
                                                   const alpha_dcu_matrix_descr_t csr_descr,
                                                   const ALPHA_INT *csr_row_ptr,
                                                   const alpha_dcu_matrix_descr_t ell_descr,
                                                   ALPHA_INT *ell_width) {
  if (handle == NULL) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  if (csr_descr == NULL || ell_descr == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (!descr_ok(csr_descr) || !descr_ok(ell_descr)) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (csr_descr->type != ALPHA_SPARSE_MATRIX_TYPE_GENERAL ||
      ell_descr->type != ALPHA_SPARSE_MATRIX_TYPE_GENERAL)
    return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  if (m < 0) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (ell_width == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (m == 0) {
    *ell_width = 0;
    return ALPHA_SPARSE_STATUS_SUCCESS;
  }
  if (csr_row_ptr == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  ASAMD_HIP_STATUS(asamd_csr2ell_width(handle->stream, m, csr_row_ptr, ell_width));
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

#define ASAMD_CSR2ELL(NAME, T, KERNEL)                                                             \
  alphasparse_status_t NAME(alphasparse_dcu_handle_t handle, ALPHA_INT m,                          \
                            const alpha_dcu_matrix_descr_t csr_descr, const T *csr_val,            \
                            const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,            \
                            const alpha_dcu_matrix_descr_t ell_descr, ALPHA_INT ell_width,         \
                            T *ell_val, ALPHA_INT *ell_col_ind) {                                  \
    if (handle == NULL) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;                                 \
    if (csr_descr == NULL || ell_descr == NULL) return ALPHA_SPARSE_STATUS_INVALID_POINTER;        \
    if (!descr_ok(csr_descr) || !descr_ok(ell_descr)) return ALPHA_SPARSE_STATUS_INVALID_VALUE;    \
    if (csr_descr->type != ALPHA_SPARSE_MATRIX_TYPE_GENERAL ||                                     \
        ell_descr->type != ALPHA_SPARSE_MATRIX_TYPE_GENERAL)                                       \
      return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;                                                    \
    if (m < 0 || ell_width < 0) return ALPHA_SPARSE_STATUS_INVALID_VALUE;                          \
    /* the host converter refuses width*m >= 2^31 (convert_ell_x_coo.c:53-56) */                  \
    if ((uint64_t)ell_width * (uint64_t)m >= ((uint64_t)1 << 31))                                  \
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;                                                    \
    if (m == 0 || ell_width == 0) return ALPHA_SPARSE_STATUS_SUCCESS;                              \
    if (csr_val == NULL || csr_row_ptr == NULL || csr_col_ind == NULL || ell_val == NULL ||        \
        ell_col_ind == NULL)                                                                       \
      return ALPHA_SPARSE_STATUS_INVALID_POINTER;                                                  \
    if (ASAMD_MISALIGNED(T, csr_val) || ASAMD_MISALIGNED(T, ell_val))                              \
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;                                                    \
    ASAMD_HIP_STATUS(KERNEL(handle->stream, m, csr_val, csr_row_ptr, csr_col_ind,                  \
                            (int32_t)csr_descr->base, (int32_t)ell_descr->base, ell_width,         \
                            ell_val, ell_col_ind));                                                \
    return ALPHA_SPARSE_STATUS_SUCCESS;                                                            \
  }

ASAMD_CSR2ELL(alphasparse_dcu_scsr2ell, float, asamd_s_csr2ell)
ASAMD_CSR2ELL(alphasparse_dcu_dcsr2ell, double, asamd_d_csr2ell)
ASAMD_CSR2ELL(alphasparse_dcu_ccsr2ell, ALPHA_Complex8, asamd_c_csr2ell)
ASAMD_CSR2ELL(alphasparse_dcu_zcsr2ell, ALPHA_Complex16, asamd_z_csr2ell)
