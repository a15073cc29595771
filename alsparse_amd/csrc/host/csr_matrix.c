/* CSR matrix handles: construction, export, device mirror, destruction.
 * Reference behaviour: src/core/format/alphasparse_x_create_csr.c:7-57,
 * alphasparse_x_export_csr.c:5-26, host2device_x_csr.cpp:14-41,
 * src/core/op_/alphasparse_destroy.c:186-195, destroy_x_csr.c:5-13. */
#include <stdlib.h>

#include "internal.h"

static size_t asamd_round64(size_t n) { return (n + 63) & ~(size_t)63; }

static void asamd_release_mirror(void *d_row_ptr, void *d_col, void *d_val) {
  asamd_registry_erase(ASAMD_KEY_MATRIX, d_row_ptr);
  (void)hipFree(d_row_ptr);
  (void)hipFree(d_col);
  (void)hipFree(d_val);
}

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_CSR spmat_csr_s_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT
#include "csr_matrix.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_CSR spmat_csr_d_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE
#include "csr_matrix.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_CSR spmat_csr_c_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX
#include "csr_matrix.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_CSR spmat_csr_z_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX
#include "csr_matrix.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT

alphasparse_status_t alphasparse_destroy(alphasparse_matrix_t A) {
  if (!A) return ALPHA_SPARSE_STATUS_SUCCESS;
  if (A->mat) {
    if (A->format != ALPHA_SPARSE_FORMAT_CSR && A->format != ALPHA_SPARSE_FORMAT_COO &&
        A->format != ALPHA_SPARSE_FORMAT_ELL)
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    if (A->datatype < ALPHA_SPARSE_DATATYPE_FLOAT || A->datatype > ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX)
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    if (A->format == ALPHA_SPARSE_FORMAT_ELL) { /* src/core/format/destroy_x_ell.c */
      spmat_ell_s_t *e = (spmat_ell_s_t *)A->mat;
      (void)hipFree(e->d_values);
      (void)hipFree(e->d_indices);
      free(e->values);
      free(e->indices);
      free(e);
      free(A);
      return ALPHA_SPARSE_STATUS_SUCCESS;
    }
    if (A->format == ALPHA_SPARSE_FORMAT_COO) { /* src/core/format/destroy_x_coo.c */
      spmat_coo_s_t *c = (spmat_coo_s_t *)A->mat;
      (void)hipFree(c->d_values);
      (void)hipFree(c->d_rows_indx);
      (void)hipFree(c->d_cols_indx);
      free(c->values);
      free(c->row_indx);
      free(c->col_indx);
      free(c);
      free(A);
      return ALPHA_SPARSE_STATUS_SUCCESS;
    }
    /* the payload structs of all value types share one layout up to the value pointer types */
    spmat_csr_s_t *m = (spmat_csr_s_t *)A->mat;
    if (m->d_row_ptr && asamd_registry_find(ASAMD_KEY_MATRIX, m->d_row_ptr))
      asamd_release_mirror(m->d_row_ptr, m->d_col_indx, m->d_values);
    free(m->values);
    free(m->rows_start); /* rows_end aliases rows_start + 1 */
    free(m->col_indx);
    free(m);
  }
  free(A);
  return ALPHA_SPARSE_STATUS_SUCCESS;
}
