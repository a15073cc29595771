/* alphasparse_?_mv / alphasparse_?_mm: the reference's host-pointer entry
 * points (include/alphasparse/spapi.h:685-699, :899-923).  In the reference
 * they run OpenMP CPU kernels; here the multiplication runs on the GPU: the
 * matrix is mirrored to the device on first use, x / X is staged in, y / Y
 * staged out on the default handle's stream, and the call returns after the
 * result has landed in host memory (these entry points are synchronous in the
 * reference too).  There is no CPU compute path: without a usable device the
 * status is the mapped HIP error. */
#include <stdlib.h>

#include "internal.h"

/* Make sure A has a device mirror built by this library and return its record. */
static alphasparse_status_t asamd_host_prepare(const alphasparse_matrix_t A, alphasparse_dcu_handle_t *h,
                                               asamd_record **rec) {
  alphasparse_status_t st = asamd_default_handle(h);
  if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
  spmat_csr_s_t *m = (spmat_csr_s_t *)A->mat; /* the payloads of all value types share the layout */
  asamd_record *r = m->d_row_ptr ? asamd_registry_find(ASAMD_KEY_MATRIX, m->d_row_ptr) : NULL;
  if (!r) {
    switch (A->datatype) {
      case ALPHA_SPARSE_DATATYPE_FLOAT: st = host2device_s_csr(A); break;
      case ALPHA_SPARSE_DATATYPE_DOUBLE: st = host2device_d_csr(A); break;
      case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX: st = host2device_c_csr(A); break;
      default: st = host2device_z_csr(A); break;
    }
    if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
    r = asamd_registry_find(ASAMD_KEY_MATRIX, m->d_row_ptr);
    if (!r) return ALPHA_SPARSE_STATUS_INTERNAL_ERROR;
  }
  /* The host arrays stay the caller's to change (alphasparse_?_export_csr hands out pointers into them, and
   * the reference's CPU kernels read them on every call).  A cheap fingerprint of a sample of the values tells
   * when they have been rewritten: the mirror's values are copied again and the copies that its analysis
   * keeps are refreshed.  (A change of a few single values can slip through the sample: host2device_?_csr
   * mirrors afresh.) */
  static const size_t kElem[4] = {4, 8, 8, 16};
  const size_t elem = kElem[A->datatype & 3];
  const size_t nnz = (size_t)(m->rows > 0 && m->rows_end[m->rows - 1] > 0 ? m->rows_end[m->rows - 1] : 0);
  if (nnz > 0 && r->plan) {
    const uint64_t fp = asamd_host_fingerprint(m->values, nnz, elem);
    if (fp != r->host_val_fingerprint) {
      ASAMD_HIP_STATUS(hipStreamSynchronize((*h)->stream));
      ASAMD_HIP_STATUS(hipMemcpy(m->d_values, m->values, nnz * elem, hipMemcpyHostToDevice));
      ASAMD_HIP_STATUS(asamd_csr_plan_refresh_values((*h)->stream, r->plan, m->d_row_ptr, m->d_col_indx, m->d_values));
      r->host_val_fingerprint = fp;
    }
  }
  *rec = r;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

/* Grow the record's device staging buffers to at least the given sizes. */
static alphasparse_status_t asamd_host_stage(asamd_record *rec, size_t in_bytes, size_t out_bytes) {
  if (rec->d_in_bytes < in_bytes) {
    if (rec->d_in) (void)hipFree(rec->d_in);
    rec->d_in = NULL;
    rec->d_in_bytes = 0;
    ASAMD_HIP_STATUS(hipMalloc(&rec->d_in, in_bytes));
    rec->d_in_bytes = in_bytes;
  }
  if (rec->d_out_bytes < out_bytes) {
    if (rec->d_out) (void)hipFree(rec->d_out);
    rec->d_out = NULL;
    rec->d_out_bytes = 0;
    ASAMD_HIP_STATUS(hipMalloc(&rec->d_out, out_bytes));
    rec->d_out_bytes = out_bytes;
  }
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

/* beta*y with the operation order of the reference's cmp_mule
 * (include/alphasparse/complex_compute.h:76-82, :103) */
#define ASAMD_CX_SCALE(R, y, b)                            \
  do {                                                     \
    const R re_ = (b).real * (y).real - (b).imag * (y).imag; \
    const R im_ = (b).imag * (y).real + (b).real * (y).imag; \
    (y).real = re_;                                        \
    (y).imag = im_;                                        \
  } while (0)

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_CSR spmat_csr_s_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT
#define ASAMD_IS_COMPLEX 0
#define ASAMD_IS_ZERO(v) ((v) == 0)
#define ASAMD_SCALE(y, b) ((y) *= (b))
#include "host_api.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_IS_ZERO
#undef ASAMD_SCALE

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_CSR spmat_csr_d_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE
#define ASAMD_IS_COMPLEX 0
#define ASAMD_IS_ZERO(v) ((v) == 0)
#define ASAMD_SCALE(y, b) ((y) *= (b))
#include "host_api.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_IS_ZERO
#undef ASAMD_SCALE

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_CSR spmat_csr_c_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX
#define ASAMD_IS_COMPLEX 1
#define ASAMD_IS_ZERO(v) ((v).real == 0 && (v).imag == 0)
#define ASAMD_SCALE(y, b) ASAMD_CX_SCALE(float, y, b)
#include "host_api.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_IS_ZERO
#undef ASAMD_SCALE

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_CSR spmat_csr_z_t
#define ASAMD_DT ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX
#define ASAMD_IS_COMPLEX 1
#define ASAMD_IS_ZERO(v) ((v).real == 0 && (v).imag == 0)
#define ASAMD_SCALE(y, b) ASAMD_CX_SCALE(double, y, b)
#include "host_api.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_CSR
#undef ASAMD_DT
#undef ASAMD_IS_COMPLEX
#undef ASAMD_IS_ZERO
#undef ASAMD_SCALE
