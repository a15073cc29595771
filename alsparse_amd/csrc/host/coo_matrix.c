/* COO matrix handles and COO -> CSR conversion: what the reference's drivers
 * call between reading a coordinate file and exporting CSR arrays.
 * Reference behaviour: src/core/format/alphasparse_x_create_coo.c:7-48,
 * src/core/format/convert_csr_x_coo.c:14-81,
 * src/core/op_/alphasparse_convert_csr.c:125-141. */
#include <stdlib.h>
#include <string.h>

#include "internal.h"

#define ASAMD_CREATE_COO(NAME, T, COO, DT)                                                          \
  alphasparse_status_t NAME(alphasparse_matrix_t *A, const alphasparse_index_base_t indexing,       \
                            const ALPHA_INT rows, const ALPHA_INT cols, const ALPHA_INT nnz,        \
                            ALPHA_INT *row_indx, ALPHA_INT *col_indx, T *values) {                  \
    if (!A) return ALPHA_SPARSE_STATUS_INVALID_POINTER;                                             \
    *A = NULL;                                                                                      \
    if (rows <= 0 || cols <= 0 || nnz < 0) return ALPHA_SPARSE_STATUS_INVALID_VALUE;                \
    if (indexing != ALPHA_SPARSE_INDEX_BASE_ZERO && indexing != ALPHA_SPARSE_INDEX_BASE_ONE)        \
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;                                                     \
    if (nnz > 0 && (!row_indx || !col_indx || !values)) return ALPHA_SPARSE_STATUS_INVALID_POINTER; \
    const ALPHA_INT shift = indexing == ALPHA_SPARSE_INDEX_BASE_ONE ? 1 : 0;                        \
    alphasparse_matrix *AA = (alphasparse_matrix *)calloc(1, sizeof(*AA));                          \
    COO *mat = (COO *)calloc(1, sizeof(*mat));                                                      \
    const size_t cnt = (size_t)(nnz ? nnz : 1);                                                     \
    ALPHA_INT *r = (ALPHA_INT *)malloc(cnt * sizeof(ALPHA_INT));                                    \
    ALPHA_INT *c = (ALPHA_INT *)malloc(cnt * sizeof(ALPHA_INT));                                    \
    T *v = (T *)malloc(cnt * sizeof(T));                                                            \
    if (!AA || !mat || !r || !c || !v) {                                                            \
      free(AA); free(mat); free(r); free(c); free(v);                                               \
      return ALPHA_SPARSE_STATUS_ALLOC_FAILED;                                                      \
    }                                                                                               \
    for (ALPHA_INT i = 0; i < nnz; ++i) {                                                           \
      r[i] = row_indx[i] - shift;                                                                   \
      c[i] = col_indx[i] - shift;                                                                   \
      v[i] = values[i];                                                                             \
    }                                                                                               \
    mat->values = v;                                                                                \
    mat->row_indx = r;                                                                              \
    mat->col_indx = c;                                                                              \
    mat->rows = rows;                                                                               \
    mat->cols = cols;                                                                               \
    mat->nnz = nnz;                                                                                 \
    AA->mat = mat;                                                                                  \
    AA->format = ALPHA_SPARSE_FORMAT_COO;                                                           \
    AA->datatype = DT;                                                                              \
    *A = AA;                                                                                        \
    return ALPHA_SPARSE_STATUS_SUCCESS;                                                             \
  }
ASAMD_CREATE_COO(alphasparse_s_create_coo, float, spmat_coo_s_t, ALPHA_SPARSE_DATATYPE_FLOAT)
ASAMD_CREATE_COO(alphasparse_d_create_coo, double, spmat_coo_d_t, ALPHA_SPARSE_DATATYPE_DOUBLE)
ASAMD_CREATE_COO(alphasparse_c_create_coo, ALPHA_Complex8, spmat_coo_c_t, ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX)
ASAMD_CREATE_COO(alphasparse_z_create_coo, ALPHA_Complex16, spmat_coo_z_t, ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX)

/* bytes per value of a datatype tag, 0 for an unknown tag */
static size_t value_size(alphasparse_datatype_t dt) {
  switch (dt) {
    case ALPHA_SPARSE_DATATYPE_FLOAT: return sizeof(float);
    case ALPHA_SPARSE_DATATYPE_DOUBLE: return sizeof(double);
    case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX: return sizeof(ALPHA_Complex8);
    case ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX: return sizeof(ALPHA_Complex16);
    default: return 0;
  }
}

/* Position of every entry in (row, column) order, ties in source order: a
 * counting sort by row, then each row's slice ordered by (column, position). */
typedef struct {
  ALPHA_INT col;
  ALPHA_INT pos;
} col_pos;

static int col_pos_cmp(const void *a, const void *b) {
  const col_pos *x = (const col_pos *)a, *y = (const col_pos *)b;
  if (x->col != y->col) return x->col < y->col ? -1 : 1;
  return x->pos < y->pos ? -1 : (x->pos > y->pos);
}

alphasparse_status_t alphasparse_convert_csr(const alphasparse_matrix_t source,
                                             const alphasparse_operation_t operation,
                                             alphasparse_matrix_t *dest) {
  if (!source || !source->mat) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
  if (!dest) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  *dest = NULL;
  if (source->format != ALPHA_SPARSE_FORMAT_COO) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  const size_t vsize = value_size(source->datatype);
  if (vsize == 0) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (operation != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  /* the COO payloads of all value types share one layout up to the value pointer type */
  const spmat_coo_s_t *coo = (const spmat_coo_s_t *)source->mat;
  const ALPHA_INT m = coo->rows, nnz = coo->nnz;
  for (ALPHA_INT i = 0; i < nnz; ++i)
    if (coo->row_indx[i] < 0 || coo->row_indx[i] >= m || coo->col_indx[i] < 0 || coo->col_indx[i] >= coo->cols)
      return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  ALPHA_INT *offsets = (ALPHA_INT *)calloc((size_t)m + 1, sizeof(ALPHA_INT));
  ALPHA_INT *fill = (ALPHA_INT *)malloc(((size_t)m + 1) * sizeof(ALPHA_INT));
  col_pos *order = (col_pos *)malloc((size_t)(nnz ? nnz : 1) * sizeof(col_pos));
  ALPHA_INT *cols = (ALPHA_INT *)malloc((size_t)(nnz ? nnz : 1) * sizeof(ALPHA_INT));
  if (!offsets || !fill || !order || !cols) {
    free(offsets); free(fill); free(order); free(cols);
    return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  }
  for (ALPHA_INT i = 0; i < nnz; ++i) offsets[coo->row_indx[i] + 1]++;
  for (ALPHA_INT r = 0; r < m; ++r) offsets[r + 1] += offsets[r];
  memcpy(fill, offsets, ((size_t)m + 1) * sizeof(ALPHA_INT));
  for (ALPHA_INT i = 0; i < nnz; ++i) {
    const ALPHA_INT at = fill[coo->row_indx[i]]++;
    order[at].col = coo->col_indx[i];
    order[at].pos = i;
  }
  for (ALPHA_INT r = 0; r < m; ++r)
    qsort(order + offsets[r], (size_t)(offsets[r + 1] - offsets[r]), sizeof(col_pos), col_pos_cmp);
  for (ALPHA_INT i = 0; i < nnz; ++i) cols[i] = order[i].col;
  alphasparse_status_t st;
  /* values are moved as opaque vsize-byte items */
  char *vals = (char *)malloc((size_t)(nnz ? nnz : 1) * vsize);
  if (!vals) {
    st = ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  } else {
    const char *src = (const char *)coo->values;
    for (ALPHA_INT i = 0; i < nnz; ++i) memcpy(vals + (size_t)i * vsize, src + (size_t)order[i].pos * vsize, vsize);
    const alphasparse_index_base_t b0 = ALPHA_SPARSE_INDEX_BASE_ZERO;
    switch (source->datatype) {
      case ALPHA_SPARSE_DATATYPE_FLOAT:
        st = alphasparse_s_create_csr(dest, b0, m, coo->cols, offsets, offsets + 1, cols, (float *)vals);
        break;
      case ALPHA_SPARSE_DATATYPE_DOUBLE:
        st = alphasparse_d_create_csr(dest, b0, m, coo->cols, offsets, offsets + 1, cols, (double *)vals);
        break;
      case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX:
        st = alphasparse_c_create_csr(dest, b0, m, coo->cols, offsets, offsets + 1, cols, (ALPHA_Complex8 *)vals);
        break;
      default:
        st = alphasparse_z_create_csr(dest, b0, m, coo->cols, offsets, offsets + 1, cols, (ALPHA_Complex16 *)vals);
        break;
    }
    free(vals);
  }
  free(offsets);
  free(fill);
  free(order);
  free(cols);
  return st;
}

/* ---- COO -> ELL ------------------------------------------------------------- */
alphasparse_status_t alphasparse_convert_ell(const alphasparse_matrix_t source,
                                             const alphasparse_operation_t operation,
                                             alphasparse_matrix_t *dest) {
  if (!source || !source->mat) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
  if (!dest) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  *dest = NULL;
  if (source->format != ALPHA_SPARSE_FORMAT_COO) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  if (operation != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
  /* the reference goes COO -> CSR -> ELL as well (convert_ell_x_coo.c:11-14) */
  alphasparse_matrix_t csr = NULL;
  alphasparse_status_t st = alphasparse_convert_csr(source, operation, &csr);
  if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
  const spmat_csr_s_t *c = (const spmat_csr_s_t *)csr->mat; /* layouts agree up to the value type */
  const ALPHA_INT m = c->rows;
  ALPHA_INT ld = 0;
  for (ALPHA_INT r = 0; r < m; ++r) {
    const ALPHA_INT len = c->rows_end[r] - c->rows_start[r];
    if (len > ld) ld = len;
  }
  const size_t vsize = value_size(source->datatype);
  const uint64_t slots = (uint64_t)ld * (uint64_t)m;
  alphasparse_matrix *AA = NULL;
  spmat_ell_s_t *ell = NULL;
  void *vals = NULL;
  ALPHA_INT *idx = NULL;
  if (slots >= ((uint64_t)1 << 31)) {
    st = ALPHA_SPARSE_STATUS_INVALID_VALUE;
  } else {
    AA = (alphasparse_matrix *)calloc(1, sizeof(*AA));
    ell = (spmat_ell_s_t *)calloc(1, sizeof(*ell));
    vals = calloc(slots ? slots : 1, vsize);
    idx = (ALPHA_INT *)calloc(slots ? slots : 1, sizeof(ALPHA_INT));
    if (!AA || !ell || !vals || !idx) st = ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  }
  if (st == ALPHA_SPARSE_STATUS_SUCCESS) {
    for (ALPHA_INT r = 0; r < m; ++r) {
      const ALPHA_INT b = c->rows_start[r], e = c->rows_end[r];
      for (ALPHA_INT k = b; k < e; ++k) {
        const size_t at = (size_t)(k - b) * (size_t)m + (size_t)r;
        idx[at] = c->col_indx[k];
        memcpy((char *)vals + at * vsize, (const char *)c->values + (size_t)k * vsize, vsize);
      }
    }
    ell->values = (float *)vals;
    ell->indices = idx;
    ell->rows = m;
    ell->cols = c->cols;
    ell->ld = ld;
    AA->mat = ell;
    AA->format = ALPHA_SPARSE_FORMAT_ELL;
    AA->datatype = source->datatype;
    *dest = AA;
  } else {
    free(AA); free(ell); free(vals); free(idx);
  }
  (void)alphasparse_destroy(csr);
  return st;
}

#define ASAMD_EXPORT_ELL(NAME, T, ELL, DT)                                                        \
  alphasparse_status_t NAME(const alphasparse_matrix_t source, alphasparse_index_base_t *indexing, \
                            ALPHA_INT *rows, ALPHA_INT *cols, ALPHA_INT *width,                   \
                            ALPHA_INT **col_indx, T **values) {                                   \
    if (!source || !source->mat) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;                        \
    if (source->datatype != DT) return ALPHA_SPARSE_STATUS_INVALID_VALUE;                         \
    if (source->format != ALPHA_SPARSE_FORMAT_ELL) return ALPHA_SPARSE_STATUS_INVALID_VALUE;      \
    ELL *mat = (ELL *)source->mat;                                                                \
    *indexing = ALPHA_SPARSE_INDEX_BASE_ZERO;                                                     \
    *rows = mat->rows;                                                                            \
    *cols = mat->cols;                                                                            \
    *width = mat->ld;                                                                             \
    *col_indx = mat->indices;                                                                     \
    *values = mat->values;                                                                        \
    return ALPHA_SPARSE_STATUS_SUCCESS;                                                           \
  }
ASAMD_EXPORT_ELL(alphasparse_s_export_ell, float, spmat_ell_s_t, ALPHA_SPARSE_DATATYPE_FLOAT)
ASAMD_EXPORT_ELL(alphasparse_d_export_ell, double, spmat_ell_d_t, ALPHA_SPARSE_DATATYPE_DOUBLE)
ASAMD_EXPORT_ELL(alphasparse_c_export_ell, ALPHA_Complex8, spmat_ell_c_t, ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX)
ASAMD_EXPORT_ELL(alphasparse_z_export_ell, ALPHA_Complex16, spmat_ell_z_t, ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX)

/* ---- device mirrors of COO / ELL handles ------------------------------------
 * src/core/format/host2device_x_coo.cpp:14-40, host2device_x_ell.cpp:14-33.  The
 * reference refuses a COO handle whose `ordered` flag is clear (and never sets
 * it); coomv here takes entries in any order, so the flag is not consulted.  A
 * second call replaces the mirror. */
static alphasparse_status_t upload(void **dst, const void *src, size_t bytes) {
  *dst = NULL;
  hipError_t e = hipMalloc(dst, bytes ? bytes : 1);
  if (e == hipSuccess && bytes) e = hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    if (*dst) (void)hipFree(*dst);
    *dst = NULL;
  }
  return get_alphasparse_dcu_status_for_hip_status(e);
}

static alphasparse_status_t host2device_coo(alphasparse_matrix_t mtx, alphasparse_datatype_t dt, size_t vsize) {
  if (!mtx) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (mtx->format != ALPHA_SPARSE_FORMAT_COO || mtx->datatype != dt) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  spmat_coo_s_t *A = (spmat_coo_s_t *)mtx->mat;
  if (!A || !A->row_indx || !A->col_indx || !A->values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  (void)hipFree(A->d_rows_indx);
  (void)hipFree(A->d_cols_indx);
  (void)hipFree(A->d_values);
  A->d_rows_indx = A->d_cols_indx = NULL;
  A->d_values = NULL;
  const size_t nnz = (size_t)A->nnz;
  alphasparse_status_t st = upload((void **)&A->d_rows_indx, A->row_indx, nnz * sizeof(ALPHA_INT));
  if (st == ALPHA_SPARSE_STATUS_SUCCESS) st = upload((void **)&A->d_cols_indx, A->col_indx, nnz * sizeof(ALPHA_INT));
  if (st == ALPHA_SPARSE_STATUS_SUCCESS) st = upload((void **)&A->d_values, A->values, nnz * vsize);
  return st;
}
alphasparse_status_t host2device_s_coo(alphasparse_matrix_t mtx) {
  return host2device_coo(mtx, ALPHA_SPARSE_DATATYPE_FLOAT, sizeof(float));
}
alphasparse_status_t host2device_d_coo(alphasparse_matrix_t mtx) {
  return host2device_coo(mtx, ALPHA_SPARSE_DATATYPE_DOUBLE, sizeof(double));
}
alphasparse_status_t host2device_c_coo(alphasparse_matrix_t mtx) {
  return host2device_coo(mtx, ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX, sizeof(ALPHA_Complex8));
}
alphasparse_status_t host2device_z_coo(alphasparse_matrix_t mtx) {
  return host2device_coo(mtx, ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX, sizeof(ALPHA_Complex16));
}

static alphasparse_status_t host2device_ell(alphasparse_matrix_t mtx, alphasparse_datatype_t dt, size_t vsize) {
  if (!mtx) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (mtx->format != ALPHA_SPARSE_FORMAT_ELL || mtx->datatype != dt) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
  spmat_ell_s_t *A = (spmat_ell_s_t *)mtx->mat;
  if (!A || !A->indices || !A->values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  (void)hipFree(A->d_indices);
  (void)hipFree(A->d_values);
  A->d_indices = NULL;
  A->d_values = NULL;
  const size_t slots = (size_t)A->ld * (size_t)A->rows;
  alphasparse_status_t st = upload((void **)&A->d_indices, A->indices, slots * sizeof(ALPHA_INT));
  if (st == ALPHA_SPARSE_STATUS_SUCCESS) st = upload((void **)&A->d_values, A->values, slots * vsize);
  return st;
}
alphasparse_status_t host2device_s_ell(alphasparse_matrix_t mtx) {
  return host2device_ell(mtx, ALPHA_SPARSE_DATATYPE_FLOAT, sizeof(float));
}
alphasparse_status_t host2device_d_ell(alphasparse_matrix_t mtx) {
  return host2device_ell(mtx, ALPHA_SPARSE_DATATYPE_DOUBLE, sizeof(double));
}
alphasparse_status_t host2device_c_ell(alphasparse_matrix_t mtx) {
  return host2device_ell(mtx, ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX, sizeof(ALPHA_Complex8));
}
alphasparse_status_t host2device_z_ell(alphasparse_matrix_t mtx) {
  return host2device_ell(mtx, ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX, sizeof(ALPHA_Complex16));
}
