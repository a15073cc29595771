/*
 * alphasparse.h -- host-facing C API of the CSR SpMV / SpMM path.
 *
 * This header re-declares, with identical enum values, struct field order and
 * prototypes, the part of AlphaSparse's public C API that the CSR
 * matrix-vector / matrix-matrix path needs, so that a program written against
 * the reference headers links against libalpha_spblas.so from this repository
 * without source changes.  Only the s/d (fp32/fp64) CSR entry points exist.
 *
 * Every declaration cites the reference declaration it replaces
 * (paths relative to the AlphaSparse source tree).
 *
 * Behavioural difference to know about: alphasparse_?_mv / alphasparse_?_mm
 * take HOST pointers exactly as in the reference, but the multiplication runs
 * on the GPU (device mirror of the matrix, x/B staged in, y/C staged out).
 * There is no CPU compute path in this library: without a usable HIP device
 * these entry points return ALPHA_SPARSE_STATUS_EXECUTION_FAILED.
 */
#ifndef ALSPARSE_AMD_ALPHASPARSE_H
#define ALSPARSE_AMD_ALPHASPARSE_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar / index types: include/alphasparse/types.h:59-61 ------------ */
#ifndef ALPHA_INT
#define ALPHA_INT int32_t
#endif

/* complex scalars: include/alphasparse/types.h:42-56 */
#ifndef ALPHA_COMPLEX_TYPES_DEFINED
#define ALPHA_COMPLEX_TYPES_DEFINED
typedef struct { float real, imag; } ALPHA_Complex8;
typedef struct { double real, imag; } ALPHA_Complex16;
#endif

/* ---- status codes: include/alphasparse/spdef.h:8-19 ---------------------- */
typedef enum {
  ALPHA_SPARSE_STATUS_SUCCESS = 0,
  ALPHA_SPARSE_STATUS_NOT_INITIALIZED = 1,
  ALPHA_SPARSE_STATUS_ALLOC_FAILED = 2,
  ALPHA_SPARSE_STATUS_INVALID_VALUE = 3,
  ALPHA_SPARSE_STATUS_EXECUTION_FAILED = 4,
  ALPHA_SPARSE_STATUS_INTERNAL_ERROR = 5,
  ALPHA_SPARSE_STATUS_NOT_SUPPORTED = 6,
  ALPHA_SPARSE_STATUS_INVALID_POINTER = 7,
  ALPHA_SPARSE_STATUS_INVALID_HANDLE = 8
} alphasparse_status_t;

/* ---- op(A): include/alphasparse/spdef.h:22-27 ---------------------------- */
typedef enum {
  ALPHA_SPARSE_OPERATION_NON_TRANSPOSE = 0,
  ALPHA_SPARSE_OPERATION_TRANSPOSE = 1,
  ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE = 2
} alphasparse_operation_t;

/* ---- matrix type: include/alphasparse/spdef.h:32-41 ---------------------- */
typedef enum {
  ALPHA_SPARSE_MATRIX_TYPE_GENERAL = 0,
  ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC = 1,
  ALPHA_SPARSE_MATRIX_TYPE_HERMITIAN = 2,
  ALPHA_SPARSE_MATRIX_TYPE_TRIANGULAR = 3,
  ALPHA_SPARSE_MATRIX_TYPE_DIAGONAL = 4,
  ALPHA_SPARSE_MATRIX_TYPE_BLOCK_TRIANGULAR = 5,
  ALPHA_SPARSE_MATRIX_TYPE_BLOCK_DIAGONAL = 6
} alphasparse_matrix_type_t;

/* ---- index base: include/alphasparse/spdef.h:46-50 ----------------------- */
typedef enum {
  ALPHA_SPARSE_INDEX_BASE_ZERO = 0,
  ALPHA_SPARSE_INDEX_BASE_ONE = 1
} alphasparse_index_base_t;

/* ---- fill / diag: include/alphasparse/spdef.h:55-69 ---------------------- */
typedef enum {
  ALPHA_SPARSE_FILL_MODE_LOWER = 0,
  ALPHA_SPARSE_FILL_MODE_UPPER = 1
} alphasparse_fill_mode_t;

typedef enum {
  ALPHA_SPARSE_DIAG_NON_UNIT = 0,
  ALPHA_SPARSE_DIAG_UNIT = 1
} alphasparse_diag_type_t;

/* ---- dense layout: include/alphasparse/spdef.h:73-77 --------------------- */
typedef enum {
  ALPHA_SPARSE_LAYOUT_ROW_MAJOR = 0,
  ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR = 1
} alphasparse_layout_t;

/* ---- storage format tags: include/alphasparse/spdef.h:120-133 ------------ */
typedef enum {
  ALPHA_SPARSE_FORMAT_COO = 0,
  ALPHA_SPARSE_FORMAT_CSR = 1,
  ALPHA_SPARSE_FORMAT_CSC = 2,
  ALPHA_SPARSE_FORMAT_BSR = 3,
  ALPHA_SPARSE_FORMAT_SKY = 4,
  ALPHA_SPARSE_FORMAT_DIA = 5,
  ALPHA_SPARSE_FORMAT_ELL = 6,
  ALPHA_SPARSE_FORMAT_GEBSR = 7,
  ALPHA_SPARSE_FORMAT_HYB = 8,
  ALPHA_SPARSE_FORMAT_COO_AOS = 9,
  ALPHA_SPARSE_FORMAT_CSR5 = 10
} alphasparse_format_t;

/* ---- value type tags: include/alphasparse/spdef.h:137-143 ---------------- */
typedef enum {
  ALPHA_SPARSE_DATATYPE_FLOAT = 0,
  ALPHA_SPARSE_DATATYPE_DOUBLE = 1,
  ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX = 2,
  ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX = 3
} alphasparse_datatype_t;

/* ---- type-erased matrix handle: include/alphasparse/spdef.h:160-172 ------
 * `inspector` and `dcu_info` are never dereferenced by this library unless it
 * wrote them itself: handles built by other code leave them uninitialised. */
typedef void *alpha_internal_spmat;

typedef struct {
  alpha_internal_spmat mat;
  alphasparse_format_t format;
  alphasparse_datatype_t datatype;
  void *inspector;
  void *dcu_info;
} alphasparse_matrix;

typedef alphasparse_matrix *alphasparse_matrix_t;

/* ---- host-side descriptor (passed by value): spdef.h:178-183 ------------- */
struct alpha_matrix_descr {
  alphasparse_matrix_type_t type;
  alphasparse_fill_mode_t mode;
  alphasparse_diag_type_t diag;
};

/* ---- CSR payloads: include/alphasparse/spmat.h:174-188 and :203-216 ------
 * rows_end always aliases rows_start + 1 (three-array CSR inside a four-array
 * API, src/core/format/alphasparse_x_create_csr.c:25-29).  d_* is the device
 * mirror filled by host2device_?_csr. */
typedef struct {
  float *values;
  ALPHA_INT *rows_start;
  ALPHA_INT *rows_end;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  bool ordered;
  float *d_values;
  ALPHA_INT *d_row_ptr;
  ALPHA_INT *d_col_indx;
} spmat_csr_s_t;

typedef struct {
  double *values;
  ALPHA_INT *rows_start;
  ALPHA_INT *rows_end;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  bool ordered;
  double *d_values;
  ALPHA_INT *d_row_ptr;
  ALPHA_INT *d_col_indx;
} spmat_csr_d_t;

/* ---- COO payloads: include/alphasparse/spmat.h:73-86 and :96-110 ----------- */
typedef struct {
  float *values;
  ALPHA_INT *row_indx;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT nnz;
  bool ordered;
  ALPHA_INT *d_rows_indx;
  ALPHA_INT *d_cols_indx;
  float *d_values;
} spmat_coo_s_t;

typedef struct {
  double *values;
  ALPHA_INT *row_indx;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT nnz;
  bool ordered;
  ALPHA_INT *d_rows_indx;
  ALPHA_INT *d_cols_indx;
  double *d_values;
} spmat_coo_d_t;

/* include/alphasparse/spapi.h (create_coo); src/core/format/alphasparse_x_create_coo.c:7-48:
 * deep copy of nnz entries in the order given, indices shifted to base zero.
 * This is how the reference's drivers get from a coordinate file to a handle. */
alphasparse_status_t alphasparse_s_create_coo(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              const ALPHA_INT nnz, ALPHA_INT *row_indx,
                                              ALPHA_INT *col_indx, float *values);
alphasparse_status_t alphasparse_d_create_coo(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              const ALPHA_INT nnz, ALPHA_INT *row_indx,
                                              ALPHA_INT *col_indx, double *values);

/* src/core/op_/alphasparse_convert_csr.c:125-141 over
 * src/core/format/convert_csr_x_coo.c:14-81: entries sorted by (row, column),
 * duplicates kept.  Only a COO source and NON_TRANSPOSE are supported here.
 * The reference's qsort leaves the order of duplicate coordinates unspecified;
 * here they keep the order they had in the source. */
alphasparse_status_t alphasparse_convert_csr(const alphasparse_matrix_t source,
                                             const alphasparse_operation_t operation,
                                             alphasparse_matrix_t *dest);

/* ---- ELL payloads: include/alphasparse/spmat.h:617-636 (column-major, ld slots per row) */
typedef struct {
  float *values;
  ALPHA_INT *indices;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT ld;
  float *d_values;
  ALPHA_INT *d_indices;
} spmat_ell_s_t;

typedef struct {
  double *values;
  ALPHA_INT *indices;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT ld;
  double *d_values;
  ALPHA_INT *d_indices;
} spmat_ell_d_t;

/* src/core/op_/alphasparse_convert_ell.c:122-143 over src/core/format/convert_ell_x_coo.c:9-84:
 * COO -> (row, column)-sorted -> ELL with ld = longest row, slot i of row j at [i*rows + j],
 * padding (value 0, index 0); ld*rows >= 2^31 is refused (INVALID_VALUE; the reference exits).
 * Only a COO source and NON_TRANSPOSE are supported. */
alphasparse_status_t alphasparse_convert_ell(const alphasparse_matrix_t source,
                                             const alphasparse_operation_t operation,
                                             alphasparse_matrix_t *dest);
/* include/alphasparse/spapi.h:424-438; src/core/format/alphasparse_x_export_ell.c:5-24 */
alphasparse_status_t alphasparse_s_export_ell(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing, ALPHA_INT *rows,
                                              ALPHA_INT *cols, ALPHA_INT *width,
                                              ALPHA_INT **col_indx, float **values);
alphasparse_status_t alphasparse_d_export_ell(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing, ALPHA_INT *rows,
                                              ALPHA_INT *cols, ALPHA_INT *width,
                                              ALPHA_INT **col_indx, double **values);

/* ---- handle construction -------------------------------------------------
 * include/alphasparse/spapi.h:140-156; behaviour from
 * src/core/format/alphasparse_x_create_csr.c:7-57: deep copy, indices shifted
 * to base zero, nnz = rows_end[rows-1] - rows_start[0].  Unlike the reference
 * the device-side fields are zero-initialised. */
alphasparse_status_t alphasparse_s_create_csr(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              ALPHA_INT *rows_start, ALPHA_INT *rows_end,
                                              ALPHA_INT *col_indx, float *values);
alphasparse_status_t alphasparse_d_create_csr(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              ALPHA_INT *rows_start, ALPHA_INT *rows_end,
                                              ALPHA_INT *col_indx, double *values);

/* include/alphasparse/spapi.h:352-368; src/core/format/alphasparse_x_export_csr.c:5-26.
 * Returns borrowed internal pointers; always reports base zero. */
alphasparse_status_t alphasparse_s_export_csr(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing,
                                              ALPHA_INT *rows, ALPHA_INT *cols,
                                              ALPHA_INT **rows_start, ALPHA_INT **rows_end,
                                              ALPHA_INT **col_indx, float **values);
alphasparse_status_t alphasparse_d_export_csr(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing,
                                              ALPHA_INT *rows, ALPHA_INT *cols,
                                              ALPHA_INT **rows_start, ALPHA_INT **rows_end,
                                              ALPHA_INT **col_indx, double **values);

/* include/alphasparse/spapi.h:288; src/core/op_/alphasparse_destroy.c:186-195.
 * Also releases the device mirror and any cached analysis of the handle. */
alphasparse_status_t alphasparse_destroy(alphasparse_matrix_t A);

/* ---- y = alpha*op(A)*x + beta*y ------------------------------------------
 * include/alphasparse/spapi.h:685-699; validation order from
 * src/core/op/level2/alphasparse_x_mv.c:1662-1691.  x and y are host arrays. */
alphasparse_status_t alphasparse_s_mv(const alphasparse_operation_t operation, const float alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const float *x,
                                      const float beta, float *y);
alphasparse_status_t alphasparse_d_mv(const alphasparse_operation_t operation, const double alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const double *x,
                                      const double beta, double *y);

/* ---- Y = alpha*op(A)*X + beta*Y ------------------------------------------
 * include/alphasparse/spapi.h:899-923; validation order from
 * src/core/op/level3/alphasparse_x_mm.c:2305-2338.  x and y are host arrays.  op(A) = A^T (A^H for
 * complex types) multiplies with a CSR copy of the transpose kept with the handle's device mirror,
 * as src/kernel/x86_64/level3/mm/gemm/gemm_x_csr_row_trans.c does per call. */
alphasparse_status_t alphasparse_s_mm(const alphasparse_operation_t operation, const float alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const float *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const float beta, float *y, const ALPHA_INT ldy);
alphasparse_status_t alphasparse_d_mm(const alphasparse_operation_t operation, const double alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const double *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const double beta, double *y, const ALPHA_INT ldy);

/* ---- the reference's "plain" entry points ---------------------------------------
 * include/alphasparse/spapi_plain.h:13-43 (mv), :227-275 (mm); validation of
 * src/plain/op/alphasparse_x_mv_plain.c:537-564 and alphasparse_x_mm_plain.c:912-945.  In the
 * reference they run its serial, unoptimised CPU kernels and serve as the yardstick of its own tests.
 * Here they run on the GPU as well, through the unanalysed kernels that keep the plain kernels'
 * traversal: one lane per row (per element of Y) walking the entries in storage order, transposed
 * operations as a scatter.  Same arguments and status codes as alphasparse_?_mv / _mm. */
alphasparse_status_t alphasparse_s_mv_plain(const alphasparse_operation_t operation, const float alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const float *x,
                                      const float beta, float *y);
alphasparse_status_t alphasparse_s_mm_plain(const alphasparse_operation_t operation, const float alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const float *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const float beta, float *y, const ALPHA_INT ldy);
alphasparse_status_t alphasparse_d_mv_plain(const alphasparse_operation_t operation, const double alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const double *x,
                                      const double beta, double *y);
alphasparse_status_t alphasparse_d_mm_plain(const alphasparse_operation_t operation, const double alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const double *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const double beta, double *y, const ALPHA_INT ldy);
alphasparse_status_t alphasparse_c_mv_plain(const alphasparse_operation_t operation, const ALPHA_Complex8 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const ALPHA_Complex8 *x,
                                      const ALPHA_Complex8 beta, ALPHA_Complex8 *y);
alphasparse_status_t alphasparse_c_mm_plain(const alphasparse_operation_t operation, const ALPHA_Complex8 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const ALPHA_Complex8 *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const ALPHA_Complex8 beta, ALPHA_Complex8 *y, const ALPHA_INT ldy);
alphasparse_status_t alphasparse_z_mv_plain(const alphasparse_operation_t operation, const ALPHA_Complex16 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const ALPHA_Complex16 *x,
                                      const ALPHA_Complex16 beta, ALPHA_Complex16 *y);
alphasparse_status_t alphasparse_z_mm_plain(const alphasparse_operation_t operation, const ALPHA_Complex16 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const ALPHA_Complex16 *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const ALPHA_Complex16 beta, ALPHA_Complex16 *y, const ALPHA_INT ldy);

/* ---- complex element types ---------------------------------------------------
 * Payloads and entry points for ALPHA_Complex8 (c) and ALPHA_Complex16 (z), as their
 * fp32 / fp64 namesakes above: include/alphasparse/spmat.h:120-158 (COO), :231-273
 * (CSR), :638-659 (ELL); include/alphasparse/spapi.h:111-128 (create_coo), :158-174
 * (create_csr), :370-386 (export_csr), :440-454 (export_ell), :701-715 (mv), :923-945
 * (mm).  mv additionally accepts CONJUGATE_TRANSPOSE
 * (src/plain/kernel/level2/mv/gemv/gemv_c_csr_conj_plain.c:10-27). */
typedef struct {
  ALPHA_Complex8 *values;
  ALPHA_INT *rows_start;
  ALPHA_INT *rows_end;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  bool ordered;
  ALPHA_Complex8 *d_values;
  ALPHA_INT *d_row_ptr;
  ALPHA_INT *d_col_indx;
} spmat_csr_c_t;
typedef struct {
  ALPHA_Complex8 *values;
  ALPHA_INT *row_indx;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT nnz;
  bool ordered;
  ALPHA_INT *d_rows_indx;
  ALPHA_INT *d_cols_indx;
  ALPHA_Complex8 *d_values;
} spmat_coo_c_t;
alphasparse_status_t alphasparse_c_create_coo(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              const ALPHA_INT nnz, ALPHA_INT *row_indx,
                                              ALPHA_INT *col_indx, ALPHA_Complex8 *values);
typedef struct {
  ALPHA_Complex8 *values;
  ALPHA_INT *indices;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT ld;
  ALPHA_Complex8 *d_values;
  ALPHA_INT *d_indices;
} spmat_ell_c_t;
alphasparse_status_t alphasparse_c_export_ell(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing, ALPHA_INT *rows,
                                              ALPHA_INT *cols, ALPHA_INT *width,
                                              ALPHA_INT **col_indx, ALPHA_Complex8 **values);
alphasparse_status_t alphasparse_c_create_csr(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              ALPHA_INT *rows_start, ALPHA_INT *rows_end,
                                              ALPHA_INT *col_indx, ALPHA_Complex8 *values);
alphasparse_status_t alphasparse_c_export_csr(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing,
                                              ALPHA_INT *rows, ALPHA_INT *cols,
                                              ALPHA_INT **rows_start, ALPHA_INT **rows_end,
                                              ALPHA_INT **col_indx, ALPHA_Complex8 **values);
alphasparse_status_t alphasparse_c_mv(const alphasparse_operation_t operation, const ALPHA_Complex8 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const ALPHA_Complex8 *x,
                                      const ALPHA_Complex8 beta, ALPHA_Complex8 *y);
alphasparse_status_t alphasparse_c_mm(const alphasparse_operation_t operation, const ALPHA_Complex8 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const ALPHA_Complex8 *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const ALPHA_Complex8 beta, ALPHA_Complex8 *y, const ALPHA_INT ldy);

typedef struct {
  ALPHA_Complex16 *values;
  ALPHA_INT *rows_start;
  ALPHA_INT *rows_end;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  bool ordered;
  ALPHA_Complex16 *d_values;
  ALPHA_INT *d_row_ptr;
  ALPHA_INT *d_col_indx;
} spmat_csr_z_t;
typedef struct {
  ALPHA_Complex16 *values;
  ALPHA_INT *row_indx;
  ALPHA_INT *col_indx;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT nnz;
  bool ordered;
  ALPHA_INT *d_rows_indx;
  ALPHA_INT *d_cols_indx;
  ALPHA_Complex16 *d_values;
} spmat_coo_z_t;
alphasparse_status_t alphasparse_z_create_coo(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              const ALPHA_INT nnz, ALPHA_INT *row_indx,
                                              ALPHA_INT *col_indx, ALPHA_Complex16 *values);
typedef struct {
  ALPHA_Complex16 *values;
  ALPHA_INT *indices;
  ALPHA_INT rows;
  ALPHA_INT cols;
  ALPHA_INT ld;
  ALPHA_Complex16 *d_values;
  ALPHA_INT *d_indices;
} spmat_ell_z_t;
alphasparse_status_t alphasparse_z_export_ell(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing, ALPHA_INT *rows,
                                              ALPHA_INT *cols, ALPHA_INT *width,
                                              ALPHA_INT **col_indx, ALPHA_Complex16 **values);
alphasparse_status_t alphasparse_z_create_csr(alphasparse_matrix_t *A,
                                              const alphasparse_index_base_t indexing,
                                              const ALPHA_INT rows, const ALPHA_INT cols,
                                              ALPHA_INT *rows_start, ALPHA_INT *rows_end,
                                              ALPHA_INT *col_indx, ALPHA_Complex16 *values);
alphasparse_status_t alphasparse_z_export_csr(const alphasparse_matrix_t source,
                                              alphasparse_index_base_t *indexing,
                                              ALPHA_INT *rows, ALPHA_INT *cols,
                                              ALPHA_INT **rows_start, ALPHA_INT **rows_end,
                                              ALPHA_INT **col_indx, ALPHA_Complex16 **values);
alphasparse_status_t alphasparse_z_mv(const alphasparse_operation_t operation, const ALPHA_Complex16 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr, const ALPHA_Complex16 *x,
                                      const ALPHA_Complex16 beta, ALPHA_Complex16 *y);
alphasparse_status_t alphasparse_z_mm(const alphasparse_operation_t operation, const ALPHA_Complex16 alpha,
                                      const alphasparse_matrix_t A,
                                      const struct alpha_matrix_descr descr,
                                      const alphasparse_layout_t layout, const ALPHA_Complex16 *x,
                                      const ALPHA_INT columns, const ALPHA_INT ldx,
                                      const ALPHA_Complex16 beta, ALPHA_Complex16 *y, const ALPHA_INT ldy);

#include "alphasparse_util.h"

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_ALPHASPARSE_H */
