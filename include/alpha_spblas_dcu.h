/*
 * alpha_spblas_dcu.h -- GPU ("dcu") C API of the CSR SpMV / SpMM path.
 *
 * Re-declares, with identical field order, enum values and prototypes, the
 * part of AlphaSparse's device API that the CSR path needs.  The reference
 * header set is C++-only (it includes <vector> and uses references); this one
 * compiles as C11 and as C++.  All matrix / vector arguments of the
 * alphasparse_dcu_* entry points are DEVICE pointers; alpha and beta are HOST
 * pointers (the reference dereferences them on the host,
 * src/core/op_dcu/level2/alphasparse_dcu_x_csrmv.cpp:86-87).  Work is enqueued
 * on handle->stream and the call returns without synchronising.
 *
 * Every declaration cites the reference declaration it replaces
 * (paths relative to the AlphaSparse source tree).
 */
#ifndef ALSPARSE_AMD_ALPHA_SPBLAS_DCU_H
#define ALSPARSE_AMD_ALPHA_SPBLAS_DCU_H

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

#include "alphasparse.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- device descriptor: include/alphasparse/spdef.h:187-197 --------------- */
struct alpha_dcu_matrix_descr {
  alphasparse_matrix_type_t type;
  alphasparse_fill_mode_t mode;
  alphasparse_diag_type_t diag;
  alphasparse_index_base_t base;
};
typedef struct alpha_dcu_matrix_descr *alpha_dcu_matrix_descr_t;

/* include/alphasparse/spdef.h:198-207 */
typedef enum {
  ALPHA_SPARSE_DCU_POINTER_MODE_HOST = 0,
  ALPHA_SPARSE_DCU_POINTER_MODE_DVICE = 1
} alphasparse_dcu_pointer_mode_t;

typedef enum {
  ALPHA_SPARSE_DCU_LAYER_MODE_NONE = 0,
  ALPHA_SPARSE_DCU_LAYER_MODE_LOG_TRACE = 1,
  ALPHA_SPARSE_DCU_LAYER_MODE_LOG_BENCH = 2
} alphasparse_dcu_layer_mode_t;

/* ---- library handle: include/alphasparse/handle.h:18-46 -------------------
 * Field order is ABI.  `buffer` is device scratch owned by the handle; this
 * library uses it for merge-path carries and reduction partials. */
typedef struct {
  ALPHA_INT device;
  hipDeviceProp_t properties;
  ALPHA_INT wavefront_size;
  ALPHA_INT asic_rev;
  hipStream_t stream;
  alphasparse_dcu_pointer_mode_t pointer_mode;
  alphasparse_dcu_layer_mode_t layer_mode;
  size_t buffer_size;
  void *buffer;
  float *sone;
  double *done;
  ALPHA_Complex8 *cone;
  ALPHA_Complex16 *zone;
  bool check;
} alphasparse_dcu_handle;
typedef alphasparse_dcu_handle *alphasparse_dcu_handle_t;

/* ---- csrmv analysis record: include/alphasparse/handle.h:108-138 ----------
 * Public and caller-allocatable in the reference, so it cannot carry hidden
 * state: this library keeps its real analysis results in an internal registry
 * and only mirrors summary fields here.  `row_blocks` is never followed. */
enum csrgemv_algo { NONE_ALGO, SCALAR, VECTOR, VECTOR_MEMALIGN, ROW_PARTITION, ADAPTIVE };

struct _alphasparse_dcu_csrmv_info {
  bool algo_tuning;
  enum csrgemv_algo algo;
  ALPHA_INT iter;
  size_t size;
  unsigned long long *row_blocks;
  bool csr_adaptive_has_tuned;
  alphasparse_operation_t trans;
  ALPHA_INT m;
  ALPHA_INT n;
  ALPHA_INT nnz;
  const struct alpha_dcu_matrix_descr *descr;
  const void *csr_row_ptr;
  const void *csr_col_ind;
};
typedef struct _alphasparse_dcu_csrmv_info *alphasparse_dcu_csrmv_info_t;

/* the other analysis records are out of scope; only their slots exist */
typedef struct _alphasparse_dcu_trm_info *alphasparse_dcu_trm_info_t;
typedef struct _alphasparse_dcu_csrgemm_info *alphasparse_dcu_csrgemm_info_t;

/* ---- per-matrix info bundle: include/alphasparse/handle.h:168-199 --------- */
struct _alphasparse_dcu_mat_info {
  alphasparse_dcu_trm_info_t bsrsv_upper_info;
  alphasparse_dcu_trm_info_t bsrsv_lower_info;
  alphasparse_dcu_trm_info_t bsrsvt_upper_info;
  alphasparse_dcu_trm_info_t bsrsvt_lower_info;
  alphasparse_dcu_trm_info_t bsric0_info;
  alphasparse_dcu_trm_info_t bsrilu0_info;
  alphasparse_dcu_csrmv_info_t csrmv_info;
  alphasparse_dcu_trm_info_t csric0_info;
  alphasparse_dcu_trm_info_t csrilu0_info;
  alphasparse_dcu_trm_info_t csrsv_upper_info;
  alphasparse_dcu_trm_info_t csrsv_lower_info;
  alphasparse_dcu_trm_info_t csrsvt_upper_info;
  alphasparse_dcu_trm_info_t csrsvt_lower_info;
  alphasparse_dcu_trm_info_t csrsm_upper_info;
  alphasparse_dcu_trm_info_t csrsm_lower_info;
  alphasparse_dcu_trm_info_t csrsmt_upper_info;
  alphasparse_dcu_trm_info_t csrsmt_lower_info;
  alphasparse_dcu_csrgemm_info_t csrgemm_info;
  ALPHA_INT *zero_pivot;
  int boost_enable;
  int use_double_prec_tol;
  const void *boost_tol;
  const void *boost_val;
};
typedef struct _alphasparse_dcu_mat_info *alphasparse_dcu_mat_info_t;

/* ---- lifecycle: include/alphasparse/handle.h:325-332, :207-212 ------------
 * src/util_cpp/handle.cpp:55-64 (init_handle), :66-138 (get_handle: queries
 * the active device, allocates >= 1 MiB of scratch and the device constants),
 * :143-152 (destory_handle [sic]: frees device memory, not the host struct). */
alphasparse_status_t init_handle(alphasparse_dcu_handle_t *handle);
alphasparse_status_t alphasparse_dcu_get_handle(alphasparse_dcu_handle_t *handle);
alphasparse_status_t alphasparse_dcu_destory_handle(alphasparse_dcu_handle_t handle);

/* src/util_cpp/handle.cpp:248-272; defaults {GENERAL, LOWER, NON_UNIT, BASE_ZERO} */
alphasparse_status_t alphasparse_dcu_create_mat_descr(alpha_dcu_matrix_descr_t *descr);
alphasparse_status_t alphasparse_dcu_destroy_mat_descr(alpha_dcu_matrix_descr_t descr);

/* src/util_cpp/handle.cpp:274-319 (create: every slot NULL), :334-485 (destroy) */
alphasparse_status_t alphasparse_dcu_create_mat_info(alphasparse_dcu_mat_info_t *info);
alphasparse_status_t alphasparse_dcu_destroy_mat_info(alphasparse_dcu_mat_info_t info);

/* src/util_cpp/handle.cpp:154-197 */
alphasparse_status_t alphasparse_dcu_create_csrmv_info(alphasparse_dcu_csrmv_info_t *info,
                                                       bool algo_tuning);
alphasparse_status_t alphasparse_dcu_destroy_csrmv_info(alphasparse_dcu_csrmv_info_t info);

/* src/util_cpp/handle.cpp:21-53 */
alphasparse_status_t get_alphasparse_dcu_status_for_hip_status(hipError_t status);

/* ---- device mirror of a CSR handle ----------------------------------------
 * include/alphasparse/spapi_dcu.h:4402-4403; src/core/format/host2device_x_csr.cpp:14-41.
 * Additionally runs the CSR analysis once, so alphasparse_?_mv_dcu never pays
 * for it inside a timed loop. */
alphasparse_status_t host2device_s_csr(alphasparse_matrix_t A);
alphasparse_status_t host2device_d_csr(alphasparse_matrix_t A);
/* src/core/format/host2device_x_coo.cpp:14-40, host2device_x_ell.cpp:14-33: device
 * mirrors of COO / ELL handles, which alphasparse_?_mv_dcu then multiplies with
 * the coomv / ellmv kernels.  The COO `ordered` flag is not required. */
alphasparse_status_t host2device_s_coo(alphasparse_matrix_t mtx);
alphasparse_status_t host2device_d_coo(alphasparse_matrix_t mtx);
alphasparse_status_t host2device_s_ell(alphasparse_matrix_t mtx);
alphasparse_status_t host2device_d_ell(alphasparse_matrix_t mtx);

/* ---- handle-based SpMV on device vectors ----------------------------------
 * include/alphasparse/spapi_dcu.h:4441-4457;
 * src/core/op_dcu/generic/alphasparse_x_mv_dcu.cpp:16-103. */
alphasparse_status_t alphasparse_s_mv_dcu(alphasparse_dcu_handle_t handle,
                                          const alphasparse_operation_t operation,
                                          const float *alpha, const alphasparse_matrix_t A,
                                          const alpha_dcu_matrix_descr_t descr, const float *x,
                                          const float *beta, float *y);
alphasparse_status_t alphasparse_d_mv_dcu(alphasparse_dcu_handle_t handle,
                                          const alphasparse_operation_t operation,
                                          const double *alpha, const alphasparse_matrix_t A,
                                          const alpha_dcu_matrix_descr_t descr, const double *x,
                                          const double *beta, double *y);

/* ---- CSR analysis ----------------------------------------------------------
 * include/alphasparse/spapi_dcu.h:527-547; validation order from
 * src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:269-333.  Runs on the GPU:
 * row-length statistics and histogram, kernel selection, merge-path block
 * coordinates, and -- where a timing run inside the analysis shows that it pays --
 * a re-ordered copy of the matrix (tiled, ELL, transposed) that later multiplies
 * read INSTEAD of csr_val.  The reference's analysis keeps structure only
 * (:382-388), so the rule for callers is one the reference does not have:
 *   after writing new values into csr_val, call the analysis again
 * with the same arguments.  It notices that the structure arrays are unchanged
 * (a fingerprint of csr_row_ptr / csr_col_ind: one streaming pass) and only
 * gathers the values again; a changed structure is laid out afresh.  With the
 * environment variable ALSPARSE_AMD_ANALYSIS=structure no analysis keeps values
 * at all: multiplies then always read csr_val, at the speed of the row kernels.
 * Call alphasparse_dcu_csrmv_clear to forget an analysis. */
alphasparse_status_t alphasparse_dcu_s_csrmv_analysis(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const alpha_dcu_matrix_descr_t descr, const float *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info);
alphasparse_status_t alphasparse_dcu_d_csrmv_analysis(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const alpha_dcu_matrix_descr_t descr, const double *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info);

/* include/alphasparse/spapi_dcu.h:573 (declared, never defined in the reference) */
alphasparse_status_t alphasparse_dcu_csrmv_clear(alphasparse_dcu_handle_t handle,
                                                 alphasparse_dcu_mat_info_t info);

/* ---- y = alpha*op(A)*x + beta*y on raw device arrays -----------------------
 * include/alphasparse/spapi_dcu.h:577-605; validation order from
 * src/core/op_dcu/level2/alphasparse_dcu_x_csrmv.cpp:36-97.  Only
 * trans == NON_TRANSPOSE and descr->type == GENERAL are implemented; both index
 * bases are honoured (the reference validates descr->base but ignores it).
 * info may be NULL or uninitialised memory. */
alphasparse_status_t alphasparse_dcu_s_csrmv(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const float *alpha, const alpha_dcu_matrix_descr_t descr, const float *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info,
    const float *x, const float *beta, float *y);
alphasparse_status_t alphasparse_dcu_d_csrmv(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const double *alpha, const alpha_dcu_matrix_descr_t descr,
    const double *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    alphasparse_dcu_mat_info_t info, const double *x, const double *beta, double *y);

/* ---- C = alpha*op(A)*op(B) + beta*C on raw device arrays -------------------
 * include/alphasparse/spapi_dcu.h:1190-1226; validation order from
 * src/core/op_dcu/level3/alphasparse_dcu_x_csrmm.cpp:54-219.  A is m x k,
 * C is m x n.  Implemented: trans_A == NON_TRANSPOSE with
 *   row-major    B (k x n), trans_B == NON_TRANSPOSE   (the reference returns
 *                NOT_SUPPORTED here; src/kernel/dcu/level3/mm/csrmm/dcu_gemm_x_csr_row.cpp:35)
 *   column-major B (k x n), trans_B == NON_TRANSPOSE
 *   column-major B stored n x k, trans_B == TRANSPOSE. */
alphasparse_status_t alphasparse_dcu_s_csrmm(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans_A,
    alphasparse_operation_t trans_B, alphasparse_layout_t layout, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT k, ALPHA_INT nnz, const float *alpha, const alpha_dcu_matrix_descr_t descr,
    const float *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const float *B, ALPHA_INT ldb, const float *beta, float *C, ALPHA_INT ldc);
alphasparse_status_t alphasparse_dcu_d_csrmm(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans_A,
    alphasparse_operation_t trans_B, alphasparse_layout_t layout, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT k, ALPHA_INT nnz, const double *alpha, const alpha_dcu_matrix_descr_t descr,
    const double *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const double *B, ALPHA_INT ldb, const double *beta, double *C, ALPHA_INT ldc);

/* ---- CSR -> COO row indices -------------------------------------------------
 * include/alphasparse/spapi_dcu.h:3113-3118 (declared, never defined in the
 * reference).  Output convention from the host converter
 * src/core/format/convert_coo_x_csr.c:30-37: coo_row_ind[k] = r for
 * k in [row_ptr[r], row_ptr[r+1]); idx_base shifts both the input offsets and
 * the output indices. */
alphasparse_status_t alphasparse_dcu_csr2coo(alphasparse_dcu_handle_t handle,
                                             const ALPHA_INT *csr_row_ptr, ALPHA_INT nnz,
                                             ALPHA_INT m, ALPHA_INT *coo_row_ind,
                                             alphasparse_index_base_t idx_base);

/* ---- CSR -> ELL --------------------------------------------------------------
 * include/alphasparse/spapi_dcu.h:3303-3308 and :3312-3332 (declared, never
 * defined in the reference).  Output convention from the host converter
 * src/core/format/convert_ell_x_coo.c:46-79: width = longest row; arrays of
 * width*m entries, column-major (slot i of row j at [i*m + j],
 * include/alphasparse/handle.h:252-254); padding is value 0 and index 0 (plus
 * the ELL base); width*m >= 2^31 is an error (INVALID_VALUE here, where the
 * reference host code exits).  ell_width is a HOST pointer. */
alphasparse_status_t alphasparse_dcu_csr2ell_width(alphasparse_dcu_handle_t handle, ALPHA_INT m,
                                                   const alpha_dcu_matrix_descr_t csr_descr,
                                                   const ALPHA_INT *csr_row_ptr,
                                                   const alpha_dcu_matrix_descr_t ell_descr,
                                                   ALPHA_INT *ell_width);
alphasparse_status_t alphasparse_dcu_scsr2ell(
    alphasparse_dcu_handle_t handle, ALPHA_INT m, const alpha_dcu_matrix_descr_t csr_descr,
    const float *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const alpha_dcu_matrix_descr_t ell_descr, ALPHA_INT ell_width, float *ell_val,
    ALPHA_INT *ell_col_ind);
alphasparse_status_t alphasparse_dcu_dcsr2ell(
    alphasparse_dcu_handle_t handle, ALPHA_INT m, const alpha_dcu_matrix_descr_t csr_descr,
    const double *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const alpha_dcu_matrix_descr_t ell_descr, ALPHA_INT ell_width, double *ell_val,
    ALPHA_INT *ell_col_ind);

/* ---- SpMV on the converters' output formats ------------------------------------
 * include/alphasparse/spapi_dcu.h:469-481, :483-495 (coomv) and :858-869, :871-882
 * (ellmv); validation order of src/core/op_dcu/level2/alphasparse_dcu_x_coomv.cpp:50-95
 * and alphasparse_dcu_x_ellmv.cpp:48-93: only NON_TRANSPOSE and GENERAL are
 * supported, as there.  Unlike the reference's kernels, which read indices as
 * zero-based whatever the descriptor says, descr->base is honoured. */
alphasparse_status_t alphasparse_dcu_s_coomv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             ALPHA_INT nnz, const float *alpha,
                                             const alpha_dcu_matrix_descr_t descr, const float *coo_val,
                                             const ALPHA_INT *coo_row_ind, const ALPHA_INT *coo_col_ind,
                                             const float *x, const float *beta, float *y);
alphasparse_status_t alphasparse_dcu_d_coomv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             ALPHA_INT nnz, const double *alpha,
                                             const alpha_dcu_matrix_descr_t descr, const double *coo_val,
                                             const ALPHA_INT *coo_row_ind, const ALPHA_INT *coo_col_ind,
                                             const double *x, const double *beta, double *y);
alphasparse_status_t alphasparse_dcu_s_ellmv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             const float *alpha, const alpha_dcu_matrix_descr_t descr,
                                             const float *ell_val, const ALPHA_INT *ell_col_ind,
                                             ALPHA_INT ell_width, const float *x, const float *beta,
                                             float *y);
alphasparse_status_t alphasparse_dcu_d_ellmv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             const double *alpha, const alpha_dcu_matrix_descr_t descr,
                                             const double *ell_val, const ALPHA_INT *ell_col_ind,
                                             ALPHA_INT ell_width, const double *x, const double *beta,
                                             double *y);

/* ---- complex element types ---------------------------------------------------
 * The same entry points for ALPHA_Complex8 (c) and ALPHA_Complex16 (z), with the
 * semantics, validation order and extensions described at their fp32 / fp64
 * namesakes above: include/alphasparse/spapi_dcu.h:4404-4405, :4414-4415, :4419-4420
 * (host2device), :4459-4476 (mv_dcu), :549-570 (csrmv_analysis), :607-636 (csrmv),
 * :1228-1265 (csrmm), :3334-3355 (csr2ell), :497-524 (coomv), :884-909 (ellmv).
 * csrmv additionally accepts trans == CONJUGATE_TRANSPOSE, the third entry of the
 * reference's dispatch table for complex types
 * (src/core/op_dcu/level2/alphasparse_dcu_x_csrmv.cpp:17-35 over
 * src/kernel/dcu/level2/mv/csrmv/dcu_gemv_c_csr_conj.cpp:22-75); an analysis asked
 * for that operation keeps a CSR copy of A^H.  Device arrays of complex values must
 * be aligned to the element size (INVALID_VALUE otherwise). */
alphasparse_status_t host2device_c_csr(alphasparse_matrix_t A);
alphasparse_status_t host2device_c_coo(alphasparse_matrix_t mtx);
alphasparse_status_t host2device_c_ell(alphasparse_matrix_t mtx);
alphasparse_status_t alphasparse_c_mv_dcu(alphasparse_dcu_handle_t handle,
                                          const alphasparse_operation_t operation,
                                          const ALPHA_Complex8 *alpha, const alphasparse_matrix_t A,
                                          const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex8 *x,
                                          const ALPHA_Complex8 *beta, ALPHA_Complex8 *y);
alphasparse_status_t alphasparse_dcu_c_csrmv_analysis(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex8 *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info);
alphasparse_status_t alphasparse_dcu_c_csrmv(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const ALPHA_Complex8 *alpha, const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex8 *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info,
    const ALPHA_Complex8 *x, const ALPHA_Complex8 *beta, ALPHA_Complex8 *y);
alphasparse_status_t alphasparse_dcu_c_csrmm(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans_A,
    alphasparse_operation_t trans_B, alphasparse_layout_t layout, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT k, ALPHA_INT nnz, const ALPHA_Complex8 *alpha, const alpha_dcu_matrix_descr_t descr,
    const ALPHA_Complex8 *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const ALPHA_Complex8 *B, ALPHA_INT ldb, const ALPHA_Complex8 *beta, ALPHA_Complex8 *C, ALPHA_INT ldc);
alphasparse_status_t alphasparse_dcu_ccsr2ell(
    alphasparse_dcu_handle_t handle, ALPHA_INT m, const alpha_dcu_matrix_descr_t csr_descr,
    const ALPHA_Complex8 *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const alpha_dcu_matrix_descr_t ell_descr, ALPHA_INT ell_width, ALPHA_Complex8 *ell_val,
    ALPHA_INT *ell_col_ind);
alphasparse_status_t alphasparse_dcu_c_coomv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             ALPHA_INT nnz, const ALPHA_Complex8 *alpha,
                                             const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex8 *coo_val,
                                             const ALPHA_INT *coo_row_ind, const ALPHA_INT *coo_col_ind,
                                             const ALPHA_Complex8 *x, const ALPHA_Complex8 *beta, ALPHA_Complex8 *y);
alphasparse_status_t alphasparse_dcu_c_ellmv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             const ALPHA_Complex8 *alpha, const alpha_dcu_matrix_descr_t descr,
                                             const ALPHA_Complex8 *ell_val, const ALPHA_INT *ell_col_ind,
                                             ALPHA_INT ell_width, const ALPHA_Complex8 *x, const ALPHA_Complex8 *beta,
                                             ALPHA_Complex8 *y);

alphasparse_status_t host2device_z_csr(alphasparse_matrix_t A);
alphasparse_status_t host2device_z_coo(alphasparse_matrix_t mtx);
alphasparse_status_t host2device_z_ell(alphasparse_matrix_t mtx);
alphasparse_status_t alphasparse_z_mv_dcu(alphasparse_dcu_handle_t handle,
                                          const alphasparse_operation_t operation,
                                          const ALPHA_Complex16 *alpha, const alphasparse_matrix_t A,
                                          const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex16 *x,
                                          const ALPHA_Complex16 *beta, ALPHA_Complex16 *y);
alphasparse_status_t alphasparse_dcu_z_csrmv_analysis(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex16 *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info);
alphasparse_status_t alphasparse_dcu_z_csrmv(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT nnz, const ALPHA_Complex16 *alpha, const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex16 *csr_val,
    const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind, alphasparse_dcu_mat_info_t info,
    const ALPHA_Complex16 *x, const ALPHA_Complex16 *beta, ALPHA_Complex16 *y);
alphasparse_status_t alphasparse_dcu_z_csrmm(
    alphasparse_dcu_handle_t handle, alphasparse_operation_t trans_A,
    alphasparse_operation_t trans_B, alphasparse_layout_t layout, ALPHA_INT m, ALPHA_INT n,
    ALPHA_INT k, ALPHA_INT nnz, const ALPHA_Complex16 *alpha, const alpha_dcu_matrix_descr_t descr,
    const ALPHA_Complex16 *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const ALPHA_Complex16 *B, ALPHA_INT ldb, const ALPHA_Complex16 *beta, ALPHA_Complex16 *C, ALPHA_INT ldc);
alphasparse_status_t alphasparse_dcu_zcsr2ell(
    alphasparse_dcu_handle_t handle, ALPHA_INT m, const alpha_dcu_matrix_descr_t csr_descr,
    const ALPHA_Complex16 *csr_val, const ALPHA_INT *csr_row_ptr, const ALPHA_INT *csr_col_ind,
    const alpha_dcu_matrix_descr_t ell_descr, ALPHA_INT ell_width, ALPHA_Complex16 *ell_val,
    ALPHA_INT *ell_col_ind);
alphasparse_status_t alphasparse_dcu_z_coomv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             ALPHA_INT nnz, const ALPHA_Complex16 *alpha,
                                             const alpha_dcu_matrix_descr_t descr, const ALPHA_Complex16 *coo_val,
                                             const ALPHA_INT *coo_row_ind, const ALPHA_INT *coo_col_ind,
                                             const ALPHA_Complex16 *x, const ALPHA_Complex16 *beta, ALPHA_Complex16 *y);
alphasparse_status_t alphasparse_dcu_z_ellmv(alphasparse_dcu_handle_t handle,
                                             alphasparse_operation_t trans, ALPHA_INT m, ALPHA_INT n,
                                             const ALPHA_Complex16 *alpha, const alpha_dcu_matrix_descr_t descr,
                                             const ALPHA_Complex16 *ell_val, const ALPHA_INT *ell_col_ind,
                                             ALPHA_INT ell_width, const ALPHA_Complex16 *x, const ALPHA_Complex16 *beta,
                                             ALPHA_Complex16 *y);

/* ---- generic (descriptor) SpMV -------------------------------------------------
 * Enums: include/alphasparse/spdef.h:209-213 (index types), :244-251 (algorithms).
 * Descriptors: include/alphasparse/handle.h:272-304.  The reference has no
 * constructors for them: callers fill the structs themselves (init = true).
 * For an ELL matrix `nnz` holds the ELL width and col_data / val_data the
 * column-major arrays (src/core/op_dcu/generic/alphasparse_dcu_spmv.cpp:215-229). */
typedef enum {
  ALPHA_SPARSE_DCU_INDEXTYPE_U16 = 1,
  ALPHA_SPARSE_DCU_INDEXTYPE_I32 = 2,
  ALPHA_SPARSE_DCU_INDEXTYPE_I64 = 3
} alphasparse_dcu_indextype_t;

typedef enum {
  ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT = 0,
  ALPHA_SPARSE_DCU_SPMV_ALG_COO = 1,
  ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE = 2,
  ALPHA_SPARSE_DCU_SPMV_ALG_CSR_STREAM = 3,
  ALPHA_SPARSE_DCU_SPMV_ALG_ELL = 4
} alphasparse_dcu_spmv_alg_t;

struct _alphasparse_dcu_spmat_descr {
  bool init;
  bool analysed;
  int64_t rows;
  int64_t cols;
  int64_t nnz;
  void *row_data;
  void *col_data;
  void *ind_data;
  void *val_data;
  alphasparse_dcu_indextype_t row_type;
  alphasparse_dcu_indextype_t col_type;
  alphasparse_datatype_t data_type;
  alphasparse_index_base_t idx_base;
  alphasparse_format_t format;
  struct alpha_dcu_matrix_descr *descr;
  alphasparse_dcu_mat_info_t info;
};
struct _alphasparse_dcu_dnvec_descr {
  bool init;
  int64_t size;
  void *values;
  alphasparse_datatype_t data_type;
};
typedef struct _alphasparse_dcu_spmat_descr *alphasparse_dcu_spmat_descr_t;
typedef struct _alphasparse_dcu_dnvec_descr *alphasparse_dcu_dnvec_descr_t;

/* include/alphasparse/spapi_dcu.h:4371-4381; behaviour of
 * src/core/op_dcu/generic/alphasparse_dcu_spmv.cpp:17-275: a call with
 * temp_buffer == NULL reports *buffer_size = 4 and, for a CSR matrix under the
 * DEFAULT / CSR_ADAPTIVE algorithm, runs the csrmv analysis once; a call with a
 * buffer multiplies (COO, CSR or ELL; fp32 / fp64).  Differences: the analysis
 * is run in the matrix's own precision (the reference always calls the fp32
 * one, :68-71), and a successful CSR / ELL multiply returns its status
 * (SUCCESS) where the reference falls through to NOT_SUPPORTED (:274).
 * All four data types are served. */
alphasparse_status_t alphasparse_dcu_spmv(alphasparse_dcu_handle_t handle, alphasparse_operation_t trans,
                                          const void *alpha, const alphasparse_dcu_spmat_descr_t mat,
                                          const alphasparse_dcu_dnvec_descr_t x, const void *beta,
                                          const alphasparse_dcu_dnvec_descr_t y,
                                          alphasparse_datatype_t compute_type,
                                          alphasparse_dcu_spmv_alg_t alg, size_t *buffer_size,
                                          void *temp_buffer);

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_ALPHA_SPBLAS_DCU_H */
