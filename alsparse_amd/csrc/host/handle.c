/* Library handle, matrix descriptor and info-bundle lifecycle.
 * Behaviour follows src/util_cpp/handle.cpp of the reference:
 *   init_handle :55-64, alphasparse_dcu_get_handle :66-138,
 *   alphasparse_dcu_destory_handle :143-152, csrmv info :154-197,
 *   mat descr :248-272, mat info :274-319 / :334-485,
 *   hip status mapping :21-53. */
#include <stdlib.h>
#include <string.h>

#include "internal.h"

alphasparse_status_t get_alphasparse_dcu_status_for_hip_status(hipError_t status) {
  switch (status) {
    case hipSuccess:
      return ALPHA_SPARSE_STATUS_SUCCESS;
    case hipErrorOutOfMemory: /* hipErrorMemoryAllocation is the same code */
      return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    case hipErrorLaunchOutOfResources:
      return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    case hipErrorInvalidDevicePointer:
      return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    case hipErrorInvalidDevice:
    case hipErrorInvalidResourceHandle:
      return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    case hipErrorInvalidValue: /* the library misused HIP */
      return ALPHA_SPARSE_STATUS_INTERNAL_ERROR;
    case hipErrorNoDevice:
    case hipErrorUnknown:
    default:
      return ALPHA_SPARSE_STATUS_INTERNAL_ERROR;
  }
}

alphasparse_status_t init_handle(alphasparse_dcu_handle_t *handle) {
  if (!handle) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  alphasparse_dcu_handle *h = (alphasparse_dcu_handle *)calloc(1, sizeof(*h));
  if (!h) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  h->stream = 0;
  h->pointer_mode = ALPHA_SPARSE_DCU_POINTER_MODE_HOST;
  h->check = false;
  *handle = h;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_get_handle(alphasparse_dcu_handle_t *handle) {
  if (!handle) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  if (*handle == NULL) {
    alphasparse_status_t st = init_handle(handle);
    if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
  }
  alphasparse_dcu_handle *h = *handle;
  ASAMD_HIP_STATUS(hipGetDevice(&h->device));
  ASAMD_HIP_STATUS(hipGetDeviceProperties(&h->properties, h->device));
  h->wavefront_size = h->properties.warpSize;
  h->asic_rev = h->properties.asicRevision;

  const char *layer = getenv("ALPHA_SPARSE_DCU_LAYER");
  h->layer_mode = layer ? (alphasparse_dcu_layer_mode_t)atoi(layer) : ALPHA_SPARSE_DCU_LAYER_MODE_NONE;

  /* scratch: at least 1 MiB, as the reference sizes it (handle.cpp:94-105) */
  h->buffer_size = (size_t)1 << 20;
  const float s1 = 1.0f;
  const double d1 = 1.0;
  const ALPHA_Complex8 c1 = {1.0f, 0.0f};
  const ALPHA_Complex16 z1 = {1.0, 0.0};
  hipError_t e = hipMalloc(&h->buffer, h->buffer_size);
  if (e == hipSuccess) e = hipMalloc((void **)&h->sone, sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void **)&h->done, sizeof(double));
  if (e == hipSuccess) e = hipMalloc((void **)&h->cone, sizeof(ALPHA_Complex8));
  if (e == hipSuccess) e = hipMalloc((void **)&h->zone, sizeof(ALPHA_Complex16));
  if (e == hipSuccess) e = (hipError_t)asamd_warmup(h->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(h->sone, &s1, sizeof s1, hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(h->done, &d1, sizeof d1, hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(h->cone, &c1, sizeof c1, hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(h->zone, &z1, sizeof z1, hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(h->stream); /* the constants above live on this stack frame */
  if (e != hipSuccess) {
    (void)alphasparse_dcu_destory_handle(h); /* releases whatever was allocated; the struct stays the caller's */
    return get_alphasparse_dcu_status_for_hip_status(e);
  }
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_destory_handle(alphasparse_dcu_handle_t handle) {
  if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  asamd_registry_drop_handle(handle); /* the analyses this handle made on its own for un-analysed matrices */
  (void)hipFree(handle->buffer);
  (void)hipFree(handle->sone);
  (void)hipFree(handle->done);
  (void)hipFree(handle->cone);
  (void)hipFree(handle->zone);
  handle->buffer = NULL;
  handle->sone = NULL;
  handle->done = NULL;
  handle->cone = NULL;
  handle->zone = NULL;
  handle->buffer_size = 0;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_create_mat_descr(alpha_dcu_matrix_descr_t *descr) {
  if (!descr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  struct alpha_dcu_matrix_descr *d = (struct alpha_dcu_matrix_descr *)malloc(sizeof(*d));
  *descr = d;
  if (!d) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  d->type = ALPHA_SPARSE_MATRIX_TYPE_GENERAL;
  d->mode = ALPHA_SPARSE_FILL_MODE_LOWER;
  d->diag = ALPHA_SPARSE_DIAG_NON_UNIT;
  d->base = ALPHA_SPARSE_INDEX_BASE_ZERO;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_destroy_mat_descr(alpha_dcu_matrix_descr_t descr) {
  free(descr);
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_create_csrmv_info(alphasparse_dcu_csrmv_info_t *info,
                                                       bool algo_tuning) {
  if (!info) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  struct _alphasparse_dcu_csrmv_info *p = (struct _alphasparse_dcu_csrmv_info *)calloc(1, sizeof(*p));
  *info = p;
  if (!p) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
  p->algo_tuning = algo_tuning;
  p->algo = NONE_ALGO;
  p->iter = 0;
  p->size = 0;
  p->row_blocks = NULL;
  p->csr_adaptive_has_tuned = false;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_destroy_csrmv_info(alphasparse_dcu_csrmv_info_t info) {
  /* row_blocks is never allocated by this library, so there is nothing
   * device-side to release; a NULL info is fine (handle.cpp:176-180). */
  free(info);
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparse_status_t alphasparse_dcu_create_mat_info(alphasparse_dcu_mat_info_t *info) {
  if (!info) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
  struct _alphasparse_dcu_mat_info *p = (struct _alphasparse_dcu_mat_info *)calloc(1, sizeof(*p));
  *info = p;
  return p ? ALPHA_SPARSE_STATUS_SUCCESS : ALPHA_SPARSE_STATUS_ALLOC_FAILED;
}

alphasparse_status_t alphasparse_dcu_destroy_mat_info(alphasparse_dcu_mat_info_t info) {
  if (!info) return ALPHA_SPARSE_STATUS_SUCCESS;
  /* only a csrmv record that this library created is released: a bundle that
   * the caller filled by hand may hold anything in that slot */
  asamd_record *rec = asamd_registry_find(ASAMD_KEY_INFO, info);
  if (rec) {
    alphasparse_dcu_destroy_csrmv_info(info->csrmv_info);
    asamd_registry_erase(ASAMD_KEY_INFO, info);
  }
  free(info);
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

/* The handle's scratch buffer serves whatever the current call needs (reference: sized once,
 * src/util_cpp/handle.cpp:94-105): multiplies carve their per-call scratch from it, column-major csrmm
 * keeps a row-major copy of B in it.  Calls on one handle are ordered by its stream, so they can share it. */
int asamd_handle_reserve(void *handle, size_t bytes) {
  alphasparse_dcu_handle_t h = (alphasparse_dcu_handle_t)handle;
  if (!h) return (int)ALPHA_SPARSE_STATUS_INVALID_HANDLE;
  if (bytes <= h->buffer_size) return (int)ALPHA_SPARSE_STATUS_SUCCESS;
  /* a stream that is being captured can neither be waited for nor may memory be allocated under it:
   * the buffer stays, and the caller makes do with it */
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(h->stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return (int)ALPHA_SPARSE_STATUS_SUCCESS;
  }
  ASAMD_HIP_STATUS(hipStreamSynchronize(h->stream));
  void *bigger = NULL;
  if (hipMalloc(&bigger, bytes) != hipSuccess) {
    (void)hipGetLastError(); /* no room: the caller makes do with the buffer there is */
    return (int)ALPHA_SPARSE_STATUS_SUCCESS;
  }
  (void)hipFree(h->buffer);
  h->buffer = bigger;
  h->buffer_size = bytes;
  return (int)ALPHA_SPARSE_STATUS_SUCCESS;
}

/* The stream lives in a public struct field (handle->stream), which C callers set themselves as
 * with the reference; these two are for bindings that cannot see the struct layout. */
int asamd_handle_set_stream(void *handle, hipStream_t stream) {
  if (!handle) return (int)hipErrorInvalidValue;
  ((alphasparse_dcu_handle_t)handle)->stream = stream;
  return (int)hipSuccess;
}

hipStream_t asamd_handle_get_stream(void *handle) {
  return handle ? ((alphasparse_dcu_handle_t)handle)->stream : NULL;
}

int asamd_env_algo(void) {
  const char *e = getenv("ALSPARSE_AMD_SPMV_ALGO");
  if (!e || !*e) return ASAMD_SPMV_AUTO;
  if (!strcmp(e, "vector")) return ASAMD_SPMV_VECTOR;
  if (!strcmp(e, "rowconst")) return ASAMD_SPMV_ROWCONST;
  if (!strcmp(e, "merge")) return ASAMD_SPMV_MERGE;
  if (!strcmp(e, "scalar")) return ASAMD_SPMV_SCALAR;
  if (!strcmp(e, "tiled")) return ASAMD_SPMV_TILED;
  if (!strcmp(e, "stream")) return ASAMD_SPMV_STREAM;
  if (!strcmp(e, "ell")) return ASAMD_SPMV_ELL;
  if (!strcmp(e, "hot")) return ASAMD_SPMV_MERGE_HOT;
  if (!strcmp(e, "binned")) return ASAMD_SPMV_BINNED;
  if (!strcmp(e, "xlds")) return ASAMD_SPMV_XLDS;
  return ASAMD_SPMV_AUTO;
}

int asamd_env_structure_only(void) {
  const char *e = getenv("ALSPARSE_AMD_ANALYSIS");
  return e && !strcmp(e, "structure");
}
