/* alphasparse_?_mv / alphasparse_?_mm: the reference's host-pointer entry
 * points (include/alphasparse/spapi.h:685-699, :899-923).  In the reference
 * they run OpenMP CPU kernels; here the multiplication runs on the GPU: the
 * matrix is mirrored to the device on first use, x / X is staged in, y / Y
 * staged out on the default handle's stream, and the call returns after the
 * result has landed in host memory (these entry points are synchronous in the
 * reference too).  There is no CPU compute path: without a usable device the
 * status is the mapped HIP error. */
#include <omp.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

/* ---- host <-> device through pinned bounce buffers -------------------------------------------
 * The vectors of these entry points live in the caller's pageable memory.  hipMemcpy stages such memory
 * through a pinned buffer of its own with one thread; here the processor's copy into (out of) a ring of
 * pinned chunks is spread over the OpenMP threads and overlaps the DMA of the chunk before (after) it.
 * (Registering the caller's memory would avoid the copy, but costs more than the transfer it saves.)
 * One ring per process, used under a lock; transfers below one chunk go through hipMemcpyAsync as before. */
enum { kStageChunks = 4 };
static const size_t kStageChunk = (size_t)8 << 20;
static pthread_mutex_t g_stage_lock = PTHREAD_MUTEX_INITIALIZER;
static void *g_stage_buf[kStageChunks];
static hipEvent_t g_stage_ev[kStageChunks];
static int g_stage_state; /* 0: not tried, 1: ready, -1: no pinned memory (plain copies) */

static int asamd_stage_ready(void) {
  if (g_stage_state) return g_stage_state > 0;
  for (int i = 0; i < kStageChunks; ++i) {
    if (hipHostMalloc(&g_stage_buf[i], kStageChunk, hipHostMallocDefault) != hipSuccess ||
        hipEventCreateWithFlags(&g_stage_ev[i], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      g_stage_state = -1;
      return 0;
    }
  }
  g_stage_state = 1;
  return 1;
}

static void asamd_parallel_copy(void *dst, const void *src, size_t bytes) {
  const size_t piece = (size_t)1 << 20;
  const long pieces = (long)((bytes + piece - 1) / piece);
  int threads = omp_get_max_threads();
  if (threads > 16) threads = 16;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (long i = 0; i < pieces; ++i) {
    const size_t off = (size_t)i * piece;
    memcpy((char *)dst + off, (const char *)src + off, bytes - off < piece ? bytes - off : piece);
  }
}

/* Stream-ordered like hipMemcpyAsync; src may be reused when the call returns. */
static hipError_t asamd_staged_h2d(hipStream_t s, void *dst, const void *src, size_t bytes) {
  if (bytes < kStageChunk) return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s);
  pthread_mutex_lock(&g_stage_lock);
  hipError_t e = hipSuccess;
  if (!asamd_stage_ready()) {
    e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s);
  } else {
    int slot = 0;
    for (size_t off = 0; off < bytes && e == hipSuccess; off += kStageChunk, slot = (slot + 1) % kStageChunks) {
      const size_t n = bytes - off < kStageChunk ? bytes - off : kStageChunk;
      e = hipEventSynchronize(g_stage_ev[slot]); /* the chunk's earlier transfer has left it */
      if (e != hipSuccess) break;
      asamd_parallel_copy(g_stage_buf[slot], (const char *)src + off, n);
      e = hipMemcpyAsync((char *)dst + off, g_stage_buf[slot], n, hipMemcpyHostToDevice, s);
      if (e == hipSuccess) e = hipEventRecord(g_stage_ev[slot], s);
    }
  }
  pthread_mutex_unlock(&g_stage_lock);
  return e;
}

/* Returns after everything queued on s before it, and the copy, have finished. */
static hipError_t asamd_staged_d2h_sync(hipStream_t s, void *dst, const void *src, size_t bytes) {
  hipError_t e;
  if (bytes < kStageChunk) {
    e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s);
    return e == hipSuccess ? hipStreamSynchronize(s) : e;
  }
  pthread_mutex_lock(&g_stage_lock);
  if (!asamd_stage_ready()) {
    e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
  } else {
    const size_t chunks = (bytes + kStageChunk - 1) / kStageChunk;
    e = hipSuccess;
    /* the ring is filled ahead; chunk c is copied out once its transfer has landed, then its slot takes
     * chunk c + kStageChunks */
    for (size_t c = 0; c < chunks + kStageChunks && e == hipSuccess; ++c) {
      if (c >= kStageChunks) {
        const size_t d = c - kStageChunks, off = d * kStageChunk;
        const int slot = (int)(d % kStageChunks);
        e = hipEventSynchronize(g_stage_ev[slot]);
        if (e != hipSuccess) break;
        asamd_parallel_copy((char *)dst + off, g_stage_buf[slot], bytes - off < kStageChunk ? bytes - off : kStageChunk);
      }
      if (c < chunks) {
        const size_t off = c * kStageChunk;
        const int slot = (int)(c % kStageChunks);
        e = hipMemcpyAsync(g_stage_buf[slot], (const char *)src + off, bytes - off < kStageChunk ? bytes - off : kStageChunk,
                           hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipEventRecord(g_stage_ev[slot], s);
      }
    }
  }
  pthread_mutex_unlock(&g_stage_lock);
  return e;
}

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
   * the reference's CPU kernels read them on every call).  Every call therefore fingerprints ALL of the values
   * and of the structure arrays (one streaming pass over the OpenMP threads): changed values are copied to the
   * mirror again and the copies that its analysis keeps are refreshed; a changed structure gets a new mirror
   * and a new analysis.  ALSPARSE_AMD_HOST_CHECK=off promises that the host arrays stay as they were when they
   * were mirrored and skips the pass. */
  static int check = -1;
  if (check < 0) {
    const char *ev = getenv("ALSPARSE_AMD_HOST_CHECK");
    check = !(ev && !strcmp(ev, "off"));
  }
  static const size_t kElem[4] = {4, 8, 8, 16};
  const size_t elem = kElem[A->datatype & 3];
  const size_t nnz = (size_t)(m->rows > 0 && m->rows_end[m->rows - 1] > 0 ? m->rows_end[m->rows - 1] : 0);
  if (check) {
    const uint64_t ifp = asamd_host_fingerprint(m->rows_start, sizeof(ALPHA_INT) * (size_t)(m->rows + 1)) ^
                         (asamd_host_fingerprint(m->col_indx, sizeof(ALPHA_INT) * nnz) * 3);
    if (ifp != r->host_idx_fingerprint || (int32_t)nnz != r->nnz) {
      ASAMD_HIP_STATUS(hipStreamSynchronize((*h)->stream));
      switch (A->datatype) {
        case ALPHA_SPARSE_DATATYPE_FLOAT: st = host2device_s_csr(A); break;
        case ALPHA_SPARSE_DATATYPE_DOUBLE: st = host2device_d_csr(A); break;
        case ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX: st = host2device_c_csr(A); break;
        default: st = host2device_z_csr(A); break;
      }
      if (st != ALPHA_SPARSE_STATUS_SUCCESS) return st;
      r = asamd_registry_find(ASAMD_KEY_MATRIX, m->d_row_ptr);
      if (!r) return ALPHA_SPARSE_STATUS_INTERNAL_ERROR;
    } else if (nnz > 0 && r->plan) {
      const uint64_t fp = asamd_host_fingerprint(m->values, nnz * elem);
      if (fp != r->host_val_fingerprint) {
        ASAMD_HIP_STATUS(hipStreamSynchronize((*h)->stream));
        ASAMD_HIP_STATUS(hipMemcpy(m->d_values, m->values, nnz * elem, hipMemcpyHostToDevice));
        ASAMD_HIP_STATUS(asamd_csr_plan_refresh_values((*h)->stream, r->plan, m->d_row_ptr, m->d_col_indx, m->d_values));
        r->host_val_fingerprint = fp;
      }
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
