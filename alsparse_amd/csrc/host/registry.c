/* Library-side registry of CSR analysis results.
 *
 * The reference keeps analysis output inside the caller-visible
 * _alphasparse_dcu_csrmv_info record (include/alphasparse/handle.h:118-138),
 * which its own tests allocate by hand and leave uninitialised
 * (test/dcu/level2/mv_csr_d_dcu_test.cpp:210-213).  Nothing in such a record
 * can therefore be trusted; results live here, keyed by the address of the
 * object they belong to and confirmed against the call's arguments before use. */
#include <pthread.h>
#include <stdlib.h>

#include "internal.h"

static pthread_mutex_t g_lock = PTHREAD_MUTEX_INITIALIZER;
static asamd_record *g_head[3];

asamd_record *asamd_registry_find(asamd_key_kind kind, const void *key) {
  pthread_mutex_lock(&g_lock);
  asamd_record *r = g_head[kind];
  while (r && r->key != key) r = r->next;
  pthread_mutex_unlock(&g_lock);
  return r;
}

asamd_record *asamd_registry_insert(asamd_key_kind kind, const void *key) {
  asamd_record *r = (asamd_record *)calloc(1, sizeof(*r));
  if (!r) return NULL;
  r->kind = kind;
  r->key = key;
  pthread_mutex_lock(&g_lock);
  r->next = g_head[kind];
  g_head[kind] = r;
  pthread_mutex_unlock(&g_lock);
  return r;
}

void asamd_record_release_device(asamd_record *rec) {
  if (!rec) return;
  if (rec->plan) asamd_csr_plan_destroy(rec->plan);
  if (rec->d_in) (void)hipFree(rec->d_in);
  if (rec->d_out) (void)hipFree(rec->d_out);
  rec->plan = NULL;
  rec->d_in = rec->d_out = NULL;
  rec->d_in_bytes = rec->d_out_bytes = 0;
}

void asamd_registry_erase(asamd_key_kind kind, const void *key) {
  pthread_mutex_lock(&g_lock);
  asamd_record **pp = &g_head[kind];
  while (*pp && (*pp)->key != key) pp = &(*pp)->next;
  asamd_record *r = *pp;
  if (r) *pp = r->next;
  pthread_mutex_unlock(&g_lock);
  if (r) {
    asamd_record_release_device(r);
    free(r);
  }
}

static int record_matches(const asamd_record *r, const void *row_ptr, const void *col_ind,
                          int32_t m, int32_t n, int32_t nnz, int32_t base, int32_t dtype) {
  return r->plan && r->row_ptr == row_ptr && (col_ind == NULL || r->col_ind == col_ind) &&
         r->m == m && r->n == n && r->nnz == nnz && r->base == base && r->dtype == dtype;
}

alphasparse_status_t asamd_plan_for_call(alphasparse_dcu_handle_t handle, const void *info,
                                         const void *row_ptr, const void *col_ind, int32_t m,
                                         int32_t n, int32_t nnz, int32_t base, int32_t dtype,
                                         asamd_csr_plan **plan) {
  /* 1. an explicit analysis of exactly these arrays (info may be garbage: it is
   *    only ever compared by address, never dereferenced) */
  if (info) {
    asamd_record *r = asamd_registry_find(ASAMD_KEY_INFO, info);
    if (r && record_matches(r, row_ptr, col_ind, m, n, nnz, base, dtype)) {
      *plan = r->plan;
      return ALPHA_SPARSE_STATUS_SUCCESS;
    }
  }
  /* 2. a device mirror that this library built (alphasparse_?_mv_dcu path) */
  {
    asamd_record *r = asamd_registry_find(ASAMD_KEY_MATRIX, row_ptr);
    if (r && record_matches(r, row_ptr, col_ind, m, n, nnz, base, dtype)) {
      *plan = r->plan;
      return ALPHA_SPARSE_STATUS_SUCCESS;
    }
  }
  /* 3. lazy: statistics cached per row_ptr address.  The structure behind the
   *    address may change without notice, so the plan is untrusted: it only
   *    steers the kernel choice, and every kernel it can pick reads row_ptr
   *    afresh on each call. */
  asamd_record *r = asamd_registry_find(ASAMD_KEY_LAZY, row_ptr);
  if (r && !record_matches(r, row_ptr, NULL, m, n, nnz, base, dtype)) {
    asamd_registry_erase(ASAMD_KEY_LAZY, row_ptr);
    r = NULL;
  }
  if (!r) {
    asamd_csr_plan *p = NULL;
    ASAMD_HIP_STATUS(asamd_csr_plan_create_dtype(handle->stream, m, n, nnz, (const int32_t *)row_ptr,
                                           NULL, NULL, base, dtype, /*trusted=*/0, &p));
    r = asamd_registry_insert(ASAMD_KEY_LAZY, row_ptr);
    if (!r) {
      asamd_csr_plan_destroy(p);
      return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    }
    r->row_ptr = row_ptr;
    r->col_ind = col_ind;
    r->m = m;
    r->n = n;
    r->nnz = nnz;
    r->base = base;
    r->dtype = dtype;
    r->plan = p;
    const int forced = asamd_env_algo();
    if (forced != ASAMD_SPMV_AUTO) (void)asamd_csr_plan_set_algo(p, forced);
  }
  *plan = r->plan;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

uint64_t asamd_host_fingerprint(const void *values, size_t count, size_t elem) {
  const unsigned char *p = (const unsigned char *)values;
  const size_t samples = count < 1024 ? count : 1024;
  uint64_t h = 0x9E3779B97F4A7C15ull ^ (uint64_t)count;
  for (size_t s = 0; s < samples; ++s) {
    /* sample s sits at a fixed position of its 1/samples share of the array */
    const size_t i = (size_t)(((unsigned __int128)s * count) / samples) + (s * 2654435761u) % (count / samples ? count / samples : 1);
    const unsigned char *q = p + (i < count ? i : count - 1) * elem;
    for (size_t b = 0; b < elem; ++b) h = (h ^ q[b]) * 0x100000001B3ull;
  }
  return h;
}

static alphasparse_dcu_handle_t g_default_handle;

alphasparse_status_t asamd_default_handle(alphasparse_dcu_handle_t *handle) {
  alphasparse_status_t st = ALPHA_SPARSE_STATUS_SUCCESS;
  pthread_mutex_lock(&g_lock);
  if (!g_default_handle) {
    alphasparse_dcu_handle_t h = NULL;
    st = alphasparse_dcu_get_handle(&h);
    if (st == ALPHA_SPARSE_STATUS_SUCCESS) {
      g_default_handle = h;
    } else {
      free(h);
    }
  }
  *handle = g_default_handle;
  pthread_mutex_unlock(&g_lock);
  return st;
}

static asamd_record *find_any(const void *key) {
  asamd_record *r = asamd_registry_find(ASAMD_KEY_INFO, key);
  if (!r) r = asamd_registry_find(ASAMD_KEY_MATRIX, key);
  if (!r) r = asamd_registry_find(ASAMD_KEY_LAZY, key);
  return r;
}

const asamd_csr_stats *asamd_analysis_stats(const void *key) {
  asamd_record *r = find_any(key);
  return r && r->plan ? asamd_csr_plan_stats(r->plan) : NULL;
}

const asamd_csr_stats *asamd_analysis_transpose_stats(const void *key) {
  asamd_record *r = find_any(key);
  return r && r->plan ? asamd_csr_plan_transpose_stats(r->plan) : NULL;
}

int asamd_analysis_set_algo(const void *key, int32_t algo) {
  asamd_record *r = find_any(key);
  if (!r || !r->plan) return (int)hipErrorInvalidValue;
  return asamd_csr_plan_set_algo(r->plan, algo);
}
