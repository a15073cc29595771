/* Library-side registry of CSR analysis results.
 *
 * The reference keeps analysis output inside the caller-visible
 * _alphasparse_dcu_csrmv_info record (include/alphasparse/handle.h:118-138),
 * which its own tests allocate by hand and leave uninitialised
 * (test/dcu/level2/mv_csr_d_dcu_test.cpp:210-213).  Nothing in such a record
 * can therefore be trusted; results live here, keyed by the address of the
 * object they belong to and confirmed against the call's arguments before use. */
#include <omp.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

static pthread_mutex_t g_lock = PTHREAD_MUTEX_INITIALIZER;
static asamd_record *g_head[3];
static int g_lazy_count;       /* live ASAMD_KEY_LAZY records */
static uint64_t g_tick;        /* use counter: the lazy record with the smallest stamp is the oldest */

/* At most this many lazily analysed matrices are remembered (each holds a few small device buffers); the
 * least recently used one makes room.  A process that streams many un-analysed matrices through csrmv
 * therefore holds a bounded amount of device memory. */
#define ASAMD_LAZY_CAP 64

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

/* ---- lazy records ------------------------------------------------------------------------------
 * Keyed by (csr_row_ptr, handle): each handle analyses an un-analysed matrix for itself, so the
 * scratch of such a plan (merge-path carries, rewritten by every multiply) is only ever used on one
 * handle's stream.  A record is found, unlinked and freed under the lock; a multiply holds a lease
 * (`leases`) from lookup until its kernels are enqueued, and a record that is replaced or evicted
 * meanwhile (`dead`) is freed by the last lease that lets go.  hipFree waits for work in flight. */
static asamd_record *lazy_unlink_locked(asamd_record *victim) {
  asamd_record **pp = &g_head[ASAMD_KEY_LAZY];
  while (*pp && *pp != victim) pp = &(*pp)->next;
  if (*pp) {
    *pp = victim->next;
    victim->next = NULL;
    victim->dead = 1;
    --g_lazy_count;
  }
  return victim->leases == 0 ? victim : NULL; /* the caller frees it outside the lock */
}

static void promo_release(asamd_record *r) {
  if (r->promo_plan) asamd_csr_plan_destroy(r->promo_plan);
  if (r->d_watch) (void)hipFree(r->d_watch);
  if (r->h_changed) (void)hipHostFree(r->h_changed);
  if (r->promo_event) (void)hipEventDestroy((hipEvent_t)r->promo_event);
  r->promo_plan = NULL;
  r->d_watch = NULL;
  r->h_changed = NULL;
  r->promo_event = NULL;
  r->promo_pending = 0;
}

static void lazy_free(asamd_record *r) {
  if (!r) return;
  promo_release(r);
  asamd_record_release_device(r);
  free(r);
}

void asamd_plan_release(asamd_record *lease) {
  if (!lease) return;
  asamd_record *to_free = NULL;
  pthread_mutex_lock(&g_lock);
  if (--lease->leases == 0 && lease->dead) to_free = lease;
  pthread_mutex_unlock(&g_lock);
  lazy_free(to_free);
}

int asamd_registry_lazy_count(void) {
  pthread_mutex_lock(&g_lock);
  const int n = g_lazy_count;
  pthread_mutex_unlock(&g_lock);
  return n;
}

alphasparse_status_t asamd_plan_for_call(alphasparse_dcu_handle_t handle, const void *info,
                                         const void *row_ptr, const void *col_ind, int32_t m,
                                         int32_t n, int32_t nnz, int32_t base, int32_t dtype,
                                         asamd_csr_plan **plan, asamd_record **lease) {
  *lease = NULL;
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
  /* 3. lazy: statistics cached per (row_ptr address, handle).  The structure behind the
   *    address may change without notice, so the plan is untrusted: it only
   *    steers the kernel choice, and every kernel it can pick reads row_ptr
   *    afresh on each call. */
  asamd_record *stale = NULL, *found = NULL;
  pthread_mutex_lock(&g_lock);
  for (asamd_record *r = g_head[ASAMD_KEY_LAZY]; r; r = r->next) {
    if (r->key != row_ptr || r->owner != (const void *)handle) continue;
    if (record_matches(r, row_ptr, NULL, m, n, nnz, base, dtype)) {
      found = r;
      ++r->leases;
      r->last_use = ++g_tick;
    } else {
      stale = lazy_unlink_locked(r); /* another matrix lives at this address now */
    }
    break;
  }
  pthread_mutex_unlock(&g_lock);
  lazy_free(stale);
  if (!found) {
    asamd_csr_plan *p = NULL;
    ASAMD_HIP_STATUS(asamd_csr_plan_create_dtype(handle->stream, m, n, nnz, (const int32_t *)row_ptr,
                                                 NULL, NULL, base, dtype, /*trusted=*/0, &p));
    asamd_record *r = (asamd_record *)calloc(1, sizeof(*r));
    if (!r) {
      asamd_csr_plan_destroy(p);
      return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    }
    r->kind = ASAMD_KEY_LAZY;
    r->key = row_ptr;
    r->owner = (const void *)handle;
    r->row_ptr = row_ptr;
    r->col_ind = col_ind;
    r->m = m;
    r->n = n;
    r->nnz = nnz;
    r->base = base;
    r->dtype = dtype;
    r->plan = p;
    r->leases = 1;
    const int forced = asamd_env_algo();
    if (forced != ASAMD_SPMV_AUTO) (void)asamd_csr_plan_set_algo(p, forced);
    asamd_record *evicted = NULL;
    pthread_mutex_lock(&g_lock);
    r->last_use = ++g_tick;
    r->next = g_head[ASAMD_KEY_LAZY];
    g_head[ASAMD_KEY_LAZY] = r;
    if (++g_lazy_count > ASAMD_LAZY_CAP) {
      asamd_record *oldest = NULL;
      for (asamd_record *q = g_head[ASAMD_KEY_LAZY]; q; q = q->next)
        if (q != r && (!oldest || q->last_use < oldest->last_use)) oldest = q;
      if (oldest) evicted = lazy_unlink_locked(oldest);
    }
    pthread_mutex_unlock(&g_lock);
    lazy_free(evicted);
    found = r;
  }
  *plan = found->plan;
  *lease = found;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

/* ---- lazy records that keep coming back --------------------------------------------------------
 * The reference's own programs multiply with info == NULL (test/dcu/level2/mv_csr_s_dcu_test.cpp:220-222), and
 * its kernel reads the caller's arrays on every call.  A caller like that promises nothing, so nothing is
 * assumed: a copy is only ever used behind a fingerprint of every byte of all three arrays, taken on the
 * device in front of every multiply (asamd_csr_plan_csrmv_watched). */
static int env_number(const char *name, int fallback) {
  const char *v = getenv(name);
  return v && *v ? atoi(v) : fallback;
}

static int stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return 1; /* unknown: do nothing that a capture forbids */
  }
  return st != hipStreamCaptureStatusNone;
}

/* lays out the watched copy if the analysis' model expects it to pay with the fingerprints' cost on top */
static void promo_try(alphasparse_dcu_handle_t handle, asamd_record *r, const void *val) {
  r->promo_state = 2; /* whatever happens below is not tried again for this record */
  static const int kValSize[4] = {4, 8, 8, 16};
  const double vs = (double)kValSize[r->dtype], nnz = (double)r->nnz;
  /* the tiled copy is for large matrices whose x outgrows an L2 (the plan checks again) */
  if (r->nnz < (1 << 22) || (double)r->n * vs < (double)(4 << 20)) return;
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if ((double)free_b < nnz * (3.0 * vs + 40.0)) return; /* copy, its layout's scratch, the product array */
  asamd_csr_plan *p = NULL;
  if (asamd_csr_plan_create_dtype(handle->stream, r->m, r->n, r->nnz, (const int32_t *)r->row_ptr,
                                  (const int32_t *)r->col_ind, val, r->base, r->dtype, /*trusted=*/3, &p) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  const asamd_csr_stats *st = asamd_csr_plan_stats(p);
  /* three more passes: 4 bytes of row_ptr per row, 4 of col_ind and one value per entry, at 4.5 TB/s */
  const double watch_ms = (nnz * (4.0 + vs) + 4.0 * (double)r->m) / 4.5e9;
  int ok = st->algo == ASAMD_SPMV_TILED && st->tiled_built && st->tune_ms_base > 0.f &&
           (double)st->tune_ms_tiled + watch_ms < 0.6 * (double)st->tune_ms_base;
  hipEvent_t ev = NULL;
  if (ok) ok = hipMalloc((void **)&r->d_watch, 2 * sizeof(uint64_t)) == hipSuccess;
  if (ok) ok = hipHostMalloc((void **)&r->h_changed, sizeof(int32_t), hipHostMallocDefault) == hipSuccess;
  if (ok) ok = hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess;
  if (ok) {
    r->promo_event = (void *)ev;
    *r->h_changed = 0;
    ok = asamd_handle_reserve(handle, asamd_csr_plan_watched_workspace_bytes(p)) == ALPHA_SPARSE_STATUS_SUCCESS;
  }
  if (ok)
    ok = asamd_csr_plan_watch_begin(handle->stream, p, (const int32_t *)r->row_ptr, (const int32_t *)r->col_ind, val,
                                    r->d_watch, handle->buffer, handle->buffer_size) == hipSuccess;
  if (!ok) {
    (void)hipGetLastError();
    r->promo_plan = p;
    promo_release(r);
    return;
  }
  r->promo_plan = p;
  r->promo_state = 1;
  r->promo_misses = 0;
}

alphasparse_status_t asamd_lazy_multiply(alphasparse_dcu_handle_t handle, asamd_record *r, int32_t trans,
                                         const void *alpha, const void *val, const void *row_ptr,
                                         const void *col_ind, const void *x, const void *beta, void *y, int *done) {
  *done = 0;
  if (!r || r->kind != ASAMD_KEY_LAZY || r->promo_state == 2 || trans != 0) return ALPHA_SPARSE_STATUS_SUCCESS;
  static int enabled = -1, after = 4;
  if (enabled < 0) {
    after = env_number("ALSPARSE_AMD_LAZY_AFTER", 4);
    if (after < 1) after = 1;
    enabled = env_number("ALSPARSE_AMD_LAZY_COPIES", 1) != 0 && asamd_env_algo() == ASAMD_SPMV_AUTO &&
              !asamd_env_structure_only();
  }
  if (!enabled) return ALPHA_SPARSE_STATUS_SUCCESS;
  (void)row_ptr; /* (the record was found by it) */
  if (col_ind != r->col_ind || val != r->lazy_val) {
    /* other arrays than last time: the count starts again, and a copy of the old ones goes */
    r->col_ind = col_ind;
    r->lazy_val = val;
    r->lazy_calls = 1;
    if (r->promo_state == 1) {
      promo_release(r);
      r->promo_state = 0;
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
  }
  ++r->lazy_calls;
  const int capturing = stream_is_capturing(handle->stream);
  if (r->promo_state == 0) {
    if (r->lazy_calls < (uint32_t)after || capturing) return ALPHA_SPARSE_STATUS_SUCCESS;
    promo_try(handle, r, val);
    if (r->promo_state != 1) return ALPHA_SPARSE_STATUS_SUCCESS;
  }
  /* what the watched multiplies before this one found, if it has arrived (never waited for) */
  if (capturing) {
    /* (a capture forbids even asking) */
  } else if (r->promo_pending && hipEventQuery((hipEvent_t)r->promo_event) == hipSuccess) {
    r->promo_pending = 0;
    r->promo_misses = *r->h_changed ? r->promo_misses + 1 : 0;
    if (r->promo_misses >= 2) {
      /* the arrays keep changing: the copy only costs */
      promo_release(r);
      r->promo_state = 2;
      return ALPHA_SPARSE_STATUS_SUCCESS;
    }
  } else if (r->promo_pending) {
    (void)hipGetLastError(); /* hipErrorNotReady is not an error */
  }
  const size_t need = asamd_csr_plan_watched_workspace_bytes(r->promo_plan);
  if (handle->buffer_size < need) {
    if (capturing || asamd_handle_reserve(handle, need) != ALPHA_SPARSE_STATUS_SUCCESS)
      return ALPHA_SPARSE_STATUS_SUCCESS; /* the ordinary plan needs less */
  }
  const int32_t *changed = NULL;
  ASAMD_HIP_STATUS(asamd_csr_plan_csrmv_watched(handle->stream, r->promo_plan, alpha, val, (const int32_t *)r->row_ptr,
                                                (const int32_t *)col_ind, x, beta, y, r->d_watch, handle->buffer,
                                                handle->buffer_size, &changed));
  if (!capturing && !r->promo_pending && changed) {
    if (hipMemcpyAsync(r->h_changed, changed, sizeof(int32_t), hipMemcpyDeviceToHost, handle->stream) == hipSuccess &&
        hipEventRecord((hipEvent_t)r->promo_event, handle->stream) == hipSuccess)
      r->promo_pending = 1;
    else
      (void)hipGetLastError();
  }
  *done = 1;
  return ALPHA_SPARSE_STATUS_SUCCESS;
}

int asamd_registry_lazy_promoted(const void *handle, const void *row_ptr) {
  int promoted = 0;
  pthread_mutex_lock(&g_lock);
  for (asamd_record *r = g_head[ASAMD_KEY_LAZY]; r; r = r->next)
    if (r->key == row_ptr && r->owner == handle) promoted = r->promo_state == 1;
  pthread_mutex_unlock(&g_lock);
  return promoted;
}

/* every lazy record of a handle goes with the handle */
void asamd_registry_drop_handle(const void *handle) {
  for (;;) {
    asamd_record *victim = NULL, *to_free = NULL;
    pthread_mutex_lock(&g_lock);
    for (asamd_record *r = g_head[ASAMD_KEY_LAZY]; r; r = r->next)
      if (r->owner == handle) {
        victim = r;
        break;
      }
    if (victim) to_free = lazy_unlink_locked(victim);
    pthread_mutex_unlock(&g_lock);
    if (!victim) break;
    lazy_free(to_free);
  }
}

/* Every byte counts: pieces of 1 MiB are hashed by the OpenMP threads (four independent multiply-add
 * chains over 8-byte words, memory-bound), and the pieces' words are combined with their positions. */
static uint64_t hash_piece(const unsigned char *p, size_t bytes) {
  uint64_t h0 = 0x9E3779B97F4A7C15ull, h1 = 0xBF58476D1CE4E5B9ull, h2 = 0x94D049BB133111EBull, h3 = 0xD6E8FEB86659FD93ull;
  size_t i = 0;
  for (; i + 32 <= bytes; i += 32) {
    uint64_t w[4];
    memcpy(w, p + i, 32);
    h0 = (h0 ^ w[0]) * 0x100000001B3ull + 0x632BE59BD9B4E019ull;
    h1 = (h1 ^ w[1]) * 0xFF51AFD7ED558CCDull + 1;
    h2 = (h2 ^ w[2]) * 0xC4CEB9FE1A85EC53ull + 2;
    h3 = (h3 ^ w[3]) * 0x2545F4914F6CDD1Dull + 3;
  }
  for (; i < bytes; ++i) h0 = (h0 ^ p[i]) * 0x100000001B3ull;
  uint64_t h = h0 ^ (h1 >> 7) ^ (h2 << 11) ^ (h3 >> 17) ^ (h1 << 31) ^ (h3 << 23);
  h ^= h >> 29;
  h *= 0xBF58476D1CE4E5B9ull;
  return h ^ (h >> 32);
}

uint64_t asamd_host_fingerprint(const void *data, size_t bytes) {
  const unsigned char *p = (const unsigned char *)data;
  const size_t piece = (size_t)1 << 20;
  const long pieces = (long)((bytes + piece - 1) / piece);
  uint64_t sum = 0x9E3779B97F4A7C15ull ^ (uint64_t)bytes;
  int threads = omp_get_max_threads();
  if (threads > 16) threads = 16;
#pragma omp parallel for num_threads(threads) schedule(static) reduction(+ : sum) if (pieces > 4)
  for (long i = 0; i < pieces; ++i) {
    const size_t off = (size_t)i * piece;
    const uint64_t h = hash_piece(p + off, bytes - off < piece ? bytes - off : piece);
    sum += (h ^ ((uint64_t)i * 0x9E3779B97F4A7C15ull)) * 0xD6E8FEB86659FD93ull;
  }
  return sum;
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
