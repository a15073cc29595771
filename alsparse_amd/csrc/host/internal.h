/* Internals of the C host library: the analysis registry, the process-wide
 * default handle used by the host-pointer entry points, and small helpers.
 * Nothing here is part of the drop-in ABI. */
#ifndef ALSPARSE_AMD_HOST_INTERNAL_H
#define ALSPARSE_AMD_HOST_INTERNAL_H

#include <stdint.h>

#include "alpha_spblas_dcu.h"
#include "alsparse_amd_kernels.h"
#include "alsparse_amd_plan.h"

/* How an analysis record is looked up. */
typedef enum {
  ASAMD_KEY_MATRIX = 0, /* by alphasparse_matrix_t: device mirror owned by the library      */
  ASAMD_KEY_INFO = 1,   /* by alphasparse_dcu_mat_info_t: explicit *_csrmv_analysis call      */
  ASAMD_KEY_LAZY = 2    /* by csr_row_ptr: first multiply without analysis, structure unknown */
} asamd_key_kind;

typedef struct asamd_record {
  asamd_key_kind kind;
  const void *key;
  /* lazy records only: the handle the record belongs to, the multiplies that hold it at the moment, its
   * last use (for evicting the oldest) and whether it has been taken out of the registry */
  const void *owner;
  int leases;
  int dead;
  uint64_t last_use;
  /* what the plan was built for; a lookup must match all of these */
  const void *row_ptr;
  const void *col_ind;
  int32_t m, n, nnz, base, dtype; /* dtype: enum asamd_dtype == alphasparse_datatype_t */
  asamd_csr_plan *plan;
  /* explicit analyses: fingerprint of the structure arrays at analysis time (asamd_csr_structure_hash) */
  uint64_t structure_hash;
  int has_structure_hash;
  /* library-built mirrors: fingerprints of the HOST values and structure arrays at the time they were copied */
  uint64_t host_val_fingerprint;
  uint64_t host_idx_fingerprint;
  /* lazy records only: a caller who never analyses but multiplies the same arrays again and again is given a
   * tiled copy that is WATCHED (asamd_csr_plan_csrmv_watched) where the analysis' model expects it to pay:
   * calls seen in a row on the same three arrays, the value array they named, and the state of the promotion
   * (0 not tried, 1 in use, 2 not again) with what it owns */
  uint32_t lazy_calls;
  const void *lazy_val;
  int promo_state;
  asamd_csr_plan *promo_plan;
  uint64_t *d_watch;    /* fingerprints of row_ptr and col_ind at promotion (device) */
  int32_t *h_changed;   /* pinned: the last watched multiply's verdict, copied behind it */
  void *promo_event;    /* hipEvent_t recorded behind that copy */
  int promo_pending;    /* a copy is on its way */
  int promo_misses;     /* watched multiplies in a row that found the structure changed */
  /* host-pointer entry points: device staging for x / y (ASAMD_KEY_MATRIX only) */
  void *d_in;
  size_t d_in_bytes;
  void *d_out;
  size_t d_out_bytes;
  struct asamd_record *next;
} asamd_record;

/* All registry calls are serialised by one mutex.  Records of explicit analyses and of mirrors belong to
 * an object of the caller's (an info bundle, a matrix handle) and are returned unlocked, which is safe as
 * long as that object is not destroyed while another thread multiplies with it (the reference gives no such
 * guarantee either).  Lazy records come and go on their own: see asamd_plan_for_call. */
asamd_record *asamd_registry_find(asamd_key_kind kind, const void *key);
asamd_record *asamd_registry_insert(asamd_key_kind kind, const void *key);
void asamd_registry_erase(asamd_key_kind kind, const void *key);
void asamd_record_release_device(asamd_record *rec);

/* Plan for a multiply through the raw-pointer API: explicit analysis if `info`
 * is known and matches, else the mirror's, else the handle's lazy record for this row_ptr (created on
 * first use; at most 64 are kept, the least recently used one makes room).  *lease is non-NULL when the plan
 * belongs to a lazy record: pass it to asamd_plan_release once the multiply's kernels are enqueued. */
alphasparse_status_t asamd_plan_for_call(alphasparse_dcu_handle_t handle, const void *info,
                                         const void *row_ptr, const void *col_ind, int32_t m,
                                         int32_t n, int32_t nnz, int32_t base, int32_t dtype,
                                         asamd_csr_plan **plan, asamd_record **lease);
void asamd_plan_release(asamd_record *lease);
/* A multiply without analysis (lease: the lazy record asamd_plan_for_call returned).  Counts repeated calls on
 * the same arrays, promotes the record to a watched tiled copy when that pays, and then multiplies through it:
 * *done = 1 if y has been enqueued, 0 if the caller is to go on with the record's ordinary plan.
 * ALSPARSE_AMD_LAZY_COPIES=0 switches the promotion off, ALSPARSE_AMD_LAZY_AFTER=<calls> sets how many calls on
 * the same arrays it takes (default 4). */
alphasparse_status_t asamd_lazy_multiply(alphasparse_dcu_handle_t handle, asamd_record *lease, int32_t trans,
                                         const void *alpha, const void *val, const void *row_ptr,
                                         const void *col_ind, const void *x, const void *beta, void *y, int *done);

/* forgets the lazy records of a handle that is being destroyed */
void asamd_registry_drop_handle(const void *handle);
/* number of lazy records alive (tests) */
int asamd_registry_lazy_count(void);

/* Fingerprint of EVERY byte of a host array (one streaming pass spread over the OpenMP threads): taken on
 * every host-pointer multiply of the values and of both index arrays, because the reference's CPU kernels
 * read the caller's arrays on every call and alphasparse_?_export_csr hands out pointers into them. */
uint64_t asamd_host_fingerprint(const void *data, size_t bytes);

/* Process-wide handle for alphasparse_?_mv / _mm (host pointers). */
alphasparse_status_t asamd_default_handle(alphasparse_dcu_handle_t *handle);

/* ALSPARSE_AMD_SPMV_ALGO = auto | vector | rowconst | merge | scalar | tiled | stream | ell | hot | binned */
int asamd_env_algo(void);
/* ALSPARSE_AMD_ANALYSIS = structure: analyses keep no copies of the matrix values (as the reference's);
 * the default lets an analysis keep re-ordered copies, which every multiply checks against csr_val. */
int asamd_env_structure_only(void);

/* device arrays of values must be aligned to their element size (one element = one load) */
#define ASAMD_MISALIGNED(T, p) (((uintptr_t)(p)) % sizeof(T) != 0)

#define ASAMD_HIP_STATUS(expr)                                           \
  do {                                                                   \
    hipError_t asamd_e_ = (hipError_t)(expr);                            \
    if (asamd_e_ != hipSuccess)                                          \
      return get_alphasparse_dcu_status_for_hip_status(asamd_e_);        \
  } while (0)

#endif
