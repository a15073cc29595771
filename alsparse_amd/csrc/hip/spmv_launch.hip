// Stateless launchers of the CSR SpMV kernel families that work on the caller's CSR arrays
// (gfx950, wave64).  Each stands in for csr_gemv_vector_dispatch,
// src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182, for one mapping of rows to lanes; which
// one runs is decided by the host library's plan.  Nothing here allocates, copies or waits.

#include <hip/hip_runtime.h>

#include <atomic>

#include "alsparse_amd_kernels.h"
#include "launch_utils.hpp"
#include "spmv_merge.hpp"
#include "spmv_rows.hpp"
#include "spmv_trans.hpp"
#include "spmv_xlds.hpp"
#include "stream_policy.hpp"

using namespace asamd;

static_assert(kMergeThreads == ASAMD_MERGE_THREADS, "the header documents the merge block size");
static_assert(kStreamMaxGroup == ASAMD_STREAM_MAX_GROUP, "the header documents the widest lane group");

// the cache policy of a CSR multiply's two matrix streams (stream_policy.hpp) from its sizes
static int csr_stream_policy(const asamd_spmv_args* a, size_t val_size, bool wide_both = false) {
  return asamd::stream_policy((double)a->nnz, val_size,
                              ((double)a->m + 1.0) * 4.0 + ((double)a->m + (double)a->n) * (double)val_size, wide_both);
}

// ---- W lanes per row ----------------------------------------------------------------------------
template <typename T, int W>
static void launch_vector(hipStream_t s, const asamd_spmv_args* a, const int32_t* run_if) {
  constexpr int rows_per_block = kRowsBlock / W;
  const unsigned grid = (unsigned)(((int64_t)a->m + rows_per_block - 1) / rows_per_block);
  if (run_if)
    spmv_vector_standin_kernel<T, W><<<grid < 2048u ? grid : 2048u, kRowsBlock, 0, s>>>(
        a->m, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr, a->col_ind, (const T*)a->x, scalar_of<T>(a->beta),
        (T*)a->y, a->base, grid, run_if);
  else
    spmv_vector_kernel<T, W><<<grid, kRowsBlock, 0, s>>>(a->m, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr,
                                                         a->col_ind, (const T*)a->x, scalar_of<T>(a->beta), (T*)a->y,
                                                         a->base);
}

extern "C" int asamd_spmv_vector_if(hipStream_t s, const asamd_spmv_args* a, int32_t width, const int32_t* run_if) {
  if (!a) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a)) return hipErrorInvalidValue;
    switch (width) {
      case 2: launch_vector<T, 2>(s, a, run_if); break;
      case 4: launch_vector<T, 4>(s, a, run_if); break;
      case 8: launch_vector<T, 8>(s, a, run_if); break;
      case 16: launch_vector<T, 16>(s, a, run_if); break;
      case 32: launch_vector<T, 32>(s, a, run_if); break;
      case 64: launch_vector<T, 64>(s, a, run_if); break;
      default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
  });
}

extern "C" int asamd_spmv_vector(hipStream_t s, const asamd_spmv_args* a, int32_t width) {
  return asamd_spmv_vector_if(s, a, width, nullptr);
}

// ---- x in LDS ---------------------------------------------------------------------------------------
static int xlds_compute_units() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}
// A kernel may use more than 64 KB of dynamic LDS only after it has been told so, on every device it runs on:
// `done` (one word per kernel: a static of the launcher's instantiation) remembers the devices.
static hipError_t allow_full_lds(const void* kernel, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return hipGetLastError();
  if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_relaxed) >> dev) & 1u)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ASAMD_XLDS_MAX_BYTES);
  if (e == hipSuccess && dev >= 0 && dev < 64) done.fetch_or((uint64_t)1 << dev, std::memory_order_relaxed);
  return e;
}
extern "C" int asamd_spmv_xlds_fits(int32_t dtype, int32_t n) {
  return n >= 1 && (int64_t)n * (int64_t)dtype_size(dtype) <= (int64_t)ASAMD_XLDS_MAX_BYTES;
}

template <typename T, int W, bool NT>
static int launch_xlds_as(hipStream_t s, const asamd_spmv_args* a) {
  const int cus = xlds_compute_units();
  const size_t lds = ((size_t)a->n * sizeof(T) + 15) / 16 * 16;
  static std::atomic<uint64_t> allowed{0};
  if (const hipError_t e = allow_full_lds((const void*)spmv_xlds_kernel<T, W, NT>, allowed); e != hipSuccess) return e;
  constexpr int rows_per_trip = (kXldsThreads / W) * kXldsRows;
  int64_t grid = ((int64_t)a->m + rows_per_trip - 1) / rows_per_trip;
  if (grid > cus) grid = cus;
  spmv_xlds_kernel<T, W, NT><<<(unsigned)grid, kXldsThreads, lds, s>>>(a->m, a->n, scalar_of<T>(a->alpha), (const T*)a->val,
                                                                  a->row_ptr, a->col_ind, (const T*)a->x,
                                                                  scalar_of<T>(a->beta), (T*)a->y, a->base);
  return hipGetLastError();
}

template <typename T, int W>
static int launch_xlds(hipStream_t s, const asamd_spmv_args* a) {
  return (int64_t)a->nnz <= (int64_t)a->m * W ? launch_xlds_as<T, W, true>(s, a) : launch_xlds_as<T, W, false>(s, a);
}

// four entries per lane and load: W lanes take the first 4 W entries of a row.  L: column slices (their sums go to
// `partials`, slices * m elements, and are added up by a second kernel), or null.
template <typename T, int W, bool NT>
static int launch_xlds4_narrow_as(hipStream_t s, const asamd_spmv_args* a, const uint16_t* col16) {
  const size_t lds = ((size_t)a->n * sizeof(T) + 15) / 16 * 16;
  static std::atomic<uint64_t> allowed{0};
  if (const hipError_t e = allow_full_lds((const void*)spmv_xlds4_kernel<T, W, NT, unsigned short>, allowed);
      e != hipSuccess)
    return e;
  constexpr int rows_per_trip = (kXldsThreads / W) * kXlds4Rows;
  int64_t grid = ((int64_t)a->m + rows_per_trip - 1) / rows_per_trip;
  if (grid > xlds_compute_units()) grid = xlds_compute_units();
  spmv_xlds4_kernel<T, W, NT, unsigned short><<<(unsigned)grid, kXldsThreads, lds, s>>>(
      a->m, a->n, a->n, (int64_t)a->nnz, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr, a->row_ptr + 1, 0, col16,
      (const T*)a->x, scalar_of<T>(a->beta), (T*)a->y, 0, a->base);
  return hipGetLastError();
}
template <typename T, int W>
static int launch_xlds4_narrow(hipStream_t s, const asamd_spmv_args* a, const uint16_t* col16) {
  return (int64_t)a->nnz <= (int64_t)a->m * 4 * W ? launch_xlds4_narrow_as<T, W, true>(s, a, col16)
                                                  : launch_xlds4_narrow_as<T, W, false>(s, a, col16);
}

template <typename T, int W, bool NT>
static int launch_xlds4_as(hipStream_t s, const asamd_spmv_args* a, const asamd_xlds_layout* L, void* partials) {
  const int cus = xlds_compute_units();
  const int slices = L ? L->slices : 1, slice_cols = L ? L->slice_cols : a->n;
  const size_t lds = ((size_t)slice_cols * sizeof(T) + 15) / 16 * 16;
  static std::atomic<uint64_t> allowed{0};
  if (const hipError_t e = allow_full_lds((const void*)spmv_xlds4_kernel<T, W, NT>, allowed); e != hipSuccess) return e;
  constexpr int rows_per_trip = (kXldsThreads / W) * kXlds4Rows;
  int64_t grid = ((int64_t)a->m + rows_per_trip - 1) / rows_per_trip;
  const int64_t per_slice = cus / slices > 0 ? cus / slices : 1;  // the workgroups share the compute units
  if (grid > per_slice) grid = per_slice;
  if (!L) {
    spmv_xlds4_kernel<T, W, NT><<<(unsigned)grid, kXldsThreads, lds, s>>>(
        a->m, a->n, a->n, (int64_t)a->nnz, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr, a->row_ptr + 1, 0,
        a->col_ind, (const T*)a->x, scalar_of<T>(a->beta), (T*)a->y, 0, a->base);
    return hipGetLastError();
  }
  if (L->val) {
    // the copy, slice by slice: a CSR matrix per slice, base 0, 16-bit columns
    static std::atomic<uint64_t> allowed_copy{0};
    if (const hipError_t e = allow_full_lds((const void*)spmv_xlds4_kernel<T, W, NT, unsigned short>, allowed_copy);
        e != hipSuccess)
      return e;
    spmv_xlds4_kernel<T, W, NT, unsigned short><<<dim3((unsigned)grid, (unsigned)slices), kXldsThreads, lds, s>>>(
        a->m, a->n, slice_cols, (int64_t)a->nnz + 4, T(1), (const T*)L->val, L->off, L->off + 1, (int64_t)a->m, L->col,
        (const T*)a->x, T(0), (T*)partials, (int64_t)a->m, 0);
  } else {
    spmv_xlds4_kernel<T, W, NT><<<dim3((unsigned)grid, (unsigned)slices), kXldsThreads, lds, s>>>(
        a->m, a->n, slice_cols, (int64_t)a->nnz, T(1), (const T*)a->val, L->seg, L->seg + a->m, (int64_t)a->m,
        a->col_ind, (const T*)a->x, T(0), (T*)partials, (int64_t)a->m, a->base);
  }
  xlds_slices_sum_kernel<T><<<(unsigned)(((int64_t)a->m + 255) / 256), 256, 0, s>>>(
      a->m, slices, scalar_of<T>(a->alpha), (const T*)partials, scalar_of<T>(a->beta), (T*)a->y);
  return hipGetLastError();
}
// (non-temporal first loads where the pieces of the rows hold at most 4 W entries on average)
template <typename T, int W>
static int launch_xlds4(hipStream_t s, const asamd_spmv_args* a, const asamd_xlds_layout* L = nullptr,
                        void* partials = nullptr) {
  const int64_t pieces = (int64_t)a->m * (L ? L->slices : 1);
  // (the pieces of a copy are neighbours in memory and of many lengths: what one piece's load leaves of a cache line,
  // the next piece or the piece's own second load takes from the caches)
  if (L && L->val) return launch_xlds4_as<T, W, false>(s, a, L, partials);
  return (int64_t)a->nnz <= pieces * 4 * W ? launch_xlds4_as<T, W, true>(s, a, L, partials)
                                           : launch_xlds4_as<T, W, false>(s, a, L, partials);
}

extern "C" int asamd_spmv_xlds(hipStream_t s, const asamd_spmv_args* a, int32_t width) {
  if (!a) return hipErrorInvalidValue;
  if (!asamd_spmv_xlds_fits(a->dtype, a->n) || a->nnz < 1 || a->m < 1) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a)) return hipErrorInvalidValue;
    if constexpr (kIsReal<T>) {
      // rows of four entries or more on average, at least four entries in the arrays: 16-byte loads, `width` / 4 lanes
      static const bool narrow_only = getenv("ALSPARSE_AMD_XLDS_WIDE") && atoi(getenv("ALSPARSE_AMD_XLDS_WIDE")) == 0;
      if (!narrow_only && a->nnz >= 4 && (int64_t)a->nnz >= 4 * (int64_t)a->m) {
        switch (width) {
          case 2:
          case 4: return launch_xlds4<T, 1>(s, a);
          case 8: return launch_xlds4<T, 2>(s, a);
          case 16: return launch_xlds4<T, 4>(s, a);
          case 32: return launch_xlds4<T, 8>(s, a);
          case 64: return launch_xlds4<T, 16>(s, a);
          default: return hipErrorInvalidValue;
        }
      }
    }
    switch (width) {
      case 2: return launch_xlds<T, 2>(s, a);
      case 4: return launch_xlds<T, 4>(s, a);
      case 8: return launch_xlds<T, 8>(s, a);
      case 16: return launch_xlds<T, 16>(s, a);
      case 32: return launch_xlds<T, 32>(s, a);
      case 64: return launch_xlds<T, 64>(s, a);
      default: return hipErrorInvalidValue;
    }
  });
}

extern "C" int asamd_narrow_columns(hipStream_t s, int32_t nnz, int32_t base, const int32_t* col_ind, uint16_t* col16) {
  if (!col_ind || !col16 || nnz < 1) return hipErrorInvalidValue;
  int64_t grid = ((int64_t)nnz + 4 + 256 * 8 - 1) / (256 * 8);
  if (grid > 8192) grid = 8192;
  narrow_columns_kernel<<<(unsigned)grid, 256, 0, s>>>((int64_t)nnz, base, col_ind, col16);
  return hipGetLastError();
}

extern "C" int asamd_spmv_xlds_narrow(hipStream_t s, const asamd_spmv_args* a, int32_t width, const uint16_t* col16) {
  if (!a || !col16) return hipErrorInvalidValue;
  if (!asamd_spmv_xlds_fits(a->dtype, a->n) || a->n > 65536 || a->nnz < 4 || a->m < 1 ||
      (int64_t)a->nnz < 4 * (int64_t)a->m)
    return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if constexpr (!kIsReal<T>) {
      return hipErrorInvalidValue;
    } else {
      if (!args_ok<T>(a)) return hipErrorInvalidValue;
      switch (width) {
        case 2:
        case 4: return launch_xlds4_narrow<T, 1>(s, a, col16);
        case 8: return launch_xlds4_narrow<T, 2>(s, a, col16);
        case 16: return launch_xlds4_narrow<T, 4>(s, a, col16);
        case 32: return launch_xlds4_narrow<T, 8>(s, a, col16);
        case 64: return launch_xlds4_narrow<T, 16>(s, a, col16);
        default: return hipErrorInvalidValue;
      }
    }
  });
}

// `width`: lanes per piece of a row if every lane took ONE entry (2 .. 64, from the pieces' mean length)
extern "C" int asamd_spmv_xlds_sliced(hipStream_t s, const asamd_spmv_args* a, int32_t width, const asamd_xlds_layout* L,
                                      void* partials) {
  if (!a || !L || !L->seg || !partials || L->slices < 2 || L->m != a->m || a->nnz < 4 || a->m < 1)
    return hipErrorInvalidValue;
  if ((int64_t)L->slice_cols * dtype_size(a->dtype) > (int64_t)ASAMD_XLDS_MAX_BYTES ||
      (int64_t)L->slices * L->slice_cols < (int64_t)a->n)
    return hipErrorInvalidValue;
  if (L->val && (!L->off || !L->col || L->dtype != a->dtype || L->nnz != a->nnz || L->slice_cols > 65536))
    return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if constexpr (!kIsReal<T>) {
      return hipErrorInvalidValue;
    } else {
      if (!args_ok<T>(a) || (uintptr_t)partials % alignof(T)) return hipErrorInvalidValue;
      switch (width) {
        case 2:
        case 4: return launch_xlds4<T, 1>(s, a, L, partials);
        case 8: return launch_xlds4<T, 2>(s, a, L, partials);
        case 16: return launch_xlds4<T, 4>(s, a, L, partials);
        case 32: return launch_xlds4<T, 8>(s, a, L, partials);
        case 64: return launch_xlds4<T, 16>(s, a, L, partials);
        default: return hipErrorInvalidValue;
      }
    }
  });
}

extern "C" int asamd_spmv_scalar(hipStream_t s, const asamd_spmv_args* a) {
  if (!a) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a)) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)(((int64_t)a->m + kRowsBlock - 1) / kRowsBlock);
    spmv_scalar_kernel<T><<<grid, kRowsBlock, 0, s>>>(a->m, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr,
                                                      a->col_ind, (const T*)a->x, scalar_of<T>(a->beta), (T*)a->y,
                                                      a->base);
    return hipGetLastError();
  });
}

// ---- every row has 4 * G entries ---------------------------------------------------------------
template <typename T, int G>
static void launch_rowconst(hipStream_t s, const asamd_spmv_args* a) {
  constexpr int R = G >= 16 ? 1 : 2;
  constexpr int rows_per_block = (kRowsBlock / G) * R;
  const unsigned grid = (unsigned)(((int64_t)a->m + rows_per_block - 1) / rows_per_block);
  spmv_rowconst_kernel<T, G, R><<<grid, kRowsBlock, 0, s>>>(a->m, scalar_of<T>(a->alpha), (const T*)a->val,
                                                            a->col_ind, (const T*)a->x, scalar_of<T>(a->beta),
                                                            (T*)a->y, a->base, csr_stream_policy(a, sizeof(T)));
}

template <typename T>
static int rowconst_impl(hipStream_t s, const asamd_spmv_args* a, int row_len) {
  if (!args_ok<T>(a)) return hipErrorInvalidValue;
  // 128-bit loads need 16-byte aligned streams
  if ((((uintptr_t)a->val | (uintptr_t)a->col_ind) & 15u) != 0) return hipErrorInvalidValue;
  switch (row_len) {
    case 4: launch_rowconst<T, 1>(s, a); break;
    case 8: launch_rowconst<T, 2>(s, a); break;
    case 16: launch_rowconst<T, 4>(s, a); break;
    case 32: launch_rowconst<T, 8>(s, a); break;
    case 64: launch_rowconst<T, 16>(s, a); break;
    case 128: launch_rowconst<T, 32>(s, a); break;
    case 256: launch_rowconst<T, 64>(s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

extern "C" int asamd_spmv_rowconst(hipStream_t s, const asamd_spmv_args* a, int32_t row_len) {
  if (!a) return hipErrorInvalidValue;
  // the kernel loads four values as one 128-bit piece: real element types only
  if (a->dtype == ASAMD_DTYPE_FLOAT) return rowconst_impl<float>(s, a, row_len);
  if (a->dtype == ASAMD_DTYPE_DOUBLE) return rowconst_impl<double>(s, a, row_len);
  return hipErrorInvalidValue;
}

// ---- a block of rows staged in LDS, G lanes per row ----------------------------------------------
extern "C" int asamd_spmv_stream(hipStream_t s, const asamd_spmv_args* a, int32_t g, int32_t max_len,
                                 int32_t first_offset) {
  if (!a) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a)) return hipErrorInvalidValue;
    constexpr int kCap = 64 / (int)sizeof(T);  // 16 KiB of products per workgroup
    if (g < 1 || g > kStreamMaxGroup || (g & (g - 1)) != 0) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)(((int64_t)a->m * g + kStreamRows - 1) / kStreamRows);
    // 128-bit loads need 16-byte aligned streams
    const bool wide = (((uintptr_t)a->val | (uintptr_t)a->col_ind) & 15u) == 0;
    const int64_t limit = (int64_t)first_offset + a->nnz;
    const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
    const T* val = (const T*)a->val;
    const T* x = (const T*)a->x;
    T* y = (T*)a->y;
    const int policy = csr_stream_policy(a, sizeof(T));
#define ASAMD_STREAM_LAUNCH(CAP, G)                                                                                \
  do {                                                                                                             \
    if (wide)                                                                                                      \
      spmv_stream_wide_kernel<T, CAP, G><<<grid, kStreamRows, 0, s>>>(a->m, alpha, val, a->row_ptr, a->col_ind, x, \
                                                                      beta, y, a->base, limit, policy);            \
    else                                                                                                           \
      spmv_stream_kernel<T, CAP, G><<<grid, kStreamRows, 0, s>>>(a->m, alpha, val, a->row_ptr, a->col_ind, x,      \
                                                                 beta, y, a->base);                                \
  } while (0)
    if (g == 1) {
      // the smallest staging area that holds the longest row
      if (max_len <= 4) {
        ASAMD_STREAM_LAUNCH(4, 1);
      } else if constexpr (kCap >= 8) {
        if (max_len <= 8) {
          ASAMD_STREAM_LAUNCH(8, 1);
        } else if constexpr (kCap >= 16) {
          ASAMD_STREAM_LAUNCH(16, 1);
        } else {
          ASAMD_STREAM_LAUNCH(8, 1);
        }
      } else {
        ASAMD_STREAM_LAUNCH(4, 1);
      }
    } else if (g == 2) {
      ASAMD_STREAM_LAUNCH(kCap, 2);
    } else if (g == 4) {
      ASAMD_STREAM_LAUNCH(kCap, 4);
    } else if (g == 8) {
      ASAMD_STREAM_LAUNCH(kCap, 8);
    } else {
      ASAMD_STREAM_LAUNCH(kCap, 16);
    }
#undef ASAMD_STREAM_LAUNCH
    return hipGetLastError();
  });
}

// The same with 16-bit column distances (real element types, val 16-byte aligned, row_ptr[0] == base; `g` must be the
// group the distances were made for).
extern "C" int asamd_narrow_rel_columns(hipStream_t s, int32_t m, int32_t nnz, int32_t base, int32_t g,
                                        const int32_t* row_ptr, const int32_t* col_ind, int16_t* rel16, int32_t* too_far) {
  if (!row_ptr || !col_ind || !rel16 || !too_far || m < 1 || nnz < 1) return hipErrorInvalidValue;
  if (g < 1 || g > kStreamMaxGroup || (g & (g - 1)) != 0) return hipErrorInvalidValue;
  const int rows_per_group = kStreamRows / g;
  narrow_rel_columns_kernel<<<(unsigned)(((int64_t)m + rows_per_group - 1) / rows_per_group), 256, 0, s>>>(
      m, (int64_t)nnz, base, rows_per_group, row_ptr, col_ind, rel16, too_far);
  return hipGetLastError();
}

template <typename T>
static int stream_rel16_impl(hipStream_t s, const asamd_spmv_args* a, int g, int max_len, const int16_t* rel16) {
  if (!args_ok<T>(a)) return hipErrorInvalidValue;
  constexpr int kCap = 64 / (int)sizeof(T);
  if (g < 1 || g > kStreamMaxGroup || (g & (g - 1)) != 0) return hipErrorInvalidValue;
  if ((((uintptr_t)a->val) & 15u) != 0 || (((uintptr_t)rel16) & 7u) != 0) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)(((int64_t)a->m * g + kStreamRows - 1) / kStreamRows);
  const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
  // Measured with neither / the values / the distances / both non-temporal, ms per multiply:
  //   27-point stencil 160^3      fp32 0.192 / 0.176 / 0.191 / 0.186      fp64 0.276 / 0.299 / 0.276 / 0.299
  //   5-point Laplacian 4096^2    fp32 0.199 / 0.188 / 0.197 / 0.170      fp64 0.274 / 0.295 / 0.275 / 0.280
  // 4-byte values always bypass the caches; the distances too unless they fit the memory-side cache beside what is
  // not a matrix stream (49 MB of row offsets, x and y on the stencil, 201 MB on the Laplacian); 8-byte values: nothing.
  // (y past the caches as well gained 2 % on the fp64 Laplacian and lost 6 % on the fp32 one, and the branch in the
  // kernel's last lines cost the 27-point stencil, fp64, about 3 % whether taken or not: left out.)
  static const int forced = getenv("ALSPARSE_AMD_STREAM_POLICY") ? atoi(getenv("ALSPARSE_AMD_STREAM_POLICY")) : -1;
  const double rest = ((double)a->m + 1.0) * 4.0 + ((double)a->m + (double)a->n) * (double)sizeof(T);
  int policy = 0;
  if (sizeof(T) == 4) policy = kStreamNtValues | (rest + 2.0 * (double)a->nnz > 300.0e6 ? kStreamNtIndices : 0);
  if (forced >= 0) policy = forced & (kStreamNtValues | kStreamNtIndices);
#define ASAMD_STREAM_REL16(CAP, G)                                                                                   \
  spmv_stream_wide_kernel<T, CAP, G, true><<<grid, kStreamRows, 0, s>>>(a->m, alpha, (const T*)a->val, a->row_ptr,   \
                                                                        a->col_ind, (const T*)a->x, beta, (T*)a->y,  \
                                                                        a->base, (int64_t)a->nnz, policy, rel16)
  if (g == 1) {
    if (max_len <= 4) ASAMD_STREAM_REL16(4, 1);
    else if (max_len <= 8 || kCap < 16) ASAMD_STREAM_REL16(8, 1);
    else ASAMD_STREAM_REL16(kCap, 1);
  } else if (g == 2) {
    ASAMD_STREAM_REL16(kCap, 2);
  } else if (g == 4) {
    ASAMD_STREAM_REL16(kCap, 4);
  } else if (g == 8) {
    ASAMD_STREAM_REL16(kCap, 8);
  } else {
    ASAMD_STREAM_REL16(kCap, 16);
  }
#undef ASAMD_STREAM_REL16
  return hipGetLastError();
}
extern "C" int asamd_spmv_stream_rel16(hipStream_t s, const asamd_spmv_args* a, int32_t g, int32_t max_len,
                                       const int16_t* rel16) {
  if (!a || !rel16) return hipErrorInvalidValue;
  if (a->dtype == ASAMD_DTYPE_FLOAT) return stream_rel16_impl<float>(s, a, g, max_len, rel16);
  if (a->dtype == ASAMD_DTYPE_DOUBLE) return stream_rel16_impl<double>(s, a, g, max_len, rel16);
  return hipErrorInvalidValue;
}

// ---- merge-path ------------------------------------------------------------------------------------
extern "C" int asamd_merge_partition(hipStream_t s, int32_t m, int32_t nnz, const int32_t* row_ptr, int32_t base,
                                     int32_t blocks, int32_t items_per_block, int32_t* block_row) {
  if (!row_ptr || !block_row || m <= 0 || nnz < 0 || blocks < 1 || items_per_block < 1) return hipErrorInvalidValue;
  merge_partition_kernel<<<(unsigned)(((int64_t)blocks + 1 + 255) / 256), 256, 0, s>>>(m, nnz, row_ptr, base, blocks,
                                                                                     items_per_block, block_row);
  return hipGetLastError();
}

extern "C" int asamd_spmv_merge(hipStream_t s, const asamd_spmv_args* a, int32_t ipt, const int32_t* block_row,
                                int32_t* carry_row, void* carry_val, void* head_val) {
  if (!a || !block_row || !carry_row || !carry_val || !head_val) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a)) return hipErrorInvalidValue;
    if (ipt != 4 && ipt != 8 && ipt != 16) return hipErrorInvalidValue;
    // LDS per workgroup grows with ipt * sizeof(T): 16-byte values run 4 items only, 8 complex bytes up to 8
    if ((sizeof(T) == 16 && ipt != 4) || (!kIsReal<T> && ipt == 16)) return hipErrorInvalidValue;
    const int64_t items = (int64_t)kMergeThreads * ipt;
    const int nb = (int)(((int64_t)a->m + a->nnz + items - 1) / items);
    const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
    const T* val = (const T*)a->val;
    const T* x = (const T*)a->x;
    T* y = (T*)a->y;
    // 128-bit loads of the streams need them 16-byte aligned
    const bool wide = (((uintptr_t)a->val | (uintptr_t)a->col_ind) & 15u) == 0;
    const int policy = csr_stream_policy(a, sizeof(T), true);
#define ASAMD_LAUNCH_MERGE(IPT)                                                                                      \
  do {                                                                                                               \
    if (wide)                                                                                                        \
      spmv_merge_kernel<T, IPT, true><<<nb, kMergeThreads, 0, s>>>(a->m, a->nnz, alpha, val, a->row_ptr, a->col_ind, \
                                                                   x, beta, y, a->base, block_row, carry_row,        \
                                                                   (T*)carry_val, (T*)head_val, policy);             \
    else                                                                                                             \
      spmv_merge_kernel<T, IPT><<<nb, kMergeThreads, 0, s>>>(a->m, a->nnz, alpha, val, a->row_ptr, a->col_ind, x,    \
                                                             beta, y, a->base, block_row, carry_row, (T*)carry_val,  \
                                                             (T*)head_val);                                          \
  } while (0)
    if constexpr (sizeof(T) <= 8) {
      if constexpr (kIsReal<T>) {
        if (ipt == 16) ASAMD_LAUNCH_MERGE(16);
        else if (ipt == 8) ASAMD_LAUNCH_MERGE(8);
        else ASAMD_LAUNCH_MERGE(4);
      } else {
        if (ipt == 8) ASAMD_LAUNCH_MERGE(8);
        else ASAMD_LAUNCH_MERGE(4);
      }
    } else {
      ASAMD_LAUNCH_MERGE(4);
    }
#undef ASAMD_LAUNCH_MERGE
    if (nb > 1)
      merge_fixup_kernel<T><<<(nb + 255) / 256, 256, 0, s>>>(nb, a->m, alpha, beta, carry_row, (const T*)carry_val,
                                                             (const T*)head_val, y);
    return hipGetLastError();
  });
}

// ---- transposed product with y in LDS --------------------------------------------------------------
// workgroups of the launch: as many as compute units, fewer for few rows (lanes per row do not matter: the least)
static int64_t trans_ylds_groups(int32_t m) {
  const int64_t rows_per_trip = (int64_t)(kXldsThreads / kWave) * kXldsRows;
  int64_t grid = ((int64_t)m + rows_per_trip - 1) / rows_per_trip;
  return grid > xlds_compute_units() ? xlds_compute_units() : (grid < 1 ? 1 : grid);
}
extern "C" size_t asamd_spmv_trans_ylds_bytes(int32_t dtype, int32_t m, int32_t n) {
  if (m < 1 || !asamd_spmv_xlds_fits(dtype, n)) return 0;
  return (size_t)trans_ylds_groups(m) * (size_t)n * (size_t)dtype_size(dtype);
}

template <typename T, int W, bool CONJ>
static int launch_trans_ylds(hipStream_t s, const asamd_spmv_args* a, void* partials) {
  const size_t lds = ((size_t)a->n * sizeof(T) + 15) / 16 * 16;
  static std::atomic<uint64_t> allowed{0};
  if (const hipError_t e = allow_full_lds((const void*)spmv_trans_ylds_kernel<T, W, CONJ>, allowed); e != hipSuccess)
    return e;
  const int64_t grid = trans_ylds_groups(a->m);
  spmv_trans_ylds_kernel<T, W, CONJ><<<(unsigned)grid, kXldsThreads, lds, s>>>(
      a->m, a->n, scalar_of<T>(a->alpha), (const T*)a->val, a->row_ptr, a->col_ind, (const T*)a->x, (T*)partials, a->base);
  trans_partials_sum_kernel<T><<<(unsigned)(((int64_t)a->n + 255) / 256), 256, 0, s>>>(
      a->n, (int)grid, (const T*)partials, scalar_of<T>(a->beta), (T*)a->y);
  return hipGetLastError();
}
template <typename T, bool CONJ>
static int trans_ylds(hipStream_t s, const asamd_spmv_args* a, int width, void* partials) {
  switch (width) {
    case 1:
    case 2: return launch_trans_ylds<T, 2, CONJ>(s, a, partials);
    case 4: return launch_trans_ylds<T, 4, CONJ>(s, a, partials);
    case 8: return launch_trans_ylds<T, 8, CONJ>(s, a, partials);
    case 16: return launch_trans_ylds<T, 16, CONJ>(s, a, partials);
    case 32: return launch_trans_ylds<T, 32, CONJ>(s, a, partials);
    case 64: return launch_trans_ylds<T, 64, CONJ>(s, a, partials);
    default: return hipErrorInvalidValue;
  }
}
// partials: asamd_spmv_trans_ylds_bytes(dtype, m, n) bytes of per-call scratch
extern "C" int asamd_spmv_trans_ylds(hipStream_t s, const asamd_spmv_args* a, int32_t width, int32_t conj, void* partials) {
  if (!a || !partials) return hipErrorInvalidValue;
  if (asamd_spmv_trans_ylds_bytes(a->dtype, a->m, a->n) == 0 || a->nnz < 1) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a) || (conj && kIsReal<T>) || (uintptr_t)partials % alignof(T)) return hipErrorInvalidValue;
    if constexpr (!kIsReal<T>) {
      if (conj) return trans_ylds<T, true>(s, a, width, partials);
    }
    return trans_ylds<T, false>(s, a, width, partials);
  });
}

// ---- transposed product as an atomic scatter ------------------------------------------------------
template <typename T, int W, bool CONJ>
static void launch_trans_scatter(hipStream_t s, const asamd_spmv_args* a) {
  constexpr int rows_per_block = kTransThreads / W;
  const unsigned grid = (unsigned)(((int64_t)a->m + rows_per_block - 1) / rows_per_block);
  csrmv_trans_scatter_kernel<T, W, CONJ><<<grid, kTransThreads, 0, s>>>(a->m, a->n, scalar_of<T>(a->alpha),
                                                                         (const T*)a->val, a->row_ptr, a->col_ind,
                                                                         (const T*)a->x, (T*)a->y, a->base);
}

template <typename T, bool CONJ>
static int trans_scatter(hipStream_t s, const asamd_spmv_args* a, int width) {
  switch (width) {
    case 1: launch_trans_scatter<T, 1, CONJ>(s, a); break;
    case 2: launch_trans_scatter<T, 2, CONJ>(s, a); break;
    case 4: launch_trans_scatter<T, 4, CONJ>(s, a); break;
    case 8: launch_trans_scatter<T, 8, CONJ>(s, a); break;
    case 16: launch_trans_scatter<T, 16, CONJ>(s, a); break;
    case 32: launch_trans_scatter<T, 32, CONJ>(s, a); break;
    case 64: launch_trans_scatter<T, 64, CONJ>(s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

extern "C" int asamd_spmv_trans_scatter(hipStream_t s, const asamd_spmv_args* a, int32_t width, int32_t conj) {
  if (!a) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a) || a->n <= 0 || (conj && kIsReal<T>)) return hipErrorInvalidValue;
    const T beta = scalar_of<T>(a->beta);
    if (beta != T(1))
      scale_vec_kernel<T><<<(unsigned)(((int64_t)a->n + 255) / 256), 256, 0, s>>>(a->n, beta, (T*)a->y);
    if constexpr (!kIsReal<T>) {
      if (conj) return trans_scatter<T, true>(s, a, width);
    }
    return trans_scatter<T, false>(s, a, width);
  });
}

// ---- the unanalysed, one-lane-per-row path ("plain") ---------------------------------------------
// op 0: every row summed by one lane in storage order; op 1 / 2: y scaled by beta, then one lane per
// row scatters alpha*op(a)*x[row] with atomics, the traversal of the reference's own transposed kernels.
template <typename T>
static int csrmv_plain_impl(hipStream_t s, int32_t op, int32_t m, int32_t n, int32_t base, T alpha, const T* val,
                            const int* rp, const int* ci, const T* x, T beta, T* y) {
  if (m <= 0 || n <= 0 || op < 0 || op > 2 || (op == 2 && kIsReal<T>)) return hipErrorInvalidValue;
  asamd_spmv_args a;
  a.dtype = DtypeOf<T>::value;
  a.m = m;
  a.n = n;
  a.nnz = 0;  // not read by these two kernels
  a.base = base;
  a.alpha = &alpha;
  a.beta = &beta;
  a.val = val;
  a.row_ptr = rp;
  a.col_ind = ci;
  a.x = x;
  a.y = y;
  if (op == 0) return asamd_spmv_scalar(s, &a);
  return asamd_spmv_trans_scatter(s, &a, 1, op == 2);
}

extern "C" int asamd_s_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, float alpha,
                                   const float* val, const int32_t* row_ptr, const int32_t* col_ind, const float* x,
                                   float beta, float* y) {
  return csrmv_plain_impl<float>(stream, op, m, n, base, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_d_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base, double alpha,
                                   const double* val, const int32_t* row_ptr, const int32_t* col_ind, const double* x,
                                   double beta, double* y) {
  return csrmv_plain_impl<double>(stream, op, m, n, base, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_c_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base,
                                   asamd_complex8 alpha, const asamd_complex8* val, const int32_t* row_ptr,
                                   const int32_t* col_ind, const asamd_complex8* x, asamd_complex8 beta,
                                   asamd_complex8* y) {
  using T = Cx<float>;
  return csrmv_plain_impl<T>(stream, op, m, n, base, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind,
                             (const T*)x, T(beta.real, beta.imag), (T*)y);
}

extern "C" int asamd_z_csrmv_plain(hipStream_t stream, int32_t op, int32_t m, int32_t n, int32_t base,
                                   asamd_complex16 alpha, const asamd_complex16* val, const int32_t* row_ptr,
                                   const int32_t* col_ind, const asamd_complex16* x, asamd_complex16 beta,
                                   asamd_complex16* y) {
  using T = Cx<double>;
  return csrmv_plain_impl<T>(stream, op, m, n, base, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind,
                             (const T*)x, T(beta.real, beta.imag), (T*)y);
}
