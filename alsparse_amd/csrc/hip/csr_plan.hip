// CSR analysis on the GPU and SpMV kernel dispatch for gfx950.
//
// asamd_csr_plan_create stands in for the reference's host-side, serial row
// block builder (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267 and
// its D2H/H2D round trip at :348-379): one pass over row_ptr on the device
// yields min/max row length and a log2 histogram, from which the kernel family
// is chosen; for the merge-path family the workgroup coordinates are computed
// by a second small kernel.  asamd_?_csrmv stands in for
// csr_gemv_vector_dispatch (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:59-182).

#include <hip/hip_runtime.h>

#include <new>

#include "alsparse_amd_kernels.h"
#include "spmv_merge.hpp"
#include "spmv_rows.hpp"

using namespace asamd;

// ---------------------------------------------------------------------------
// Row-length statistics.  out[0] = min, out[1] = max, out[2] = row_ptr[0],
// out[3 .. 3+2*33) = 64-bit histogram counters as (lo, hi) int pairs summed
// with 32-bit atomics on the low word only: a bin can hold at most m < 2^31.
// ---------------------------------------------------------------------------
constexpr int kStatWords = 3 + ASAMD_HIST_BINS;

__global__ __launch_bounds__(256) void row_stats_kernel(int m, const int* __restrict__ row_ptr,
                                                        int* __restrict__ out) {
  __shared__ int s_hist[ASAMD_HIST_BINS];
  __shared__ int s_min, s_max;
  if (threadIdx.x < ASAMD_HIST_BINS) s_hist[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    s_min = 0x7fffffff;
    s_max = 0;
  }
  __syncthreads();
  int lmin = 0x7fffffff, lmax = 0;
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < m;
       r += (int64_t)gridDim.x * blockDim.x) {
    int len = row_ptr[r + 1] - row_ptr[r];
    if (len < 0) len = 0;  // malformed offsets: counted as empty, never indexed with
    lmin = len < lmin ? len : lmin;
    lmax = len > lmax ? len : lmax;
    const int bin = len == 0 ? 0 : 32 - __builtin_clz((unsigned)len);
    atomicAdd(&s_hist[bin], 1);
  }
  atomicMin(&s_min, lmin);
  atomicMax(&s_max, lmax);
  __syncthreads();
  if (threadIdx.x < ASAMD_HIST_BINS && s_hist[threadIdx.x] != 0)
    atomicAdd(&out[3 + threadIdx.x], s_hist[threadIdx.x]);
  if (threadIdx.x == 0) {
    atomicMin(&out[0], s_min);
    atomicMax(&out[1], s_max);
    if (blockIdx.x == 0) out[2] = row_ptr[0];
  }
}

__global__ void stats_init_kernel(int* out) {
  const int t = threadIdx.x;
  if (t < kStatWords) out[t] = t == 0 ? 0x7fffffff : 0;
}

__global__ void warmup_kernel() {}

__global__ __launch_bounds__(256) void copy_bytes_kernel(Int4* __restrict__ dst,
                                                         const Int4* __restrict__ src, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// ---------------------------------------------------------------------------
struct asamd_csr_plan {
  asamd_csr_stats st;
  int auto_algo;
  int auto_width;
  int val_size;
  int* d_block_row;   // merge-path coordinates, merge_blocks + 1 ints
  int* d_carry_row;   // merge_blocks ints
  void* d_carry_val;  // merge_blocks values
  void* d_head_val;   // merge_blocks values: partial sum of each workgroup's first row
  bool coords_valid;  // d_block_row filled for a structure promised fixed
};

static int width_for_mean(double mean) {
  // lanes per row from the mean row length; same break points as the
  // reference's dispatch (dcu_gemv_vector.h:77,94,111,128,145,162)
  if (mean < 4) return 2;
  if (mean < 8) return 4;
  if (mean < 16) return 8;
  if (mean < 32) return 16;
  if (mean < 64) return 32;
  return 64;
}

static bool rowconst_ok(const asamd_csr_stats& st) {
  const int L = st.const_len;
  return st.trusted && st.first_offset == 0 &&
         (L == 4 || L == 8 || L == 16 || L == 32 || L == 64 || L == 128 || L == 256);
}

static void choose_algo(asamd_csr_plan* p) {
  asamd_csr_stats& st = p->st;
  const double mean = st.m > 0 ? (double)st.nnz / st.m : 0.0;
  const int w = width_for_mean(mean);
  p->auto_width = w;
  if (rowconst_ok(st)) {
    p->auto_algo = ASAMD_SPMV_ROWCONST;
  } else if ((int64_t)st.max_len <= (int64_t)w * 16 && mean >= 6.0) {
    // regular rows: a lane group per row wastes little and needs no LDS
    p->auto_algo = ASAMD_SPMV_VECTOR;
  } else {
    p->auto_algo = ASAMD_SPMV_MERGE;
  }
  st.algo = p->auto_algo;
  st.vector_width = p->auto_width;
}

extern "C" int asamd_csr_plan_create(hipStream_t stream, int32_t m, int32_t n, int32_t nnz,
                                     const int32_t* row_ptr, int32_t base, int32_t val_size,
                                     int32_t trusted, asamd_csr_plan** out) {
  if (!out || !row_ptr || m <= 0 || nnz < 0 || (val_size != 4 && val_size != 8))
    return hipErrorInvalidValue;
  asamd_csr_plan* p = new (std::nothrow) asamd_csr_plan();
  if (!p) return hipErrorOutOfMemory;
  p->st.m = m;
  p->st.n = n;
  p->st.nnz = nnz;
  p->st.base = base;
  p->st.trusted = trusted ? 1 : 0;
  p->val_size = val_size;

  int* d_stats = nullptr;
  hipError_t e = hipMalloc(&d_stats, kStatWords * sizeof(int));
  if (e != hipSuccess) {
    delete p;
    return e;
  }
  stats_init_kernel<<<1, 64, 0, stream>>>(d_stats);
  int grid = (m + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;
  row_stats_kernel<<<grid, 256, 0, stream>>>(m, row_ptr, d_stats);
  int h[kStatWords];
  e = hipMemcpyAsync(h, d_stats, sizeof(h), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(d_stats);
  if (e != hipSuccess) {
    delete p;
    return e;
  }
  p->st.min_len = h[0];
  p->st.max_len = h[1];
  p->st.first_offset = h[2] - base;
  p->st.const_len = h[0] == h[1] ? h[0] : -1;
  for (int b = 0; b < ASAMD_HIST_BINS; ++b) p->st.hist[b] = h[3 + b];

  const int64_t total = (int64_t)m + nnz;
  const int64_t nb = (total + kMergeItems - 1) / kMergeItems;
  p->st.merge_blocks = (int)nb;
  choose_algo(p);

  // merge-path buffers are sized by m + nnz only, so they stay valid even if
  // the structure behind row_ptr changes under an untrusted plan
  e = hipMalloc(&p->d_block_row, (nb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_carry_row, nb * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&p->d_carry_val, nb * (size_t)val_size);
  if (e == hipSuccess) e = hipMalloc(&p->d_head_val, nb * (size_t)val_size);
  if (e != hipSuccess) {
    asamd_csr_plan_destroy(p);
    return e;
  }
  if (p->st.trusted) {
    merge_partition_kernel<<<(int)((nb + 1 + 255) / 256), 256, 0, stream>>>(
        m, nnz, row_ptr, base, (int)nb, p->d_block_row);
    e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      asamd_csr_plan_destroy(p);
      return e;
    }
    p->coords_valid = true;
  }
  *out = p;
  return hipSuccess;
}

extern "C" void asamd_csr_plan_destroy(asamd_csr_plan* p) {
  if (!p) return;
  if (p->d_block_row) (void)hipFree(p->d_block_row);
  if (p->d_carry_row) (void)hipFree(p->d_carry_row);
  if (p->d_carry_val) (void)hipFree(p->d_carry_val);
  if (p->d_head_val) (void)hipFree(p->d_head_val);
  delete p;
}

extern "C" const asamd_csr_stats* asamd_csr_plan_stats(const asamd_csr_plan* p) {
  return p ? &p->st : nullptr;
}

extern "C" int asamd_csr_plan_set_algo(asamd_csr_plan* p, int32_t algo) {
  if (!p) return hipErrorInvalidValue;
  switch (algo) {
    case ASAMD_SPMV_AUTO:
      p->st.algo = p->auto_algo;
      return hipSuccess;
    case ASAMD_SPMV_ROWCONST:
      if (!rowconst_ok(p->st)) return hipErrorInvalidValue;
      p->st.algo = algo;
      return hipSuccess;
    case ASAMD_SPMV_VECTOR:
    case ASAMD_SPMV_MERGE:
    case ASAMD_SPMV_SCALAR:
      p->st.algo = algo;
      return hipSuccess;
    default:
      return hipErrorInvalidValue;
  }
}

// ---------------------------------------------------------------------------
template <typename T, int W>
static void launch_vector(hipStream_t s, const asamd_csr_stats& st, T alpha, const T* val,
                          const int* rp, const int* ci, const T* x, T beta, T* y) {
  constexpr int rows_per_block = kRowsBlock / W;
  const unsigned grid = (unsigned)(((int64_t)st.m + rows_per_block - 1) / rows_per_block);
  spmv_vector_kernel<T, W><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base);
}

template <typename T, int G>
static void launch_rowconst(hipStream_t s, const asamd_csr_stats& st, T alpha, const T* val,
                            const int* ci, const T* x, T beta, T* y) {
  constexpr int R = G >= 16 ? 1 : 2;
  constexpr int rows_per_block = (kRowsBlock / G) * R;
  const unsigned grid = (unsigned)(((int64_t)st.m + rows_per_block - 1) / rows_per_block);
  spmv_rowconst_kernel<T, G, R><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, ci, x, beta, y, st.base);
}

template <typename T>
static int csrmv_impl(hipStream_t s, asamd_csr_plan* p, T alpha, const T* val, const int* rp,
                      const int* ci, const T* x, T beta, T* y) {
  if (!p || !val || !rp || !ci || !x || !y) return hipErrorInvalidValue;
  if (p->val_size != (int)sizeof(T)) return hipErrorInvalidValue;
  const asamd_csr_stats& st = p->st;
  int algo = st.algo;
  if (algo == ASAMD_SPMV_ROWCONST) {
    // 128-bit loads need 16-byte aligned streams; fall back otherwise
    const bool aligned = (((uintptr_t)val | (uintptr_t)ci) & 15u) == 0;
    if (!aligned || !rowconst_ok(st)) algo = ASAMD_SPMV_VECTOR;
  }
  switch (algo) {
    case ASAMD_SPMV_ROWCONST:
      switch (st.const_len / 4) {
        case 1: launch_rowconst<T, 1>(s, st, alpha, val, ci, x, beta, y); break;
        case 2: launch_rowconst<T, 2>(s, st, alpha, val, ci, x, beta, y); break;
        case 4: launch_rowconst<T, 4>(s, st, alpha, val, ci, x, beta, y); break;
        case 8: launch_rowconst<T, 8>(s, st, alpha, val, ci, x, beta, y); break;
        case 16: launch_rowconst<T, 16>(s, st, alpha, val, ci, x, beta, y); break;
        case 32: launch_rowconst<T, 32>(s, st, alpha, val, ci, x, beta, y); break;
        default: launch_rowconst<T, 64>(s, st, alpha, val, ci, x, beta, y); break;
      }
      break;
    case ASAMD_SPMV_SCALAR: {
      const unsigned grid = (unsigned)(((int64_t)st.m + kRowsBlock - 1) / kRowsBlock);
      spmv_scalar_kernel<T><<<grid, kRowsBlock, 0, s>>>(st.m, alpha, val, rp, ci, x, beta, y, st.base);
      break;
    }
    case ASAMD_SPMV_MERGE: {
      const int nb = st.merge_blocks;
      if (!p->coords_valid) {
        merge_partition_kernel<<<(nb + 1 + 255) / 256, 256, 0, s>>>(st.m, st.nnz, rp, st.base, nb,
                                                                    p->d_block_row);
      }
      spmv_merge_kernel<T><<<nb, kMergeThreads, 0, s>>>(st.m, st.nnz, alpha, val, rp, ci, x, beta, y,
                                                        st.base, p->d_block_row, p->d_carry_row,
                                                        (T*)p->d_carry_val, (T*)p->d_head_val);
      if (nb > 1)
        merge_fixup_kernel<T><<<(nb + 255) / 256, 256, 0, s>>>(nb, st.m, alpha, beta, p->d_carry_row,
                                                               (const T*)p->d_carry_val,
                                                               (const T*)p->d_head_val, y);
      break;
    }
    case ASAMD_SPMV_VECTOR:
    default:
      switch (p->auto_width) {
        case 2: launch_vector<T, 2>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 4: launch_vector<T, 4>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 8: launch_vector<T, 8>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 16: launch_vector<T, 16>(s, st, alpha, val, rp, ci, x, beta, y); break;
        case 32: launch_vector<T, 32>(s, st, alpha, val, rp, ci, x, beta, y); break;
        default: launch_vector<T, 64>(s, st, alpha, val, rp, ci, x, beta, y); break;
      }
      break;
  }
  return hipGetLastError();
}

extern "C" int asamd_s_csrmv(hipStream_t stream, asamd_csr_plan* plan, float alpha,
                             const float* val, const int32_t* row_ptr, const int32_t* col_ind,
                             const float* x, float beta, float* y) {
  return csrmv_impl<float>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_d_csrmv(hipStream_t stream, asamd_csr_plan* plan, double alpha,
                             const double* val, const int32_t* row_ptr, const int32_t* col_ind,
                             const double* x, double beta, double* y) {
  return csrmv_impl<double>(stream, plan, alpha, val, row_ptr, col_ind, x, beta, y);
}

extern "C" int asamd_copy_bytes(hipStream_t stream, void* dst, const void* src, size_t nbytes) {
  if (!dst || !src || (nbytes & 15u) || (((uintptr_t)dst | (uintptr_t)src) & 15u))
    return hipErrorInvalidValue;
  const size_t n16 = nbytes / 16;
  if (n16 == 0) return hipSuccess;
  size_t grid = (n16 + 255) / 256;
  if (grid > 256 * 64) grid = 256 * 64;
  copy_bytes_kernel<<<(unsigned)grid, 256, 0, stream>>>((Int4*)dst, (const Int4*)src, n16);
  return hipGetLastError();
}

extern "C" int asamd_warmup(hipStream_t stream) {
  warmup_kernel<<<1, 1, 0, stream>>>();
  return hipGetLastError();
}
