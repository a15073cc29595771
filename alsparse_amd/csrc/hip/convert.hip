// CSR -> COO and CSR -> ELL on the GPU for gfx950 (wave64).
//
// The reference declares these device conversions but never defines them
// (include/alphasparse/spapi_dcu.h:3113, :3303, :3312); the output conventions
// are those of its host converters:
//   COO  src/core/format/convert_coo_x_csr.c:30-37   row index of every entry
//   ELL  src/core/format/convert_ell_x_coo.c:46-79   width = longest row,
//        column-major [slot*m + row], padding value 0 / index 0.
// Pure index streaming: outputs are bit-exact functions of the inputs.

#include <hip/hip_runtime.h>

#include "alsparse_amd_kernels.h"
#include "device_utils.hpp"

using namespace asamd;

// ---------------------------------------------------------------------------
// csr2coo: each workgroup owns kCooChunk consecutive entries.  It finds the
// rows that overlap its chunk with two binary searches over row_ptr, stages
// their offsets in LDS and lets every entry locate its row by a binary search
// in LDS; the row-index stream is written fully coalesced.  Chunks overlapped
// by more rows than the LDS window holds (long runs of empty rows) search
// row_ptr in global memory instead.
// ---------------------------------------------------------------------------
constexpr int kCooThreads = 256;
constexpr int kCooPerThread = 16;
constexpr int kCooChunk = kCooThreads * kCooPerThread;  // 4096 entries
constexpr int kCooWindow = 4096;                        // staged row offsets

// largest r in [lo, hi] with row_ptr[r] - base <= k   (row_ptr[lo] - base <= k holds)
template <typename P>
__device__ __forceinline__ int last_row_not_after(P offsets, int lo, int hi, int64_t k) {
  while (lo < hi) {
    const int mid = (int)(((int64_t)lo + hi + 1) >> 1);
    if ((int64_t)offsets(mid) <= k) {
      lo = mid;
    } else {
      hi = mid - 1;
    }
  }
  return lo;
}

__global__ __launch_bounds__(kCooThreads) void csr2coo_kernel(const int* __restrict__ row_ptr,
                                                              int nnz, int m,
                                                              int* __restrict__ coo_row, int base) {
  __shared__ int s_off[kCooWindow + 1];
  __shared__ int s_r0, s_r1;
  const int64_t k0 = (int64_t)blockIdx.x * kCooChunk;
  int64_t k1 = k0 + kCooChunk;
  if (k1 > nnz) k1 = nnz;
  auto global_off = [&](int r) { return row_ptr[r] - base; };
  if (threadIdx.x == 0) {
    // rows [r0, r1] contain entries k0 .. k1-1 (empty rows in between included)
    const int r0 = last_row_not_after(global_off, 0, m - 1, k0);
    const int r1 = last_row_not_after(global_off, r0, m - 1, k1 - 1);
    s_r0 = r0;
    s_r1 = r1;
  }
  __syncthreads();
  const int r0 = s_r0, r1 = s_r1;
  const int span = r1 - r0 + 1;
  if (span <= kCooWindow) {
    for (int i = threadIdx.x; i < span; i += kCooThreads) s_off[i] = row_ptr[r0 + i] - base;
    __syncthreads();
    auto lds_off = [&](int i) { return s_off[i]; };
#pragma unroll 4
    for (int s = 0; s < kCooPerThread; ++s) {
      const int64_t k = k0 + threadIdx.x + (int64_t)s * kCooThreads;
      if (k < k1) coo_row[k] = r0 + last_row_not_after(lds_off, 0, span - 1, k) + base;
    }
  } else {
    for (int s = 0; s < kCooPerThread; ++s) {
      const int64_t k = k0 + threadIdx.x + (int64_t)s * kCooThreads;
      if (k < k1) coo_row[k] = last_row_not_after(global_off, r0, r1, k) + base;
    }
  }
}

extern "C" int asamd_csr2coo(hipStream_t stream, const int32_t* row_ptr, int32_t nnz, int32_t m,
                             int32_t* coo_row, int32_t base) {
  if (!row_ptr || !coo_row || m <= 0 || nnz <= 0) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)(((int64_t)nnz + kCooChunk - 1) / kCooChunk);
  csr2coo_kernel<<<grid, kCooThreads, 0, stream>>>(row_ptr, nnz, m, coo_row, base);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// csr2ell_width: max over rows of row_ptr[r+1] - row_ptr[r].
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void max_row_len_kernel(int m, const int* __restrict__ row_ptr,
                                                          int* __restrict__ out) {
  __shared__ int s_max;
  if (threadIdx.x == 0) s_max = 0;
  __syncthreads();
  int lmax = 0;
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < m;
       r += (int64_t)gridDim.x * blockDim.x) {
    const int len = row_ptr[r + 1] - row_ptr[r];
    lmax = len > lmax ? len : lmax;
  }
  atomicMax(&s_max, lmax);
  __syncthreads();
  if (threadIdx.x == 0) atomicMax(out, s_max);
}

__global__ void zero_int_kernel(int* p) { *p = 0; }

extern "C" int asamd_csr2ell_width(hipStream_t stream, int32_t m, const int32_t* row_ptr,
                                   int32_t* width_host) {
  if (!row_ptr || !width_host || m <= 0) return hipErrorInvalidValue;
  int* d = nullptr;
  hipError_t e = hipMalloc(&d, sizeof(int));
  if (e != hipSuccess) return e;
  zero_int_kernel<<<1, 1, 0, stream>>>(d);
  int grid = (m + 255) / 256;
  if (grid > 4096) grid = 4096;
  max_row_len_kernel<<<grid, 256, 0, stream>>>(m, row_ptr, d);
  e = hipMemcpyAsync(width_host, d, sizeof(int), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(d);
  return e;
}

// ---------------------------------------------------------------------------
// csr2ell: a workgroup owns kEllRows consecutive rows.  Their entries form one
// contiguous range of the CSR streams, which is read coalesced into LDS in
// windows; slot s of row j is then written to [s*m + j], consecutive lanes on
// consecutive rows, so both sides of the transpose stay coalesced.  Rows longer
// than the LDS window are read from global memory directly.
// ---------------------------------------------------------------------------
constexpr int kEllRows = 256;
constexpr int kEllWindow = 4096;  // staged entries per workgroup pass (half of it for 16-byte values)

template <typename T>
__global__ __launch_bounds__(kEllRows) void csr2ell_kernel(
    int m, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int csr_base, int ell_base, int width,
    T* __restrict__ ell_val, int* __restrict__ ell_col) {
  constexpr int kWindow = sizeof(T) > 8 ? kEllWindow / 2 : kEllWindow;  // at most 32 KiB of staged values
  __shared__ T s_val[kWindow];
  __shared__ int s_col[kWindow];
  const int64_t row_first = (int64_t)blockIdx.x * kEllRows;
  const int64_t row = row_first + threadIdx.x;
  int64_t row_last = row_first + kEllRows;
  if (row_last > m) row_last = m;
  const int64_t blk_begin = (int64_t)row_ptr[row_first] - csr_base;
  const int64_t blk_end = (int64_t)row_ptr[row_last] - csr_base;
  int64_t my_begin = 0, my_end = 0;
  if (row < m) {
    my_begin = (int64_t)row_ptr[row] - csr_base;
    my_end = (int64_t)row_ptr[row + 1] - csr_base;
  }
  const bool staged = blk_end - blk_begin <= kWindow;  // workgroup-uniform
  if (staged) {
    for (int64_t k = blk_begin + threadIdx.x; k < blk_end; k += kEllRows) {
      s_val[k - blk_begin] = val[k];
      s_col[k - blk_begin] = col_ind[k];
    }
    __syncthreads();
  }
  if (row >= m) return;
  const int len = (int)(my_end - my_begin);
  for (int s = 0; s < width; ++s) {
    T v = T(0);
    int c = ell_base;
    if (s < len) {
      if (staged) {
        v = s_val[my_begin - blk_begin + s];
        c = s_col[my_begin - blk_begin + s] - csr_base + ell_base;
      } else {
        v = val[my_begin + s];
        c = col_ind[my_begin + s] - csr_base + ell_base;
      }
    }
    const int64_t o = (int64_t)s * m + row;
    ell_val[o] = v;
    ell_col[o] = c;
  }
}

template <typename T>
static int csr2ell_impl(hipStream_t stream, int m, const T* val, const int* rp, const int* ci,
                        int csr_base, int ell_base, int width, T* ell_val, int* ell_col) {
  if (!val || !rp || !ci || !ell_val || !ell_col || m <= 0 || width < 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)ell_val) % alignof(T)) return hipErrorInvalidValue;
  if (width == 0) return hipSuccess;
  const unsigned grid = (unsigned)(((int64_t)m + kEllRows - 1) / kEllRows);
  csr2ell_kernel<T><<<grid, kEllRows, 0, stream>>>(m, val, rp, ci, csr_base, ell_base, width, ell_val,
                                                   ell_col);
  return hipGetLastError();
}

extern "C" int asamd_s_csr2ell(hipStream_t stream, int32_t m, const float* val,
                               const int32_t* row_ptr, const int32_t* col_ind, int32_t csr_base,
                               int32_t ell_base, int32_t width, float* ell_val, int32_t* ell_col) {
  return csr2ell_impl<float>(stream, m, val, row_ptr, col_ind, csr_base, ell_base, width, ell_val,
                             ell_col);
}

extern "C" int asamd_d_csr2ell(hipStream_t stream, int32_t m, const double* val,
                               const int32_t* row_ptr, const int32_t* col_ind, int32_t csr_base,
                               int32_t ell_base, int32_t width, double* ell_val, int32_t* ell_col) {
  return csr2ell_impl<double>(stream, m, val, row_ptr, col_ind, csr_base, ell_base, width, ell_val,
                              ell_col);
}

// Complex values are copied bit for bit and the padding is all-zero bits, so the 8-byte
// complex type runs the fp64 instantiation; the 16-byte one has its own.
extern "C" int asamd_c_csr2ell(hipStream_t stream, int32_t m, const asamd_complex8* val,
                               const int32_t* row_ptr, const int32_t* col_ind, int32_t csr_base,
                               int32_t ell_base, int32_t width, asamd_complex8* ell_val, int32_t* ell_col) {
  return csr2ell_impl<double>(stream, m, (const double*)val, row_ptr, col_ind, csr_base, ell_base, width,
                              (double*)ell_val, ell_col);
}

extern "C" int asamd_z_csr2ell(hipStream_t stream, int32_t m, const asamd_complex16* val,
                               const int32_t* row_ptr, const int32_t* col_ind, int32_t csr_base,
                               int32_t ell_base, int32_t width, asamd_complex16* ell_val, int32_t* ell_col) {
  using T = asamd::Cx<double>;
  return csr2ell_impl<T>(stream, m, (const T*)val, row_ptr, col_ind, csr_base, ell_base, width, (T*)ell_val,
                         ell_col);
}
