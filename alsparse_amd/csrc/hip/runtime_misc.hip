// Library start-up, the multiply that allocates nothing, and the one C++-typed helper of the reference's
// test drivers.

#include <hip/hip_runtime.h>

#include <atomic>
#include <vector>

#include "alsparse_amd_kernels.h"
#include "launch_utils.hpp"
#include "spmv_merge.hpp"
#include "spmv_trans.hpp"

using namespace asamd;

__global__ void warmup_kernel() {}

// ---- the multiply that allocates nothing -----------------------------------------------------
// Merge-path SpMV (the kernels of spmv_merge.hpp, 8 items per thread) whose workgroup coordinates,
// carries and head sums live in a fixed device array instead of a caller's workspace.
// The array has four equal quarters of kStaticSlots 4-byte slots: block_row | carry_row | carry_val |
// head_val.  Every slot that a call reads is written by that call first, so nothing has to be cleared
// between calls; two calls that overlap on one device share the array and race.
constexpr int kStaticIpt = 8;
constexpr int kStaticSlots = ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES / 16;
static_assert((int64_t)(kStaticSlots - 1) * kMergeThreads * kStaticIpt == ASAMD_CSRMV_NOALLOC_MAX_ITEMS,
              "the documented limit is what the array holds");
static __device__ __align__(256) unsigned char scratch[ASAMD_CSRMV_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` per device: every GPU holds its own copy of the array.  In host code
// the array's name is only a handle for hipGetSymbolAddress, never a pointer a kernel can take.
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static hipError_t static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

extern "C" int asamd_s_csrmv_noalloc(hipStream_t stream, int32_t m, int32_t n, int32_t nnz, int32_t base,
                                     float alpha, const float* val, const int32_t* row_ptr,
                                     const int32_t* col_ind, const float* x, float beta, float* y) {
  if (m <= 0 || n <= 0 || nnz < 0 || (base != 0 && base != 1) || !row_ptr || !x || !y) return hipErrorInvalidValue;
  if (nnz > 0 && (!val || !col_ind)) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)x | (uintptr_t)y) % alignof(float)) return hipErrorInvalidValue;
  const int64_t total = (int64_t)m + nnz;
  // larger problems need more workgroup slots than the fixed array has, and this call may not allocate
  if (total > ASAMD_CSRMV_NOALLOC_MAX_ITEMS) return hipErrorOutOfMemory;
  if (nnz == 0) {  // y = beta*y
    scale_vec_kernel<float><<<(unsigned)(((int64_t)m + 255) / 256), 256, 0, stream>>>(m, beta, y);
    return hipGetLastError();
  }
  void* base_ptr = nullptr;
  const hipError_t e = static_scratch(&base_ptr);
  if (e != hipSuccess) return e;
  int* block_row = (int*)base_ptr;
  int* carry_row = block_row + kStaticSlots;
  float* carry_val = (float*)(carry_row + kStaticSlots);
  float* head_val = carry_val + kStaticSlots;
  constexpr int kItems = kMergeThreads * kStaticIpt;
  const int nb = (int)((total + kItems - 1) / kItems);
  merge_partition_kernel<<<(nb + 1 + 255) / 256, 256, 0, stream>>>(m, nnz, row_ptr, base, nb, kItems, block_row);
  spmv_merge_kernel<float, kStaticIpt><<<nb, kMergeThreads, 0, stream>>>(m, nnz, alpha, val, row_ptr, col_ind, x, beta,
                                                                         y, base, block_row, carry_row, carry_val,
                                                                         head_val);
  if (nb > 1)
    merge_fixup_kernel<float><<<(nb + 255) / 256, 256, 0, stream>>>(nb, m, alpha, beta, carry_row, carry_val, head_val,
                                                                    y);
  return hipGetLastError();
}

extern "C" int asamd_warmup(hipStream_t stream) {
  // the library's init call: also resolves, for the current device, the address of the fixed array that
  // asamd_s_csrmv_noalloc works in, so that its first call has nothing left to set up
  void* p = nullptr;
  const hipError_t e = static_scratch(&p);
  if (e != hipSuccess) return e;
  warmup_kernel<<<1, 1, 0, stream>>>();
  return hipGetLastError();
}

// Mean of the samples below twice the plain mean: src/util_cpp/handle.cpp:495-510.
extern "C" double get_avg_time(std::vector<double> times) {
  if (times.empty()) return 0.0;
  double avg = 0.0;
  for (double t : times) avg += t;
  avg /= (double)times.size();
  double kept = 0.0;
  int cnt = 0;
  for (double t : times)
    if (t < 2 * avg) {
      kept += t;
      ++cnt;
    }
  return cnt ? kept / cnt : avg;
}
