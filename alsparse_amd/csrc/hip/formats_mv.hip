// SpMV for the two formats the CSR converters produce, y = alpha*A*x + beta*y:
//
//   ELL (column-major slots, slot s of row r at [s*m + r]): one lane per row,
//   so the lanes of a wave read consecutive addresses in every slot.  Replaces
//   src/kernel/dcu/level2/mv/dcu_gemv_x_ell.cpp:10-43 (same traversal; the
//   slot loop is unrolled so that four independent gathers are in flight, and
//   the index base of the descriptor is honoured).
//
//   COO (entries grouped by row, as csr2coo leaves them): every wave owns one
//   contiguous run of entries and reduces it 64 at a time with a segmented
//   scan across its lanes (DPP only); the last lane of every row segment adds the
//   segment's sum to y, the open segment at the end of a step is carried into
//   the next one in registers.  Replaces
//   src/kernel/dcu/level2/mv/dcu_gemv_x_coo.cpp:10-195, which stages the same
//   scan through LDS with a barrier per step, writes y without atomics (a row
//   shared by two waves races there) and finishes with a one-workgroup pass.
//   Here the first and the last segment of every wave go to boundary slots and
//   a second kernel adds the slots of one row up in wave order (the
//   reference's carry-out and block reduction, :169-255, as one ordered pass);
//   every sum reaches y through one hardware float atomic.  Entries grouped by
//   row therefore give the same result from run to run, and entries that are
//   not grouped by row at all are still summed correctly (then the order of the
//   additions to a row that turns up in several places is not fixed).  y is
//   scaled by beta beforehand, as in the reference (:161-169).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "alsparse_amd_kernels.h"
#include "device_utils.hpp"
#include "spmv_ell.hpp"
#include "stream_policy.hpp"

namespace asamd {
namespace {

// y <- beta * y ahead of an accumulating kernel (beta == 0 stores zeros without reading)
template <typename T>
__global__ __launch_bounds__(256) void scale_y_kernel(int m, T beta, T* __restrict__ y) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= m) return;
  y[i] = beta == T(0) ? T(0) : y[i] * beta;
}

constexpr int kCooThreads = 256;
constexpr int kCooSteps = 16;                        // 64-entry steps per wave (more when the workspace is short)
constexpr int kCooWaves = kCooThreads / kWave;

// With boundary slots (b_row != nullptr): the wave's first and last row segment -- the ones that may belong
// to rows shared with the neighbouring waves -- do not go to y but to slots 2w (head) and 2w + 1 (tail) of
// the wave; coomv_boundary_kernel adds the runs of equal rows up in wave order and adds each run once.
// Entries that are grouped by row therefore reach every y through a single addition of a sum formed in a
// fixed order: the result is the same from run to run.
// NTI / NTV: the index streams / the values are loaded non-temporally (see stream_policy.hpp)
template <typename T, bool NTI, bool NTV>
__global__ __launch_bounds__(kCooThreads) void coomv_kernel(int64_t nnz, int m, int n, T alpha,
                                                            const T* __restrict__ coo_val,
                                                            const int* __restrict__ coo_row,
                                                            const int* __restrict__ coo_col, int base,
                                                            const T* __restrict__ x, T* __restrict__ y, int per_wave,
                                                            int* __restrict__ b_row, T* __restrict__ b_val) {
  const int lane = threadIdx.x % kWave;
  const int64_t wave = (int64_t)blockIdx.x * kCooWaves + threadIdx.x / kWave;
  const int64_t begin = wave * per_wave;
  const int64_t end = begin + per_wave < nnz ? begin + per_wave : nnz;
  if (begin >= end) {
    if (b_row && lane < 2) b_row[2 * wave + lane] = -1;  // a wave past the end: empty slots
    return;
  }
  const bool slots = b_row != nullptr;
  bool emitted = !slots;  // whether the wave's first segment has gone out (wave-uniform); without slots: nothing special
  int carry_row = -1;     // open segment handed from one step to the next (same in all lanes)
  T carry_val = T(0);
  int head_row = -1;
  T head_val = T(0);
  for (int64_t k0 = begin; k0 < end; k0 += kWave) {
    const int64_t k = k0 + lane;
    int r = -1;
    T v = T(0);
    if (k < end) {
      const int rr = (NTI ? __builtin_nontemporal_load(&coo_row[k]) : coo_row[k]) - base;
      const int c = (NTI ? __builtin_nontemporal_load(&coo_col[k]) : coo_col[k]) - base;
      if ((unsigned)rr < (unsigned)m && (unsigned)c < (unsigned)n) {
        r = rr;
        v = (NTV ? nt_load(coo_val + k) : coo_val[k]) * x[c];
      }
    }
    const int r0 = lane_bcast(r, 0);
    const bool flush = carry_row != r0 && carry_row >= 0;  // the carried segment ended with the last step
    if (flush && !emitted) {
      head_row = carry_row;
      head_val = carry_val;
    }
    if (lane == 0) {
      if (carry_row == r) v += carry_val;
      else if (flush && emitted) atomic_add(&y[carry_row], alpha * carry_val);
    }
    if (flush) emitted = true;
    // rows of the neighbouring lanes through DPP wave shifts (lane 0 sees -2, lane 63 sees -2: never a row)
    const int r_prev = __builtin_amdgcn_update_dpp(-2, r, 0x138, 0xF, 0xF, false);  // wave_shr:1
    const int r_next = __builtin_amdgcn_update_dpp(-2, r, 0x130, 0xF, 0xF, false);  // wave_shl:1
    const bool head = lane == 0 || r_prev != r;
    v = segmented_scan(v, head);
    // the last lane of every row segment adds the segment's sum; lane 63's segment stays open
    const bool ends = lane < kWave - 1 && r_next != r && r >= 0;
    const uint64_t end_mask = __builtin_amdgcn_ballot_w64(ends);
    const int first_end = end_mask ? __builtin_ctzll(end_mask) : kWave;
    if (!emitted && end_mask) {  // the wave's first segment ends inside this step
      head_row = lane_bcast(r, first_end);
      head_val = lane_bcast(v, first_end);
    }
    if (ends && (emitted || lane != first_end)) atomic_add(&y[r], alpha * v);
    if (end_mask) emitted = true;
    carry_row = lane_bcast(r, kWave - 1);
    carry_val = lane_bcast(v, kWave - 1);
  }
  if (!slots) {
    if (lane == 0 && carry_row >= 0) atomic_add(&y[carry_row], alpha * carry_val);
    return;
  }
  if (!emitted) {  // one segment (or none) in the whole wave: it is the head, there is no tail
    head_row = carry_row;
    head_val = carry_val;
    carry_row = -1;
  }
  if (lane == 0) {
    b_row[2 * wave] = head_row;
    b_val[2 * wave] = head_val;
    b_row[2 * wave + 1] = carry_row;
    b_val[2 * wave + 1] = carry_val;
  }
}

// Slot i starts a run if the nearest filled slot below it names another row; the run's sums are added in
// slot order and reach y through one addition (atomic: entries that are not grouped by row may have put the
// same row elsewhere).
template <typename T>
__global__ __launch_bounds__(256) void coomv_boundary_kernel(int64_t slots, T alpha, const int* __restrict__ b_row,
                                                             const T* __restrict__ b_val, T* __restrict__ y) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= slots) return;
  const int r = b_row[i];
  if (r < 0) return;
  int64_t q = i - 1;
  while (q >= 0 && b_row[q] < 0) --q;
  if (q >= 0 && b_row[q] == r) return;
  T sum = b_val[i];
  for (int64_t j = i + 1; j < slots; ++j) {
    const int rj = b_row[j];
    if (rj < 0) continue;
    if (rj != r) break;
    sum += b_val[j];
  }
  atomic_add(&y[r], alpha * sum);
}

template <typename T>
int ellmv_impl(hipStream_t stream, int32_t m, int32_t n, T alpha, const T* ell_val, const int32_t* ell_col,
               int32_t width, int32_t base, const T* x, T beta, T* y) {
  if (m < 0 || n < 0 || width < 0) return (int)hipErrorInvalidValue;
  if (((uintptr_t)ell_val | (uintptr_t)x | (uintptr_t)y) % alignof(T)) return (int)hipErrorInvalidValue;
  if (m == 0) return (int)hipSuccess;
  if constexpr (sizeof(T) <= 8) {
    // two rows per lane where the caller's arrays allow aligned pairs
    if (m % 2 == 0 && (uintptr_t)ell_val % (2 * sizeof(T)) == 0 && (uintptr_t)ell_col % 8 == 0) {
      const unsigned grid2 = (unsigned)(((int64_t)m / 2 + kEllThreads - 1) / kEllThreads);
      const int policy = stream_policy((double)m * width, sizeof(T), ((double)m + (double)n) * (double)sizeof(T), true);
#define ASAMD_ELL_LAUNCH(NTV, NTC) \
  ellmv_multi_kernel<T, 2, NTV, NTC><<<grid2, kEllThreads, 0, stream>>>(m, n, alpha, ell_val, ell_col, width, base, x, beta, y)
      if (policy == 0) ASAMD_ELL_LAUNCH(false, false);
      else if (policy == kStreamNtValues) ASAMD_ELL_LAUNCH(true, false);
      else if (policy == kStreamNtIndices) ASAMD_ELL_LAUNCH(false, true);
      else ASAMD_ELL_LAUNCH(true, true);
#undef ASAMD_ELL_LAUNCH
      return (int)hipGetLastError();
    }
  }
  const unsigned grid = (unsigned)(((int64_t)m + kEllThreads - 1) / kEllThreads);
  ellmv_kernel<T><<<grid, kEllThreads, 0, stream>>>(m, n, alpha, ell_val, ell_col, width, base, x, beta, y);
  return (int)hipGetLastError();
}

template <typename T>
int coomv_impl(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, T alpha, const T* coo_val,
               const int32_t* coo_row, const int32_t* coo_col, int32_t base, const T* x, T beta, T* y, void* workspace,
               size_t workspace_bytes) {
  if (m < 0 || n < 0 || nnz < 0) return (int)hipErrorInvalidValue;
  if (((uintptr_t)coo_val | (uintptr_t)x | (uintptr_t)y) % alignof(T)) return (int)hipErrorInvalidValue;
  if (m == 0) return (int)hipSuccess;
  if (beta != T(1)) {
    scale_y_kernel<T><<<(unsigned)(((int64_t)m + 255) / 256), 256, 0, stream>>>(m, beta, y);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  if (nnz == 0) return (int)hipSuccess;
  // two boundary slots (row, sum) per wave in the workspace; a short workspace means longer waves
  int per_wave = kWave * kCooSteps;
  int* b_row = nullptr;
  T* b_val = nullptr;
  const size_t slot_bytes = 2 * (sizeof(T) + sizeof(int));
  if (workspace && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= 64 * slot_bytes) {
    const int64_t max_waves = (int64_t)(workspace_bytes / slot_bytes) / kCooWaves * kCooWaves;
    int64_t waves = (nnz + per_wave - 1) / per_wave;
    if (waves > max_waves) {
      const int64_t steps = (nnz + max_waves * kWave - 1) / (max_waves * kWave);
      if (steps * kWave < INT32_MAX / 2) per_wave = (int)(steps * kWave);
      waves = (nnz + per_wave - 1) / per_wave;
    }
    if (waves <= max_waves) {
      b_val = (T*)workspace;
      b_row = (int*)((char*)workspace + (size_t)max_waves * 2 * sizeof(T));
    }
  }
  const int64_t per_block = (int64_t)per_wave * kCooWaves;
  const int64_t grid = (nnz + per_block - 1) / per_block;
  if (grid > 0x7fffffff) return (int)hipErrorInvalidValue;
  // (21 M-entry Laplacian, fp64: indices non-temporal and values not 100 us, all three non-temporal 107 us)
  const int policy = stream_policy((double)nnz, sizeof(T), ((double)m + (double)n) * (double)sizeof(T), false, 8.0);
#define ASAMD_COO_LAUNCH(NTI, NTV)                                                                                    \
  coomv_kernel<T, NTI, NTV><<<(unsigned)grid, kCooThreads, 0, stream>>>(nnz, m, n, alpha, coo_val, coo_row, coo_col, base, \
                                                                        x, y, per_wave, b_row, b_val)
  if (policy == 0) ASAMD_COO_LAUNCH(false, false);
  else if (policy == kStreamNtValues) ASAMD_COO_LAUNCH(false, true);
  else if (policy == kStreamNtIndices) ASAMD_COO_LAUNCH(true, false);
  else ASAMD_COO_LAUNCH(true, true);
#undef ASAMD_COO_LAUNCH
  if (b_row) {
    const int64_t slots = grid * kCooWaves * 2;
    coomv_boundary_kernel<T><<<(unsigned)((slots + 255) / 256), 256, 0, stream>>>(slots, alpha, b_row, b_val, y);
  }
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace asamd

extern "C" {

int asamd_s_ellmv(hipStream_t stream, int32_t m, int32_t n, float alpha, const float* ell_val,
                  const int32_t* ell_col_ind, int32_t ell_width, int32_t base, const float* x, float beta,
                  float* y) {
  return asamd::ellmv_impl<float>(stream, m, n, alpha, ell_val, ell_col_ind, ell_width, base, x, beta, y);
}

int asamd_d_ellmv(hipStream_t stream, int32_t m, int32_t n, double alpha, const double* ell_val,
                  const int32_t* ell_col_ind, int32_t ell_width, int32_t base, const double* x, double beta,
                  double* y) {
  return asamd::ellmv_impl<double>(stream, m, n, alpha, ell_val, ell_col_ind, ell_width, base, x, beta, y);
}

int asamd_s_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, float alpha, const float* coo_val,
                  const int32_t* coo_row_ind, const int32_t* coo_col_ind, int32_t base, const float* x,
                  float beta, float* y, void* workspace, size_t workspace_bytes) {
  return asamd::coomv_impl<float>(stream, m, n, nnz, alpha, coo_val, coo_row_ind, coo_col_ind, base, x, beta, y, workspace,
                                  workspace_bytes);
}

int asamd_d_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, double alpha, const double* coo_val,
                  const int32_t* coo_row_ind, const int32_t* coo_col_ind, int32_t base, const double* x,
                  double beta, double* y, void* workspace, size_t workspace_bytes) {
  return asamd::coomv_impl<double>(stream, m, n, nnz, alpha, coo_val, coo_row_ind, coo_col_ind, base, x, beta,
                                   y, workspace, workspace_bytes);
}

// complex element types: the same kernels over Cx<float> / Cx<double>
int asamd_c_ellmv(hipStream_t stream, int32_t m, int32_t n, asamd_complex8 alpha, const asamd_complex8* ell_val,
                  const int32_t* ell_col_ind, int32_t ell_width, int32_t base, const asamd_complex8* x,
                  asamd_complex8 beta, asamd_complex8* y) {
  using T = asamd::Cx<float>;
  return asamd::ellmv_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)ell_val, ell_col_ind, ell_width,
                              base, (const T*)x, T(beta.real, beta.imag), (T*)y);
}

int asamd_z_ellmv(hipStream_t stream, int32_t m, int32_t n, asamd_complex16 alpha, const asamd_complex16* ell_val,
                  const int32_t* ell_col_ind, int32_t ell_width, int32_t base, const asamd_complex16* x,
                  asamd_complex16 beta, asamd_complex16* y) {
  using T = asamd::Cx<double>;
  return asamd::ellmv_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)ell_val, ell_col_ind, ell_width,
                              base, (const T*)x, T(beta.real, beta.imag), (T*)y);
}

int asamd_c_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, asamd_complex8 alpha,
                  const asamd_complex8* coo_val, const int32_t* coo_row_ind, const int32_t* coo_col_ind,
                  int32_t base, const asamd_complex8* x, asamd_complex8 beta, asamd_complex8* y, void* workspace,
                  size_t workspace_bytes) {
  using T = asamd::Cx<float>;
  return asamd::coomv_impl<T>(stream, m, n, nnz, T(alpha.real, alpha.imag), (const T*)coo_val, coo_row_ind,
                              coo_col_ind, base, (const T*)x, T(beta.real, beta.imag), (T*)y, workspace, workspace_bytes);
}

int asamd_z_coomv(hipStream_t stream, int32_t m, int32_t n, int64_t nnz, asamd_complex16 alpha,
                  const asamd_complex16* coo_val, const int32_t* coo_row_ind, const int32_t* coo_col_ind,
                  int32_t base, const asamd_complex16* x, asamd_complex16 beta, asamd_complex16* y, void* workspace,
                  size_t workspace_bytes) {
  using T = asamd::Cx<double>;
  return asamd::coomv_impl<T>(stream, m, n, nnz, T(alpha.real, alpha.imag), (const T*)coo_val, coo_row_ind,
                              coo_col_ind, base, (const T*)x, T(beta.real, beta.imag), (T*)y, workspace, workspace_bytes);
}

}  // extern "C"
