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
// rows that overlap its chunk -- the largest r with row_ptr[r] - base <= k for
// its first and its last entry -- with two searches over row_ptr in which all
// of its threads probe at once: thread t probes lo + (t + 1) * step, the probes
// are monotone, so the number of them that are not after k says which of the
// 257 pieces holds the answer (three dependent rounds for 2^24 rows).  Every such row then marks the chunk position where it starts
// with its number (LDS integer max, so the last of several empty rows wins),
// and an inclusive running maximum over the positions -- four per thread,
// DPP inside the wave, one LDS word per wave across waves -- gives every
// entry its row.  Work is linear in entries + rows; a binary search per entry
// was LDS-bound (nine dependent reads each: 0.90 ms for 2^28 entries against
// 0.3 ms).  The row-index stream is written as 128-bit pieces, 1 KiB of
// consecutive bytes per wave instruction.
// ---------------------------------------------------------------------------
// Output that the L2s (8 x 4 MiB) cannot hold is written with non-temporal stores: measured on 84 MB to
// 2 GiB of output, csr2coo 30 -> 25 us and 0.266 -> 0.198 ms, csr2ell 129 -> 87 us and 0.90 -> 0.86 ms.
static bool stores_bypass_caches(size_t out_bytes) { return out_bytes > ((size_t)32 << 20); }

constexpr int kCooThreads = 256;
constexpr int kCooRound = kCooThreads * 4;  // entries per scan round
constexpr int kCooRounds = 8;
constexpr int kCooChunk = kCooRound * kCooRounds;  // 8192 entries

// inclusive running maximum of non-negative values over the 64 lanes of a wave (DPP only)
__device__ __forceinline__ int wave_max_scan(int v) {
  v = max(v, dpp_mov_rows<0x111, 0xF>(v));  // row_shr:1
  v = max(v, dpp_mov_rows<0x112, 0xF>(v));  // row_shr:2
  v = max(v, dpp_mov_rows<0x114, 0xF>(v));  // row_shr:4
  v = max(v, dpp_mov_rows<0x118, 0xF>(v));  // row_shr:8
  v = max(v, dpp_mov_rows<0x142, 0xA>(v));  // row_bcast:15 into rows 1 and 3
  v = max(v, dpp_mov_rows<0x143, 0xC>(v));  // row_bcast:31 into rows 2 and 3
  return v;
}

// chunk_row[b] = largest r with row_ptr[r] - base <= b * kCooChunk, for b in [0, chunks]: one thread and
// one binary search per chunk boundary, all of them in flight together (inside the chunk kernel the
// same searches are a chain of dependent loads that each workgroup waits for)
__global__ __launch_bounds__(256) void csr2coo_chunk_rows_kernel(const int* __restrict__ row_ptr, int nnz, int m,
                                                                 int base, int chunks, int* __restrict__ chunk_row) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b > chunks) return;
  int64_t k = (int64_t)b * kCooChunk;
  if (k > nnz - 1) k = nnz - 1;  // the last boundary: the row of the last entry
  int lo = 0, hi = m - 1;
  while (lo < hi) {
    const int mid = (int)(((int64_t)lo + hi + 1) >> 1);
    if ((int64_t)row_ptr[mid] - base <= k) lo = mid;
    else hi = mid - 1;
  }
  chunk_row[b] = lo;
}

// chunk_row: the table above, or null (then every workgroup searches for its own rows)
template <bool NTS>
__global__ __launch_bounds__(kCooThreads) void csr2coo_kernel(const int* __restrict__ row_ptr,
                                                              int nnz, int m,
                                                              int* __restrict__ coo_row, int base,
                                                              const int* __restrict__ chunk_row) {
  __shared__ __align__(16) int s_mark[kCooChunk];
  __shared__ int s_part[kCooRounds * (kCooThreads / kWave)];
  const int64_t k0 = (int64_t)blockIdx.x * kCooChunk;
  int64_t k1 = k0 + kCooChunk;
  if (k1 > nnz) k1 = nnz;
  auto global_off = [&](int r) { return row_ptr[r] - base; };
  // rows [r0, r1] contain entries k0 .. k1-1 (empty rows in between included); the two searches run
  // side by side, so their probes share the memory latency of each round
  int lo0 = 0, hi0 = m - 1, lo1 = 0, hi1 = m - 1;
  if (chunk_row) {
    // rows that start exactly at the next chunk's first entry are included in [r0, r1] this way;
    // their marks fall outside the chunk and are dropped below
    lo0 = hi0 = chunk_row[blockIdx.x];
    lo1 = hi1 = chunk_row[blockIdx.x + 1];
  }
  while (lo0 < hi0 || lo1 < hi1) {
    const int64_t step0 = ((int64_t)hi0 - lo0 + kCooThreads - 1) / kCooThreads;
    const int64_t step1 = ((int64_t)hi1 - lo1 + kCooThreads - 1) / kCooThreads;
    const int64_t p0 = lo0 + ((int64_t)threadIdx.x + 1) * step0;
    const int64_t p1 = lo1 + ((int64_t)threadIdx.x + 1) * step1;
    const bool in0 = step0 > 0 && p0 <= hi0, in1 = step1 > 0 && p1 <= hi1;
    const int64_t off0 = in0 ? global_off((int)p0) : 0, off1 = in1 ? global_off((int)p1) : 0;
    const int below0 = __syncthreads_count(in0 && off0 <= k0);
    const int below1 = __syncthreads_count(in1 && off1 <= k1 - 1);
    if (step0 > 0) {
      const int64_t nlo = lo0 + below0 * step0, nhi = nlo + step0 - 1;
      lo0 = (int)nlo;
      hi0 = (int)(nhi < hi0 ? nhi : hi0);
    }
    if (step1 > 0) {
      const int64_t nlo = lo1 + below1 * step1, nhi = nlo + step1 - 1;
      lo1 = (int)nlo;
      hi1 = (int)(nhi < hi1 ? nhi : hi1);
    }
  }
  const int r0 = lo0, r1 = lo1;
  for (int i = threadIdx.x; i < kCooChunk / 4; i += kCooThreads) reinterpret_cast<Int4*>(s_mark)[i] = Int4{0, 0, 0, 0};
  __syncthreads();
  // row r0 + i (i >= 1) starts after k0 and not after k1 - 1: inside the chunk
  for (int64_t i = 1 + threadIdx.x; i <= (int64_t)r1 - r0; i += kCooThreads) {
    const int64_t pos = (int64_t)row_ptr[r0 + i] - base - k0;
    if (pos > 0 && pos < kCooChunk) atomicMax(&s_mark[pos], (int)i);  // always true for ascending offsets
  }
  __syncthreads();
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const bool wide = (uintptr_t)coo_row % 16 == 0;
  constexpr int kWaves = kCooThreads / kWave;
  // round j covers positions [j * kCooRound, (j + 1) * kCooRound), four per thread.  First every wave
  // scans its part of every round and leaves the part's maximum in LDS; after ONE barrier every
  // thread folds the maxima of the parts before its own into its values.
  int v[kCooRounds][4], before[kCooRounds];
#pragma unroll
  for (int j = 0; j < kCooRounds; ++j) {
    const Int4 mk = reinterpret_cast<const Int4*>(s_mark)[j * kCooThreads + threadIdx.x];
    v[j][0] = mk.x;
    v[j][1] = max(v[j][0], mk.y);
    v[j][2] = max(v[j][1], mk.z);
    v[j][3] = max(v[j][2], mk.w);
    const int incl = wave_max_scan(v[j][3]);
    before[j] = __builtin_amdgcn_update_dpp(0, incl, 0x138, 0xF, 0xF, true);  // wave_shr:1, lane 0 gets 0
    if (lane == kWave - 1) s_part[j * kWaves + wave] = incl;
  }
  __syncthreads();
  int run = 0;  // maximum over all parts before (round j, this wave)
  const int rb = r0 + base;
#pragma unroll
  for (int j = 0; j < kCooRounds; ++j) {
    int lead = run;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int pw = s_part[j * kWaves + w];
      if (w < wave) lead = max(lead, pw);
      run = max(run, pw);
    }
    lead = max(lead, before[j]);
    const int64_t k = k0 + (int64_t)j * kCooRound + 4 * threadIdx.x;
    const int o[4] = {rb + max(lead, v[j][0]), rb + max(lead, v[j][1]), rb + max(lead, v[j][2]), rb + max(lead, v[j][3])};
    if (wide && k + 4 <= k1) {
      if constexpr (NTS) {
        typedef int V4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(V4{o[0], o[1], o[2], o[3]}, reinterpret_cast<V4*>(coo_row + k));
      } else {
        *reinterpret_cast<Int4*>(coo_row + k) = Int4{o[0], o[1], o[2], o[3]};
      }
    } else {
      for (int q = 0; q < 4 && k + q < k1; ++q) coo_row[k + q] = o[q];
    }
  }
}

extern "C" size_t asamd_csr2coo_workspace_bytes(int32_t nnz) {
  if (nnz <= 0) return 0;
  return (size_t)(((int64_t)nnz + kCooChunk - 1) / kCooChunk + 1) * sizeof(int);
}

extern "C" int asamd_csr2coo_ws(hipStream_t stream, const int32_t* row_ptr, int32_t nnz, int32_t m,
                                int32_t* coo_row, int32_t base, void* workspace, size_t workspace_bytes) {
  if (!row_ptr || !coo_row || m <= 0 || nnz <= 0) return hipErrorInvalidValue;
  const int chunks = (int)(((int64_t)nnz + kCooChunk - 1) / kCooChunk);
  int* chunk_row = nullptr;
  if (workspace && workspace_bytes >= asamd_csr2coo_workspace_bytes(nnz) && (uintptr_t)workspace % alignof(int) == 0) {
    chunk_row = (int*)workspace;
    csr2coo_chunk_rows_kernel<<<(unsigned)((chunks + 1 + 255) / 256), 256, 0, stream>>>(row_ptr, nnz, m, base, chunks,
                                                                                        chunk_row);
  }
  if (stores_bypass_caches((size_t)nnz * sizeof(int)))
    csr2coo_kernel<true><<<(unsigned)chunks, kCooThreads, 0, stream>>>(row_ptr, nnz, m, coo_row, base, chunk_row);
  else
    csr2coo_kernel<false><<<(unsigned)chunks, kCooThreads, 0, stream>>>(row_ptr, nnz, m, coo_row, base, chunk_row);
  return hipGetLastError();
}

extern "C" int asamd_csr2coo(hipStream_t stream, const int32_t* row_ptr, int32_t nnz, int32_t m,
                             int32_t* coo_row, int32_t base) {
  return asamd_csr2coo_ws(stream, row_ptr, nnz, m, coo_row, base, nullptr, 0);
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
  // eight rows per thread and trip, all sixteen loads issued before the first is used
  constexpr int kU = 8;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t r0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r0 < m; r0 += kU * stride) {
    int lo[kU], hi[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int64_t r = r0 + u * stride;
      const int64_t q = r < m ? r : r0;  // unconditional loads
      lo[u] = row_ptr[q];
      hi[u] = row_ptr[q + 1];
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) lmax = max(lmax, hi[u] - lo[u]);
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
  // every workgroup ends with one atomic on the same word: few, long-running workgroups
  int grid = (int)(((int64_t)m + 256 * 8 - 1) / (256 * 8));
  if (grid > 1024) grid = 1024;
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

// WIDE: val and col_ind are 16-byte aligned; the staged range is then read as pieces of four entries from the
// multiple of four at or before its start (a quarter of the load instructions); pieces that would reach past
// the end of the arrays -- in the last workgroup only -- are read entry by entry.
template <typename T, bool NTS, bool WIDE>
__global__ __launch_bounds__(kEllRows) void csr2ell_kernel(
    int m, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int csr_base, int ell_base, int width,
    T* __restrict__ ell_val, int* __restrict__ ell_col, const int* __restrict__ gate) {
  if (gate && *gate == 0) return;  // a refresh behind the value guard: nothing has changed
  constexpr int kWindow = sizeof(T) > 8 ? kEllWindow / 2 : kEllWindow;  // at most 32 KiB of staged values
  // staged entry p lives at p + p / 32: lanes read slot s of consecutive rows, i.e. positions a row
  // length apart, and without the skew rows of 16 or 32 entries would all fall into a few LDS banks
  auto at = [](int p) { return p + (p >> 5); };
  __shared__ T s_val[kWindow + kWindow / 32];
  __shared__ int s_col[kWindow + kWindow / 32];
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
  if (staged && WIDE) {
    const int count = (int)(blk_end - blk_begin);
    const int64_t limit = (int64_t)row_ptr[m] - csr_base;  // entries in the arrays
    const int64_t a0 = blk_begin & ~(int64_t)3;
    const int head = (int)(blk_begin - a0);
    const int span = count + head;
    constexpr int kU = 4;  // pieces of each stream in flight per thread before the first LDS write
    for (int p0 = 4 * threadIdx.x; p0 < span; p0 += 4 * kU * kEllRows) {
      Quad<T> v[kU];
      Int4 c[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int k = p0 + u * 4 * kEllRows;
        if (k < span) {
          if (a0 + k + 4 <= limit) {
            v[u].load(val + a0 + k);
            c[u] = *reinterpret_cast<const Int4*>(col_ind + a0 + k);
          } else {
            alignas(32) T tv[4] = {T(0), T(0), T(0), T(0)};
            int tc[4] = {0, 0, 0, 0};
            for (int j = 0; j < 4 && a0 + k + j < limit; ++j) {
              tv[j] = val[a0 + k + j];
              tc[j] = col_ind[a0 + k + j];
            }
            v[u].load(tv);
            c[u] = Int4{tc[0], tc[1], tc[2], tc[3]};
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int k = p0 + u * 4 * kEllRows;
        if (k < span) {
          const int cc[4] = {c[u].x, c[u].y, c[u].z, c[u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int p = k + j - head;
            if (p >= 0 && p < count) {
              s_val[at(p)] = v[u].get(j);
              s_col[at(p)] = cc[j];
            }
          }
        }
      }
    }
    __syncthreads();
  } else if (staged) {
    // eight loads of each stream in flight per thread before the first LDS write: a load-wait-write
    // loop pays the memory latency once per trip
    constexpr int kU = 8;
    const int count = (int)(blk_end - blk_begin);
    for (int p0 = threadIdx.x; p0 < count; p0 += kU * kEllRows) {
      T v[kU];
      int c[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int p = p0 + u * kEllRows;
        const int q = p < count ? p : p0;  // unconditional loads: the tail re-reads a staged entry
        v[u] = val[blk_begin + q];
        c[u] = col_ind[blk_begin + q];
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int p = p0 + u * kEllRows;
        if (p < count) {
          s_val[at(p)] = v[u];
          s_col[at(p)] = c[u];
        }
      }
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
        const int p = (int)(my_begin - blk_begin) + s;
        v = s_val[at(p)];
        c = s_col[at(p)] - csr_base + ell_base;
      } else {
        v = val[my_begin + s];
        c = col_ind[my_begin + s] - csr_base + ell_base;
      }
    }
    const int64_t o = (int64_t)s * m + row;
    if constexpr (NTS) {
      nt_store(v, ell_val + o);
      nt_store(c, ell_col + o);
    } else {
      ell_val[o] = v;
      ell_col[o] = c;
    }
  }
}

template <typename T>
static int csr2ell_impl(hipStream_t stream, int m, const T* val, const int* rp, const int* ci,
                        int csr_base, int ell_base, int width, T* ell_val, int* ell_col,
                        const int* gate = nullptr) {
  if (!val || !rp || !ci || !ell_val || !ell_col || m <= 0 || width < 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)ell_val) % alignof(T)) return hipErrorInvalidValue;
  if (width == 0) return hipSuccess;
  const unsigned grid = (unsigned)(((int64_t)m + kEllRows - 1) / kEllRows);
  const bool nts = stores_bypass_caches((size_t)m * (size_t)width * (sizeof(T) + sizeof(int)));
  const bool wide = (((uintptr_t)val | (uintptr_t)ci) & 15u) == 0;
#define ASAMD_CSR2ELL(NTS, WIDE) \
  csr2ell_kernel<T, NTS, WIDE><<<grid, kEllRows, 0, stream>>>(m, val, rp, ci, csr_base, ell_base, width, ell_val, ell_col, gate)
  if (nts && wide) ASAMD_CSR2ELL(true, true);
  else if (nts) ASAMD_CSR2ELL(true, false);
  else if (wide) ASAMD_CSR2ELL(false, true);
  else ASAMD_CSR2ELL(false, false);
#undef ASAMD_CSR2ELL
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

// Elements copied bit for bit: only their size matters.  gate: see asamd_value_guard.
extern "C" int asamd_csr2ell_gated(hipStream_t stream, int32_t elem_bytes, int32_t m, const void* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, int32_t csr_base, int32_t ell_base,
                                   int32_t width, void* ell_val, int32_t* ell_col, const int32_t* gate) {
  if (elem_bytes == 4)
    return csr2ell_impl<float>(stream, m, (const float*)val, row_ptr, col_ind, csr_base, ell_base, width,
                               (float*)ell_val, ell_col, gate);
  if (elem_bytes == 8)
    return csr2ell_impl<double>(stream, m, (const double*)val, row_ptr, col_ind, csr_base, ell_base, width,
                                (double*)ell_val, ell_col, gate);
  if (elem_bytes == 16) {
    using T = asamd::Cx<double>;
    return csr2ell_impl<T>(stream, m, (const T*)val, row_ptr, col_ind, csr_base, ell_base, width, (T*)ell_val,
                           ell_col, gate);
  }
  return hipErrorInvalidValue;
}
