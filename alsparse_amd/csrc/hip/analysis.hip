// Analysis building blocks on the GPU (gfx950): row-length statistics, fingerprints of the structure
// arrays and of the values.  Each entry point is one self-contained operation on plain device arrays;
// the host library's plan strings them together.  The row statistics replace the host-side walk over
// row_ptr of src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:58-267 and its device-to-host round trip
// at :348-379; the fingerprints have no counterpart (the reference's analysis keeps nothing that a change
// of values could invalidate, :382-388).

#include <hip/hip_runtime.h>

#include "alsparse_amd_kernels.h"
#include "launch_utils.hpp"

using namespace asamd;

// ---------------------------------------------------------------------------
// Row-length statistics.  out[0] = min, out[1] = max, out[2] = row_ptr[0],
// out[3 .. 3+33) = histogram counters: a bin can hold at most m < 2^31.
// ---------------------------------------------------------------------------
constexpr int kStatWords = ASAMD_ROW_STATS_WORDS;

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

extern "C" int asamd_csr_row_stats(hipStream_t stream, int32_t m, const int32_t* row_ptr, int32_t* d_scratch,
                                   int32_t* stats_host) {
  if (!row_ptr || !d_scratch || !stats_host || m <= 0) return hipErrorInvalidValue;
  stats_init_kernel<<<1, 64, 0, stream>>>(d_scratch);
  int64_t grid = ((int64_t)m + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;
  row_stats_kernel<<<(unsigned)grid, 256, 0, stream>>>(m, row_ptr, d_scratch);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess)
    e = hipMemcpyAsync(stats_host, d_scratch, kStatWords * sizeof(int), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  return e;
}

// ---------------------------------------------------------------------------
// hash[0] += sum over i of mix(a[i], i + salt): a fingerprint of an index array that does not depend on
// the order of the (integer, wrapping) additions.
// ---------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long mix_index(unsigned long long v, unsigned long long i) {
  unsigned long long z = (v + 0x9E3779B97F4A7C15ull) * 0xBF58476D1CE4E5B9ull ^ (i * 0x94D049BB133111EBull);
  z = (z ^ (z >> 29)) * 0xD6E8FEB86659FD93ull;
  return z ^ (z >> 32);
}

__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long mine) {
  __shared__ unsigned long long s_sum[256 / kWave];
  for (int d = kWave / 2; d > 0; d >>= 1) mine += __shfl_down(mine, d, kWave);
  if (threadIdx.x % kWave == 0) s_sum[threadIdx.x / kWave] = mine;
  __syncthreads();
  unsigned long long total = 0;
  if (threadIdx.x == 0)
    for (int w = 0; w < 256 / kWave; ++w) total += s_sum[w];
  return total;  // valid in thread 0
}

__global__ __launch_bounds__(256) void index_hash_kernel(int64_t n, const int* __restrict__ a, unsigned long long salt,
                                                         unsigned long long* __restrict__ hash) {
  unsigned long long mine = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    mine += mix_index((unsigned long long)(unsigned)nt_load(a + i), (unsigned long long)i + salt);
  const unsigned long long total = block_sum_u64(mine);
  if (threadIdx.x == 0) atomicAdd(hash, total);
}

__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0; }

extern "C" int asamd_csr_structure_hash(hipStream_t stream, int32_t m, int32_t nnz, const int32_t* row_ptr,
                                        const int32_t* col_ind, void* d_scratch, uint64_t* hash_host) {
  if (!row_ptr || !hash_host || !d_scratch || ((uintptr_t)d_scratch & 7u) || m < 0 || nnz < 0 || (nnz > 0 && !col_ind))
    return hipErrorInvalidValue;
  unsigned long long* d_hash = (unsigned long long*)d_scratch;
  zero_u64_kernel<<<1, 1, 0, stream>>>(d_hash);
  index_hash_kernel<<<256 * 8, 256, 0, stream>>>((int64_t)m + 1, row_ptr, 0x1234567ull, d_hash);
  if (nnz > 0) index_hash_kernel<<<256 * 16, 256, 0, stream>>>((int64_t)nnz, col_ind, 0xABCDEF01ull << 8, d_hash);
  hipError_t e = hipGetLastError();
  unsigned long long h = 0;
  if (e == hipSuccess) e = hipMemcpyAsync(&h, d_hash, sizeof(h), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  *hash_host = (uint64_t)h;
  return e;
}

// ---------------------------------------------------------------------------
// Value guard.  The array is taken as 4-byte words in runs of run_words words (64 times a power of two); of
// every run one wave reads 64 consecutive words (256 bytes) at a position that varies from run to run
// (a fixed stride would sample the same memory channels and the same residues over and over), each
// word is mixed with its position, and the sums of all lanes add up to the fingerprint -- integer
// additions, so the order does not matter and equal arrays give equal words.  run_words == 64 reads
// everything.
// ---------------------------------------------------------------------------
constexpr int kGuardBlocks = 2048;
constexpr int kGuardUnroll = 8;
static_assert(ASAMD_GUARD_WS_BYTES >= kGuardBlocks * 8 + 16, "guard scratch holds the partial sums, the word and the flag");

struct GuardWs {
  unsigned long long partial[kGuardBlocks];
  unsigned long long fp;
  int flag;
};
static_assert(offsetof(GuardWs, flag) == 8 * kGuardBlocks + 8, "ASAMD_GUARD_FLAG points at the flag");

// Three 32-bit multiplications per word (they run at a quarter of the rate of an addition, and hashing a
// whole array must stay a memory-bound pass).  For a fixed position the low half is a bijection of the word, so
// one changed word always changes the sum; the position enters both halves, so words that change places do too.
__device__ __forceinline__ unsigned long long mix_word(unsigned w, unsigned long long idx) {
  const unsigned i = (unsigned)idx ^ ((unsigned)(idx >> 32) * 0x9E3779B1u);  // (the high part is wave-uniform)
  const unsigned t = i * 0x85EBCA6Bu;
  unsigned a = (w ^ t) * 0x9E3779B1u;
  a ^= a >> 15;
  unsigned b = (w + ((t >> 7) | (t << 25))) * 0x27D4EB2Fu;
  b ^= b >> 16;
  return ((unsigned long long)b << 32) | a;
}

__global__ __launch_bounds__(256) void value_hash_kernel(const unsigned* __restrict__ words, int64_t total_words,
                                                         int64_t run_words, unsigned long long* __restrict__ partial) {
  const int lane = threadIdx.x % kWave;
  const int64_t waves = (int64_t)gridDim.x * (256 / kWave);
  // (wave-uniform values are made so for the compiler: the position arithmetic then runs on the scalar unit)
  const int64_t wave = (int64_t)blockIdx.x * (256 / kWave) + __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
  const int64_t runs = (total_words + run_words - 1) / run_words;
  const unsigned slot_mask = (unsigned)(run_words / kWave) - 1u;  // positions inside a run: a power of two
  unsigned long long mine = 0;
  for (int64_t r0 = wave; r0 < runs; r0 += waves * kGuardUnroll) {
    unsigned w[kGuardUnroll];
    int64_t idx[kGuardUnroll];
#pragma unroll
    for (int u = 0; u < kGuardUnroll; ++u) {
      const int64_t r = r0 + (int64_t)u * waves;
      const int64_t start = r * run_words;
      int64_t pos = start + (int64_t)((((unsigned)r * 2654435761u) >> 7) & slot_mask) * kWave;
      if (pos >= total_words) pos = start;  // the last, short run
      idx[u] = r < runs && pos + lane < total_words ? pos + lane : -1;
      w[u] = idx[u] >= 0 ? nt_load(words + idx[u]) : 0u;
    }
#pragma unroll
    for (int u = 0; u < kGuardUnroll; ++u)
      if (idx[u] >= 0) mine += mix_word(w[u], (unsigned long long)idx[u]);
  }
  const unsigned long long total = block_sum_u64(mine);
  if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

// Every word of a 16-byte aligned array, four per lane and load: the same sum as value_hash_kernel with runs
// of 64 words (each word is mixed with its own position, and sums do not mind the order).
__global__ __launch_bounds__(256) void value_hash_all_kernel(const Int4* __restrict__ quads, int64_t total_quads,
                                                             unsigned long long* __restrict__ partial) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  unsigned long long mine = 0;
  for (int64_t q0 = (int64_t)blockIdx.x * 256 + threadIdx.x; q0 < total_quads; q0 += stride * kGuardUnroll) {
    Int4 w[kGuardUnroll];
#pragma unroll
    for (int u = 0; u < kGuardUnroll; ++u) {
      const int64_t q = q0 + (int64_t)u * stride;
      w[u] = nt_load_object(quads + (q < total_quads ? q : q0));
    }
#pragma unroll
    for (int u = 0; u < kGuardUnroll; ++u) {
      const int64_t q = q0 + (int64_t)u * stride;
      if (q < total_quads) {
        const unsigned long long i = (unsigned long long)q * 4;
        mine += mix_word((unsigned)w[u].x, i) + mix_word((unsigned)w[u].y, i + 1) + mix_word((unsigned)w[u].z, i + 2) +
                mix_word((unsigned)w[u].w, i + 3);
      }
    }
  }
  const unsigned long long total = block_sum_u64(mine);
  if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

__global__ __launch_bounds__(256) void value_verdict_kernel(GuardWs* __restrict__ ws, int64_t total_words,
                                                            const unsigned long long* __restrict__ stored) {
  unsigned long long mine = 0;
  for (int i = threadIdx.x; i < kGuardBlocks; i += 256) mine += ws->partial[i];
  unsigned long long fp = block_sum_u64(mine);
  if (threadIdx.x == 0) {
    fp ^= (unsigned long long)total_words * 0x9E3779B97F4A7C15ull;
    ws->fp = fp;
    ws->flag = (!stored || *stored != fp) ? 1 : 0;
  }
}

__global__ void value_commit_kernel(const GuardWs* __restrict__ ws, unsigned long long* __restrict__ stored) {
  if (ws->flag) *stored = ws->fp;
}

extern "C" size_t asamd_value_guard_run(size_t nbytes) {
  // 256 bytes of every run, 32 MiB in all at the most: the run is the smallest power of two (in 256-byte
  // units) that gets there
  size_t run = 256;
  while (nbytes / run * 256 > ASAMD_GUARD_FULL_BYTES) run *= 2;
  return run;
}

extern "C" int asamd_value_guard(hipStream_t stream, const void* val, size_t nbytes, int32_t full,
                                 const uint64_t* stored, void* ws) {
  if (!val || !ws || ((uintptr_t)ws & 7u) || ((uintptr_t)val & 3u) || (nbytes & 3u) || nbytes == 0)
    return hipErrorInvalidValue;
  const int64_t total_words = (int64_t)(nbytes / 4);
  const int64_t run_words = (int64_t)((full || nbytes <= ASAMD_GUARD_FULL_BYTES ? (size_t)256 : asamd_value_guard_run(nbytes)) / 4);
  GuardWs* g = (GuardWs*)ws;
  if (run_words == kWave && total_words % 4 == 0 && ((uintptr_t)val & 15u) == 0)
    value_hash_all_kernel<<<kGuardBlocks, 256, 0, stream>>>((const Int4*)val, total_words / 4, g->partial);
  else
    value_hash_kernel<<<kGuardBlocks, 256, 0, stream>>>((const unsigned*)val, total_words, run_words, g->partial);
  value_verdict_kernel<<<1, 256, 0, stream>>>(g, total_words, (const unsigned long long*)stored);
  return hipGetLastError();
}

__global__ void guard_any_kernel(const GuardWs* __restrict__ a, const GuardWs* __restrict__ b, int* __restrict__ out) {
  *out = (a->flag | b->flag) ? 1 : 0;
}

extern "C" int asamd_value_guard_any(hipStream_t stream, const void* ws_a, const void* ws_b, int32_t* out) {
  if (!ws_a || !ws_b || !out) return hipErrorInvalidValue;
  guard_any_kernel<<<1, 1, 0, stream>>>((const GuardWs*)ws_a, (const GuardWs*)ws_b, out);
  return hipGetLastError();
}

extern "C" int asamd_value_guard_commit(hipStream_t stream, const void* ws, uint64_t* stored) {
  if (!ws || !stored) return hipErrorInvalidValue;
  value_commit_kernel<<<1, 1, 0, stream>>>((const GuardWs*)ws, (unsigned long long*)stored);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Locality probe: where do the columns of consecutive entries fall?  `segments` runs of kProbeSegment
// consecutive entries, spread evenly over the entry stream, one workgroup each.  Two counts, both of
// 128-byte lines of x:
//   wave scale     distinct lines among every 64 consecutive entries (one gather instruction of a wave in the
//                  row and merge-path kernels issues that many requests to the L1),
//   segment scale  distinct lines in the whole run (a bitmap in LDS; what a compute unit's neighbourhood of
//                  the stream touches, reuse included).
// Deterministic: the same arrays always give the same counts.
// ---------------------------------------------------------------------------
constexpr int kProbeSegment = 1 << 15;
constexpr int kProbeBits = 1 << 18;  // 32 KiB bitmap

__global__ __launch_bounds__(256) void locality_probe_kernel(int nnz, int base, int elem_shift, int segments,
                                                             const int* __restrict__ col_ind,
                                                             unsigned long long* __restrict__ out) {
  __shared__ unsigned bitmap[kProbeBits / 32];
  for (int i = threadIdx.x; i < kProbeBits / 32; i += 256) bitmap[i] = 0;
  __syncthreads();
  const int lane = threadIdx.x % kWave;
  const int64_t seg_len = nnz < kProbeSegment ? nnz : kProbeSegment;
  const int64_t room = (int64_t)nnz - seg_len;
  const int64_t begin = segments > 1 ? room * blockIdx.x / (segments - 1) : 0;
  unsigned wave_lines = 0, seg_lines = 0, entries = 0;
  for (int64_t k0 = begin + (threadIdx.x / kWave) * kWave; k0 < begin + seg_len; k0 += 256) {
    const int64_t k = k0 + lane;
    const bool live = k < begin + seg_len;
    // 128-byte line of x that the entry's gather touches
    const unsigned line = live ? (unsigned)(((int64_t)(col_ind[k] - base) << elem_shift) >> 7) : 0xFFFFFFFFu;
    // wave scale: a lane counts if no lower lane of the wave has its line
    bool first = live;
    for (int j = 0; j < kWave; ++j) {
      const unsigned other = __shfl(line, j, kWave);
      if (j < lane && other == line) first = false;
    }
    wave_lines += first ? 1u : 0u;
    entries += live ? 1u : 0u;
    if (live) {
      // lines beyond the bitmap fold onto it (a hash: two lines rarely share a bit within one run)
      const unsigned bit = (line ^ (line >> 18) * 0x9E3779B1u) & (kProbeBits - 1);
      const unsigned old = atomicOr(&bitmap[bit >> 5], 1u << (bit & 31));
      seg_lines += (old >> (bit & 31)) & 1u ? 0u : 1u;
    }
  }
  unsigned long long v[3] = {wave_lines, seg_lines, entries};
  for (int q = 0; q < 3; ++q) {
    __syncthreads();  // block_sum_u64 reuses one LDS array
    const unsigned long long total = block_sum_u64(v[q]);
    if (threadIdx.x == 0 && total) atomicAdd(&out[q], total);
  }
}

__global__ void zero3_u64_kernel(unsigned long long* p) {
  if (threadIdx.x < 3) p[threadIdx.x] = 0;
}

extern "C" int asamd_csr_locality_probe(hipStream_t stream, int32_t nnz, int32_t base, int32_t elem_bytes,
                                        const int32_t* col_ind, int32_t segments, void* d_scratch, float* out_host) {
  if (!col_ind || !d_scratch || !out_host || ((uintptr_t)d_scratch & 7u) || nnz < 1 || segments < 1)
    return hipErrorInvalidValue;
  int shift = 0;
  while ((1 << shift) < elem_bytes) ++shift;
  if ((1 << shift) != elem_bytes || elem_bytes > 16) return hipErrorInvalidValue;
  unsigned long long* d = (unsigned long long*)d_scratch;
  zero3_u64_kernel<<<1, 64, 0, stream>>>(d);
  locality_probe_kernel<<<segments, 256, 0, stream>>>(nnz, base, shift, segments, col_ind, d);
  hipError_t e = hipGetLastError();
  unsigned long long h[3] = {0, 0, 0};
  if (e == hipSuccess) e = hipMemcpyAsync(h, d, sizeof(h), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  out_host[0] = h[2] ? (float)((double)h[0] / (double)h[2]) : 0.f;
  out_host[1] = h[2] ? (float)((double)h[1] / (double)h[2]) : 0.f;
  return e;
}
